"""A plain, slow Rabapel on the CPU, written from the design's equations, one function per
mechanism: the oracle of the tests.  It shares no code with the engine: it materialises every
head's keys and values from the latent rows, masks with a full matrix and loops over experts.

Everything is computed in the dtype of the tensors it is handed (the tests pass float64).
`cfg` is the dict of a config.json; `w` maps tensor names to tensors.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms(x, eps) * weight


def rotary_frequencies(rot: dict, dtype=torch.float64):
    """(frequencies [dims/2], factor that multiplies cos and sin) of a `rot` entry."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=dtype)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):                   # the dimension whose wave makes `turns` turns over `orig`
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """Rotate the pairs (2i, 2i+1), i < dims/2, of the last axis of x [T, ..., n] by p * f_i."""
    dims = int(rot["dims"])
    f, gain = rotary_frequencies(rot, x.dtype)
    ang = positions.to(x.dtype)[:, None] * f[None, :]                 # [T, dims/2]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = (torch.cos(ang) * gain).view(shape), (torch.sin(ang) * gain).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def window_mask(T: int, size: Optional[int]) -> torch.Tensor:
    """[T, T] True where query i sees key j: 0 <= i - j (< size)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = (i - j) >= 0
    if size:
        ok &= (i - j) < int(size)
    return ok


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                     positions: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The mixer on the rows h [T, width] of one sequence; tensors `p + name`."""
    T = h.shape[0]
    H, dn, dr, dv, R = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(T) if positions is None else positions
    q = (h @ w[p + "q"].T).view(T, H, dn + dr)
    down = h @ w[p + "dkv"].T
    c = rms_norm(down[:, :R], w[p + "dkv.norm"], eps)
    k_rot = down[:, R:]
    k_plain = (c @ w[p + "uk"].T).view(T, H, dn)
    val = (c @ w[p + "uv"].T).view(T, H, dv)
    q_rot, k_rot = q[..., dn:], k_rot[:, None, :]
    if m.get("rot"):
        q_rot = rotate(q_rot, pos, m["rot"])
        k_rot = rotate(k_rot, pos, m["rot"])
    s = torch.einsum("ihd,jhd->hij", q[..., :dn], k_plain)
    s = s + torch.einsum("ihd,jd->hij", q_rot, k_rot[:, 0, :])
    s = s * float(m["scale"])
    see = window_mask(T, (m.get("mask") or {}).get("size"))
    s = s.masked_fill(~see[None], float("-inf"))
    a = torch.softmax(s, dim=-1)
    o = torch.einsum("hij,jhd->ihd", a, val)
    gate = torch.sigmoid(h @ w[p + "g"].T)                            # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * dv) @ w[p + "o"].T


def dense_ff(h, w, p):
    return torch.relu(h @ w[p + "up"].T) ** 2 @ w[p + "down"].T


def gated_ff(h, w, p):
    g = h @ w[p + "gate"].T
    return (g * torch.sigmoid(g) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, w, p, r: dict):
    """(chosen [T, top], weights [T, top]) over real experts followed by identity experts."""
    z = h @ w[p + "router"].T
    s = torch.softmax(z, dim=-1)
    pick = s + w[p + "correction"] if (p + "correction") in w else s
    chosen = torch.topk(pick, int(r["top"]), dim=-1).indices
    return chosen, torch.gather(s, 1, chosen)


def moe_ff(h, w, p, mlp: dict):
    r = mlp["router"]
    n_real = int(r["experts"])
    chosen, weight = route(h, w, p, r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(chosen[t].tolist(), weight[t]):
            y = gated_ff(h[t:t + 1], w, f"{p}e{e}.")[0] if e < n_real else h[t]
            out[t] += g * y
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ w[p + "shared.sg"].T) * gated_ff(h, w, p + "shared.")
    return out


def feed_forward(h, w, p, mlp: Optional[dict]):
    if mlp is None:
        return torch.zeros_like(h)
    if mlp["kind"] == "dense":
        return dense_ff(h, w, p)
    if mlp["kind"] == "moe":
        return moe_ff(h, w, p, mlp)
    raise ValueError(mlp["kind"])


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], layers_out: Optional[list] = None):
    """Logits [T, vocab] of one sequence; `layers_out` collects the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] != "latent_attention":
            raise ValueError(layer["type"])
        h = rms_norm(x, w[f"l{i}.norm1"], eps)
        x = x + (latent_attention(h, w, f"l{i}.mix.", layer["mixer"], eps)
                 + feed_forward(h, w, f"l{i}.mlp.", layer.get("mlp")))
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T


def generate_greedy(cfg, w, prompt: List[int], n: int) -> List[int]:
    seq, out = list(prompt), []
    for _ in range(n):
        tok = int(torch.argmax(forward(cfg, w, seq)[-1]))
        out.append(tok)
        seq.append(tok)
    return out
