"""Kukupel, plainly: one function per mechanism, written from the design's equations in float64 on
the CPU, token by token where the design is recurrent.  It shares no code with the library; the
tests compare the engine with it.

Notation: h holds a sublayer's input rows [T, E]; a matrix W [out, in] acts on a row as W h,
which for all rows at once is h @ W.T.
"""
from __future__ import annotations

import math

import torch


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def short_conv_silu(x, w):
    """x [T, C], w [C, taps]: y[t] = sum_j w[:, j] x[t - (taps - 1 - j)] with zeros before t = 0,
    then y * sigmoid(y)."""
    T, taps = x.shape[0], w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                y[t] += w[:, j] * x[src]
    return y * torch.sigmoid(y)


def unit(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def delta_recurrence(q, k, v, beta, g):
    """q, k [T, H, dk]; v [T, H, dv]; beta [T, H]; g [T, H, dk].  Per head, from S = 0:
    S <- g * S (rows); u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, dk, dv, dtype=q.dtype)
    o = torch.zeros(T, H, dv, dtype=q.dtype)
    for t in range(T):
        for h in range(H):
            Sh = S[h] * g[t, h][:, None]
            u = beta[t, h] * (v[t, h] - Sh.T @ k[t, h])
            Sh = Sh + torch.outer(k[t, h], u)
            o[t, h] = Sh.T @ q[t, h]
            S[h] = Sh
    return o


def delta_rule(h, w, p, m, eps, beside_attention):
    """The gated delta rule mixer with the tensors `p`*; `beside_attention`: a decay a key channel
    and a sigmoid gate, both through a low rank, else a decay a head and a silu gate."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T, rep = h.shape[0], m["heads"] // m["kv_heads"]
    q = short_conv_silu(h @ w[p + "q"].T, w[p + "q.conv"]).view(T, G, dk)
    k = short_conv_silu(h @ w[p + "k"].T, w[p + "k.conv"]).view(T, G, dk)
    v = short_conv_silu(h @ w[p + "v"].T, w[p + "v.conv"]).view(T, H, dv)
    q = (unit(q) * dk ** -0.5).repeat_interleave(rep, dim=1)
    k = unit(k).repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(h @ w[p + "b"].T)
    rate = torch.exp(w[p + "A_log"])
    if beside_attention:
        a = ((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).view(T, H, dk)
        g = torch.exp(-rate[None, :, None] * softplus(a))
        gate = torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).view(T, H, dv)
    else:
        a = h @ w[p + "a"].T + w[p + "dt_bias"]
        g = torch.exp(-rate[None, :] * softplus(a))[:, :, None].expand(T, H, dk)
        z = (h @ w[p + "g"].T).view(T, H, dv)
        gate = z * torch.sigmoid(z)
    o = delta_recurrence(q, k, v, beta, g)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * w[p + "norm"] * gate
    return o.reshape(T, H * dv) @ w[p + "o"].T


def capped_attention(h, w, p, m):
    """softmax over j <= i of softcap * tanh(q_i . k_j * scale / softcap), times the values."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T, rep = h.shape[0], m["heads"] // m["kv_heads"]
    q = (h @ w[p + "q"].T).view(T, H, dk)
    k = (h @ w[p + "k"].T).view(T, G, dk)
    v = (h @ w[p + "v"].T).view(T, G, dv)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    cap = m.get("softcap", 0) or 0
    for i in range(T):
        for hh in range(H):
            s = (k[: i + 1, hh // rep] @ q[i, hh]) * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            out[i, hh] = torch.softmax(s, 0) @ v[: i + 1, hh // rep]
    return out.reshape(T, H * dv) @ w[p + "o"].T


def experts(h, w, p, mlp, margins=None):
    """Every token's `top` experts by sigmoid(router); out = sum expert(score * h);
    expert(x) = W_down (g sigmoid(1.702 g) (u + 1)), g = min(W_gate x, limit), u = clamp(W_up x).
    `margins` (a tensor [T]) is lowered to the distance between the last chosen and the first
    unchosen score, for tests of arithmetic that rounds: a close call may go either way there."""
    top, lim = mlp["router"]["top"], mlp["expert"]["limit"]
    s = torch.sigmoid(h @ w[p + "router"].T)
    if margins is not None and top < s.shape[1]:
        ranked = torch.sort(s, dim=1, descending=True).values
        margins.copy_(torch.minimum(margins, ranked[:, top - 1] - ranked[:, top]))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in torch.topk(s[t], top).indices.tolist():
            x = s[t, e] * h[t]
            g = torch.clamp(w[f"{p}e{e}.gate"] @ x, max=lim)
            u = torch.clamp(w[f"{p}e{e}.up"] @ x, -lim, lim)
            out[t] += w[f"{p}e{e}.down"] @ (g * torch.sigmoid(1.702 * g) * (u + 1))
    return out


def mixer(h, w, i, layer, eps):
    m, p = layer["mixer"], f"l{i}.mix."
    if layer["type"] == "delta":
        return delta_rule(h, w, p, m, eps, False)
    return (m["left_scale"] * capped_attention(h, w, p + "left.", m["left"])
            + m["right_scale"] * delta_rule(h, w, p + "right.", m["right"], eps, True))


def forward(config, w, tokens, layers_out=None, margins=None):
    """Logits [T, vocab] of one sequence from its first token.  `margins`: see `experts`."""
    eps, S = config["norm"]["eps"], config.get("streams", 0)
    x = w["embed"][torch.tensor(list(tokens))]
    xs = [x.clone() for _ in range(max(S, 1))]
    for i, layer in enumerate(config["layers"]):
        for q in (1, 2):
            hc = f"l{i}.hc{q}."
            if q == 2 and layer.get("mlp") is None:
                if S and hc + "mix" in w:        # no sublayer, but a mix matrix: the streams are still mixed
                    xs = [sum(w[hc + "mix"][s, t] * xs[s] for s in range(S)) for t in range(S)]
                continue
            u = sum(w[hc + "in"][s] * xs[s] for s in range(S)) if S else xs[0]
            hn = rms_norm(u, w[f"l{i}.norm{q}"], eps)
            y = mixer(hn, w, i, layer, eps) if q == 1 else experts(hn, w, f"l{i}.mlp.", layer["mlp"], margins)
            if S:
                xs = [sum(w[hc + "mix"][s, t] * xs[s] for s in range(S)) + w[hc + "out"][t] * y
                      for t in range(S)]
            else:
                xs = [xs[0] + y]
        if layers_out is not None:
            layers_out.append(sum(xs))
    return rms_norm(sum(xs), w["final.norm"], eps) @ w["embed"].T


def greedy(config, w, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(torch.argmax(forward(config, w, ids)[-1])))
    return ids[len(prompt):]


def decided_rows(config, w, tokens, least=0.01):
    """The number of leading positions at which every router's choice is decided by at least
    `least`: arithmetic that rounds activations gives the same experts there; from the first
    close call on it may choose otherwise, and a recurrent layer carries that to every later
    position."""
    margins = torch.full((len(tokens),), math.inf, dtype=torch.float64)
    forward(config, w, tokens, margins=margins)
    close_calls = (margins < least).nonzero()
    return int(close_calls[0]) if len(close_calls) else len(tokens)
