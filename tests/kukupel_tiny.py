"""Tiny Kukupel configurations and helpers for the tests.  Sizes differ from layer to layer and
avoid equal or trivial values: attention with 6/2, 4/4 and 3/1 heads, key sizes above and below the
value size, delta-rule heads with and without shared q/k heads, 2 to 5 taps, 1 to 3 experts a
token, 2 and 5 residual streams and none, layers without feed-forward, every order of the two
kinds of layer."""
from __future__ import annotations

import os

import torch

import plain_kukupel as P


def _par(left, right, ls=0.9, rs=1.3):
    heads, kv, dim, vdim, scale, cap = left
    rh, rkv, rdim, rvdim, conv, ra, rg = right
    return {"left": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "softcap": cap},
            "right": {"heads": rh, "kv_heads": rkv, "dim": rdim, "vdim": rvdim, "conv": conv,
                      "decay_rank": ra, "gate_rank": rg},
            "left_scale": ls, "right_scale": rs}


def _delta(heads, kv, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}


def _moe(ff, n, top, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": n, "top": top}}


MIXED = {"architecture": "Kukupel", "vocab": 300, "width": 96, "norm": {"eps": 1e-5}, "streams": 2,
         "layers": [
             {"type": "delta", "mixer": _delta(3, 3, 24, 40, 2), "mlp": _moe(48, 5, 2, 1.5)},
             {"type": "parallel", "mixer": _par((6, 2, 16, 40, 0.3, 8.0), (4, 2, 20, 12, 4, 7, 9)),
              "mlp": _moe(40, 3, 1, 0.8)},
             {"type": "parallel", "mixer": _par((4, 4, 48, 24, 0.2, 3.0), (2, 1, 36, 28, 5, 5, 3), 1.4, 0.6),
              "mlp": None},
             {"type": "delta", "mixer": _delta(6, 2, 12, 20, 3), "mlp": _moe(24, 7, 3, 2.0)},
         ]}

# a width that is no multiple of 4, five streams, equal key and value sizes (the shared attention
# kernels in bfloat16), no cap in one layer, a delta rule with one head
ODD = {"architecture": "Kukupel", "vocab": 131, "width": 90, "norm": {"eps": 3e-6}, "streams": 5,
       "layers": [
           {"type": "parallel", "mixer": _par((3, 1, 32, 32, 0.15, 5.0), (1, 1, 30, 50, 3, 4, 6)),
            "mlp": _moe(30, 2, 2, 1.0)},
           {"type": "parallel", "mixer": _par((4, 2, 16, 16, 0.3, 0), (5, 5, 10, 6, 2, 3, 3)),
            "mlp": _moe(20, 4, 1, 3.0)},
       ]}

# one residual stream: plain pre-norm layers
PLAIN = {"architecture": "Kukupel", "vocab": 150, "width": 64, "norm": {"eps": 1e-6},
         "layers": [
             {"type": "parallel", "mixer": _par((2, 1, 24, 16, 0.25, 6.0), (2, 2, 16, 24, 4, 6, 6)),
              "mlp": _moe(32, 3, 2, 1.2)},
             {"type": "delta", "mixer": _delta(4, 1, 16, 8, 4), "mlp": _moe(16, 2, 1, 0.9)},
         ]}

# delta-rule layers only: nothing is kept per token
NO_KEYS = {"architecture": "Kukupel", "vocab": 120, "width": 48, "norm": {"eps": 1e-5}, "streams": 3,
           "layers": [{"type": "delta", "mixer": _delta(2, 2, 20, 12, 3), "mlp": _moe(24, 3, 1, 1.0)},
                      {"type": "delta", "mixer": _delta(3, 1, 8, 16, 4), "mlp": None}]}


def single(kind="parallel", streams=3, left=(4, 2, 16, 24, 0.25, 10.0), right=(2, 2, 16, 12, 3, 4, 4),
           delta=(2, 2, 16, 12, 4), mlp=None, width=64, vocab=200):
    """One layer, for tests that plant a key or a memory."""
    mixer = _par(left, right) if kind == "parallel" else _delta(*delta)
    cfg = {"architecture": "Kukupel", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
           "layers": [{"type": kind, "mixer": mixer, "mlp": mlp}]}
    if streams:
        cfg["streams"] = streams
    return cfg


def write_model(tmp, config: dict, seed: int, dtype=torch.float32, gain: float = 4.0, edit=None) -> str:
    """A random model folder for `config`; every matrix of the layers times `gain` (with the
    library's small random weights a wrong key or a lost state moves nothing), the decays' biases
    spread so that heads forget at different speeds; `edit(weights)` may change the float64
    weights before they are written."""
    import inferllm_amd as I
    from inferllm_amd.weights.safetensors_io import write_safetensors
    from tiny import read_weights
    d = os.path.join(str(tmp), f"kukupel_{seed}_{abs(hash(repr(config))) % 10**8}_{str(dtype)[6:]}")
    I.write_random_model(d, I.config_from_dict(config), seed=seed, dtype=torch.float32)
    w = {}
    g = torch.Generator().manual_seed(seed)
    for n, t in read_weights(d).items():
        t = t.double()
        if n.endswith("dt_bias") or n.endswith("A_log"):
            t = torch.randn(t.shape, generator=g, dtype=torch.float64) * 1.5 - 1.0
        elif n.endswith(".conv"):
            t = t * 20
        elif t.dim() == 2 and ".hc" not in n and n != "embed":
            t = t * gain
        elif n == "embed":
            t = t * 10
        w[n] = t
    if edit is not None:
        edit(w)
    write_safetensors(os.path.join(d, "model.safetensors"), [(n, t.to(dtype)) for n, t in w.items()],
                      metadata={"format": "pt"})
    return d


def weights64(model_dir: str):
    from tiny import read_weights
    return {n: t.double() for n, t in read_weights(model_dir).items()}


def plant_key(w, config: dict, key_token: int, query_token: int, strength: float = 6.0) -> None:
    """Change layer 0's attention so that `query_token`'s score for `key_token` stands far above
    what random weights give, in every head: one query dim and one key dim are raised for exactly
    these two tokens (their layer-0 inputs are known: the normed read of the embeddings).  Whether
    the key is seen then decides the logits.  `strength` is the raw score before the cap."""
    m, eps, S = config["layers"][0]["mixer"]["left"], config["norm"]["eps"], config.get("streams", 0)
    read = float(w["l0.hc1.in"].sum()) if S else 1.0
    hid = lambda t: P.rms_norm(w["embed"][t] * read, w["l0.norm1"], eps)
    h_key, h_query = hid(key_token), hid(query_token)
    a = (strength / m["scale"]) ** 0.5
    rep = m["heads"] // m["kv_heads"]
    for h in range(m["heads"]):
        w["l0.mix.left.q"][h * m["dim"]] += a * h_query / (h_query @ h_query)
    for g in range(m["kv_heads"]):
        w["l0.mix.left.k"][g * m["dim"]] += a * h_key / (h_key @ h_key)
    # and a value that shows: the key token's value rows are large
    w["l0.mix.left.v"] += 3.0 * torch.outer(torch.ones(w["l0.mix.left.v"].shape[0], dtype=torch.float64),
                                            h_key / (h_key @ h_key))


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    return float((got.double().cpu() - want).abs().max() / want.abs().max())
