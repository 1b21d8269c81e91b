"""Tiny Rabapel configurations and helpers for the tests.  The sizes differ from layer to layer
and avoid equal or trivial values: head counts 3, 5, 16 and 2, plain and rotated head parts of
different sizes, a value size above and below the query size, latent ranks that are no multiple
of 64, rotated dims below the rot part, windows of 70 and 33 beside layers without one, routers
with and without identity experts and shared experts, a layer without feed-forward."""
from __future__ import annotations

import os

import torch

import plain_rabapel as P


def _mixer(heads, dim, rot_dim, vdim, rank, scale, window=None, dims=None, base=10000.0, scaling=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale,
         "rot": {"base": base, "dims": dims or rot_dim}}
    if window:
        m["mask"] = {"size": window}
    if scaling:
        m["rot"]["scaling"] = scaling
    return m


def _moe(ff, experts, top, identity=0, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top}}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


YARN = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}

MIXED = {"architecture": "Rabapel", "vocab": 300, "width": 96, "norm": {"eps": 1e-5},
         "embedding": {"scale": 0.7},
         "layers": [
             {"type": "latent_attention", "mixer": _mixer(3, 16, 8, 24, 40, 0.3, window=70, scaling=YARN),
              "mlp": {"kind": "dense", "ff": 200}},
             {"type": "latent_attention", "mixer": _mixer(5, 8, 16, 40, 64, 0.2, dims=12, base=5000.0),
              "mlp": _moe(48, 5, 3, identity=2, shared=72)},
             {"type": "latent_attention", "mixer": _mixer(16, 4, 4, 6, 130, 0.5, window=33), "mlp": None},
             {"type": "latent_attention", "mixer": _mixer(2, 32, 32, 20, 24, 0.11, base=300000.0,
                                                           scaling={"factor": 5.0, "original": 96, "fast": 20.0, "slow": 1.5}),
              "mlp": _moe(40, 3, 1)},
         ]}

# a width that is no multiple of 4 (the kernels' element-by-element paths), one expert of two chosen
ODD = {"architecture": "Rabapel", "vocab": 131, "width": 90, "norm": {"eps": 3e-6},
       "embedding": {"scale": 1.25},
       "layers": [
           {"type": "latent_attention", "mixer": _mixer(7, 10, 6, 14, 50, 0.25, window=20, dims=4),
            "mlp": _moe(30, 2, 2, identity=1, shared=50)},
           {"type": "latent_attention", "mixer": _mixer(1, 24, 8, 48, 96, 0.2),
            "mlp": {"kind": "dense", "ff": 77}},
       ]}

# one layer, for tests that plant a key (`plant_key`)
def single(window=None, heads=4, dim=16, rot_dim=8, vdim=12, rank=48, mlp=None, width=64, vocab=200):
    return {"architecture": "Rabapel", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
            "embedding": {"scale": 0.6},
            "layers": [{"type": "latent_attention",
                        "mixer": _mixer(heads, dim, rot_dim, vdim, rank, 0.25, window=window, scaling=YARN),
                        "mlp": mlp}]}


def write_model(tmp, config: dict, seed: int, dtype=torch.float32, gain: float = 4.0, edit=None) -> str:
    """A random model folder for `config`; every matrix times `gain` (see tests/tiny.py: with the
    library's small random weights a wrong key moves nothing); `edit(weights)` may change the
    float64 weights before they are written."""
    import inferllm_amd as I
    from inferllm_amd.weights.safetensors_io import write_safetensors
    from tiny import read_weights
    d = os.path.join(str(tmp), f"rabapel_{seed}_{abs(hash(repr(config))) % 10**8}_{str(dtype)[6:]}")
    I.write_random_model(d, I.config_from_dict(config), seed=seed, dtype=torch.float32)
    w = {n: (t.double() * gain if t.dim() == 2 else t.double()) for n, t in read_weights(d).items()}
    if edit is not None:
        edit(w)
    write_safetensors(os.path.join(d, "model.safetensors"), [(n, t.to(dtype)) for n, t in w.items()],
                      metadata={"format": "pt"})
    return d


def weights64(model_dir: str):
    from tiny import read_weights
    return {n: t.double() for n, t in read_weights(model_dir).items()}


def plant_key(w, config: dict, key_token: int, query_token: int, strength: float = 30.0) -> None:
    """Change layer 0 so that `query_token`'s score for `key_token` stands `strength` above what
    random weights give, in every head: one plain query dim and one plain key dim are raised for
    exactly these two tokens (their layer-0 inputs are known: the normed embeddings).  Whether the
    key is seen then decides the logits."""
    m, eps = config["layers"][0]["mixer"], config["norm"]["eps"]
    H, dn, dr, R = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"]
    hid = lambda t: P.rms_norm(w["embed"][t] * config["embedding"]["scale"], w["l0.norm1"], eps)
    h_key, h_query = hid(key_token), hid(query_token)
    c_key = P.rms_norm((w["l0.mix.dkv"] @ h_key)[:R], w["l0.mix.dkv.norm"], eps)
    a = (strength / m["scale"]) ** 0.5
    for h in range(H):
        w["l0.mix.q"][h * (dn + dr)] += a * h_query / (h_query @ h_query)
        w["l0.mix.uk"][h * dn] += a * c_key / (c_key @ c_key)


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    return float((got.double().cpu() - want).abs().max() / want.abs().max())
