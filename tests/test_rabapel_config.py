"""Rabapel without a GPU: its configuration, the tensors it asks for, the scaled rotary
frequencies of the position part against the plain model's, and the plain model's own parts."""
import copy

import pytest
import torch

import plain_rabapel as P
from rabapel_tiny import MIXED, ODD, YARN


def test_config_reads_back_and_names_its_tensors():
    import inferllm_amd as I
    from inferllm_amd.engine.model import expected_tensors
    cfg = I.config_from_dict(MIXED)
    assert I.config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    want = expected_tensors(cfg.to_spec())
    assert want["embed"].shape == (300, 96) and want["final.norm"].shape == (96,)
    assert want["l0.mix.q"].shape == (3 * 24, 96) and want["l0.mix.dkv"].shape == (48, 96)
    assert want["l0.mix.uk"].shape == (48, 40) and want["l0.mix.uv"].shape == (72, 40)
    assert want["l0.mix.g"].shape == (3, 96) and want["l0.mix.o"].shape == (96, 72)
    assert want["l0.mlp.up"].shape == (200, 96) and want["l0.mlp.down"].shape == (96, 200)
    assert want["l1.mlp.router"].shape == (7, 96) and want["l1.mlp.correction"].shape == (7,)
    assert want["l1.mlp.e4.down"].shape == (96, 48) and "l1.mlp.e5.gate" not in want
    assert want["l1.mlp.shared.sg"].shape == (1, 96) and want["l1.mlp.shared.up"].shape == (72, 96)
    assert not any(n.startswith("l2.mlp") for n in want)
    assert "l3.mlp.shared.gate" not in want and want["l3.mlp.e2.gate"].shape == (40, 96)
    spec = cfg.to_spec()
    assert [l.block for l in spec.layers] == ["parallel"] * 4
    assert spec.layers[2].mixer.params["window"] == 33 and spec.layers[1].mixer.params["window"] is None


@pytest.mark.parametrize("change", [
    lambda c: c.pop("vocab"),
    lambda c: c["layers"].clear(),
    lambda c: c["layers"][0].update(type="attention"),
    lambda c: c["layers"][0]["mixer"].update(heads=0),
    lambda c: c["layers"][0]["mixer"]["rot"].update(dims=9),
    lambda c: c["layers"][0]["mlp"].update(kind="swiglu"),
    lambda c: c["layers"][1]["mlp"]["router"].update(top=9),
    lambda c: c["norm"].update(eps=0),
])
def test_config_errors_name_the_key(change):
    import inferllm_amd as I
    c = copy.deepcopy(MIXED)
    change(c)
    with pytest.raises(I.ConfigError):
        I.config_from_dict(c)


@pytest.mark.parametrize("rot", [
    {"base": 10000.0, "dims": 8, "scaling": YARN},
    {"base": 300000.0, "dims": 24, "scaling": {"factor": 5.0, "original": 256, "fast": 20.0, "slow": 1.5}},
    {"base": 5000.0, "dims": 12},
    {"base": 100.0, "dims": 4, "scaling": {"factor": 2.0, "original": 16, "fast": 1.0, "slow": 1.0}},
])
def test_scaled_rotary_table_equals_the_plain_angles(rot):
    from inferllm_amd.parts.position import rotary_table
    table = rotary_table(rot["base"], rot["dims"], 300, "cpu", rot.get("scaling"))
    f, gain = P.rotary_frequencies(rot)
    ang = torch.arange(300, dtype=torch.float64)[:, None] * f[None, :]
    assert float((table[..., 0].double() - torch.cos(ang) * gain).abs().max()) < 1e-6
    assert float((table[..., 1].double() - torch.sin(ang) * gain).abs().max()) < 1e-6
    if rot.get("scaling"):
        plain, _ = P.rotary_frequencies({"base": rot["base"], "dims": rot["dims"]})
        assert float(f[0]) == pytest.approx(float(plain[0])) or rot["dims"] <= 4    # fast pairs keep their turn
        assert gain > 1.0


def test_plain_parts():
    g = torch.Generator().manual_seed(0)
    x = torch.randn((5, 12), generator=g, dtype=torch.float64)
    assert torch.allclose((P.rms(x, 0.0) ** 2).mean(-1), torch.ones(5, dtype=torch.float64))
    # rotation keeps lengths (times the gain) and leaves the dims beyond `dims` alone
    rot = {"base": 100.0, "dims": 8}
    y = P.rotate(x, torch.arange(5), rot)
    assert torch.allclose(y[:, 8:], x[:, 8:]) and torch.allclose(y[:, :8].norm(dim=-1), x[:, :8].norm(dim=-1))
    assert torch.allclose(y[0], x[0])
    # the window: itself and size - 1 before it
    m = P.window_mask(6, 3)
    assert m[5].tolist() == [False, False, False, True, True, True] and m[1].tolist() == [True, True] + [False] * 4
    # an identity expert hands the input back, weighted, not renormalised
    w = {"r.router": torch.tensor([[0.0] * 12, [1.0] * 12], dtype=torch.float64),
         "r.correction": torch.tensor([-10.0, 0.0], dtype=torch.float64)}
    mlp = {"kind": "moe", "router": {"experts": 1, "identity": 1, "top": 1}}
    out = P.moe_ff(x, w, "r.", mlp)
    s = torch.softmax(x @ w["r.router"].T, -1)[:, 1:2]
    assert torch.allclose(out, s * x)


def test_plain_model_runs_the_tiny_configurations():
    import inferllm_amd as I
    from inferllm_amd.engine.model import expected_tensors
    from inferllm_amd.weights.random_init import random_tensors
    for config in (MIXED, ODD):
        want = expected_tensors(I.config_from_dict(config).to_spec())
        w = {n: t.double() * (4 if t.dim() == 2 else 1) for n, t in random_tensors(want, 1, torch.float32)}
        toks = [1, 5, 9, 2, 77, 30]
        full = P.forward(config, w, toks)
        assert full.shape == (6, config["vocab"]) and torch.isfinite(full).all()
        # causal: a prefix gives the same logits
        assert torch.allclose(P.forward(config, w, toks[:4]), full[:4], atol=1e-9)
