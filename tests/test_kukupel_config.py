"""Kukupel without a GPU: its configuration, the tensors it asks for, the parts it is translated
into, and the plain model's own mechanisms against each other."""
import copy

import pytest
import torch

import plain_kukupel as P
from kukupel_tiny import MIXED, NO_KEYS, ODD, PLAIN


def test_config_reads_back_and_names_its_tensors():
    import inferllm_amd as I
    from inferllm_amd.engine.model import expected_tensors
    cfg = I.config_from_dict(MIXED)
    assert I.config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    want = expected_tensors(cfg.to_spec())
    assert want["embed"].shape == (300, 96) and want["final.norm"].shape == (96,)
    # layer 0: the delta rule alone, a decay a head and a full gate
    assert want["l0.mix.q"].shape == (3 * 24, 96) and want["l0.mix.v"].shape == (3 * 40, 96)
    assert want["l0.mix.q.conv"].shape == (72, 2) and want["l0.mix.v.conv"].shape == (120, 2)
    assert want["l0.mix.a"].shape == (3, 96) and want["l0.mix.dt_bias"].shape == (3,)
    assert want["l0.mix.g"].shape == (120, 96) and want["l0.mix.norm"].shape == (40,)
    assert "l0.mix.a1" not in want and "l0.mix.left.q" not in want
    # layer 1: attention beside the delta rule, a decay a key channel through a low rank
    assert want["l1.mix.left.q"].shape == (6 * 16, 96) and want["l1.mix.left.k"].shape == (2 * 16, 96)
    assert want["l1.mix.left.v"].shape == (2 * 40, 96) and want["l1.mix.left.o"].shape == (96, 6 * 40)
    assert want["l1.mix.right.k"].shape == (2 * 20, 96) and want["l1.mix.right.v"].shape == (4 * 12, 96)
    assert want["l1.mix.right.a1"].shape == (7, 96) and want["l1.mix.right.a2"].shape == (4 * 20, 7)
    assert want["l1.mix.right.g1"].shape == (9, 96) and want["l1.mix.right.g2"].shape == (4 * 12, 9)
    assert want["l1.mix.right.dt_bias"].shape == (80,) and want["l1.mix.right.A_log"].shape == (4,)
    assert want["l1.mlp.router"].shape == (3, 96) and want["l1.mlp.e2.down"].shape == (96, 40)
    assert "l1.mlp.e3.gate" not in want and "l1.mlp.correction" not in want
    # the streams' weights; a layer without a feed-forward has the first sublayer's alone
    assert want["l1.hc1.in"].shape == (2,) and want["l1.hc2.mix"].shape == (2, 2)
    assert "l2.hc2.in" not in want and "l2.norm2" not in want and want["l2.hc1.out"].shape == (2,)
    spec = cfg.to_spec()
    assert [l.block for l in spec.layers] == ["hyper_connections"] * 4
    assert [l.mixer.kind for l in spec.layers] == ["gated_delta_rule", "side_by_side", "side_by_side",
                                                   "gated_delta_rule"]
    assert spec.embedding.params["streams"] == 2 and "read" not in spec.final_norm.tensors
    ff = spec.layers[0].feed_forward.params
    assert (ff["score"], ff["activation"], ff["weight_on"], ff["limit"]) == ("sigmoid", "clamped_swish", "input", 1.5)


def test_one_stream_is_the_plain_pre_norm_layer():
    import inferllm_amd as I
    from inferllm_amd.engine.model import expected_tensors
    spec = I.config_from_dict(PLAIN).to_spec()
    assert [l.block for l in spec.layers] == ["pre_norm", "pre_norm"]
    assert spec.final_norm.kind == "rms_norm" and not any(".hc" in n for n in expected_tensors(spec))


def test_cache_needs_follow_the_mixers():
    import inferllm_amd as I
    from inferllm_amd.engine.model import DecoderModel
    m = DecoderModel(I.config_from_dict(MIXED).to_spec())
    kv, st = m.kv_lines(), m.state_lines()
    assert sorted(kv) == [1, 2] and sorted(st) == [0, 1, 2, 3]
    assert [t.shape for t in kv[1].tensors] == [(2, 16), (2, 40)]
    assert st[0]["S"].shape == (3, 24, 40) and st[0]["tail"].shape == (1, 2 * 72 + 120)
    assert st[2]["S"].shape == (2, 36, 28) and st[2]["tail"].shape == (4, 2 * 36 + 56)
    assert not m.one_token_mixers and m.graph_safe and m.graph_safe_prompts
    assert not DecoderModel(I.config_from_dict(NO_KEYS).to_spec()).kv_lines()


def test_low_ranks_are_taken_from_tensor_shapes():
    import inferllm_amd as I
    c = copy.deepcopy(ODD)
    for key in ("decay_rank", "gate_rank"):
        del c["layers"][0]["mixer"]["right"][key]
    cfg = I.config_from_dict(c).with_tensor_shapes({"l0.mix.right.a1": (11, 90), "l0.mix.right.g1": (13, 90)})
    p = cfg.to_spec().layers[0].mixer.params["right"].params
    assert (p["decay_rank"], p["gate_rank"]) == (11, 13)
    stated = I.config_from_dict(ODD).with_tensor_shapes({"l0.mix.right.a1": (11, 90)})
    assert stated.to_spec().layers[0].mixer.params["right"].params["decay_rank"] == 4


@pytest.mark.parametrize("change", [
    lambda c: c.pop("width"),
    lambda c: c["layers"].clear(),
    lambda c: c.update(streams=9),
    lambda c: c["layers"][0].update(type="attention"),
    lambda c: c["layers"][0]["mixer"].update(kv_heads=2),
    lambda c: c["layers"][0]["mixer"].pop("conv"),
    lambda c: c["layers"][1]["mixer"]["left"].update(softcap=-1),
    lambda c: c["layers"][1]["mixer"].pop("right_scale"),
    lambda c: c["layers"][1]["mlp"].update(kind="dense"),
    lambda c: c["layers"][1]["mlp"]["router"].update(top=4),
    lambda c: c["layers"][3]["mlp"]["expert"].pop("limit"),
    lambda c: c["norm"].update(eps=0),
])
def test_config_errors_name_the_key(change):
    import inferllm_amd as I
    c = copy.deepcopy(MIXED)
    change(c)
    with pytest.raises(I.ConfigError):
        I.config_from_dict(c)


def test_plain_recurrence_equals_its_unrolled_sum():
    """Without decay and with beta = 1 and orthonormal keys the delta rule stores each value under
    its key: o_t = sum over j <= t of (q_t . k_j) v_j, which the plain recurrence must give."""
    g = torch.Generator().manual_seed(1)
    T, dk, dv = 6, 8, 5
    k = torch.linalg.qr(torch.randn(dk, dk, generator=g, dtype=torch.float64))[0][:T]
    q, v = torch.randn(T, dk, generator=g, dtype=torch.float64), torch.randn(T, dv, generator=g, dtype=torch.float64)
    o = P.delta_recurrence(q[:, None], k[:, None], v[:, None], torch.ones(T, 1, dtype=torch.float64),
                           torch.ones(T, 1, dk, dtype=torch.float64))[:, 0]
    want = torch.stack([sum((q[t] @ k[j]) * v[j] for j in range(t + 1)) for t in range(T)])
    assert float((o - want).abs().max()) < 1e-12


def test_plain_convolution_sees_only_the_past():
    x = torch.zeros(7, 2, dtype=torch.float64)
    x[3] = 1.0
    w = torch.tensor([[1.0, 2.0, 3.0], [0.5, 0.0, -1.0]], dtype=torch.float64)
    y = P.short_conv_silu(x, w)
    silu = lambda z: z * torch.sigmoid(z)
    assert torch.equal(y[:3], torch.zeros(3, 2, dtype=torch.float64)) and torch.equal(y[6], torch.zeros(2, dtype=torch.float64))
    assert torch.allclose(y[3], silu(w[:, 2])) and torch.allclose(y[4], silu(w[:, 1])) and torch.allclose(y[5], silu(w[:, 0]))


def test_a_layer_without_feed_forward_tolerates_the_second_sublayers_tensors():
    """A folder may hold norm2 and hc2.* of a layer whose mlp is null: nothing acts on the norm and
    the read and output weights; the mix matrix, if there, still mixes the streams."""
    import inferllm_amd as I
    from inferllm_amd.engine.model import expected_tensors
    shapes = {"l2.norm2": (96,), "l2.hc2.in": (2,), "l2.hc2.out": (2,), "l2.hc2.mix": (2, 2)}
    cfg = I.config_from_dict(MIXED).with_tensor_shapes(shapes)
    spec = cfg.to_spec()
    want = expected_tensors(spec)
    assert want["l2.hc2.mix"].shape == (2, 2) and "l2.hc2.in" not in want and "l2.norm2" not in want
    assert sorted(spec.ignored_tensor_suffixes) == ["l2.hc2.in", "l2.hc2.out", "l2.norm2"]
    assert "l2.hc2.mix" not in expected_tensors(I.config_from_dict(MIXED).to_spec())
