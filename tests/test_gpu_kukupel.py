"""Kukupel through the engine against the plain model (tests/plain_kukupel.py): every mechanism in
a layer of its own, whole prompts, token-by-token decoding, prompts cut into portions down to two
tokens, batches of unequal requests, slots and pages used again, planted keys far away and at page
borders, the first tokens, long decoding, ranks read from the tensors, greedy generation through
the engine's own loop; and the new kernels alone.  Configurations: tests/kukupel_tiny.py."""
import json
import os

import pytest
import torch

import plain_kukupel as P
from kukupel_tiny import MIXED, NO_KEYS, ODD, PLAIN, _moe, plant_key, single, weights64, write_model
from tiny import random_ids

pytestmark = pytest.mark.gpu

BUDGET = {"float32": 3e-5, "bfloat16": 4e-2}
STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16}
CONFIGS = {"MIXED": MIXED, "ODD": ODD, "PLAIN": PLAIN, "NO_KEYS": NO_KEYS}


def engine_for(d, dtype, **kw):
    import inferllm_amd as I
    kw.setdefault("max_batch", 8)
    kw.setdefault("max_seq_len", 1024)
    kw.setdefault("poison_freed", True)
    return I.Engine.from_pretrained(d, dtype=dtype, device="cuda:0", **kw)


def feed(eng, slot, tokens, cuts):
    """Logits of every position of `tokens`, fed in steps that end at `cuts` (then one by one)."""
    from inferllm_amd import StepEntry
    rows, at = [], 0
    for c in list(cuts) + list(range((cuts[-1] if cuts else 0) + 1, len(tokens) + 1)):
        if c <= at:
            continue
        rows.append(eng.step([StepEntry(slot, tokens[at:c], list(range(c - at)))]).clone())
        at = c
    return torch.cat(rows)


def close(got, want, dtype, what="", decided=None):
    """float32: every row within the budget.  bfloat16: rounding of the activations can turn a
    router's close call, and the recurrent layers carry another choice of experts to every later
    position: the rows before the first close call (`decided`, from `P.decided_rows`; None: all)
    are compared, and all of them but a few are within the budget."""
    scale = want.abs().max()
    if dtype != "float32" and decided is not None:
        got, want = got[:decided], want[:decided]
        if decided == 0:
            return
    err = (got.double().cpu() - want).abs().amax(dim=-1) / scale
    assert not torch.isnan(got).any(), what
    if dtype == "float32":
        assert float(err.max()) < BUDGET[dtype], (what, float(err.max()))
    else:
        over = int((err > BUDGET[dtype]).sum())
        assert over <= max(1, len(err) // 20) and float(err.median()) < BUDGET[dtype] / 2, \
            (what, over, len(err), float(err.median()))


# ------------------------------------------------------------------ each mechanism in a layer of its own
MECHANISMS = {
    "delta_head_decay": single("delta", streams=0, delta=(4, 2, 24, 20, 4)),
    "delta_shared_qk_two_taps": single("delta", streams=0, delta=(6, 1, 12, 36, 2)),
    "attention_beside_delta": single("parallel", streams=0, left=(6, 3, 16, 40, 0.25, 4.0),
                                     right=(3, 3, 20, 12, 3, 5, 7)),
    "attention_wide_keys": single("parallel", streams=0, left=(2, 2, 80, 24, 0.1, 2.5),
                                  right=(2, 1, 8, 8, 5, 2, 2)),
    "experts": single("delta", streams=0, mlp=_moe(40, 6, 2, 0.7)),
    "experts_top_is_all": single("delta", streams=0, mlp=_moe(24, 3, 3, 2.0)),
    "streams": single("delta", streams=4, mlp=_moe(24, 3, 1, 1.0)),
    "one_stream_with_weights": single("parallel", streams=1, mlp=_moe(24, 3, 1, 1.0)),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_mechanism_alone_prompt_and_tokens(tmp_path_factory, name, dtype):
    """A one-layer model that has the mechanism: a prompt of 70 tokens, then 10 single tokens."""
    config = MECHANISMS[name]
    d = write_model(tmp_path_factory.getbasetemp(), config, seed=5, dtype=STORE[dtype])
    eng = engine_for(d, dtype)
    ids = random_ids(80, config["vocab"], 17)
    slot = eng.alloc_slot()
    w = weights64(d)
    close(feed(eng, slot, ids, [70]), P.forward(config, w, ids), dtype, name, P.decided_rows(config, w, ids))
    eng.free_slot(slot)
    eng.cache.check()


# ------------------------------------------------------------------ whole models
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompts_of_unequal_lengths_then_tokens(tmp_path_factory, name, dtype):
    """Several prompts in one step (1 to 140 tokens, the first tokens of each included), then
    four steps of one token each for all of them, against the plain model of each alone."""
    from inferllm_amd import StepEntry
    config = CONFIGS[name]
    d = write_model(tmp_path_factory.getbasetemp(), config, seed=3, dtype=STORE[dtype])
    w = weights64(d)
    eng = engine_for(d, dtype)
    reqs = [random_ids(n + 4, config["vocab"], 11 * n) for n in (1, 2, 140, 65, 33, 71)]
    slots = [eng.alloc_slot() for _ in reqs]
    got = [[] for _ in reqs]
    out = eng.step([StepEntry(s, r[:-4], list(range(len(r) - 4))) for s, r in zip(slots, reqs)])
    at = 0
    for i, r in enumerate(reqs):
        got[i].append(out[at:at + len(r) - 4].clone())
        at += len(r) - 4
    for t in (4, 3, 2, 1):
        out = eng.step([StepEntry(s, [r[-t]], [0]) for s, r in zip(slots, reqs)])
        for i in range(len(reqs)):
            got[i].append(out[i:i + 1].clone())
    for i, r in enumerate(reqs):
        close(torch.cat(got[i]), P.forward(config, w, r), dtype, f"request {i}", P.decided_rows(config, w, r))
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cuts", [[], [1], [2, 4, 6], [63, 64, 65, 130], [17, 19, 100], [128]])
def test_token_by_token_and_portions_equal_the_whole_prompt(tmp_path_factory, cuts, dtype):
    """140 tokens one by one ([]), or in portions that end at `cuts` (portions of one and two
    tokens, portions that end at, before and after a page's border) and then one by one."""
    d = write_model(tmp_path_factory.getbasetemp(), MIXED, seed=4, dtype=STORE[dtype])
    eng = engine_for(d, dtype)
    ids = random_ids(140, MIXED["vocab"], 23)
    want = P.forward(MIXED, weights64(d), ids)
    slot = eng.alloc_slot()
    close(feed(eng, slot, ids if cuts else ids[:40], cuts), want if cuts else want[:40], dtype, str(cuts),
          P.decided_rows(MIXED, weights64(d), ids))
    eng.free_slot(slot)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_with_keys_and_values_of_one_width(tmp_path_factory, dtype):
    """ODD's attention has keys and values of one width: in bfloat16 its prompts, portions (over
    the paged cache) and single tokens run the shared matrix-core kernels with the cap."""
    d = write_model(tmp_path_factory.getbasetemp(), ODD, seed=21, dtype=STORE[dtype])
    w = weights64(d)
    eng = engine_for(d, dtype)
    ids = random_ids(150, ODD["vocab"], 29)
    slot = eng.alloc_slot()
    close(feed(eng, slot, ids, [40, 42, 43, 128, 140]), P.forward(ODD, w, ids), dtype, "",
          P.decided_rows(ODD, w, ids))
    eng.free_slot(slot)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32"])
def test_mixed_steps_of_portions_starts_and_single_tokens(tmp_path_factory, dtype):
    """Steps that hold a sequence that starts, one that goes on by a portion and one that goes on
    by two tokens, against each alone; every mixer goes on from what it kept."""
    from inferllm_amd import StepEntry
    d = write_model(tmp_path_factory.getbasetemp(), ODD, seed=9, dtype=STORE[dtype])
    w = weights64(d)
    eng = engine_for(d, dtype)
    a, b, c = (random_ids(n, ODD["vocab"], n) for n in (90, 70, 30))
    sa, sb, sc = (eng.alloc_slot() for _ in range(3))
    rows = {"a": [], "b": [], "c": []}
    out = eng.step([StepEntry(sa, a[:50], list(range(50)))])
    rows["a"].append(out.clone())
    out = eng.step([StepEntry(sa, a[50:88], list(range(38))), StepEntry(sb, b[:66], list(range(66)))])
    rows["a"].append(out[:38].clone()); rows["b"].append(out[38:].clone())
    out = eng.step([StepEntry(sc, c, list(range(30))), StepEntry(sa, a[88:], [0, 1]),
                    StepEntry(sb, b[66:], list(range(4)))])
    rows["c"].append(out[:30].clone()); rows["a"].append(out[30:32].clone()); rows["b"].append(out[32:].clone())
    for name, ids in (("a", a), ("b", b), ("c", c)):
        close(torch.cat(rows[name]), P.forward(ODD, w, ids), dtype, name)
    for s in (sa, sb, sc):
        eng.free_slot(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_slots_and_pages_used_again(tmp_path_factory, dtype):
    """Requests come and go in a cache with little room: later ones run in slots, pages and states
    that earlier ones used (freed pages are poisoned), and equal what they give alone."""
    from inferllm_amd import StepEntry
    d = write_model(tmp_path_factory.getbasetemp(), MIXED, seed=6, dtype=STORE[dtype])
    w = weights64(d)
    eng = engine_for(d, dtype, max_batch=2, max_tokens=384, max_seq_len=256)
    for round_ in range(3):
        reqs = [random_ids(n, MIXED["vocab"], 100 * round_ + n) for n in (100 + round_ * 30, 40 + round_)]
        slots = [eng.alloc_slot() for _ in reqs]
        out = eng.step([StepEntry(s, r[:-3], list(range(len(r) - 3))) for s, r in zip(slots, reqs)])
        got = [[out[:len(reqs[0]) - 3].clone()], [out[len(reqs[0]) - 3:].clone()]]
        for t in (3, 2, 1):
            out = eng.step([StepEntry(s, [r[-t]], [0]) for s, r in zip(slots, reqs)])
            got[0].append(out[:1].clone()); got[1].append(out[1:].clone())
        for i, r in enumerate(reqs):
            close(torch.cat(got[i]), P.forward(MIXED, w, r), dtype, f"round {round_} request {i}",
                  P.decided_rows(MIXED, w, r))
        eng.free_slot(slots[0])                      # the short one stays a round longer in its slot
        eng.free_slot(slots[1])
        eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key_at", [0, 1, 63, 64, 65, 127, 128, 400])
def test_a_planted_key_is_seen_from_far_in_prompts_and_in_decoding(tmp_path_factory, key_at, dtype):
    """One token's key is made to stand out for one query token.  The query comes at the end of a
    prompt of 520 tokens and again as a decoded token; the key lies at the sequence's first tokens,
    on both sides of page borders, or far back.  With the key left out the logits differ by far
    more than the budget, so a key that is lost shows."""
    config = single("parallel", streams=2, vocab=260)
    KEY, QUERY = 250, 251
    edit = lambda w: plant_key(w, config, KEY, QUERY)
    d = write_model(tmp_path_factory.getbasetemp(), config, seed=8, dtype=STORE[dtype], edit=edit)
    w = weights64(d)
    ids = [t % 250 for t in random_ids(522, 250, 31)]
    ids[key_at] = KEY
    ids[519] = QUERY
    ids[521] = QUERY
    want = P.forward(config, w, ids)
    without = list(ids); without[key_at] = 7
    moved = (P.forward(config, w, without)[[519, 521]] - want[[519, 521]]).abs().max() / want.abs().max()
    assert float(moved) > 8 * BUDGET[dtype], float(moved)
    eng = engine_for(d, dtype)
    slot = eng.alloc_slot()
    got = feed(eng, slot, ids, [520])
    close(got[[519, 521]], want[[519, 521]], dtype, f"key at {key_at}")
    close(got, want, dtype, "all rows")
    eng.free_slot(slot)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tmp_path_factory, dtype):
    """A prompt of 20 tokens, then 300 tokens one by one (over five pages, through decode graphs)."""
    d = write_model(tmp_path_factory.getbasetemp(), PLAIN, seed=12, dtype=STORE[dtype])
    eng = engine_for(d, dtype)
    ids = random_ids(320, PLAIN["vocab"], 41)
    slot = eng.alloc_slot()
    w = weights64(d)
    close(feed(eng, slot, ids, [20]), P.forward(PLAIN, w, ids), dtype, "", P.decided_rows(PLAIN, w, ids))
    eng.free_slot(slot)


def test_state_starts_at_zero_in_a_slot_used_before(tmp_path_factory):
    """The recurrent state and the convolution's tail of a slot are cleared when it is handed out:
    the same request twice in the same slot gives the same bits, with another request between."""
    from inferllm_amd import StepEntry
    d = write_model(tmp_path_factory.getbasetemp(), NO_KEYS, seed=2, dtype=torch.float32)
    eng = engine_for(d, "float32", max_batch=1)
    a, b = random_ids(50, NO_KEYS["vocab"], 1), random_ids(77, NO_KEYS["vocab"], 2)
    outs = []
    for ids in (a, b, a):
        slot = eng.alloc_slot()
        outs.append(eng.step([StepEntry(slot, ids, [len(ids) - 1])]).clone())
        eng.free_slot(slot)
    assert torch.equal(outs[0], outs[2])
    close(outs[0], P.forward(NO_KEYS, weights64(d), a)[-1:], "float32")


def test_low_ranks_come_from_the_tensors(tmp_path_factory):
    """A configuration that does not state the low ranks of the decay and gate projections: the
    engine reads them from the folder's tensors."""
    config = single("parallel", streams=2, right=(2, 2, 16, 12, 3, 5, 9))
    d = write_model(tmp_path_factory.getbasetemp(), config, seed=13, dtype=torch.float32)
    path = os.path.join(d, "config.json")
    with open(path) as f:
        stored = json.load(f)
    for key in ("decay_rank", "gate_rank"):
        del stored["layers"][0]["mixer"]["right"][key]
    with open(path, "w") as f:
        json.dump(stored, f)
    eng = engine_for(d, "float32")
    ids = random_ids(30, config["vocab"], 3)
    slot = eng.alloc_slot()
    close(feed(eng, slot, ids, [30]), P.forward(config, weights64(d), ids), "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(tmp_path_factory, dtype):
    """`Engine.generate` (the scheduler's batches, decode graphs, the sampler's arg-max): four
    prompts of unequal lengths with room for two at a time, against the plain model's greedy
    tokens; in bfloat16 a close call may differ, after which the texts part."""
    d = write_model(tmp_path_factory.getbasetemp(), MIXED, seed=7, dtype=STORE[dtype])
    w = weights64(d)
    eng = engine_for(d, dtype, max_batch=2, poison_freed=False)
    prompts = [random_ids(n, MIXED["vocab"], 5 + n) for n in (3, 40, 66, 9)]
    got = eng.generate(prompts, max_new_tokens=12)
    same = 0
    for p, g in zip(prompts, got):
        want = P.greedy(MIXED, w, p, 12)
        assert len(g) == 12
        if dtype == "float32":
            assert g == want
        same += sum(1 for x, y in zip(g, want) if x == y) >= 6
    assert same >= 3
    portions = eng.generate(prompts, max_new_tokens=12, max_step_tokens=16)
    if dtype == "float32":
        assert portions == got


def test_the_command_line_and_the_trace_replay(tmp_path):
    """`bin/chat` with token-id prompts, greedy, names the design by `--type`; `bin/trace_run`
    replays two requests that start together and go on by one token."""
    import subprocess
    import sys
    import numpy as np
    d = write_model(tmp_path, PLAIN, seed=14, dtype=torch.float32)
    w = weights64(d)
    ids = random_ids(9, PLAIN["vocab"], 2)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "chat"), "-m", d, "-d", "float32", "--temp", "0",
                        "-n", "5", "--prompt-ids", " ".join(map(str, ids)), "-c", "64", "--type", "kukupel"],
                       capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    assert [int(t) for t in r.stdout.split()] == P.greedy(PLAIN, w, ids, 5)
    a, b = random_ids(70, PLAIN["vocab"], 4), random_ids(5, PLAIN["vocab"], 6)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:68], "want": [0, 67]},
                                     {"id": "b", "tokens": b[:3], "want": [2]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[68:69], "want": []},
                                     {"id": "b", "tokens": b[3:4], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[69:], "want": [0]},
                                     {"id": "b", "tokens": b[4:], "want": [0]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    wa, wb = P.forward(PLAIN, w, a), P.forward(PLAIN, w, b)
    V = PLAIN["vocab"]
    got = {i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V)) for i in range(3)}
    close(got[0], torch.stack([wa[0], wa[67], wb[2]]), "float32")
    close(got[1], wb[3:4], "float32")
    close(got[2], torch.stack([wa[69], wb[4]]), "float32")


def test_a_conversation_in_one_slot(tmp_path):
    """`Engine.session`: the turns of a conversation go on from what the slot holds (keys and
    values, states, the convolutions' tails) by several tokens; a model with states is decoded in
    step, so no token is ever taken back."""
    d = write_model(tmp_path, MIXED, seed=17)
    w = weights64(d)
    eng = engine_for(d, "float32")
    first = random_ids(6, MIXED["vocab"], 54)
    with eng.session(stop_token_ids=[]) as chat:
        a1 = chat.say(first, max_new_tokens=4)
        assert a1 == P.greedy(MIXED, w, first, 4)
        turn = random_ids(5, MIXED["vocab"], 77)
        a2 = chat.say(turn, max_new_tokens=3)
        # the token that max_new_tokens cut off is fed in front of the next turn
        assert a2 == P.greedy(MIXED, w, first + a1 + turn, 3)
    eng.cache.check()


# ------------------------------------------------------------------ kernels alone
def test_stream_mix_norm_against_plain_torch():
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    for S, E, T in ((3, 90, 5), (1, 64, 3), (8, 130, 9)):
        x = torch.randn(T, S, E, generator=g)
        y1, y2 = torch.randn(T, E, generator=g), torch.randn(T, E, generator=g)
        mix, out, read, w = (torch.randn(S, S, generator=g), torch.randn(S, generator=g),
                             torch.randn(S, generator=g), torch.randn(E, generator=g))
        y = 0.7 * y1.double() + 1.9 * y2.double()
        xn = torch.stack([sum(mix[s, t].double() * x[:, s].double() for s in range(S)) + out[t].double() * y
                          for t in range(S)], dim=1)
        u = sum(read[s].double() * xn[:, s] for s in range(S))
        want = P.rms_norm(u, w.double(), 1e-5)
        xg = x.cuda()
        write = ops.StreamWrite(y1.cuda(), mix.cuda(), out.cuda(), y2=y2.cuda(), ya=0.7, yb=1.9)
        rows = torch.tensor([T - 1, 0], dtype=torch.int32, device="cuda")
        picked = ops.stream_mix_norm(xg, write, read.cuda(), w.cuda(), 1e-5, torch.float32, rows)
        assert torch.equal(xg.cpu(), x)                  # picking rows leaves the streams alone
        got = ops.stream_mix_norm(xg, write, read.cuda(), w.cuda(), 1e-5, torch.float32)
        assert float((got.double().cpu() - want).abs().max()) < 1e-4
        assert float((picked.double().cpu() - want[[T - 1, 0]]).abs().max()) < 1e-4
        assert float((xg.double().cpu() - xn).abs().max()) < 1e-4
        plain = ops.stream_mix_norm(xg, None, None, w.cuda(), 1e-5, torch.float32)
        assert float((plain.double().cpu() - P.rms_norm(xn.sum(1), w.double(), 1e-5)).abs().max()) < 1e-4


def test_sigmoid_routing_and_weighted_inputs_against_the_plain_experts():
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    T, E, F, N, top, lim = 37, 48, 20, 6, 3, 0.6
    h = torch.randn(T, E, generator=g)
    w = {"router": torch.randn(N, E, generator=g) * 0.3}
    for e in range(N):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = (torch.randn(F, E, generator=g) * 0.3,
                                                          torch.randn(F, E, generator=g) * 0.3,
                                                          torch.randn(E, F, generator=g) * 0.3)
    want = P.experts(h.double(), {"m." + k: v.double() for k, v in w.items()}, "m.",
                     _moe(F, N, top, lim))
    wgu = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(N)]).cuda()
    wd = torch.stack([w[f"e{e}.down"] for e in range(N)]).cuda()
    hg = h.cuda()
    idx, wt, grouped = ops.moe_plan(hg, w["router"].cuda(), None, top, wgu, "sigmoid")
    y = ops.moe_experts(hg, idx, wgu, wd, grouped, "clamped_swish", lim, wt)
    got = ops.moe_combine(hg, idx, None, y, N)
    assert float((got.double().cpu() - want).abs().max() / want.abs().max()) < 1e-5
