"""Rabapel through the engine against the plain model (tests/plain_rabapel.py): whole prompts,
token-by-token decoding, prompts cut into portions, batches of unequal requests, slots and pages
used again, planted keys at window edges, page borders and far away, greedy generation; and the
router and expert kernels alone.  Configurations: tests/rabapel_tiny.py."""
import pytest
import torch

import plain_rabapel as P
from rabapel_tiny import MIXED, ODD, plant_key, rel_err, single, weights64, write_model
from tiny import random_ids

pytestmark = pytest.mark.gpu

BUDGET = {"float32": 2e-5, "bfloat16": 4e-2}
STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16}


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


def close(got, want, dtype, what=""):
    """float32: every row within the budget.  bfloat16: rounding of the activations can turn a
    router's close call, which moves one token's output; all rows but a few within the budget."""
    scale = want.abs().max()
    err = (got.double().cpu() - want).abs().amax(dim=-1) / scale
    if dtype == "float32":
        assert float(err.max()) < BUDGET[dtype], (what, float(err.max()))
    else:
        over = int((err > BUDGET[dtype]).sum())
        assert over <= max(1, len(err) // 20) and float(err.median()) < BUDGET[dtype] / 2, \
            (what, over, len(err), float(err.median()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["MIXED", "ODD"])
def test_whole_prompts_of_unequal_lengths_then_tokens(tmp_path_factory, name, dtype):
    """Several prompts in one step (1 to 140 tokens, the first tokens of each included), then
    four steps of one token each for all of them, against the plain model of each alone."""
    from inferllm_amd import StepEntry
    config = {"MIXED": MIXED, "ODD": ODD}[name]
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
        close(torch.cat(got[i]), P.forward(config, w, r), dtype, f"request {i}")
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_past_windows_and_pages(tmp_path_factory, dtype):
    """A prompt of 9 tokens, then 190 tokens one by one: the windows of 70 and 33 keys pass over
    decoded tokens, pages of 64 fill up and the windows' rings of pages come round."""
    d = write_model(tmp_path_factory.getbasetemp(), MIXED, seed=5, dtype=STORE[dtype])
    w = weights64(d)
    eng = engine_for(d, dtype, step_rows=16)
    toks = random_ids(199, MIXED["vocab"], 1)
    s = eng.alloc_slot()
    close(feed(eng, s, toks, [9]), P.forward(MIXED, w, toks), dtype)
    eng.free_slot(s)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,dim,rot_dim,vdim,rank,window", [(20, 64, 32, 96, 256, 70), (3, 160, 64, 224, 208, None),
                                                                (33, 16, 16, 24, 512, 129)])
def test_wide_heads_and_long_latents(tmp_path_factory, heads, dim, rot_dim, vdim, rank, window, dtype):
    """Heads of up to 224 dims, latents of 208 to 512, 3 to 33 heads (the kernels' other branches:
    more accumulators, several groups of heads, generic prompt attention)."""
    from inferllm_amd import StepEntry
    config = single(window=window, heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, rank=rank,
                    mlp={"kind": "dense", "ff": 96}, width=128)
    d = write_model(tmp_path_factory.getbasetemp(), config, seed=heads, dtype=STORE[dtype], gain=2.0)
    w = weights64(d)
    eng = engine_for(d, dtype)
    reqs = [random_ids(n, config["vocab"], n) for n in (170, 66)]
    slots = [eng.alloc_slot() for _ in reqs]
    cut = [len(r) - 12 for r in reqs]
    out = eng.step([StepEntry(s, r[:k], list(range(k))) for s, r, k in zip(slots, reqs, cut)])
    got = [[out[:cut[0]].clone()], [out[cut[0]:].clone()]]
    for t in range(12):
        o = eng.step([StepEntry(slots[i], [reqs[i][cut[i] + t]], [0]) for i in range(2)])
        for i in range(2):
            got[i].append(o[i:i + 1].clone())
    for i, r in enumerate(reqs):
        close(torch.cat(got[i]), P.forward(config, w, r), dtype, f"request {i}")


@pytest.mark.parametrize("graphs", [True, False])
def test_portions_of_a_prompt(tmp_path_factory, graphs):
    """A prompt fed in portions of 2 to 90 tokens (and single ones between) gives what the whole
    prompt gives; the portions cross pages and are longer and shorter than the windows."""
    d = write_model(tmp_path_factory.getbasetemp(), MIXED, seed=7)
    w = weights64(d)
    eng = engine_for(d, "float32", use_graphs=graphs)
    toks = random_ids(230, MIXED["vocab"], 2)
    want = P.forward(MIXED, w, toks)
    for cuts in ([2, 4, 7, 71, 73, 163, 228], [64, 128, 129, 131, 221], [90, 92, 180, 230]):
        s = eng.alloc_slot()
        got = feed(eng, s, toks, cuts)
        eng.free_slot(s)
        assert rel_err(got, want) < BUDGET["float32"], cuts


def test_a_request_alone_and_in_company(tmp_path_factory):
    """The logits of a request do not depend on what else is in the batch beyond rounding, and
    slots and pages that were freed (and filled with NaN) are used again."""
    from inferllm_amd import StepEntry
    d = write_model(tmp_path_factory.getbasetemp(), MIXED, seed=9)
    eng = engine_for(d, "float32")
    reqs = [random_ids(n, MIXED["vocab"], 7 * n) for n in (40, 141, 9, 90)]
    alone = []
    for r in reqs:
        s = eng.alloc_slot()
        alone.append(feed(eng, s, r, [len(r) - 6]))
        eng.free_slot(s)
    for order in ([0, 1, 2, 3], [3, 1, 0, 2]):
        slots = {i: eng.alloc_slot() for i in order}
        out = eng.step([StepEntry(slots[i], reqs[i][:-6], list(range(len(reqs[i]) - 6))) for i in order])
        at, got = 0, {i: [] for i in order}
        for i in order:
            got[i].append(out[at:at + len(reqs[i]) - 6].clone())
            at += len(reqs[i]) - 6
        for t in range(6, 0, -1):
            live = [i for i in order if not (i == 2 and t < 4)]      # one request ends earlier
            if t == 3:
                eng.free_slot(slots[2])
            out = eng.step([StepEntry(slots[i], [reqs[i][-t]], [0]) for i in live])
            for k, i in enumerate(live):
                got[i].append(out[k:k + 1].clone())
        for i in order:
            g = torch.cat(got[i])
            n = g.shape[0]
            assert rel_err(g, alone[i][:n].double().cpu()) < 1e-5, (order, i)
            if i != 2:
                eng.free_slot(slots[i])
    eng.cache.check()


def _planted(tmp, window, mlp=None):
    config = single(window=window, mlp=mlp)
    A, B = 17, 23
    d = write_model(tmp, config, seed=window or 1, edit=lambda w: plant_key(w, config, A, B))
    return config, d, A, B


def _sequence(config, A, B, at, gap, tail=0):
    """Filler tokens with the planted key token at place `at` and the query token `gap` later."""
    fill = [t for t in random_ids(at + gap + tail + 40, config["vocab"], at * 1000 + gap) if t not in (A, B)]
    seq = fill[:at] + [A] + fill[at:at + gap - 1] + [B] + fill[at + gap - 1:at + gap - 1 + tail]
    return seq


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_planted_key_just_inside_and_outside_the_window(tmp_path_factory, dtype):
    """The query token's score for the key token stands out, so its logits turn on whether the
    key is seen: at distance window - 1 it is, at distance window it is not.  Keys at the start
    of a sequence, at page borders and in the middle; the query in a prompt and decoded alone."""
    window = 70
    config, d, A, B = _planted(tmp_path_factory.getbasetemp(), window)
    if dtype == "bfloat16":
        d = write_model(tmp_path_factory.getbasetemp(), config, seed=window, dtype=torch.bfloat16,
                        edit=lambda w: plant_key(w, config, A, B))
    w = weights64(d)
    eng = engine_for(d, dtype)
    for at in (0, 5, 63, 64, 100, 127):
        rows = {}
        for gap in (window - 1, window):
            seq = _sequence(config, A, B, at, gap, tail=2)
            want = P.forward(config, w, seq)
            rows[gap] = want[at + gap]
            for cut in (len(seq), at + gap):              # the query in the prompt / decoded alone
                s = eng.alloc_slot()
                got = feed(eng, s, seq, [cut])
                eng.free_slot(s)
                err = rel_err(got[at + gap - 1:], want[at + gap - 1:])
                assert err < BUDGET[dtype], (at, gap, cut, err)
        # the plant works: seen or not seen is a difference of the logits' own size
        assert float((rows[window - 1] - rows[window]).abs().max() / rows[window].abs().max()) > 0.2


def test_a_planted_key_far_away(tmp_path_factory):
    """Without a window a key hundreds of tokens back, also on a page border, is still seen: the
    plain model with that key masked differs by the logits' own size."""
    config, d, A, B = _planted(tmp_path_factory.getbasetemp(), None,
                               mlp={"kind": "dense", "ff": 100})
    w = weights64(d)
    eng = engine_for(d, "float32")
    for at, gap in ((0, 300), (64, 257), (127, 400), (3, 511)):
        seq = _sequence(config, A, B, at, gap, tail=1)
        want = P.forward(config, w, seq)
        for cut in (len(seq), at + gap, at + 2):
            s = eng.alloc_slot()
            got = feed(eng, s, seq, [cut] if cut > at + 2 else [cut, at + gap])
            eng.free_slot(s)
            assert rel_err(got[at + gap:], want[at + gap:]) < BUDGET["float32"], (at, gap, cut)
        near = dict(config, layers=[dict(config["layers"][0],
                                         mixer=dict(config["layers"][0]["mixer"], mask={"size": gap}))])
        blind = P.forward(near, w, seq)[at + gap]
        assert float((blind - want[at + gap]).abs().max() / want[at + gap].abs().max()) > 0.2


def test_greedy_generation_through_the_engine(tmp_path_factory):
    """`Engine.generate` (scheduler, sampler, decode graphs) gives the plain model's greedy tokens."""
    d = write_model(tmp_path_factory.getbasetemp(), MIXED, seed=13)
    w = weights64(d)
    eng = engine_for(d, "float32")
    prompts = [random_ids(n, MIXED["vocab"], 3 * n) for n in (5, 68, 1, 31)]
    got = eng.generate(prompts, max_new_tokens=8, stop_token_ids=[])
    assert got == [P.generate_greedy(MIXED, w, p, 8) for p in prompts]
    assert eng.generate(prompts[:2], max_new_tokens=4, stop_token_ids=[], max_step_tokens=16) == \
        [g[:4] for g in got[:2]]
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_of_many_short_requests(tmp_path, dtype):
    """`bin/trace_run` on a Rabapel folder: fourteen requests of 1 to 75 tokens in one batch, then
    decoded together while the shorter ones end, with --max-tokens the tokens themselves (every
    request holds a partly filled page on top of that)."""
    from test_gpu_trace import replay
    d = write_model(tmp_path, MIXED, seed=21, dtype=STORE[dtype])
    w = weights64(d)
    lens = [1, 2, 3, 5, 8, 13, 21, 34, 55, 75, 65, 64, 63, 4]
    reqs = [random_ids(n + 2 + i % 3, MIXED["vocab"], 50 + i) for i, n in enumerate(lens)]
    plain = [P.forward(MIXED, w, r) for r in reqs]
    steps = [{"step": 0, "entries": [{"id": f"r{i}", "tokens": r[:lens[i]], "want": [lens[i] - 1]}
                                     for i, r in enumerate(reqs)], "end": []}]
    expect = {0: torch.cat([plain[i][lens[i] - 1:lens[i]] for i in range(len(reqs))])}
    at, live, n = list(lens), list(range(len(reqs))), 1
    while live:
        ends = [i for i in live if at[i] == len(reqs[i]) - 1]
        steps.append({"step": n, "entries": [{"id": f"r{i}", "tokens": [reqs[i][at[i]]], "want": [0]} for i in live],
                      "end": [f"r{i}" for i in ends]})
        expect[n] = torch.cat([plain[i][at[i]:at[i] + 1] for i in live])
        n += 1
        for i in live:
            at[i] += 1
        live = [i for i in live if i not in ends]
    got = replay(d, dtype, str(tmp_path / "out"), sum(len(r) for r in reqs), steps)
    for s_ in sorted(expect):
        close(torch.from_numpy(got[s_].copy()), expect[s_], dtype, f"step {s_}")


def test_command_line_and_a_conversation(tmp_path):
    """`bin/chat` on a Rabapel folder with token-id prompts, greedy: the plain model's tokens; and
    `Engine.session`: the turns of a conversation go on from the slot's cache by several tokens."""
    import os
    import subprocess
    import sys
    d = write_model(tmp_path, MIXED, seed=17)
    w = weights64(d)
    prompts = [random_ids(n, MIXED["vocab"], 9 * n) for n in (6, 2)]
    ids_file = tmp_path / "prompts.txt"
    ids_file.write_text("\n".join(" ".join(map(str, p)) for p in prompts) + "\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "chat"), "-m", d, "-d", "float32", "--temp", "0",
                        "-n", "7", "--prompt-ids-file", str(ids_file), "-c", "64", "--type", "rabapel"],
                       capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    got = [[int(t) for t in line.split()] for line in r.stdout.strip().splitlines()]
    assert got == [P.generate_greedy(MIXED, w, p, 7) for p in prompts]
    eng = engine_for(d, "float32")
    with eng.session(stop_token_ids=[]) as chat:
        said = list(prompts[0])
        a1 = chat.say(prompts[0], max_new_tokens=4)
        assert a1 == P.generate_greedy(MIXED, w, said, 4)
        turn = random_ids(5, MIXED["vocab"], 77)
        a2 = chat.say(turn, max_new_tokens=3)
        # the token that max_new_tokens cut off is fed in front of the next turn
        assert a2 == P.generate_greedy(MIXED, w, said + a1 + turn, 3)


def test_architecture_is_chosen_by_config_and_refuses_what_it_lacks(tmp_path_factory):
    import inferllm_amd as I
    assert "Rabapel" in I.registered_architectures()
    bad = dict(MIXED, layers=[dict(MIXED["layers"][0], type="something_else")])
    with pytest.raises(I.ConfigError):
        I.config_from_dict(bad)


# ---------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,dn,dr,dv,R,rot,window", [(3, 16, 8, 24, 40, 8, 0), (16, 8, 16, 12, 64, 12, 70),
                                                     (5, 24, 32, 40, 48, 32, 33), (20, 16, 16, 16, 128, 16, 0),
                                                     (1, 0, 8, 8, 16, 8, 65), (2, 8, 8, 8, 600, 8, 0)])
def test_latent_kernels_alone(dtype, H, dn, dr, dv, R, rot, window):
    """Norm, rotation and store of the latent rows, the packed rows for prompts, the gate, and
    one token's attention over the paged latent cache (both kernels), against plain torch
    (tests/kernel_refs.py), with scattered pages, a window's ring and unequal lengths."""
    from inferllm_amd.kernels import ops
    import kernel_refs as K
    g = torch.Generator().manual_seed(H * 100 + R)
    page, ring = 64, ((window + 62) // 64 + 1 if window else 0)
    per_seq = ring or 4
    lens = [130, 64, 200] if not window else [130, 64, 333]
    table = torch.randperm(3 * per_seq, generator=g).to(torch.int32).view(3, per_seq)
    ncols = H * (dn + dr) + R + dr + H
    cos_sin = torch.randn((512, rot // 2, 2), generator=g)
    norm_w = (torch.rand((R,), generator=g) + 0.5).to(dtype)
    w_uk = (torch.randn((H * dn, R), generator=g) * 0.3).to(dtype)
    w_uv = (torch.randn((H * dv, R), generator=g) * 0.3).to(dtype)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    transposed = dtype == torch.bfloat16 and R % 16 == 0 and (R + dr) % 8 == 0
    cache_ref = torch.zeros((3 * per_seq + 1, page, R + dr), dtype=dtype)
    cache_gpu = cache_ref.clone().cuda()
    ct_ref = torch.zeros((3 * per_seq + 1, R, page, 1), dtype=dtype) if transposed else None
    ct_gpu = ct_ref.clone().cuda() if transposed else None
    # whole prompts: all rows of the three sequences in one call
    T = sum(lens)
    y = torch.randn((T, ncols), generator=g).to(dtype)
    pos = torch.cat([torch.arange(n) for n in lens]).to(torch.int32)
    slot = torch.cat([torch.full((n,), i) for i, n in enumerate(lens)]).to(torch.int32)
    slot_len = torch.tensor(lens, dtype=torch.int32)
    y_gpu = y.clone().cuda()
    c_g, kr_g = ops.latent_rope_store(y_gpu, H, dn, dr, R, rot, cos_sin.cuda(), norm_w.cuda(), 1e-5, pos.cuda(),
                                      slot.cuda(), slot_len.cuda(), cache_gpu, table.cuda(), page, ring, True, ct_gpu)
    c_r, kr_r = K.latent_rope_store(y, H, dn, dr, R, rot, cos_sin, norm_w, 1e-5, pos, slot, slot_len, cache_ref,
                                    table, page, ring, True, ct_ref)
    for got, want in ((c_g, c_r), (kr_g, kr_r), (y_gpu, y), (cache_gpu, cache_ref)) + (((ct_gpu, ct_ref),) if transposed else ()):
        assert float((got.double().cpu() - want.double()).abs().max()) <= tol * max(1.0, float(want.double().abs().max()))
    cache_gpu.copy_(cache_ref)                      # the same bits on both sides from here on
    if transposed:
        ct_gpu.copy_(ct_ref)
    kvu = torch.randn((T, H * (dn + dv)), generator=g).to(dtype)
    P_ = -(-max(dn + dr, dv) // 16) * 16
    packed = ops.latent_pack(y_gpu, kvu.cuda(), kr_g, H, dn, dr, dv, P_)
    assert torch.equal(packed.cpu(), K.latent_pack(y_gpu.cpu(), kvu, kr_g.cpu(), H, dn, dr, dv, P_))
    attn = torch.randn((T, H * P_), generator=g).to(dtype)
    gated = ops.latent_gate(attn.cuda(), y_gpu, ncols - H, H, dv, P_)
    assert rel_err(gated, K.latent_gate(attn, y_gpu.cpu(), ncols - H, H, dv, P_).double()) < tol
    # one more token of each sequence: store and queries in one launch, then the walk over the cache
    y1 = torch.randn((3, ncols), generator=g).to(dtype)
    p1 = torch.tensor(lens, dtype=torch.int32)
    s1 = torch.arange(3, dtype=torch.int32)
    y1_gpu = y1.clone().cuda()
    for qa_dtype in ([torch.float32, torch.bfloat16] if transposed else [torch.float32]):
        ct = ct_gpu if qa_dtype == torch.bfloat16 else None
        qa_g = ops.latent_store_absorb(y1_gpu, H, dn, dr, R, rot, cos_sin.cuda(), norm_w.cuda(), 1e-5, p1.cuda(),
                                       s1.cuda(), cache_gpu, table.cuda(), page, ring, w_uk.cuda(), qa_dtype, ct_gpu)
        qa_r = K.latent_store_absorb(y1, H, dn, dr, R, rot, cos_sin, norm_w, 1e-5, p1, s1, cache_ref, table, page,
                                     ring, w_uk, qa_dtype, ct_ref)
        assert torch.equal(y1_gpu.cpu(), y1)                      # the rows keep their unrotated queries
        assert rel_err(qa_g, qa_r.double()) < (tol if qa_dtype == torch.float32 else 2e-2)
        assert float((cache_gpu.double().cpu() - cache_ref.double()).abs().max()) <= tol * max(1.0, float(cache_ref.double().abs().max()))
        cache_gpu.copy_(cache_ref)
        if transposed:
            ct_gpu.copy_(ct_ref)
        want = K.latent_attn_decode(qa_g.cpu(), y1, w_uv, ncols - H, cache_ref, table, page, ring, s1, p1 + 1, 0,
                                    H, dr, R, dv, 0.2, window, 1).double()
        for nsplit in (1, 3, 7):
            got = ops.latent_attn_decode(qa_g, y1_gpu, w_uv.cuda(), ncols - H, cache_gpu, table.cuda(), page, ring,
                                         s1.cuda(), (p1 + 1).cuda(), 0, H, dr, R, dv, 0.2, window, nsplit, ct)
            assert rel_err(got, want) < tol, (qa_dtype, nsplit)
    # the queries' product alone (rows whose queries are rotated already)
    qa2 = ops.latent_absorb_q(y_gpu[:5].contiguous(), w_uk.cuda(), H, dn, dr, R, torch.float32)
    assert rel_err(qa2, K.latent_absorb_q(y_gpu[:5].cpu(), w_uk, H, dn, dr, R, torch.float32).double()) < tol


@pytest.mark.parametrize("E", [96, 90, 2048])
def test_norm_adds_a_pair_of_outputs(E):
    """x + (a + b) and the norm in one kernel, for all rows and for picked rows."""
    from inferllm_amd.kernels import ops
    import kernel_refs as K
    g = torch.Generator().manual_seed(E)
    x = torch.randn((7, E), generator=g)
    a = torch.randn((7, E), generator=g).to(torch.bfloat16)
    b = torch.randn((7, E), generator=g)
    wt = torch.rand((E,), generator=g) + 0.5
    for rows in (None, torch.tensor([5, 0, 2], dtype=torch.int32)):
        xg, xr = x.clone().cuda(), x.clone()
        got = ops.add_rmsnorm(xg, (a.cuda(), b.cuda()), wt.cuda(), 1e-5, torch.float32,
                              rows.cuda() if rows is not None else None)
        want = K.add_rmsnorm(xr, (a, b), wt, 1e-5, torch.float32, rows)
        assert float((got.cpu() - want).abs().max()) < 1e-5
        assert float((xg.cpu() - xr).abs().max()) < 1e-6



@pytest.mark.parametrize("n_out,top", [(7, 3), (16, 2), (130, 8), (3, 1)])
def test_router_kernel(n_out, top):
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(n_out)
    z = torch.randn((50, n_out), generator=g) * 2
    corr = torch.randn((n_out,), generator=g) * 0.3
    idx, wt = ops.moe_route(z.cuda(), corr.cuda(), top)
    s = torch.softmax(z.double(), -1)
    want = torch.topk(s + corr.double(), top, dim=-1).indices
    assert torch.equal(idx.cpu().long(), want)
    assert float((wt.cpu().double() - torch.gather(s, 1, want)).abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 3, 8, 9, 40])
def test_router_product_choice_and_grouping(dtype, T):
    """A routed layer's plan: the choices and weights of the router's float32 product, and every
    (token, choice) pair in its expert's group, in tiles of no more rows than said."""
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(T)
    E, NE, n_real, top, F = 96, 11, 8, 3, 32
    h = torch.randn((T, E), generator=g).to(dtype).cuda()
    w = torch.randn((NE, E), generator=g).cuda()
    corr = (torch.randn((NE,), generator=g) * 0.05).to(dtype).cuda()
    wgu = torch.zeros((n_real, 2 * F, E), dtype=dtype).cuda()
    idx, wt, (order, tiles, max_tiles, rows, _) = ops.moe_plan(h, w, corr, top, wgu)
    idx3, wt3 = ops.moe_route(ops.few_outputs_f32(h, w), corr, top)
    assert torch.equal(idx, idx3) and torch.equal(wt, wt3)
    want = torch.topk(torch.softmax(h.double().cpu() @ w.double().cpu().T, -1) + corr.double().cpu(), top).indices
    assert torch.equal(idx.cpu().long(), want)
    n_tiles = int(tiles[3 * max_tiles])
    seen = []
    for i in range(n_tiles):
        e, first, n = (int(v) for v in tiles[3 * i:3 * i + 3])
        assert 0 < n <= rows
        pairs = order[first:first + n].cpu().tolist()
        assert all(int(idx.view(-1)[p]) == e for p in pairs)
        seen += pairs
    assert sorted(seen) == [p for p in range(T * top) if int(idx.view(-1)[p]) < n_real]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,F,n_real,n_id,top,T", [(64, 40, 5, 2, 3, 37), (90, 30, 2, 0, 1, 9),
                                                   (128, 96, 12, 4, 2, 300), (96, 64, 6, 1, 2, 3),
                                                   (160, 32, 4, 0, 3, 40), (256, 128, 3, 1, 2, 700),
                                                   (320, 64, 12, 4, 2, 1000), (512, 160, 5, 0, 1, 1)])
def test_expert_kernels(dtype, E, F, n_real, n_id, top, T):
    """Grouping, the experts' products and the weighted sum against a loop over tokens."""
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(E + T)
    h = torch.randn((T, E), generator=g).to(dtype)
    wgu = (torch.randn((n_real, 2 * F, E), generator=g) * 0.2).to(dtype)
    wd = (torch.randn((n_real, E, F), generator=g) * 0.2).to(dtype)
    idx = torch.stack([torch.randperm(n_real + n_id, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    wt = torch.rand((T, top), generator=g)
    shared = torch.randn((T, E), generator=g).to(dtype)
    sg = torch.randn((E,), generator=g).to(dtype) * 0.1
    y = ops.moe_experts(h.cuda(), idx.cuda(), wgu.cuda(), wd.cuda())
    out = ops.moe_combine(h.cuda(), idx.cuda(), wt.cuda(), y, n_real, shared.cuda(), sg.cuda())
    h64, want = h.double(), torch.zeros((T, E), dtype=torch.float64)
    for t in range(T):
        for k in range(top):
            e = int(idx[t, k])
            if e < n_real:
                gu = wgu[e].double() @ h64[t]
                v = wd[e].double() @ (torch.nn.functional.silu(gu[:F]) * gu[F:])
            else:
                v = h64[t]
            want[t] += wt[t, k].double() * v
        want[t] += torch.sigmoid(h64[t] @ sg.double()) * shared[t].double()
    assert rel_err(out, want) < (1e-5 if dtype == torch.float32 else 2e-2)
