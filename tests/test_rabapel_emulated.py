"""Rabapel through the step function, the cache and the model wiring on the CPU, with the GPU
kernels replaced by their plain torch contracts (tests/kernel_refs.py): packing, positions,
page tables and window rings, slots used again, portions of prompts, which rows get logits."""
import pytest
import torch

import kernel_refs
import plain_rabapel as P
from rabapel_tiny import MIXED, ODD, weights64, write_model
from tiny import random_ids

import inferllm_amd as I
from inferllm_amd.cache import CacheManager
from inferllm_amd.engine import DecoderModel, StepEntry, StepRunner


def build_runner(config, weights, max_tokens=2048, max_slots=4, step_rows=32):
    cfg = I.config_from_dict(config)
    model = DecoderModel(cfg.to_spec())
    model.load({k: v.to(torch.float32) for k, v in weights.items()})
    cache = CacheManager(model.kv_lines(), model.state_lines(), max_tokens=max_tokens, max_slots=max_slots,
                         max_seq_len=512, dtype=torch.float32, device="cpu", poison_freed=True,
                         step_rows=step_rows)
    return StepRunner(model, cache, torch.float32, torch.device("cpu"), use_graphs=False)


@pytest.fixture
def emulated(monkeypatch):
    kernel_refs.patch(monkeypatch)


@pytest.mark.parametrize("name", ["MIXED", "ODD"])
def test_prompts_tokens_and_portions_equal_plain(name, tmp_path, emulated):
    config = {"MIXED": MIXED, "ODD": ODD}[name]
    d = write_model(tmp_path, config, seed=2)
    w = weights64(d)
    r = build_runner(config, w)
    reqs = [random_ids(n, config["vocab"], 3 + n) for n in (90, 5, 41)]
    plain = [P.forward(config, w, ids) for ids in reqs]
    # together: prompts of unequal lengths, then three tokens each; the shortest ends first
    slots = [r.cache.alloc_slot() for _ in reqs]
    cut = [len(ids) - 3 for ids in reqs]
    out = r.step([StepEntry(s, ids[:k], [0, k - 1]) for s, ids, k in zip(slots, reqs, cut)])
    for i in range(3):
        assert (out[2 * i:2 * i + 2].double() - plain[i][[0, cut[i] - 1]]).abs().max() < 1e-5
    for t in range(3):
        live = [i for i in range(3) if not (i == 1 and t == 2)]
        if t == 2:
            r.cache.free_slot(slots[1])
        out = r.step([StepEntry(slots[i], [reqs[i][cut[i] + t]], [0]) for i in live])
        for j, i in enumerate(live):
            assert (out[j].double() - plain[i][cut[i] + t]).abs().max() < 1e-5
    for i in (0, 2):
        r.cache.free_slot(slots[i])
    # a prompt in portions (past the windows and a page border), in a slot that was used before
    s = r.cache.alloc_slot()
    at, rows = 0, []
    for c in (2, 30, 61, 67, 90):
        rows.append(r.step([StepEntry(s, reqs[0][at:c], list(range(c - at)))]))
        at = c
    assert (torch.cat(rows).double() - plain[0]).abs().max() < 1e-5
    r.cache.free_slot(s)
    r.cache.check()
