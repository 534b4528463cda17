"""Dotorax through the step function, the cache and the model wiring on the CPU, with the GPU
kernels replaced by their plain torch stand-ins (tests/kernel_refs.py): packing, page tables, the
states' slots (cleared when handed out, carried from step to step), the tails of the convolutions in
front of the sublayers and inside the recurrent unit over portions of one and two tokens, the pooled
rows of blocks that a step completes, layers that read an earlier layer's cache line, which rows get
logits."""
import pytest
import torch

import kernel_refs
import plain_dotorax as P
from dotorax_tiny import CONFIGS, MIXED, weights64, write_model
from tiny import random_ids

import inferllm_amd as I
from inferllm_amd.cache import CacheManager
from inferllm_amd.engine import DecoderModel, StepEntry, StepRunner
from inferllm_amd.weights.loader import stored_shapes


def build_runner(d, weights, max_tokens=1024, max_slots=3):
    cfg = I.load_config(d).with_tensor_shapes(stored_shapes(d))
    model = DecoderModel(cfg.to_spec())
    model.load({k: v.to(torch.float32) for k, v in weights.items() if k in model.wants()})
    cache = CacheManager(model.kv_lines(), model.state_lines(), max_tokens=max_tokens, max_slots=max_slots,
                         max_seq_len=256, dtype=torch.float32, device="cpu", poison_freed=True)
    return StepRunner(model, cache, torch.float32, torch.device("cpu"), use_graphs=False)


@pytest.fixture
def emulated(monkeypatch):
    kernel_refs.patch(monkeypatch)


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_prompts_tokens_and_portions_equal_plain(name, tmp_path, emulated):
    config = CONFIGS[name]
    d = write_model(tmp_path, config, seed=2)
    w = weights64(d)
    r = build_runner(d, w)
    reqs = [random_ids(n, config["vocab"], 3 + n) for n in (90, 5, 21)]
    plain = [P.forward(config, w, ids) for ids in reqs]
    slots = [r.cache.alloc_slot() for _ in reqs]
    cut = [len(ids) - 3 for ids in reqs]
    out = r.step([StepEntry(s, ids[:k], [0, k - 1]) for s, ids, k in zip(slots, reqs, cut)])
    for i in range(3):
        assert (out[2 * i:2 * i + 2].double() - plain[i][[0, cut[i] - 1]]).abs().max() < 1e-4
    for t in range(3):
        live = [i for i in range(3) if not (i == 1 and t == 2)]
        if t == 2:
            r.cache.free_slot(slots[1])
        out = r.step([StepEntry(slots[i], [reqs[i][cut[i] + t]], [0]) for i in live])
        for j, i in enumerate(live):
            assert (out[j].double() - plain[i][cut[i] + t]).abs().max() < 1e-4
    for i in (0, 2):
        r.cache.free_slot(slots[i])
    # a prompt in portions of one, two and more tokens (across a window's, a block's and a page's
    # border), in a slot, states and pages that were used before
    s = r.cache.alloc_slot()
    at, rows = 0, []
    for c in (1, 3, 5, 6, 30, 37, 39, 64, 66, 72, 73, 90):
        rows.append(r.step([StepEntry(s, reqs[0][at:c], list(range(c - at)))]))
        at = c
    assert (torch.cat(rows).double() - plain[0]).abs().max() < 1e-4
    r.cache.free_slot(s)
    r.cache.check()


def test_a_second_sublayers_tensors_without_a_feed_forward_stay_in_the_file(tmp_path, emulated):
    def edit(w):
        w["l2.norm2"] = torch.zeros(MIXED["width"], dtype=torch.float64)
        w["l2.canon2"] = torch.ones(MIXED["width"], MIXED["canon"]["taps"], dtype=torch.float64)
    d = write_model(tmp_path, MIXED, seed=6, edit=edit)
    w = weights64(d)
    cfg = I.load_config(d).with_tensor_shapes(stored_shapes(d))
    assert "l2.norm2" not in DecoderModel(cfg.to_spec()).wants()
    r = build_runner(d, w)
    ids = random_ids(20, MIXED["vocab"], 8)
    s = r.cache.alloc_slot()
    out = r.step([StepEntry(s, ids, list(range(20)))])
    assert (out.double() - P.forward(MIXED, w, ids)).abs().max() < 1e-4
