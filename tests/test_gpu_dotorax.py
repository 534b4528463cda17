"""Dotorax through the engine against the plain model (tests/plain_dotorax.py): every mechanism in
a layer of its own, whole prompts, token-by-token decoding, prompts cut into portions down to two
tokens, batches of unequal requests, slots, pages and states used again, planted keys far away, at
page borders and just inside and just outside a window, a pooled block that is just seen and one
that is not yet, in prompts and in decoding, a memory from far back, the first tokens, long
decoding, greedy generation through the engine's own loop, the command line and the trace replay;
and the new kernels alone.  Configurations: tests/dotorax_tiny.py."""
import json
import os

import pytest
import torch

import kernel_refs as R
import plain_dotorax as P
from dotorax_tiny import (CONFIGS, MIXED, NO_KEYS, ODD, _att, _gla, _left, _par, _rot, plant_key, plant_memory,
                          single, weights64, write_model)
from tiny import random_ids

pytestmark = pytest.mark.gpu

BUDGET = {"float32": 3e-5, "bfloat16": 4e-2}
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
    """float32: every row within the budget.  bfloat16: all rows but a few within the budget, and
    the median well inside it."""
    scale = want.abs().max()
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
    "attention_part_rotated_grouped": single("attention", _att(6, 3, 16, 40, 0.3, _rot(700.0, 6))),
    "attention_all_rotated_one_kv_head": single("attention", _att(5, 1, 24, 8, 0.2, _rot(20000.0, 24)), taps=4),
    "attention_wide_heads": single("attention", _att(2, 2, 136, 132, 0.05, _rot(100.0, 64)), taps=1),
    "window_and_pool": single("parallel", _par(_left(6, 2, 20, 12, 0.8, _rot(50.0, 10), 29, 4), 24, 2, 3, 1.0, 0.0)),
    "window_pool_of_one": single("parallel", _par(_left(2, 1, 8, 72, 1.1, _rot(9.0, 8), 17, 1), 8, 1, 1, 0.9, 0.1)),
    "recurrent_unit_three_blocks": single("parallel", _par(_left(1, 1, 8, 8, 0.5, _rot(10.0, 2), 5, 2), 66, 3, 4, 0.0, 1.0)),
    "recurrent_unit_one_wide_block": single("parallel", _par(_left(1, 1, 8, 8, 0.5, _rot(10.0, 2), 5, 2), 300, 1, 2, 0.1, 1.2)),
    "linear_attention_wide_keys": single("gla", _gla(3, 40, 12, 4.0, 6)),
    "linear_attention_wide_values": single("gla", _gla(2, 8, 72, 25.0, 2), taps=2),
    "feed_forward": single("gla", _gla(2, 8, 8, 8.0, 3), ff=88),
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
    close(feed(eng, slot, ids, [70]), P.forward(config, weights64(d), ids), dtype, name)
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
        close(torch.cat(got[i]), P.forward(config, w, r), dtype, f"request {i}")
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cuts", [[], [1], [2, 4, 6], [36, 37, 38, 63, 64, 65, 130], [17, 19, 100], [128]])
def test_token_by_token_and_portions_equal_the_whole_prompt(tmp_path_factory, cuts, dtype):
    """140 tokens one by one ([]), or in portions that end at `cuts` (portions of one and two
    tokens, portions that end at, before and after a window's, a block's and a page's border) and
    then one by one."""
    d = write_model(tmp_path_factory.getbasetemp(), MIXED, seed=4, dtype=STORE[dtype])
    eng = engine_for(d, dtype)
    ids = random_ids(140, MIXED["vocab"], 23)
    want = P.forward(MIXED, weights64(d), ids)
    slot = eng.alloc_slot()
    close(feed(eng, slot, ids if cuts else ids[:45], cuts), want if cuts else want[:45], dtype, str(cuts))
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
            close(torch.cat(got[i]), P.forward(MIXED, w, r), dtype, f"pass {round_} request {i}")
        for s in slots:
            eng.free_slot(s)
        eng.cache.check()


def test_state_starts_at_zero_in_a_slot_used_before(tmp_path_factory):
    """The states and the convolutions' tails are cleared when a slot is handed out: the same request
    twice in the same slot gives the same bits, with another request between."""
    from inferllm_amd import StepEntry
    config = single("parallel", _par(_left(2, 1, 8, 8, 0.5, _rot(10.0, 4), 9, 2), 40, 2, 4, 0.5, 1.0), ff=32)
    d = write_model(tmp_path_factory.getbasetemp(), config, seed=2, dtype=torch.float32)
    eng = engine_for(d, "float32", max_batch=1)
    a, b = random_ids(50, config["vocab"], 1), random_ids(77, config["vocab"], 2)
    outs = []
    for ids in (a, b, a):
        slot = eng.alloc_slot()
        eng.step([StepEntry(slot, ids[:-1], [])])
        outs.append(eng.step([StepEntry(slot, ids[-1:], [0])]).clone())
        eng.free_slot(slot)
    assert torch.equal(outs[0], outs[2])
    close(outs[0], P.forward(config, weights64(d), a)[-1:], "float32")


# ------------------------------------------------------------------ far keys, the edges of windows and of pooled blocks
def _planted(tmp_path_factory, config, dtype, n, query_at, key_at, p="l0.mix.", m=None, seed=8):
    KEY, QUERY = 250, 251
    ids = [t % 250 for t in random_ids(n, 250, 31)]
    ids[key_at] = KEY
    if query_at != key_at:
        ids[query_at] = QUERY
    edit = lambda w: plant_key(w, config, KEY, QUERY if query_at != key_at else KEY, p, m)
    d = write_model(tmp_path_factory.getbasetemp(), config, seed=seed, dtype=STORE[dtype], edit=edit)
    return d, ids


def _prompt_and_decoded(d, dtype, ids, want, query_at):
    eng = engine_for(d, dtype)
    slot = eng.alloc_slot()
    got = feed(eng, slot, ids, [len(ids)])
    close(got[[query_at]], want[[query_at]], dtype, "the query's row in a prompt")
    close(got, want, dtype, "prompt")
    eng.free_slot(slot)
    slot = eng.alloc_slot()
    got = feed(eng, slot, ids[:query_at + 3], [max(1, query_at - 2)])
    close(got[[query_at]], want[[query_at]], dtype, "the query's row decoded")
    close(got, want[:query_at + 3], dtype, "decoded")
    eng.free_slot(slot)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("query_at, key_at", [(399, 0), (399, 3), (300, 63), (300, 64), (257, 128), (1, 0), (5, 5)])
def test_a_planted_key_far_back_under_full_attention(tmp_path_factory, query_at, key_at, dtype):
    """One position's key is made to stand out for one query position hundreds of tokens later (at
    the sequence's first tokens, on both sides of page borders), in a prompt and as a decoded
    token; the same sequence without the key token gives logits far from the right ones."""
    config = single("attention", _att(4, 2, 16, 24, 1.0, _rot(10000.0, 8)), ff=40, vocab=260)
    d, ids = _planted(tmp_path_factory, config, dtype, 400, query_at, key_at)
    w = weights64(d)
    want = P.forward(config, w, ids)
    wrong = P.forward(config, w, ids[:key_at] + [7] + ids[key_at + 1:])
    moved = (wrong[query_at] - want[query_at]).abs().max() / want[query_at].abs().max()
    assert float(moved) > 8 * BUDGET[dtype], float(moved)
    _prompt_and_decoded(d, dtype, ids, want, query_at)


WINDOW, POOL = 37, 5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("query_at, key_at", [
    (110, 74), (110, 73),          # the window's last position, and the one beyond it (in no pooled block yet)
    (100, 64), (100, 63),          # the same on both sides of the page border at 64
    (165, 129), (165, 128),        # and of the one at 128
    (36, 0), (37, 0), (1, 0),      # the first tokens: inside the first window, just outside it
])
def test_a_planted_key_just_inside_and_just_outside_a_window(tmp_path_factory, query_at, key_at, dtype):
    """A key at the window's far edge is seen, one position further it is not (its block is not yet
    pooled either); a window that is one token off moves the logits by far more than the budget."""
    left = _left(4, 2, 16, 24, 1.0, _rot(10000.0, 8), WINDOW, POOL)
    config = single("parallel", _par(left, 16, 2, 2, 1.0, 0.05), ff=40, vocab=260)
    d, ids = _planted(tmp_path_factory, config, dtype, 170, query_at, key_at, "l0.mix.left.", left)
    w = weights64(d)
    want = P.forward(config, w, ids)
    if query_at - key_at < WINDOW - 1:             # well inside: the sequence without the key token
        wrong = P.forward(config, w, ids[:key_at] + [7] + ids[key_at + 1:])
    else:                                          # at the edge: a window that is one token off
        wrong = P.forward(config, w, ids, edge_shift=-1 if query_at - key_at < WINDOW else 1)
    moved = (wrong[query_at] - want[query_at]).abs().max() / want[query_at].abs().max()
    assert float(moved) > 8 * BUDGET[dtype], float(moved)
    _prompt_and_decoded(d, dtype, ids, want, query_at)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("query_at, key_at", [
    (46, 9), (45, 8),              # block 1 (positions 5..9) is seen from 46 = 9 + 37 on; at 45 its tokens
    (46, 5), (45, 5),              # up to 8 have left the window and nothing of them is seen
    (101, 64), (100, 61),          # the block 60..64 that ends at the page border
    (101, 60), (169, 2),           # a block's first token; a block from far back among thirty others
])
def test_a_planted_key_in_a_pooled_block_just_seen_and_not_yet(tmp_path_factory, query_at, key_at, dtype):
    """The planted key lies in a block of 5 tokens before the window: once the whole block has left
    the window its mean key and value are seen, one position earlier nothing of it is."""
    left = _left(4, 2, 16, 24, 4.0, _rot(10000.0, 8), WINDOW, POOL)
    config = single("parallel", _par(left, 16, 2, 2, 1.0, 0.05), ff=40, vocab=260)
    d, ids = _planted(tmp_path_factory, config, dtype, 170, query_at, key_at, "l0.mix.left.", left)
    w = weights64(d)
    want = P.forward(config, w, ids)
    last = key_at // POOL * POOL + POOL - 1
    if last < query_at - WINDOW:                   # seen for a while: the sequence without the key token
        wrong = P.forward(config, w, ids[:key_at] + [7] + ids[key_at + 1:])
    else:                                          # just seen, or not yet: blocks that come a token early or late
        wrong = P.forward(config, w, ids, pool_shift=-1 if last == query_at - WINDOW else 1)
    moved = (wrong[query_at] - want[query_at]).abs().max() / want[query_at].abs().max()
    assert float(moved) > 8 * BUDGET[dtype], float(moved)
    _prompt_and_decoded(d, dtype, ids, want, query_at)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_reads_the_keys_another_layer_stored(tmp_path_factory, dtype):
    """Two layers: the second has no key and value projections and reads the first one's cache line.
    With the first layer's key planted, the second layer's queries find it 200 tokens later."""
    first = _att(4, 2, 16, 24, 1.0, _rot(10000.0, 8))
    config = single("attention", first, ff=40, vocab=260)
    config["layers"].append({"type": "attention", "mixer": _att(6, 2, 16, 24, 0.7, _rot(10000.0, 8), kv_from=0),
                             "mlp": None})
    d, ids = _planted(tmp_path_factory, config, dtype, 260, 255, 40)
    w = weights64(d)
    want = P.forward(config, w, ids)
    _prompt_and_decoded(d, dtype, ids, want, 255)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["gla", "parallel"])
def test_a_memory_from_far_back(tmp_path_factory, kind, dtype):
    """A recurrent layer that hardly forgets: the sequence's first token still moves the logits 300
    tokens later, in a prompt and in decoded tokens; a state that is lost or cleared shows."""
    config = (single("gla", _gla(2, 24, 20, 2.0, 4), vocab=150) if kind == "gla" else
              single("parallel", _par(_left(1, 1, 8, 8, 0.5, _rot(10.0, 2), 4, 2), 48, 2, 3, 0.0, 1.0), vocab=150))
    ids = [149] + [t % 149 for t in random_ids(309, 149, 5)]
    edit = lambda w: plant_memory(w, config, 149)
    d = write_model(tmp_path_factory.getbasetemp(), config, seed=15, dtype=STORE[dtype], edit=edit)
    w = weights64(d)
    want = P.forward(config, w, ids)
    other = [7] + ids[1:]
    moved = (P.forward(config, w, other)[300:] - want[300:]).abs().max() / want[300:].abs().max()
    assert float(moved) > 4 * BUDGET[dtype], float(moved)
    eng = engine_for(d, dtype)
    slot = eng.alloc_slot()
    got = feed(eng, slot, ids, [300])
    close(got[300:], want[300:], dtype, kind + ", the last rows")
    close(got, want, dtype, kind)
    eng.free_slot(slot)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tmp_path_factory, dtype):
    """A prompt of 20 tokens, then 280 tokens one by one (over pages, windows and blocks, through
    decode graphs)."""
    d = write_model(tmp_path_factory.getbasetemp(), ODD, seed=12, dtype=STORE[dtype])
    eng = engine_for(d, dtype)
    ids = random_ids(300, ODD["vocab"], 41)
    slot = eng.alloc_slot()
    close(feed(eng, slot, ids, [20]), P.forward(ODD, weights64(d), ids), dtype)
    eng.free_slot(slot)


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
        want = P.generate_greedy(MIXED, w, p, 12)
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
    d = write_model(tmp_path, ODD, seed=14, dtype=torch.float32)
    w = weights64(d)
    ids = random_ids(9, ODD["vocab"], 2)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "chat"), "-m", d, "-d", "float32", "--temp", "0",
                        "-n", "5", "--prompt-ids", " ".join(map(str, ids)), "-c", "64", "--type", "dotorax"],
                       capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    assert [int(t) for t in r.stdout.split()] == P.generate_greedy(ODD, w, ids, 5)
    a, b = random_ids(70, ODD["vocab"], 4), random_ids(5, ODD["vocab"], 6)
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
    wa, wb = P.forward(ODD, w, a), P.forward(ODD, w, b)
    V = ODD["vocab"]
    got = {i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V)) for i in range(3)}
    close(got[0], torch.stack([wa[0], wa[67], wb[2]]), "float32")
    close(got[1], wb[3:4], "float32")
    close(got[2], torch.stack([wa[69], wb[4]]), "float32")


def test_a_conversation_in_one_slot(tmp_path):
    """`Engine.session`: the turns of a conversation go on from what the slot holds (keys and
    values, pooled rows, states, tails) by several tokens."""
    d = write_model(tmp_path, MIXED, seed=17)
    w = weights64(d)
    eng = engine_for(d, "float32")
    first = random_ids(6, MIXED["vocab"], 54)
    with eng.session(stop_token_ids=[]) as chat:
        a1 = chat.say(first, max_new_tokens=4)
        assert a1 == P.generate_greedy(MIXED, w, first, 4)
        turn = random_ids(5, MIXED["vocab"], 77)
        a2 = chat.say(turn, max_new_tokens=3)
        assert a2 == P.generate_greedy(MIXED, w, first + a1 + turn, 3)
    eng.cache.check()


# ------------------------------------------------------------------ kernels alone, against their plain torch stand-ins
def _cuda(*ts):
    return [t.cuda() if t is not None else None for t in ts]


def _near(got, want, tol=2e-5):
    want = want.double()
    assert float((got.double().cpu() - want).abs().max()) <= tol * max(1.0, float(want.abs().max()))


def _packed(lens, slots):
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    row_slot = torch.tensor([s for n, s in zip(lens, slots) for _ in range(n)], dtype=torch.int32)
    return cu, torch.tensor(slots, dtype=torch.int32), row_slot


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("lens", [[40, 3, 17], [1, 1, 1], [2, 1]])
def test_short_convolution_with_a_kept_tail_against_plain_torch(lens, dtype):
    """Steps of many rows, of one row (the tail moves on in the same launch) and of fewer rows than
    taps; with and without biases and the input added; then the tails kept for the next step."""
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(sum(lens))
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for C, taps, off in ((70, 4, 5), (300, 2, 0), (9, 1, 3), (33, 8, 0), (64, 3, 4), (1028, 4, 8)):
        T = sum(lens)
        cu, seq_slot, row_slot = _packed(lens, [4, 0, 2][:len(lens)])
        # (rows whose width, offset and channels are multiples of 4 take four channels a thread)
        X = torch.randn(T, C + off + (2 if C % 4 else 4), generator=g).to(dtype)
        w, bias, in_bias = torch.randn(C, taps, generator=g), torch.randn(C, generator=g), torch.randn(C, generator=g)
        tail = torch.randn(6, max(taps - 1, 1), C, generator=g).to(dtype)
        single = max(lens) == 1
        for b, ib, add in ((None, None, True), (bias, in_bias, False)):
            t_want, t_got = tail.clone(), tail.cuda()
            want = R.short_conv(X, off, C, w, t_want, row_slot, torch.float32, b, ib, add, update_tail=single)
            got = ops.short_conv(X.cuda(), off, C, w.cuda(), t_got, row_slot.cuda(), torch.float32,
                                 b.cuda() if b is not None else None, ib.cuda() if ib is not None else None, add,
                                 update_tail=single)
            _near(got, want, tol)
            if not single:
                R.short_conv_tail(X, off, t_want, cu, seq_slot, len(lens), taps, ib)
                ops.short_conv_tail(X.cuda(), off, t_got, cu.cuda(), seq_slot.cuda(), len(lens), taps,
                                    ib.cuda() if ib is not None else None)
            _near(t_got, t_want, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_with_a_gain_and_clamped_gate_against_plain_torch(dtype):
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for T, E in ((5, 90), (1, 4096), (33, 7)):
        a, w = (torch.randn(T, E, generator=g) * 3).to(dtype), torch.randn(E, generator=g) + 1
        _near(ops.rms_rows_gain(a.cuda(), w.cuda(), 1e-5, 0.3), R.rms_rows_gain(a, w, 1e-5, 0.3), 1e-5)
        gu = (torch.randn(T, 2 * E, generator=g) * 2).to(dtype)
        _near(ops.clamped_swish_mul(gu.cuda(), 1.25), R.clamped_swish_mul(gu, 1.25), tol)
        # the pass between two sublayers: the sublayer's own norm, the add, the next norm, and for
        # single tokens the convolution with its tail; or only some rows, with x left as it is
        x, w2 = torch.randn(T, E, generator=g), (torch.randn(E, generator=g) + 1).to(dtype)
        cw, tail = torch.randn(E, 3, generator=g), torch.randn(T + 1, 2, E, generator=g).to(dtype)
        slots = torch.randperm(T, generator=g).to(torch.int32)
        idx = torch.tensor([T - 1, 0], dtype=torch.int32)
        for post in (None, (a, w, 1e-5, 0.3)):
            for conv, rows in ((None, None), (None, idx), ((cw, tail, slots), None)):
                x_want, x_got, t_want, t_got = x.clone(), x.cuda(), tail.clone(), tail.cuda()
                want = R.post_add_rmsnorm(x_want, ops.PostNormed(*post) if post else None, w2, 2e-5, dtype, rows,
                                          (cw, t_want, slots) if conv else None)
                got = ops.post_add_rmsnorm(x_got, ops.PostNormed(a.cuda(), w.cuda(), 1e-5, 0.3) if post else None,
                                           w2.cuda(), 2e-5, dtype, rows.cuda() if rows is not None else None,
                                           (cw.cuda(), t_got, slots.cuda()) if conv else None)
                _near(got, want, tol); _near(x_got, x_want, 1e-5); _near(t_got, t_want, tol)


@pytest.mark.parametrize("M, F, K", [(1, 344, 256), (8, 1000, 136), (16, 33, 1000), (40, 320, 96), (64, 2816, 1024),
                                     (100, 640, 512), (300, 96, 64)])
def test_gate_and_up_with_the_clamped_gate_against_plain_torch(M, F, K):
    """The gate|up product with the clamped gate: the fused kernels of few bfloat16 rows (from the
    plain matrix and from the copy in the kernels' tile order) and the product followed by the
    activation's own kernel, in bfloat16 and float32."""
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(M + F)
    x = torch.randn(M, K, generator=g)
    w = torch.randn(2 * F, K, generator=g) * (3.0 / K ** 0.5)
    for dtype, tol in ((torch.bfloat16, 3e-2), (torch.float32, 2e-5)):
        xd, wd = x.to(dtype), w.to(dtype)
        both = xd.double() @ wd.double().T
        gate, up = torch.clamp(both[:, :F], max=1.25), torch.clamp(both[:, F:], -1.25, 1.25)
        want = gate * torch.sigmoid(1.702 * gate) * (up + 1)
        ways = [wd.cuda()]
        if dtype == torch.bfloat16:
            ways.append(ops.decode_weight(wd.cuda(), "gate_up", True))
        for wv in ways:
            _near(ops.gate_up_act(xd.cuda(), wv, 1.25), want, tol)
    # limit 0 is SiLU times up, as before
    both = x.to(torch.bfloat16).double() @ w.to(torch.bfloat16).double().T
    want = both[:, :F] * torch.sigmoid(both[:, :F]) * both[:, F:]
    _near(ops.gate_up_act(x.to(torch.bfloat16).cuda(), w.to(torch.bfloat16).cuda()), want, 3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pooled_window_attention_against_plain_torch(dtype):
    """Rotation with either pairing, the norm a head and the store; the pooled rows of completed
    blocks; then rows over the cache and single tokens, positions on both sides of window, block
    and page borders, with and without a scale a head."""
    from inferllm_amd.kernels import ops
    from inferllm_amd.parts.position import rotary_table
    g = torch.Generator().manual_seed(6)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for nh, nkv, dk, dv, window, pool, rot, pairing in ((6, 2, 20, 12, 37, 3, 8, 1), (4, 4, 16, 40, 64, 8, 16, 0),
                                                        (3, 1, 72, 8, 50, 1, 2, 1), (2, 2, 34, 130, 9, 7, 34, 0),
                                                        (2, 1, 132, 136, 20, 0, 0, 0)):
        lens, starts, slots, page, pages = [150, 3, 1], [60, 0, 129], [1, 3, 0], 64, 20
        T = sum(lens)
        table = torch.randperm(pages, generator=g).view(4, 5).to(torch.int32)
        cu, seq_slot, row_slot = _packed(lens, slots)
        row_pos = torch.tensor([s + i for n, s in zip(lens, starts) for i in range(n)], dtype=torch.int32)
        k_off, v_off = nh * dk + 3, nh * dk + 3 + nkv * dk
        rows = torch.randn(T, v_off + nkv * dv + 1, generator=g).to(dtype)
        cs = rotary_table(77.0, rot, 300, "cpu") if rot else None
        kc = torch.randn(pages, nkv, page, dk, generator=g).to(dtype)
        vc = torch.randn(pages, nkv, page, dv, generator=g).to(dtype)
        kp, vp = torch.randn(kc.shape, generator=g).to(dtype), torch.randn(vc.shape, generator=g).to(dtype)
        r_want, kc_want, vc_want = rows.clone(), kc.clone(), vc.clone()
        qs = torch.rand(nh, generator=g) + 0.5 if pairing else None        # a scale a query head, or none
        R.qk_rotate_store(r_want, k_off, v_off, cs, rot, pairing, True, 1e-5, row_pos, row_slot, kc_want, vc_want,
                          table, page, 0, nh, nkv, dk, dv, qs)
        r_got, kc_got, vc_got = rows.cuda(), kc.cuda(), vc.cuda()
        ops.qk_rotate_store(r_got, k_off, v_off, cs.cuda() if rot else None, rot, pairing, True, 1e-5, row_pos.cuda(),
                            row_slot.cuda(), kc_got, vc_got, table.cuda(), page, 0, nh, nkv, dk, dv,
                            qs.cuda() if qs is not None else None)
        _near(r_got, r_want, tol); _near(kc_got, kc_want, tol); _near(vc_got, vc_want, tol)
        kp_want, vp_want, kp_got, vp_got = kp.clone(), vp.clone(), kp.cuda(), vp.cuda()
        if pool:
            # the blocks of the first sequence that ended before this step are there already
            early = torch.arange(60, dtype=torch.int32)
            R.pool_store(early, torch.full((60,), 1, dtype=torch.int32), kc_want, vc_want, kp_want, vp_want, table,
                         page, nkv, dk, dv, pool)
            R.pool_store(row_pos, row_slot, kc_want, vc_want, kp_want, vp_want, table, page, nkv, dk, dv, pool)
            ops.pool_store(early.cuda(), torch.full((60,), 1, dtype=torch.int32).cuda(), kc_got, vc_got, kp_got,
                           vp_got, table.cuda(), page, nkv, dk, dv, pool)
            ops.pool_store(row_pos.cuda(), row_slot.cuda(), kc_got, vc_got, kp_got, vp_got, table.cuda(), page, nkv,
                           dk, dv, pool)
            _near(kp_got, kp_want, tol); _near(vp_got, vp_want, tol)
        seq_start = torch.tensor(starts, dtype=torch.int32)
        for hs in (None, torch.rand(nh, generator=g) + 0.5):
            want = R.attn_pooled_rows(r_want, cu, seq_slot, seq_start, kc_want, vc_want, kp_want, vp_want, table,
                                      page, 3, max(lens), nh, nkv, dk, dv, 0.3, hs, window, pool)
            ins = _cuda(r_want, kc_want, vc_want, kp_want, vp_want)
            got = ops.attn_pooled_rows(ins[0], cu.cuda(), seq_slot.cuda(), seq_start.cuda(), *ins[1:], table.cuda(),
                                       page, 3, max(lens), nh, nkv, dk, dv, 0.3, hs.cuda() if hs is not None else None,
                                       window, pool)
            _near(got, want, tol)
            last = torch.tensor([int(cu[b + 1]) - 1 for b in range(3)])
            q1 = r_want[last].contiguous()
            seq_len = torch.tensor([s + n for s, n in zip(starts, lens)], dtype=torch.int32)
            got = ops.attn_pooled_decode(q1.cuda(), *ins[1:], table.cuda(), page, seq_slot.cuda(), seq_len.cuda(),
                                         nh, nkv, dk, dv, 0.3, hs.cuda() if hs is not None else None, window, pool)
            _near(got, want[last], tol)
            if pool and hs is None:
                # the window's tokens by the capped attention's kernels, which leave max + log(sum) of
                # every softmax, then the pooled blocks merged in: the same attention
                lse = torch.empty(T, nh, dtype=torch.float32, device="cuda")
                o = ops.attn_cap_rows(ins[0], cu.cuda(), seq_slot.cuda(), seq_start.cuda(), ins[1], ins[2],
                                      table.cuda(), page, 0, 3, max(lens), nh, nkv, dk, dv, 0.3, 0.0, window,
                                      lse=lse)
                ops.attn_pooled_rows(ins[0], cu.cuda(), seq_slot.cuda(), seq_start.cuda(), *ins[1:], table.cuda(),
                                     page, 3, max(lens), nh, nkv, dk, dv, 0.3, None, window, pool, out=o, lse=lse)
                _near(o, want, 2 * tol)
                lse1 = torch.empty(3, nh, dtype=torch.float32, device="cuda")
                o1 = ops.attn_cap_decode(q1.cuda(), ins[1], ins[2], table.cuda(), page, 0, seq_slot.cuda(),
                                         seq_len.cuda(), nh, nkv, dk, dv, 0.3, 0.0, window, 2, lse=lse1)
                ops.attn_pooled_decode(q1.cuda(), *ins[1:], table.cuda(), page, seq_slot.cuda(), seq_len.cuda(), nh,
                                       nkv, dk, dv, 0.3, None, window, pool, out=o1, lse=lse1)
                _near(o1, want[last], 2 * tol)


@pytest.mark.parametrize("matrix_cores", [1, 0])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_with_one_gate_a_head_against_plain_torch(dtype, matrix_cores):
    """The capped attention's kernels (rows on the matrix cores and on the vector units, single
    tokens with one and with several ranges of keys) with one gate a head in place of one a value."""
    from inferllm_amd.kernels import ops
    ops._lib().illm_set_attn_cap_mfma(matrix_cores)
    try:
        g = torch.Generator().manual_seed(9)
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        for nh, nkv, dk, dv in ((6, 2, 20, 12), (4, 4, 64, 64), (5, 1, 36, 130)):
            lens, starts, slots, page, pages = [150, 3, 1], [60, 0, 129], [1, 3, 0], 64, 20
            T = sum(lens)
            table = torch.randperm(pages, generator=g).view(4, 5).to(torch.int32)
            cu, seq_slot, _ = _packed(lens, slots)
            g_off = nh * dk + 2
            rows = torch.randn(T, g_off + nh + 1, generator=g).to(dtype)
            kc = torch.randn(pages, nkv, page, dk, generator=g).to(dtype)
            vc = torch.randn(pages, nkv, page, dv, generator=g).to(dtype)
            seq_start = torch.tensor(starts, dtype=torch.int32)
            want = R.attn_cap_rows(rows, cu, seq_slot, seq_start, kc, vc, table, page, 0, 3, max(lens), nh, nkv, dk,
                                   dv, 0.2, 0.0, 0, None, 0, rows, g_off, True)
            r_in, kc_in, vc_in = _cuda(rows, kc, vc)
            got = ops.attn_cap_rows(r_in, cu.cuda(), seq_slot.cuda(), seq_start.cuda(), kc_in, vc_in, table.cuda(),
                                    page, 0, 3, max(lens), nh, nkv, dk, dv, 0.2, 0.0, 0, None, 0, r_in, g_off, True)
            _near(got, want, tol)
            last = torch.tensor([int(cu[b + 1]) - 1 for b in range(3)])
            q1 = rows[last].contiguous()
            seq_len = torch.tensor([s + n for s, n in zip(starts, lens)], dtype=torch.int32)
            for nsplit in (1, 3):
                got = ops.attn_cap_decode(q1.cuda(), kc_in, vc_in, table.cuda(), page, 0, seq_slot.cuda(),
                                          seq_len.cuda(), nh, nkv, dk, dv, 0.2, 0.0, 0, nsplit, None, 0, q1.cuda(),
                                          g_off, True)
                _near(got, want[last], tol)
    finally:
        ops._lib().illm_set_attn_cap_mfma(1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_attention_and_recurrent_unit_kernels_against_plain_torch(dtype):
    """gla_prepare, and the recurrent unit's gates and scan: steps of many rows and of one, blocks
    of 8 to 300 channels, a state that goes on from what the slot holds."""
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(11)
    for lens in ([70, 1, 19], [1, 1, 1], [200, 64, 33]):      # from 64 rows on the scan runs in chunks
        T = sum(lens)
        cu, seq_slot, _ = _packed(lens, [2, 0, 4])
        for H, dk, dv in ((3, 10, 14), (1, 40, 9)):
            U = (torch.randn(T, 2 * H * dk + H * dv + 7, generator=g) * 2).to(dtype)
            Z = (torch.randn(T, H * dk, generator=g) * 3).to(dtype)
            zb = torch.randn(H * dk, generator=g)
            want = R.gla_prepare(U, 0, H * dk + 3, 2 * H * dk + 4, Z, zb, 7.0, H, dk, dv)
            got = ops.gla_prepare(U.cuda(), 0, H * dk + 3, 2 * H * dk + 4, Z.cuda(), zb.cuda(), 7.0, H, dk, dv)
            for a, b in zip(got, want):
                _near(a, b, 1e-5)
        for C, nb in ((24, 3), (300, 1), (64, 8), (1100, 1)):
            cb = C // nb
            u = torch.randn(T, C, generator=g) * 2
            wt = torch.randn(2, nb, cb, cb, generator=g) * min(0.5, 4.0 / cb ** 0.5)    # sums of about one size
            rb, ib, lam = (torch.randn(C, generator=g) for _ in range(3))
            a_want, x_want = R.lru_gates(u, wt, rb, ib, lam, 8.0)
            a_got, x_got = ops.lru_gates(*_cuda(u, wt, rb, ib, lam), 8.0)
            _near(a_got, a_want, 1e-5); _near(x_got, x_want, 1e-5)
            Y = (torch.randn(T, C + 5, generator=g) * 2).to(dtype)
            yb = torch.randn(C, generator=g)
            state = torch.randn(6, C, generator=g)
            s_want, s_got = state.clone(), state.cuda()
            want = R.lru_scan(a_want, x_want, s_want, Y, 5, yb, cu, seq_slot, 3, max(lens), torch.float32)
            got = ops.lru_scan(a_got, x_got, s_got, Y.cuda(), 5, yb.cuda(), cu.cuda(), seq_slot.cuda(), 3, max(lens),
                               torch.float32)
            _near(got, want, 1e-4); _near(s_got, s_want, 1e-4)
