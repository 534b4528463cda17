"""Sabipel through the engine against the plain model (tests/plain_sabipel.py): every mechanism in
a layer of its own, whole prompts, token-by-token decoding, prompts cut into portions down to two
tokens, batches of unequal requests, slots, pages and states used again, planted keys just inside
and just outside a chunk, at page borders, in prompts and in decoding, a memory from far back, the
first tokens, long decoding, greedy generation through the engine's own loop, the command line and
the trace replay; and the new kernels alone.  Configurations: tests/sabipel_tiny.py."""
import json
import os

import pytest
import torch

import kernel_refs as R
import plain_sabipel as P
from sabipel_tiny import (CONFIGS, MIXED, NO_KEYS, ODD, _att, _mem, _ssm, plant_key, plant_memory, single,
                          weights64, write_model)
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
    "state_space_groups_shared": single("mamba2", _ssm(6, 12, 20, 2, 4, 3)),
    "state_space_one_head_a_group_two_taps": single("mamba2", _ssm(3, 40, 8, 3, 2, 1)),
    "state_space_wide_state_one_tap": single("mamba2", _ssm(2, 70, 96, 1, 1, 5)),
    "memory_wide_keys": single("mlstm", _mem(3, 40, 12, 7.0)),
    "memory_wide_values_cap_bites": single("mlstm", _mem(2, 8, 72, 1.2)),
    "attention_chunks": single("attention", _att(6, 3, 16, 40, 0.3, chunk=29)),
    "attention_no_chunks_one_kv_head": single("attention", _att(5, 1, 24, 8, 0.2)),
    "feed_forward": single("mamba2", _ssm(2, 8, 8, 1, 3, 2), ff=88),
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
    tokens, portions that end at, before and after a chunk's and a page's border) and then one by one."""
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
            close(torch.cat(got[i]), P.forward(MIXED, w, r), dtype, f"round {round_} request {i}")
        for s in slots:
            eng.free_slot(s)
        eng.cache.check()


def test_state_starts_at_zero_in_a_slot_used_before(tmp_path_factory):
    """The states, the convolution's tail, the running maximum and the token before a step's first
    are cleared when a slot is handed out: the same request twice in the same slot gives the same
    bits, with another request between."""
    from inferllm_amd import StepEntry
    d = write_model(tmp_path_factory.getbasetemp(), NO_KEYS, seed=2, dtype=torch.float32)
    eng = engine_for(d, "float32", max_batch=1)
    a, b = random_ids(50, NO_KEYS["vocab"], 1), random_ids(77, NO_KEYS["vocab"], 2)
    outs = []
    for ids in (a, b, a):
        slot = eng.alloc_slot()
        eng.step([StepEntry(slot, ids[:-1], [])])
        outs.append(eng.step([StepEntry(slot, ids[-1:], [0])]).clone())
        eng.free_slot(slot)
    assert torch.equal(outs[0], outs[2])
    close(outs[0], P.forward(NO_KEYS, weights64(d), a)[-1:], "float32")


# ------------------------------------------------------------------ the edges of chunks
CHUNK = 37


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("query_at, key_at", [
    (110, 74), (110, 73),         # the chunk's first position, and the one before it
    (73, 37), (74, 73), (74, 74),  # a query that is a chunk's last, a chunk's first
    (147, 111), (147, 110),       # across the page border at 128
    (66, 63), (66, 64),           # a key on both sides of the page border at 64 inside one chunk
    (36, 0), (37, 0), (1, 0),     # the first chunk and the first tokens
])
def test_a_planted_key_just_inside_and_just_outside_a_chunk(tmp_path_factory, query_at, key_at, dtype):
    """One position's key is made to stand out for one query position.  The query comes inside a
    prompt and again, with the same tokens, as a decoded token of a second run; the key lies at the
    first position of the query's chunk or just before it, on both sides of page borders, at the
    sequence's first tokens.  A key that is wrongly seen or wrongly missed moves the logits by far
    more than the budget."""
    config = single("attention", _att(4, 2, 16, 24, 1.0, chunk=CHUNK), ff=40, vocab=260)
    KEY, QUERY = 250, 251
    ids = [t % 250 for t in random_ids(150, 250, 31)]
    ids[key_at] = KEY
    if query_at != key_at:
        ids[query_at] = QUERY
    edit = lambda w: plant_key(w, config, KEY, QUERY if query_at != key_at else KEY)
    d = write_model(tmp_path_factory.getbasetemp(), config, seed=8, dtype=STORE[dtype], edit=edit)
    w = weights64(d)
    want = P.forward(config, w, ids)
    # the same weights with the key's visibility the other way round (what an implementation that
    # is off at the chunk's edge, or loses the key's row, would give): far from the right logits
    start = query_at // CHUNK * CHUNK
    if key_at == query_at:
        wrong = P.forward(config, w, ids[:key_at] + [7] + ids[key_at + 1:])
    elif key_at >= start:
        wrong = P.forward(config, w, ids, edge_shift=key_at - start + 1)
    else:
        wrong = P.forward(config, w, ids, edge_shift=key_at - start)
    moved = (wrong[query_at] - want[query_at]).abs().max() / want[query_at].abs().max()
    assert float(moved) > 8 * BUDGET[dtype], float(moved)
    eng = engine_for(d, dtype)
    slot = eng.alloc_slot()
    got = feed(eng, slot, ids, [150])
    close(got[[query_at]], want[[query_at]], dtype, "the query's row in a prompt")
    close(got, want, dtype, "prompt")
    eng.free_slot(slot)
    slot = eng.alloc_slot()
    got = feed(eng, slot, ids[:query_at + 3], [max(1, query_at - 2)])
    close(got[[query_at]], want[[query_at]], dtype, "the query's row decoded")
    close(got, want[:query_at + 3], dtype, "decoded")
    eng.free_slot(slot)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["mlstm", "mamba2"])
def test_a_memory_from_far_back(tmp_path_factory, kind, dtype):
    """A recurrent layer that hardly forgets: the sequence's first token still moves the logits 300
    tokens later, in a prompt and in decoded tokens; a state that is lost or cleared shows."""
    config = (single("mlstm", _mem(2, 24, 20, 15.0), vocab=150) if kind == "mlstm"
              else single("mamba2", _ssm(2, 20, 16, 1, 3, 1), vocab=150))
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
    """A prompt of 20 tokens, then 280 tokens one by one (over pages and chunks, through decode graphs)."""
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
                        "-n", "5", "--prompt-ids", " ".join(map(str, ids)), "-c", "64", "--type", "sabipel"],
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
    values, states, tails, the last token) by several tokens; a model with states is decoded in
    step, so no token is ever taken back."""
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


@pytest.mark.parametrize("lens", [[40, 3, 17], [1, 1, 1], [2, 9]])
def test_plain_gated_scan_against_plain_torch(lens):
    """The scan without the correction, in its layout for long steps (from 16 rows) and for short."""
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(len(lens) + lens[0])
    for G, H, dk, dv in ((2, 6, 20, 13), (1, 1, 70, 65), (3, 3, 8, 130)):
        T = sum(lens)
        cu, seq_slot, _ = _packed(lens, [4, 0, 2][:len(lens)])
        qn, kn = torch.randn(T, G, dk, generator=g), torch.randn(T, G, dk, generator=g)
        vv, beta = torch.randn(T, H, dv, generator=g), torch.rand(T, H, generator=g)
        dec = torch.rand(T, H, 1, generator=g) * 0.5 + 0.5
        state = torch.randn(6, H, dk, dv, generator=g)
        want_state = state.clone()
        want = R.delta_scan(qn, kn, vv, beta, dec, want_state, cu, seq_slot, len(lens), max(lens), correct=False)
        st = state.cuda()
        got = ops.delta_scan(*_cuda(qn, kn, vv, beta, dec), st, cu.cuda(), seq_slot.cuda(), len(lens), max(lens),
                             correct=False)
        _near(got, want, 1e-4)
        _near(st, want_state, 1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_state_space_kernels_against_plain_torch(dtype):
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    for (G, H, N, dv, taps, NG), lens in (((2, 4, 12, 10, 4, 5), [9, 1, 2]), ((1, 3, 40, 7, 2, 1), [1, 1]),
                                          ((3, 3, 8, 96, 1, 3), [5])):
        inner, C, T = H * dv, H * dv + 2 * G * N, sum(lens)
        cu, seq_slot, row_slot = _packed(lens, [3, 1, 0][:len(lens)])
        U = torch.randn(T, 2 * inner + 2 * G * N + H + 3, generator=g).to(dtype)
        conv_w, conv_b = torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
        tail = torch.randn(5, max(taps - 1, 1), C, generator=g).to(dtype)
        a_log, dt_bias = torch.randn(H, generator=g), torch.randn(H, generator=g)
        single_rows = max(lens) == 1
        t_want, t_got = tail.clone(), tail.cuda()
        want = R.ssm_prepare(U, inner, 2 * inner + 2 * G * N, conv_w, conv_b, t_want, row_slot, a_log, dt_bias,
                             G, H, N, dv, update_tail=single_rows)
        Ug = U.cuda()
        got = ops.ssm_prepare(Ug, inner, 2 * inner + 2 * G * N, conv_w.cuda(), conv_b.cuda(), t_got,
                              row_slot.cuda(), a_log.cuda(), dt_bias.cuda(), G, H, N, dv, update_tail=single_rows)
        for a, b in zip(got, want):
            _near(a, b, 1e-5)
        if not single_rows:
            R.delta_conv_tail(U, t_want, cu, seq_slot, len(lens), taps, col_off=inner)
            ops.delta_conv_tail(Ug, t_got, cu.cuda(), seq_slot.cuda(), len(lens), taps, col_off=inner)
        assert torch.equal(t_got.cpu(), t_want)
        o, x, D, w = (torch.randn(T, H, dv, generator=g), torch.randn(T, H, dv, generator=g),
                      torch.randn(H, generator=g), torch.randn(inner, generator=g).to(dtype))
        want = R.ssm_finish(o, x, D, U, 0, w, NG, 1e-5, torch.float32)
        got = ops.ssm_finish(o.cuda(), x.cuda(), D.cuda(), Ug, 0, w.cuda(), NG, 1e-5, torch.float32)
        _near(got, want, 1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_matrix_memory_kernels_against_plain_torch(dtype):
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(4)
    for (H, dk, dv, cap), lens in (((3, 10, 14, 2.0), [70, 1, 130]), ((1, 40, 9, 11.0), [1, 1, 1]),
                                   ((5, 8, 80, 0.7), [64, 65])):
        T = sum(lens)
        cu, seq_slot, _ = _packed(lens, [2, 0, 4][:len(lens)])
        width = 2 * H * dk + 2 * H * dv + 2 * H
        U = (torch.randn(T, width, generator=g) * 2).to(dtype)
        i_off = 2 * H * dk + H * dv
        i_bias, f_bias = torch.randn(H, generator=g), torch.randn(H, generator=g) + 1
        m = torch.randn(6, H, generator=g)
        m_want, m_got = m.clone(), m.cuda()
        want = R.memory_prepare(U, i_off, i_off + H, i_bias, f_bias, cap, m_want, cu, seq_slot, len(lens), H, dk, dv)
        got = ops.memory_prepare(U.cuda(), i_off, i_off + H, i_bias.cuda(), f_bias.cuda(), cap, m_got, cu.cuda(),
                                 seq_slot.cuda(), len(lens), H, dk, dv)
        for a, b in zip(got, want):
            _near(a, b, 1e-5)
        _near(m_got, m_want, 1e-5)
        o, em = torch.randn(T, H, dv + 1, generator=g), torch.rand(T, H, generator=g) * 2
        w = torch.randn(H * dv, generator=g).to(dtype)
        want = R.memory_finish(o, em, w, U, i_off + 2 * H, 1e-5, torch.float32)
        got = ops.memory_finish(o.cuda(), em.cuda(), w.cuda(), U.cuda(), i_off + 2 * H, 1e-5, torch.float32)
        _near(got, want, 1e-5)


@pytest.mark.parametrize("matrix_cores", [1, 0])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_with_bias_chunks_and_gate_against_plain_torch(dtype, matrix_cores):
    """Norms over whole q and k, value mixing and the store; then rows over the cache and single
    tokens with slopes, chunks and the gate, positions on both sides of chunk and page borders; the
    rows on the matrix cores' float32 instruction (widths up to 128 in steps of 4) and on the
    vector units (every width)."""
    from inferllm_amd.kernels import ops
    ops._lib().illm_set_attn_cap_mfma(matrix_cores)
    try:
        _attention_cases(dtype)
    finally:
        ops._lib().illm_set_attn_cap_mfma(1)


def _attention_cases(dtype):
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(6)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for nh, nkv, dk, dv, chunk, window in ((6, 2, 20, 12, 37, 0), (4, 4, 16, 40, 0, 0), (3, 1, 72, 8, 64, 50),
                                           (4, 2, 128, 128, 45, 0), (2, 2, 34, 130, 33, 0), (8, 2, 100, 36, 0, 0)):
        lens, starts, slots, page, pages = [150, 3, 1], [60, 0, 129], [1, 3, 0], 64, 20
        T = sum(lens)
        table = torch.randperm(pages, generator=g).view(4, 5).to(torch.int32)
        cu, seq_slot, row_slot = _packed(lens, slots)
        row_pos = torch.tensor([s + i for n, s in zip(lens, starts) for i in range(n)], dtype=torch.int32)
        width = nh * dk + nkv * dk + nkv * dv + nh * dv
        rows = torch.randn(T, width, generator=g).to(dtype)
        first = torch.randn(T, nkv * dv + 5, generator=g).to(dtype)
        qw, kw = torch.randn(nh * dk, generator=g).to(dtype), torch.randn(nkv * dk, generator=g).to(dtype)
        lam = torch.tensor([0.3])
        kc = (torch.randn(pages, nkv, page, dk, generator=g)).to(dtype)
        vc = (torch.randn(pages, nkv, page, dv, generator=g)).to(dtype)
        k_off, v_off, g_off = nh * dk, nh * dk + nkv * dk, nh * dk + nkv * dk + nkv * dv
        r_want, kc_want, vc_want = rows.clone(), kc.clone(), vc.clone()
        R.qkv_norm_mix_store(r_want, k_off, v_off, qw, kw, 1e-5, lam, first, 5, row_pos, row_slot, kc_want, vc_want,
                             table, page, 0, nh, nkv, dk, dv)
        r_got, kc_got, vc_got = rows.cuda(), kc.cuda(), vc.cuda()
        ops.qkv_norm_mix_store(r_got, k_off, v_off, qw.cuda(), kw.cuda(), 1e-5, lam.cuda(), first.cuda(), 5,
                               row_pos.cuda(), row_slot.cuda(), kc_got, vc_got, table.cuda(), page, 0, nh, nkv, dk, dv)
        _near(r_got, r_want, tol); _near(kc_got, kc_want, tol); _near(vc_got, vc_want, tol)
        slopes = torch.pow(2.0, -8.0 * torch.arange(1, nh + 1) / nh).float()
        seq_start = torch.tensor(starts, dtype=torch.int32)
        want = R.attn_cap_rows(r_want, cu, seq_slot, seq_start, kc_want, vc_want, table, page, 0, 3, max(lens),
                               nh, nkv, dk, dv, 0.2, 0.0, window, slopes, chunk, r_want, g_off)
        r_in, kc_in, vc_in = r_want.cuda(), kc_want.cuda(), vc_want.cuda()
        got = ops.attn_cap_rows(r_in, cu.cuda(), seq_slot.cuda(), seq_start.cuda(), kc_in, vc_in, table.cuda(),
                                page, 0, 3, max(lens), nh, nkv, dk, dv, 0.2, 0.0, window, slopes.cuda(), chunk,
                                r_in, g_off)
        _near(got, want, tol)
        # single tokens: the last row of each sequence again, as a decode step
        last = torch.tensor([int(cu[b + 1]) - 1 for b in range(3)])
        q1 = r_want[last].contiguous()
        seq_len = torch.tensor([s + n for s, n in zip(starts, lens)], dtype=torch.int32)
        for nsplit in (1, 3):
            got = ops.attn_cap_decode(q1.cuda(), kc_in, vc_in, table.cuda(), page, 0, seq_slot.cuda(),
                                      seq_len.cuda(), nh, nkv, dk, dv, 0.2, 0.0, window, nsplit, slopes.cuda(),
                                      chunk, q1.cuda(), g_off)
            _near(got, want[last], tol)


def test_pair_embedding_and_gelu_against_plain_torch():
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(9)
    V, E, buckets, places = 50, 36, 17, 40
    table, pairs, pos = (torch.randn(V, E, generator=g), torch.randn(buckets + 1, E, generator=g),
                         torch.randn(places, E, generator=g))
    tokens = torch.randint(0, V, (12,), generator=g).to(torch.int32)
    row_slot = torch.tensor([2] * 5 + [0] * 4 + [1] * 3, dtype=torch.int32)
    row_pos = torch.tensor([0, 1, 2, 3, 4, 7, 8, 9, 10, 0, 1, 2], dtype=torch.int32)
    last = torch.tensor([31, 5, 6, 9], dtype=torch.int32)
    l_want, l_got = last.clone(), last.cuda()
    want = R.embed_pairs(tokens, row_pos, row_slot, table, 2.5, pairs, buckets, 7, 3, pos, l_want, False)
    got = ops.embed_pairs(*_cuda(tokens, row_pos, row_slot, table), 2.5, pairs.cuda(), buckets, 7, 3, pos.cuda(),
                          l_got, False)
    _near(got, want, 1e-6)
    cu, seq_slot = torch.tensor([0, 5, 9, 12], dtype=torch.int32), torch.tensor([2, 0, 1], dtype=torch.int32)
    R.remember_last(tokens, cu, seq_slot, l_want, 3)
    ops.remember_last(tokens.cuda(), cu.cuda(), seq_slot.cuda(), l_got, 3)
    assert torch.equal(l_got.cpu(), l_want)
    one = torch.tensor([3, 0, 2], dtype=torch.int32)              # one row a sequence: remembered at once
    t1, p1 = tokens[:3].contiguous(), torch.tensor([4, 0, 9], dtype=torch.int32)
    want = R.embed_pairs(t1, p1, one, table, 1.0, pairs, buckets, 7, 3, None, l_want, True)
    got = ops.embed_pairs(t1.cuda(), p1.cuda(), one.cuda(), table.cuda(), 1.0, pairs.cuda(), buckets, 7, 3, None,
                          l_got, True)
    _near(got, want, 1e-6)
    assert torch.equal(l_got.cpu(), l_want)
    x = torch.randn(1000, generator=g) * 3
    _near(ops.gelu_tanh(x.cuda()), R.gelu_tanh(x), 1e-6)
    xb = (torch.randn(5, 1024, generator=g) * 3).to(torch.bfloat16)           # 8 values a thread
    _near(ops.gelu_tanh(xb.cuda()), R.gelu_tanh(xb), 1e-2)


@pytest.mark.parametrize("E, T", [(90, 3), (2048, 5), (8200, 2)])
def test_two_norms_of_the_same_rows_in_one_pass(E, T):
    from inferllm_amd.kernels import ops
    g = torch.Generator().manual_seed(E)
    x, a, b = (torch.randn(T, E, generator=g) for _ in range(3))
    w1, w2 = torch.randn(E, generator=g), torch.randn(E, generator=g)
    x_want = x.clone()
    want = R.add_rmsnorm(x_want, (a, b), w1, 1e-5, torch.float32, None, w2)
    xg = x.cuda()
    got = ops.add_rmsnorm(xg, (a.cuda(), b.cuda()), w1.cuda(), 1e-5, torch.float32, weight2=w2.cuda())
    _near(got[0], want[0], 1e-5); _near(got[1], want[1], 1e-5); _near(xg, x_want, 1e-6)
