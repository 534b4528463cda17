#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B]

Default: the LLaMA-2-7B layer sizes (32 layers, hidden 4096, 32/32 heads of 128,
feed-forward 11008, vocabulary 32000) with seeded random bfloat16 weights, a batch
of 8 sequences with 512-token prompts that decode 256 tokens (8 more to warm up),
cache context 4096.  A step is one decode step of the whole batch: step function, greedy choice on the device, the tokens
back on the host, as `Engine.generate` runs it.  One JSON line is printed: decoded tokens per second, the
prefill of 2,048 tokens, the decode step against the HBM roofline, and under
`points` decoding at batch 1 and 64, decoding from 3,800-token contexts at batch
8 and 64, milliseconds to the first token of prompts of 16, 64 and 160 tokens, prefills of
64 x 128, 8,192 and 16,384 tokens (and of 16,384 in steps of 2,048 that go on from the paged
cache), the LLaMA-3-8B shape with 16 prompts of 64 to 4,096 tokens and with 8 sequences at
8,000-token contexts, and the LLaMA-2-70B shape (prefill of 2,048 tokens, decode at batch 1 and
32 from 1,024-token prompts; `--no-70b` leaves it out).  Every decode run goes through the
engine's generation loop, whose stopwatch starts after the warm-up steps.  Every decode point has a
`..._hbm_frac` beside it: the bytes its step has to read (every weight once, the
cache of its live sequences) / its time / the HBM peak.  Peaks are the published ones
of MI355X (HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s, float32 157.3 TFLOP/s).
The run fails (non-zero) if any timed run produced a non-finite logit or the same
greedy token everywhere.

`--design rabapel`, `--design kukupel`, `--design sabipel` and `--design dotorax` are other workloads with a line of their own (the
default's stays as it is):
Rabapel (latent attention, layers that alternate a dense and a routed feed-forward) at two
sizes beside LLaMA at the same width, heads and layer count: prefill of 2,048 tokens and decoding
at batch 1, 8 and 64, each with its fraction of the matrix or HBM peak.
Kukupel likewise beside Rabapel, and Sabipel (state-space, matrix-memory and chunked-attention
layers with dense feed-forwards) beside Kukupel, and Dotorax (rotated attention with shared keys,
gated linear attention, a window with pooled blocks beside a recurrent unit, gated feed-forwards,
sublayers between two norms behind a short convolution) beside Sabipel.
"""
import argparse
import json
import sys
import time

HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

LLAMA2_7B = {"architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "intermediate_size": 11008,
             "num_hidden_layers": 32, "num_attention_heads": 32, "num_key_value_heads": 32,
             "vocab_size": 32000, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
             "max_position_embeddings": 4096, "tie_word_embeddings": False,
             "bos_token_id": 1, "eos_token_id": 2}


LLAMA3_8B = dict(LLAMA2_7B, intermediate_size=14336, num_key_value_heads=8, vocab_size=128256,
                 rope_theta=500000.0, max_position_embeddings=8192)
LLAMA2_70B = dict(LLAMA2_7B, hidden_size=8192, intermediate_size=28672, num_hidden_layers=80,
                  num_attention_heads=64, num_key_value_heads=8)
SHAPES = {"llama2-7b": ("LLaMA-2-7B shape", LLAMA2_7B), "llama3-8b": ("LLaMA-3-8B shape", LLAMA3_8B),
          "llama2-70b": ("LLaMA-2-70B shape", LLAMA2_70B)}


def weight_bytes_per_step(cfg, layers, esz):
    E, F, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim", E // nh)
    per_layer = ((nh + 2 * nkv) * hd * E + E * nh * hd + 3 * E * F + 2 * E) * esz
    return layers * per_layer + (V * E + E) * esz


def kv_bytes_per_token(cfg, layers, esz):
    nkv = cfg["num_key_value_heads"]
    hd = cfg.get("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])
    return layers * 2 * nkv * hd * esz


def prefill_flops(cfg, layers, T, out_rows=1, lens=None):
    """Flops of a prefill of T tokens (`lens`: the prompts' lengths if more than one)."""
    E, F, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim", E // nh)
    linear = 2.0 * T * ((nh + 2 * nkv) * hd * E + E * nh * hd + 3 * E * F)
    attn = sum(2.0 * 2.0 * nh * hd * (n * (n + 1) / 2) for n in (lens or [T]))
    return layers * (linear + attn) + 2.0 * out_rows * V * E


class Bench:
    """One engine of one shape and the runs on it."""

    def __init__(self, cfg, layers, dtype, max_batch, max_tokens, seed=1234):
        import torch
        from inferllm_amd import Engine
        self.torch = torch
        self.cfg = dict(cfg)
        self.full_layers = cfg["num_hidden_layers"]
        self.layers = layers or self.full_layers
        self.cfg["num_hidden_layers"] = self.layers
        self.esz = 2 if dtype == "bfloat16" else 4
        self.dkey = "bf16" if dtype == "bfloat16" else "fp32"
        t0 = time.time()
        self.eng = Engine.from_random(self.cfg, seed=0, dtype=dtype, device="cuda:0",
                                      max_batch=max_batch, max_seq_len=cfg["max_position_embeddings"],
                                      max_tokens=max_tokens)
        torch.cuda.synchronize()
        print(f"[bench] engine ready in {time.time() - t0:.1f} s "
              f"({self.layers} layers, room for {max_tokens} tokens)", file=sys.stderr, flush=True)
        self.g = torch.Generator().manual_seed(seed)

    def close(self):
        self.eng = None
        import gc
        gc.collect()
        self.torch.cuda.empty_cache()

    def ids(self, n):
        return self.torch.randint(0, self.cfg["vocab_size"], (n,), generator=self.g).tolist()

    @classmethod
    def around(cls, eng, vocab, layers, dtype, step_bytes, flops, seed=1234):
        """A bench around an engine that is there already (another design): `step_bytes(batch,
        mean_ctx)` and `flops(tokens, lens)` are the design's own counts."""
        import torch
        b = cls.__new__(cls)
        b.torch, b.eng, b.cfg, b.layers, b.full_layers = torch, eng, {"vocab_size": vocab}, layers, layers
        b.esz = 2 if dtype == "bfloat16" else 4
        b.dkey = "bf16" if dtype == "bfloat16" else "fp32"
        b.g = torch.Generator().manual_seed(seed)
        b.step_bytes = step_bytes
        b.flops = flops
        return b

    flops = None

    def step_bytes(self, batch, mean_ctx):
        return (weight_bytes_per_step(self.cfg, self.layers, self.esz)
                + batch * mean_ctx * kv_bytes_per_token(self.cfg, self.layers, self.esz))

    def decode_run(self, batch, steps, warmup, prompt):
        """(tokens/s, ms/step, fraction of the HBM peak) of `steps` timed decode steps of `batch`
        sequences that start from prompts of `prompt` tokens, through the engine's generation
        loop (greedy, no stop token): the loop runs `warmup` decode steps, waits for the device,
        and its stopwatch runs from there to the end of the batch."""
        from inferllm_amd.sampling import Sampler, SamplingParams
        torch, eng = self.torch, self.eng
        prompts = [self.ids(prompt) for _ in range(batch)]
        params = SamplingParams()                                   # greedy
        # (prompts go in steps of at most 16,384 tokens to bound the prefill's activations)
        loop = eng.generation_loop(Sampler(params, eng.device), max_step_tokens=16384)
        loop.time_after = warmup
        out = loop.run(prompts, params, warmup + steps + 1, [])
        st = loop.stats
        if st.timed_steps != steps or st.batches != 1 or any(len(o) != warmup + steps + 1 for o in out):
            raise SystemExit(f"bench: the loop timed {st.timed_steps} steps of {st.batches} batches at "
                             f"batch {batch}, not {steps} of one")
        dt = st.timed_seconds
        # what was timed must have computed something: greedy tokens that are not one and the same
        # everywhere (a run on NaN or constant logits would be as fast)
        distinct = {int(t) for o in out for t in o}
        print(f"[bench] batch {batch}, prompts of {prompt}: {dt / steps * 1e3:.3f} ms a step, "
              f"{len(distinct)} distinct greedy tokens in {steps + warmup} steps", file=sys.stderr, flush=True)
        if steps + warmup >= 16 and len(distinct) < 2:
            raise SystemExit(f"bench: the greedy token is {sorted(distinct)} in every step of every "
                             f"sequence at batch {batch}: the logits are degenerate")
        mean_ctx = prompt + 1 + warmup + (steps + 1) / 2.0
        ms = dt / steps * 1e3
        frac = self.step_bytes(batch, mean_ctx) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS
        return batch * steps / dt, ms, frac

    def prefill_run(self, T=2048, reps=6, prompts=1, max_step_tokens=None, skip=1):
        """`prompts` prompts of T tokens each in one step (or, with `max_step_tokens`, one prompt in
        steps of that many tokens that go on from the cache): tokens/s of the fastest of `reps` runs
        after the first `skip`, the time to the first token in ms, and the fraction of the matrix peak."""
        from inferllm_amd import StepEntry
        from inferllm_amd.kernels import ops
        torch, eng = self.torch, self.eng
        ids = [self.ids(T) for _ in range(prompts)]
        times = []
        for i in range(reps):
            slots = [eng.alloc_slot() for _ in ids]
            torch.cuda.synchronize()
            t = time.perf_counter()
            if max_step_tokens is None:
                logits = eng.step([StepEntry(s, p, [T - 1]) for s, p in zip(slots, ids)])
            else:
                for a in range(0, T, max_step_tokens):
                    piece = ids[0][a:a + max_step_tokens]
                    logits = eng.step([StepEntry(slots[0], piece, [len(piece) - 1] if a + len(piece) == T else [])])
            ops.argmax(logits).tolist()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            if not bool(torch.isfinite(logits).all()):
                raise SystemExit("bench: non-finite logits in the prefill")
            for s in slots:
                eng.free_slot(s)
        pt = min(times[skip:])
        fl = (self.flops(T * prompts, [T] * prompts) if self.flops is not None else
              prefill_flops(self.cfg, self.layers, T * prompts, prompts, [T] * prompts))
        return {"value": round(T * prompts / pt, 1), "tokens": T * prompts, "ms": round(pt * 1e3, 3),
                "frac": round(fl / pt / (PEAK_TFLOPS[self.dkey] * 1e12), 4)}

    def generate_run(self, lens, new_tokens):
        """Prompts of the given lengths through `Engine.generate` (all in one batch), three times
        (the first sets libraries and graphs up, the second may still take fresh memory from the
        driver for what the graphs' pools cannot lend it); the third run's figures: (prefill
        tokens/s, its fraction of the matrix peak, decode tokens/s, its fraction of the HBM peak)."""
        prompts = [self.ids(n) for n in lens]
        for _ in range(3):
            out = self.eng.generate(prompts, max_new_tokens=new_tokens, stop_token_ids=[])
            st = self.eng.last_stats
        assert all(len(o) == new_tokens for o in out)
        if len({t for o in out for t in o}) < 2:
            raise SystemExit("bench: the generation loop produced one and the same token everywhere")
        B, T = len(lens), sum(lens)
        pf = T / st.prefill_seconds
        pf_frac = (prefill_flops(self.cfg, self.layers, T, B, lens) / st.prefill_seconds
                   / (PEAK_TFLOPS[self.dkey] * 1e12))
        steps = st.decode_steps
        ms = st.decode_seconds / steps * 1e3
        mean_ctx = T / B + 1 + (steps + 1) / 2.0
        frac = self.step_bytes(B, mean_ctx) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS
        return pf, pf_frac, B * steps / st.decode_seconds, frac


# ---------------------------------------------------------------- another design beside LLaMA
def rabapel_config(width, heads, layers, dense_ff, experts, expert_ff, top, shared_ff, vocab=32000,
                   window=None):
    """Layers that alternate a dense and a routed feed-forward; heads of 128 + 64 query dims,
    128 value dims and a latent of 512, the sizes such heads have in published models."""
    mixer = {"heads": heads, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "scale": 192 ** -0.5,
             "rot": {"base": 10000.0, "dims": 64,
                     "scaling": {"factor": 40.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}
    if window:
        mixer["mask"] = {"size": window}
    dense = {"kind": "dense", "ff": dense_ff}
    moe = {"kind": "moe", "expert": {"ff": expert_ff},
           "router": {"experts": experts, "identity": 0, "top": top}, "shared": {"ff": shared_ff}}
    return {"architecture": "Rabapel", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
            "embedding": {"scale": 1.0}, "max_positions": 8192,
            "layers": [{"type": "latent_attention", "mixer": dict(mixer), "mlp": moe if i % 2 else dense}
                       for i in range(layers)]}


def rabapel_counts(cfg, esz):
    """(step_bytes(batch, mean_ctx), flops(tokens, lens)) of a Rabapel configuration: the weights
    a decode step has to read (of a routed layer: router, shared expert and the experts that
    `batch` tokens are expected to choose among them) and its cache rows; the multiply-adds of a
    prompt step with every head's keys and values made from the latent rows."""
    E, V = cfg["width"], cfg["vocab"]

    def layer_parts(layer):
        m, mlp = layer["mixer"], layer["mlp"]
        H, dq, dv, R, dr = m["heads"], m["dim"] + m["rot_dim"], m["vdim"], m["kv_rank"], m["rot_dim"]
        mix = E * (H * dq + R + dr + H) + R * H * (m["dim"] + dv) + E * H * dv
        return m, mlp, mix

    def step_bytes(batch, mean_ctx):
        total = V * E
        for layer in cfg["layers"]:
            m, mlp, mix = layer_parts(layer)
            total += mix + batch * min(mean_ctx, (m.get("mask") or {}).get("size") or mean_ctx) * (m["kv_rank"] + m["rot_dim"])
            if mlp["kind"] == "dense":
                total += 2 * E * mlp["ff"]
            else:
                n, top = mlp["router"]["experts"], mlp["router"]["top"]
                used = n * (1.0 - (1.0 - top / n) ** batch)
                total += E * n + 3 * E * mlp["shared"]["ff"] + used * 3 * E * mlp["expert"]["ff"]
        return total * esz

    def flops(tokens, lens):
        total = 2.0 * len(lens) * V * E
        for layer in cfg["layers"]:
            m, mlp, mix = layer_parts(layer)
            H, dq, dv = m["heads"], m["dim"] + m["rot_dim"], m["vdim"]
            w = (m.get("mask") or {}).get("size")
            pairs = sum(n * (n + 1) / 2 if not w or n <= w else w * (w + 1) / 2 + (n - w) * w for n in lens)
            total += 2.0 * tokens * mix + 2.0 * H * (dq + dv) * pairs
            if mlp["kind"] == "dense":
                total += 2.0 * tokens * 2 * E * mlp["ff"]
            else:
                r = mlp["router"]
                total += 2.0 * tokens * (E * r["experts"] + 3 * E * mlp["shared"]["ff"]
                                         + r["top"] * 3 * E * mlp["expert"]["ff"])
        return total

    return step_bytes, flops


def rabapel_main(args) -> int:
    """Rabapel at two sizes beside LLaMA of the same width, heads and number of layers (four: the
    figures are per design and size, tokens/s of these four-layer models, with the fraction of the
    matrix peak for prompts and of the HBM peak for decode steps)."""
    import torch
    from inferllm_amd import Engine
    layers = args.layers or 4
    esz = 2 if args.dtype == "bfloat16" else 4
    sizes = {"2048": dict(width=2048, heads=16, dense_ff=8192, experts=64, expert_ff=1408, top=6, shared_ff=2816),
             "4096": dict(width=4096, heads=32, dense_ff=11008, experts=32, expert_ff=2048, top=4, shared_ff=4096)}
    few = min(args.steps, 128)
    out = {"metric": "Rabapel beside LLaMA at equal width, heads and layers: prefill tok/s at 2,048 tokens, decode tok/s at batch 1/8/64",
           "unit": "tokens/s", "n_gpus": 1, "steps": few, "warmup": 4, "dtype": "bf16" if esz == 2 else "fp32",
           "data": "synthetic: seeded random weights N(0, 0.02), uniform random token ids",
           "layers": layers, "sizes": {}}
    for name, sz in sizes.items():
        if args.size and args.size != name:
            continue
        row = {}
        rcfg = rabapel_config(layers=layers, **sz)
        lcfg = dict(LLAMA2_7B, hidden_size=sz["width"], intermediate_size=sz["dense_ff"],
                    num_attention_heads=sz["heads"], num_key_value_heads=sz["heads"],
                    num_hidden_layers=layers, max_position_embeddings=8192)
        for design in ("rabapel", "llama"):
            if design == "rabapel":
                eng = Engine.from_random(rcfg, seed=0, dtype=args.dtype, device="cuda:0", max_batch=64,
                                         max_seq_len=4096, max_tokens=64 * 1024)
                b = Bench.around(eng, rcfg["vocab"], layers, args.dtype, *rabapel_counts(rcfg, esz))
            else:
                b = Bench(lcfg, layers, args.dtype, 64, 64 * 1024)
            torch.cuda.synchronize()
            r = {"prefill_2048": b.prefill_run(2048, reps=4)}
            for batch in (1, 8, 64):
                v, ms, f = b.decode_run(batch, few, 4, args.prompt)
                r[f"decode_b{batch}"] = {"value": round(v, 1), "ms": round(ms, 4), "hbm_frac": round(f, 4)}
            row[design] = r
            b.close()
            del b
        out["sizes"][name] = row
    print(json.dumps(out), flush=True)
    return 0


# ---------------------------------------------------------------- Kukupel beside Rabapel
def kukupel_config(width, heads, kv_heads, layers, experts, expert_ff, top, streams=4, vocab=32000):
    """Layers in the order parallel, parallel, delta, parallel ...: attention heads of 128 query
    and 128 value dims beside delta-rule heads of 128 x 128 (a decay a key channel, low ranks of
    64), delta-rule layers of the same heads alone, a routed feed-forward in every layer."""
    delta = {"heads": heads, "kv_heads": heads, "dim": 128, "vdim": 128, "conv": 4}
    par = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
                    "softcap": 30.0},
           "right": dict(delta, decay_rank=64, gate_rank=64), "left_scale": 1.0, "right_scale": 1.0}
    mlp = {"kind": "moe", "expert": {"ff": expert_ff, "limit": 7.0}, "router": {"experts": experts, "top": top}}
    return {"architecture": "Kukupel", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
            "streams": streams, "max_positions": 8192,
            "layers": [{"type": "delta", "mixer": dict(delta), "mlp": mlp} if i % 4 == 2 else
                       {"type": "parallel", "mixer": dict(par), "mlp": mlp} for i in range(layers)]}


def kukupel_counts(cfg, esz):
    """(step_bytes(batch, mean_ctx), flops(tokens, lens)) of a Kukupel configuration: the weights
    a decode step reads (of a routed layer the router and the experts that `batch` tokens are
    expected to choose), attention's cache rows and the delta rule's float32 states (read and
    written); the multiply-adds of a prompt step (the recurrence as 3 key x value products a
    token and head)."""
    E, V = cfg["width"], cfg["vocab"]

    def delta_parts(m, low):
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        w = E * (2 * G * dk + H * dv + H) + E * H * dv
        w += (E * (m["decay_rank"] + m["gate_rank"]) + m["decay_rank"] * H * dk + m["gate_rank"] * H * dv
              if low else E * (H + H * dv))
        return w, H * dk * dv

    def layer_parts(layer):
        m = layer["mixer"]
        if layer["type"] == "delta":
            w, state = delta_parts(m, False)
            return w, state, 0, 0
        l = m["left"]
        w, state = delta_parts(m["right"], True)
        w += E * (l["heads"] * l["dim"] + l["kv_heads"] * (l["dim"] + l["vdim"])) + E * l["heads"] * l["vdim"]
        return w, state, l["kv_heads"] * (l["dim"] + l["vdim"]), l["heads"] * (l["dim"] + l["vdim"])

    def step_bytes(batch, mean_ctx):
        total = V * E * esz
        for layer in cfg["layers"]:
            w, state, kv_row, _ = layer_parts(layer)
            r, ff = layer["mlp"]["router"], layer["mlp"]["expert"]["ff"]
            used = r["experts"] * (1.0 - (1.0 - r["top"] / r["experts"]) ** batch)
            total += (w + used * 3 * E * ff + batch * mean_ctx * kv_row) * esz + E * r["experts"] * 4
            total += batch * state * 4 * 2
        return total

    def flops(tokens, lens):
        total = 2.0 * len(lens) * V * E
        pairs = sum(n * (n + 1) / 2 for n in lens)
        for layer in cfg["layers"]:
            w, state, _, qk = layer_parts(layer)
            r, ff = layer["mlp"]["router"], layer["mlp"]["expert"]["ff"]
            total += 2.0 * tokens * (w + E * r["experts"] + r["top"] * 3 * E * ff) + 2.0 * qk * pairs
            total += 2.0 * 3 * state * tokens
        return total

    return step_bytes, flops


def kukupel_main(args) -> int:
    """Kukupel at two sizes beside Rabapel, the library's other design with routed feed-forwards,
    at the same width, heads, experts and number of layers (four): tokens/s of these four-layer
    models, with the fraction of the matrix peak for prompts and of the HBM peak for decode steps."""
    import torch
    from inferllm_amd import Engine
    layers = args.layers or 4
    esz = 2 if args.dtype == "bfloat16" else 4
    sizes = {"2048": dict(width=2048, heads=16, kv_heads=4, experts=64, expert_ff=1408, top=6),
             "4096": dict(width=4096, heads=32, kv_heads=8, experts=32, expert_ff=2048, top=4)}
    few = min(args.steps, 128)
    out = {"metric": "Kukupel beside Rabapel at equal width, heads, experts and layers: prefill tok/s at 2,048 tokens, decode tok/s at batch 1/8/64",
           "unit": "tokens/s", "n_gpus": 1, "steps": few, "warmup": 4, "dtype": "bf16" if esz == 2 else "fp32",
           "data": "synthetic: seeded random weights, uniform random token ids", "layers": layers, "sizes": {}}
    for name, sz in sizes.items():
        if args.size and args.size != name:
            continue
        row = {}
        kcfg = kukupel_config(layers=layers, **sz)
        rcfg = rabapel_config(width=sz["width"], heads=sz["heads"], layers=layers, dense_ff=4 * sz["width"],
                              experts=sz["experts"], expert_ff=sz["expert_ff"], top=sz["top"],
                              shared_ff=2 * sz["expert_ff"])
        for design, cfg, counts in (("kukupel", kcfg, kukupel_counts), ("rabapel", rcfg, rabapel_counts)):
            if args.only and args.only != design:
                continue
            eng = Engine.from_random(cfg, seed=0, dtype=args.dtype, device="cuda:0", max_batch=64,
                                     max_seq_len=4096, max_tokens=64 * 1024)
            b = Bench.around(eng, cfg["vocab"], layers, args.dtype, *counts(cfg, esz))
            torch.cuda.synchronize()
            r = {"prefill_2048": b.prefill_run(2048, reps=4)}
            for batch in (1, 8, 64):
                v, ms, f = b.decode_run(batch, few, 4, args.prompt)
                r[f"decode_b{batch}"] = {"value": round(v, 1), "ms": round(ms, 4), "hbm_frac": round(f, 4)}
            row[design] = r
            b.close()
            del b, eng
        out["sizes"][name] = row
    print(json.dumps(out), flush=True)
    return 0


def sabipel_config(width, heads, kv_heads, layers, chunk=1024, vocab=32000):
    """Layers in the order mamba2, attention, mlstm, attention ...: state-space heads of 64 value
    dims on a state of 128 (an inner width of twice the model's), matrix-memory heads of 128 x 128,
    attention heads of 128 query and 128 value dims in chunks of `chunk` positions, a dense
    feed-forward of four times the width in every layer."""
    ssm = {"heads": 2 * width // 64, "vdim": 64, "state": 128, "groups": 8, "conv": 4, "norm_groups": 8}
    mem = {"heads": heads, "dim": 128, "vdim": 128, "gate_cap": 15.0}
    att = {"heads": heads, "kv_heads": kv_heads, "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
           "mask": {"size": chunk}, "v_mix": True}
    mlp = {"kind": "dense", "ff": 4 * width}
    kinds = [("mamba2", ssm), ("attention", att), ("mlstm", mem), ("attention", att)]
    return {"architecture": "Sabipel", "vocab": vocab, "width": width, "max_positions": 8192,
            "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0, "bigram": {"buckets": 65521, "mul_prev": 37, "mul_cur": 11}},
            "layers": [{"type": kinds[i % 4][0], "mixer": dict(kinds[i % 4][1]), "mlp": dict(mlp)}
                       for i in range(layers)]}


def sabipel_counts(cfg, esz):
    """(step_bytes(batch, mean_ctx), flops(tokens, lens)) of a Sabipel configuration: the weights a
    decode step reads, attention's cache rows within a chunk, the recurrent layers' float32 states
    (read and written); the multiply-adds of a prompt step (attention within its chunks, the
    recurrence as 2 key x value products a token and head)."""
    E, V = cfg["width"], cfg["vocab"]

    def layer_parts(layer):
        """(weights, float32 state, cache columns a token, score columns a pair, chunk)"""
        m, kind = layer["mixer"], layer["type"]
        ff = 2 * E * layer["mlp"]["ff"] if layer.get("mlp") else 0
        if kind == "mamba2":
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            return E * (2 * inner + 2 * gn + m["heads"]) + inner * E + ff, m["heads"] * m["state"] * m["vdim"], 0, 0, 0
        if kind == "mlstm":
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            return E * (2 * H * dk + 2 * H * dv + 2 * H) + H * dv * E + ff, H * dk * (dv + 1), 0, 0, 0
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        return (E * (H * dk + G * dk + G * dv + H * dv) + H * dv * E + ff, 0, G * (dk + dv), H * (dk + dv),
                (m.get("mask") or {}).get("size", 0))

    def seen(n, chunk):
        """keys that position n - 1 sees"""
        return (n - 1) % chunk + 1 if chunk else n

    def step_bytes(batch, mean_ctx):
        total = V * E * esz + batch * 3 * E * esz
        for layer in cfg["layers"]:
            w, state, kv_row, _, chunk = layer_parts(layer)
            total += (w + batch * seen(int(mean_ctx), chunk) * kv_row) * esz + batch * state * 4 * 2
        return total

    def flops(tokens, lens):
        total = 2.0 * len(lens) * V * E
        for layer in cfg["layers"]:
            w, state, _, qk, chunk = layer_parts(layer)
            pairs = sum(sum(seen(p + 1, chunk) for p in range(n)) for n in lens) if qk else 0
            total += 2.0 * tokens * w + 2.0 * qk * pairs + 2.0 * 2 * state * tokens
        return total

    return step_bytes, flops


def sabipel_main(args) -> int:
    """Sabipel at two sizes beside Kukupel, the library's other design with recurrent layers that
    keep a matrix of state per head, at the same width, heads and number of layers (four): tokens/s
    of these four-layer models, with the fraction of the matrix peak for prompts and of the HBM peak
    for decode steps."""
    import torch
    from inferllm_amd import Engine
    layers = args.layers or 4
    esz = 2 if args.dtype == "bfloat16" else 4
    sizes = {"2048": dict(width=2048, heads=16, kv_heads=4), "4096": dict(width=4096, heads=32, kv_heads=8)}
    experts = {"2048": dict(experts=64, expert_ff=1408, top=6), "4096": dict(experts=32, expert_ff=2048, top=4)}
    few = min(args.steps, 128)
    out = {"metric": "Sabipel beside Kukupel at equal width, heads and layers: prefill tok/s at 2,048 tokens, decode tok/s at batch 1/8/64",
           "unit": "tokens/s", "n_gpus": 1, "steps": few, "warmup": 4, "dtype": "bf16" if esz == 2 else "fp32",
           "data": "synthetic: seeded random weights, uniform random token ids", "layers": layers, "sizes": {}}
    for name, sz in sizes.items():
        if args.size and args.size != name:
            continue
        row = {}
        scfg = sabipel_config(layers=layers, **sz)
        kcfg = kukupel_config(layers=layers, **sz, **experts[name])
        for design, cfg, counts in (("sabipel", scfg, sabipel_counts), ("kukupel", kcfg, kukupel_counts)):
            if args.only and args.only != design:
                continue
            eng = Engine.from_random(cfg, seed=0, dtype=args.dtype, device="cuda:0", max_batch=64,
                                     max_seq_len=4096, max_tokens=64 * 1024)
            b = Bench.around(eng, cfg["vocab"], layers, args.dtype, *counts(cfg, esz))
            torch.cuda.synchronize()
            r = {"prefill_2048": b.prefill_run(2048, reps=4)}
            if not args.prefill_only:
                for batch in (1, 8, 64):
                    v, ms, f = b.decode_run(batch, few, 4, args.prompt)
                    r[f"decode_b{batch}"] = {"value": round(v, 1), "ms": round(ms, 4), "hbm_frac": round(f, 4)}
            row[design] = r
            b.close()
            del b, eng
        out["sizes"][name] = row
    print(json.dumps(out), flush=True)
    return 0

def dotorax_config(width, heads, kv_heads, layers, window=1024, pool=8, vocab=32000):
    """Layers in the order attention, gla, parallel, attention that reads the first layer's keys ...:
    attention heads of 128 query and 128 value dims with half of each head rotated, linear-attention
    heads of 64 key and 128 value dims, a window of `window` tokens with blocks of `pool` beside a
    recurrent unit as wide as the model in blocks of 128 or 256 channels, a gated feed-forward of
    8/3 of the width in every layer, three taps in front of every sublayer."""
    rot = {"base": 10000.0, "dims": 64}
    att = {"heads": heads, "kv_heads": kv_heads, "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "rot": rot}
    gla = {"heads": heads, "dim": 64, "vdim": 128, "tau": 16.0, "rank": 16}
    par = {"left": dict(att, mask={"size": window, "pool": pool}),
           "right": {"width": width, "blocks": 16, "conv": 4}, "left_scale": 1.0, "right_scale": 1.0}
    mlp = {"kind": "dense", "ff": 8 * width // 3 // 256 * 256, "limit": 7.0}
    out = []
    for i in range(layers):
        kind = ("attention", "gla", "parallel", "attention")[i % 4]
        mixer = dict(att) if kind == "attention" else dict(gla) if kind == "gla" else \
            {k: (dict(v) if isinstance(v, dict) else v) for k, v in par.items()}
        if i % 4 == 3:
            mixer["kv_from"] = i - 3
        out.append({"type": kind, "mixer": mixer, "mlp": dict(mlp)})
    return {"architecture": "Dotorax", "vocab": vocab, "width": width, "max_positions": 8192,
            "norm": {"eps": 1e-6}, "residual_mult": 0.5, "canon": {"taps": 3}, "layers": out}


def dotorax_counts(cfg, esz):
    """(step_bytes(batch, mean_ctx), flops(tokens, lens)) of a Dotorax configuration: the weights a
    decode step reads, attention's cache rows (all of them, or a window's and the pooled rows before
    it), the recurrent layers' float32 states (read and written); the multiply-adds of a prompt step
    (attention over what each row sees, the linear attention's recurrence as 2 key x value products
    a token and head, the recurrent unit's gates)."""
    E, V = cfg["width"], cfg["vocab"]

    def att_parts(m, own=True):
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        return E * (H * dk + (G * (dk + dv) if own else 0)) + H * dv * E, G * (dk + dv), H * (dk + dv)

    def layer_parts(layer):
        """(weights, float32 state, cache columns a token, score columns a pair, window, pool, other multiply-adds a token)"""
        m, kind = layer["mixer"], layer["type"]
        ff = 3 * E * layer["mlp"]["ff"] if layer.get("mlp") else 0
        if kind == "gla":
            H, dk, dv, r = m["heads"], m["dim"], m["vdim"], m.get("rank", 16)
            return E * (2 * H * dk + 2 * H * dv + r) + r * H * dk + H * dv * E + ff, H * dk * dv, 0, 0, 0, 0, 0
        if kind == "attention":
            w, kv, qk = att_parts(m, "kv_from" not in m)
            return w + E * m["heads"] + ff, 0, kv, qk, 0, 0, 0
        w, kv, qk = att_parts(m["left"])
        C, nb = m["right"]["width"], m["right"]["blocks"]
        gates = 2 * C * (C // nb)
        return (w + 3 * E * C + gates + ff, C, kv, qk, m["left"]["mask"]["size"], m["left"]["mask"]["pool"], gates)

    def seen(n, window, pool):
        """keys that position n - 1 sees"""
        if not window or n <= window:
            return n
        return window + (n - window) // pool

    def step_bytes(batch, mean_ctx):
        total = V * E * esz + batch * 3 * E * esz
        for layer in cfg["layers"]:
            w, state, kv_row, _, window, pool, _ = layer_parts(layer)
            total += (w + batch * seen(int(mean_ctx), window, pool) * kv_row) * esz + batch * state * 4 * 2
        return total

    def flops(tokens, lens):
        total = 2.0 * len(lens) * V * E
        for layer in cfg["layers"]:
            w, state, _, qk, window, pool, other = layer_parts(layer)
            pairs = sum(sum(seen(p + 1, window, pool) for p in range(n)) for n in lens) if qk else 0
            mem = 2 * state if layer["type"] == "gla" else 0
            total += 2.0 * tokens * (w + other) + 2.0 * qk * pairs + 2.0 * mem * tokens
        return total

    return step_bytes, flops


def dotorax_main(args) -> int:
    """Dotorax at two sizes beside Sabipel, the library's closest design (recurrent layers with a
    state per sequence, attention whose scores and weights stay float32), at the same width, heads
    and number of layers (four): tokens/s of these four-layer models, with the fraction of the
    matrix peak for prompts and of the HBM peak for decode steps."""
    import torch
    from inferllm_amd import Engine
    layers = args.layers or 4
    esz = 2 if args.dtype == "bfloat16" else 4
    sizes = {"2048": dict(width=2048, heads=16, kv_heads=4), "4096": dict(width=4096, heads=32, kv_heads=8)}
    few = min(args.steps, 128)
    out = {"metric": "Dotorax beside Sabipel at equal width, heads and layers: prefill tok/s at 2,048 tokens, decode tok/s at batch 1/8/64",
           "unit": "tokens/s", "n_gpus": 1, "steps": few, "warmup": 4, "dtype": "bf16" if esz == 2 else "fp32",
           "data": "synthetic: seeded random weights, uniform random token ids", "layers": layers, "sizes": {}}
    for name, sz in sizes.items():
        if args.size and args.size != name:
            continue
        row = {}
        dcfg = dotorax_config(layers=layers, **sz)
        scfg = sabipel_config(layers=layers, **sz)
        for design, cfg, counts in (("dotorax", dcfg, dotorax_counts), ("sabipel", scfg, sabipel_counts)):
            if args.only and args.only != design:
                continue
            eng = Engine.from_random(cfg, seed=0, dtype=args.dtype, device="cuda:0", max_batch=64,
                                     max_seq_len=4096, max_tokens=64 * 1024)
            b = Bench.around(eng, cfg["vocab"], layers, args.dtype, *counts(cfg, esz))
            torch.cuda.synchronize()
            r = {"prefill_2048": b.prefill_run(2048, reps=4)}
            if not args.prefill_only:
                for batch in (1, 8, 64):
                    v, ms, f = b.decode_run(batch, few, 4, args.prompt)
                    r[f"decode_b{batch}"] = {"value": round(v, 1), "ms": round(ms, 4), "hbm_frac": round(f, 4)}
            row[design] = r
            b.close()
            del b, eng
        out["sizes"][name] = row
    print(json.dumps(out), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration (0: all)")
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--shape", default="llama2-7b", choices=sorted(SHAPES),
                    help="layer sizes (default: the headline configuration)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip everything under `points` and the prefill")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the 2,048-token prefill (for profiles); prints its own line")
    ap.add_argument("--no-70b", action="store_true",
                    help="leave the LLaMA-2-70B shape out of `points` (138 GB of weights: half a minute)")
    ap.add_argument("--with-70b", action="store_true", help="(the default now; kept for old command lines)")
    ap.add_argument("--design", default="llama", choices=["llama", "rabapel", "kukupel", "sabipel", "dotorax"],
                    help="rabapel: that design at two sizes beside LLaMA at equal size (a line of its own); "
                         "kukupel: that design at two sizes beside Rabapel at equal size (likewise); "
                         "sabipel: that design at two sizes beside Kukupel at equal size (likewise); "
                         "dotorax: that design at two sizes beside Sabipel at equal size (likewise)")
    ap.add_argument("--size", default="", help="with --design rabapel, kukupel, sabipel or dotorax: only this width (2048 or 4096)")
    ap.add_argument("--only", default="", help="with --design kukupel, sabipel or dotorax: only this one of the two designs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only (this library has no multi-GPU path); --gpus must be 1")
        return 2

    if args.design == "rabapel":
        return rabapel_main(args)
    if args.design == "kukupel":
        return kukupel_main(args)
    if args.design == "sabipel":
        return sabipel_main(args)
    if args.design == "dotorax":
        return dotorax_main(args)

    shape_name, shape_cfg = SHAPES[args.shape]
    ctx_len = shape_cfg["max_position_embeddings"]
    headline = args.shape == "llama2-7b" and args.dtype == "bfloat16" and not args.no_points
    long_ctx = 3800
    max_b = max(args.batch, 1 if args.no_points else (128 if headline else 64))
    per_seq = -(-(args.prompt + args.steps + args.warmup + 2) // 64) * 64     # whole cache pages
    room = max(max_b * max(per_seq, 1024), 4096)
    if headline:
        room = max(room, 64 * (-(-(long_ctx + 64 + 8) // 64) * 64))
    b = Bench(shape_cfg, args.layers, args.dtype, max_b, room)
    cfg, layers = b.cfg, b.layers

    if args.prefill_only:
        print(json.dumps({"prefill": b.prefill_run(reps=max(3, args.steps))}), flush=True)
        return 0

    tps, ms, frac = b.decode_run(args.batch, args.steps, args.warmup, args.prompt)
    out = {
        "metric": "decode tok/s at batch 1/8/64 + prefill tok/s at 2,048 tokens (LLaMA-2-7B)",
        "value_is": f"decode tokens/s at batch {args.batch}", "value": round(tps, 2),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": b.dkey, "data": "synthetic: seeded random weights N(0, 0.02), uniform random token ids",
        "config": {"model": shape_name, "layers": layers, "layers_full": b.full_layers,
                   "hidden_size": cfg["hidden_size"], "intermediate_size": cfg["intermediate_size"],
                   "num_attention_heads": cfg["num_attention_heads"],
                   "num_key_value_heads": cfg["num_key_value_heads"],
                   "head_dim": cfg.get("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"]),
                   "vocab_size": cfg["vocab_size"], "global_batch": args.batch,
                   "seq_len": ctx_len, "prompt_len": args.prompt, "rope_theta": cfg["rope_theta"],
                   "rms_norm_eps": cfg["rms_norm_eps"], "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(frac * HBM_PEAK_GBS, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(frac, 4)},
    }
    if not args.no_points:
        out["prefill"] = b.prefill_run()
        points = {}
        few = min(args.steps, 256)
        for name, batch in (("decode_b1", 1), ("decode_b64", 64)):
            v, _, f = b.decode_run(batch, few, 4, args.prompt)
            points[name], points[name + "_hbm_frac"] = round(v, 2), round(f, 4)
        if headline:
            v, _, f = b.decode_run(128, 64, 4, args.prompt)
            points["decode_b128"], points["decode_b128_hbm_frac"] = round(v, 2), round(f, 4)
            # long contexts: the cache's share of a step's bytes grows from a seventh to nine tenths
            for name, batch in (("decode_b8_ctx3800", 8), ("decode_b64_ctx3800", 64)):
                v, _, f = b.decode_run(batch, 64, 4, long_ctx)
                points[name], points[name + "_hbm_frac"] = round(v, 2), round(f, 4)
            # short prompts: milliseconds to the first token (their steps are replayed from graphs
            # from the second of a shape on), and 64 prompts of 128 tokens in one step
            for n in (16, 64, 160):
                points[f"first_token_ms_prompt{n}"] = b.prefill_run(n, reps=8, skip=3)["ms"]
            p = b.prefill_run(128, prompts=64)
            points["prefill_64x128"], points["prefill_64x128_frac"] = p["value"], p["frac"]
            b.close()
            # the same layer sizes with room for 16,384 positions: one long prompt whole, and in
            # steps of 2,048 tokens that go on from the paged cache
            long = Bench(dict(LLAMA2_7B, max_position_embeddings=16384), args.layers, args.dtype, 1, 16384 + 64)
            for T in (8192, 16384):
                p = long.prefill_run(T, reps=3)
                points[f"prefill_{T}"], points[f"prefill_{T}_frac"] = p["value"], p["frac"]
            p = long.prefill_run(16384, reps=3, max_step_tokens=2048)
            points["prefill_16384_in_steps_of_2048"], points["prefill_16384_in_steps_of_2048_frac"] = p["value"], p["frac"]
            long.close()
            # LLaMA-3-8B shape (grouped heads, vocabulary 128,256): 16 prompts of 64 to 4,096
            # tokens, lengths seeded, one batch through the generation loop, 128 new tokens each;
            # and 8 sequences decoding from 8,000-token contexts (its context is 8,192)
            import torch
            lens = torch.randint(64, 4097, (16,), generator=torch.Generator().manual_seed(16)).tolist()
            total = max(sum(-(-(n + 130) // 64) * 64 for n in lens), 8 * 8192)
            b8 = Bench(LLAMA3_8B, 0, args.dtype, 16, total)
            pf, pf_frac, dc, dc_frac = b8.generate_run(lens, 128)
            points.update({"llama3_8b_ragged16_prompt_tokens": sum(lens),
                           "llama3_8b_ragged16_prefill": round(pf, 1),
                           "llama3_8b_ragged16_prefill_frac": round(pf_frac, 4),
                           "llama3_8b_ragged16_decode": round(dc, 2),
                           "llama3_8b_ragged16_decode_hbm_frac": round(dc_frac, 4)})
            v, _, f = b8.decode_run(8, 64, 4, 8000)
            points["llama3_8b_decode_b8_ctx8000"], points["llama3_8b_decode_b8_ctx8000_hbm_frac"] = round(v, 2), round(f, 4)
            b8.close()
            if not args.no_70b:
                b70 = Bench(LLAMA2_70B, 0, args.dtype, 32, 32 * 1280)
                p70 = b70.prefill_run()
                points.update({"llama2_70b_prefill": p70["value"], "llama2_70b_prefill_frac": p70["frac"]})
                for name, batch in (("llama2_70b_decode_b1", 1), ("llama2_70b_decode_b32", 32)):
                    v, _, f = b70.decode_run(batch, 128, 4, 1024)
                    points[name], points[name + "_hbm_frac"] = round(v, 2), round(f, 4)
                b70.close()
        out["points"] = points
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
