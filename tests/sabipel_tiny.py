"""Tiny Sabipel configurations and helpers for the tests.  Sizes differ from layer to layer and
avoid equal or trivial values: attention with 6/2, 4/4, 3/1 and 5/5 heads, key sizes above and
below the value size, chunks of 37, 50 and 64 (a page) positions and none, layers that mix values
and layers that do not; state-space layers with 1, 2 and as many groups as heads, 2 to 5 taps, 1 to 4
norm groups; matrix memories with key sizes above and below the value size and gate caps that do
and do not bite; layers without feed-forward; every order of the three kinds of layer."""
from __future__ import annotations

import os

import torch

import plain_sabipel as P


def _att(heads, kv, dim, vdim, scale, chunk=None, v_mix=False):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk:
        m["mask"] = {"size": chunk}
    if v_mix:
        m["v_mix"] = True
    return m


def _ssm(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
            "norm_groups": norm_groups}


def _mem(heads, dim, vdim, cap):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def _layer(kind, mixer, ff=None):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def _model(layers, vocab, width, eps, positions, scale, buckets, mul_prev, mul_cur):
    return {"architecture": "Sabipel", "vocab": vocab, "width": width, "max_positions": positions,
            "norm": {"eps": eps},
            "embedding": {"scale": scale, "bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}},
            "layers": layers}


MIXED = _model([
    _layer("attention", _att(6, 2, 20, 12, 0.2, chunk=37, v_mix=True), 112),
    _layer("mlstm", _mem(3, 16, 28, 9.0), 56),
    _layer("mamba2", _ssm(4, 24, 20, 1, 4, 3), None),
    _layer("attention", _att(4, 4, 16, 6, 0.3, chunk=50, v_mix=True), 40),
    _layer("attention", _att(3, 1, 24, 40, 0.15), 72),
    _layer("mamba2", _ssm(6, 10, 12, 6, 2, 1), 64),
], vocab=310, width=80, eps=2e-5, positions=512, scale=5.5, buckets=97, mul_prev=13, mul_cur=5)

# a width that is no multiple of 4, a memory first, values mixed by the last two attention layers
# only, a chunk of exactly one page, a cap that bites
ODD = _model([
    _layer("mlstm", _mem(2, 40, 12, 1.5), 50),
    _layer("attention", _att(5, 5, 8, 16, 0.4, chunk=64), None),
    _layer("mamba2", _ssm(3, 14, 36, 3, 5, 2), 30),
    _layer("attention", _att(2, 1, 32, 18, 0.2, chunk=23, v_mix=True), 44),
    _layer("attention", _att(6, 1, 12, 18, 0.25, v_mix=True), 28),
], vocab=131, width=90, eps=3e-6, positions=300, scale=2.0, buckets=41, mul_prev=3, mul_cur=11)

# nothing is kept per token: recurrent layers only
NO_KEYS = _model([
    _layer("mamba2", _ssm(2, 16, 8, 2, 3, 4), 48),
    _layer("mlstm", _mem(4, 12, 12, 6.0), None),
    _layer("mamba2", _ssm(5, 8, 24, 1, 2, 5), 24),
], vocab=120, width=48, eps=1e-5, positions=400, scale=9.0, buckets=256, mul_prev=1, mul_cur=2)

CONFIGS = {"MIXED": MIXED, "ODD": ODD, "NO_KEYS": NO_KEYS}


def single(kind, mixer, ff=None, width=64, vocab=200, positions=700, buckets=53):
    """One layer, for tests of one mechanism and tests that plant a key or a memory."""
    return _model([_layer(kind, mixer, ff)], vocab=vocab, width=width, eps=1e-6, positions=positions,
                  scale=3.0, buckets=buckets, mul_prev=7, mul_cur=3)


def write_model(tmp, config: dict, seed: int, dtype=torch.float32, gain: float = 4.0, edit=None) -> str:
    """A random model folder for `config`; every matrix of the layers times `gain` (with the
    library's small random weights a wrong key or a lost state moves nothing), decays and gate
    biases spread so that heads forget at different speeds, the value-mixing weights away from 0,
    the tables of pairs and positions as large as the token rows; `edit(weights)` may change the
    float64 weights before they are written."""
    import inferllm_amd as I
    from inferllm_amd.weights.safetensors_io import write_safetensors
    from tiny import read_weights
    d = os.path.join(str(tmp), f"sabipel_{seed}_{abs(hash(repr(config))) % 10**8}_{str(dtype)[6:]}")
    I.write_random_model(d, I.config_from_dict(config), seed=seed, dtype=torch.float32)
    w = {}
    g = torch.Generator().manual_seed(seed)
    rnd = lambda shape: torch.randn(shape, generator=g, dtype=torch.float64)
    for n, t in read_weights(d).items():
        t = t.double()
        if n.endswith("dt_bias") or n.endswith("A_log"):
            t = rnd(t.shape) * 1.5 - 1.0
        elif n.endswith(".i.b"):
            t = rnd(t.shape)
        elif n.endswith(".f.b"):
            t = rnd(t.shape) * 1.5 + 2.0
        elif n.endswith(".conv"):
            t = t * 20
        elif n.endswith(".conv.b"):
            t = rnd(t.shape) * 0.3
        elif n.endswith(".vmix"):
            t = torch.tensor(0.2 + 0.5 * float(torch.rand((), generator=g)), dtype=torch.float64)
        elif n in ("embed", "bigram", "pos"):
            t = t * (10 if n == "embed" else 30)
        elif t.dim() == 2:
            t = t * gain
        w[n] = t
    if edit is not None:
        edit(w)
    write_safetensors(os.path.join(d, "model.safetensors"), [(n, t.to(dtype)) for n, t in w.items()],
                      metadata={"format": "pt"})
    return d


def weights64(model_dir: str):
    from tiny import read_weights
    return {n: t.double() for n, t in read_weights(model_dir).items()}


def _mark(w, token: int, column: int) -> None:
    """Give `token` alone a large entry in `column` of the embedded rows: the column is cleared in
    every table that the embedding adds up, then set in the token's row."""
    for table in ("embed", "bigram", "pos"):
        w[table][:, column] = 0.0
    w["embed"][token, column] = 3.0


def plant_key(w, config: dict, key_token: int, query_token: int) -> None:
    """Change layer 0's attention so that `query_token`'s score for `key_token` stands far above
    every other score, in every head: each of the two tokens alone has a large entry in a column of
    its own of the layer's input, one query dim of every head reads the query token's column and
    the same dim of every key head the key token's, and the key token's values are made large.  After
    the norms over whole q and k the raised dims carry most of each; whether the key is seen then
    decides the logits.  Both tokens must occur nowhere else in the sequence."""
    m = config["layers"][0]["mixer"]
    _mark(w, key_token, 0)
    _mark(w, query_token, 1)
    for hh in range(m["heads"]):
        w["l0.mix.q"][hh * m["dim"], 1] += 8.0
    for g in range(m["kv_heads"]):
        w["l0.mix.k"][g * m["dim"], 0] += 8.0
    w["l0.mix.v"][:, 0] += 2.0


def plant_memory(w, config: dict, token: int) -> None:
    """Change layer 0's recurrent mixer so that `token` is written into the state with a weight far
    above every other token's (its input gate, or its step size, reads a column in which that token
    alone has a large entry) and is hardly forgotten afterwards."""
    m = config["layers"][0]["mixer"]
    _mark(w, token, 0)
    if config["layers"][0]["type"] == "mlstm":
        w["l0.mix.i"][:, 0] += 2.0
        w["l0.mix.i.b"][:] = -6.0
        w["l0.mix.f.b"][:] = 9.0
    else:
        inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
        w["l0.mix.in"][2 * inner + 2 * gn:, 0] += 1.5
        w["l0.mix.dt_bias"][:] = -5.0
        w["l0.mix.A_log"][:] = -7.0


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    return float((got.double().cpu() - want).abs().max() / want.abs().max())
