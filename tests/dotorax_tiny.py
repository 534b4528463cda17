"""Tiny Dotorax configurations and helpers for the tests.  Sizes differ from layer to layer and avoid
equal or trivial values: attention with 6/2, 4/4 and 3/1 heads, key sizes above and below the value
size, rotations of part of a head and of all of it, layers that read an earlier layer's keys;
windows of 37, 64 (a page) and 70 tokens with pools of 3, 8 and 5; recurrent units with 1, 2 and 3
blocks and 1 to 4 taps; gated linear attention with key sizes above and below the value size and
ranks of 3 to 9; input convolutions of 1 to 4 taps; layers without feed-forward; every order of the
three kinds of layer."""
from __future__ import annotations

import os

import torch

import plain_dotorax as P


def _rot(base, dims):
    return {"base": base, "dims": dims}


def _att(heads, kv, dim, vdim, scale, rot, kv_from=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _left(heads, kv, dim, vdim, scale, rot, size, pool):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot,
            "mask": {"size": size, "pool": pool}}


def _par(left, width, blocks, conv, left_scale, right_scale):
    return {"left": left, "right": {"width": width, "blocks": blocks, "conv": conv},
            "left_scale": left_scale, "right_scale": right_scale}


def _gla(heads, dim, vdim, tau, rank):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}


def _layer(kind, mixer, ff=None, limit=1.5):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def _model(layers, vocab, width, eps, positions, mult, taps):
    return {"architecture": "Dotorax", "vocab": vocab, "width": width, "max_positions": positions,
            "norm": {"eps": eps}, "residual_mult": mult, "canon": {"taps": taps}, "layers": layers}


MIXED = _model([
    _layer("attention", _att(6, 2, 20, 12, 0.2, _rot(5000.0, 8)), 112),
    _layer("gla", _gla(3, 16, 28, 5.0, 5), 56, limit=0.8),
    _layer("parallel", _par(_left(4, 2, 24, 16, 0.3, _rot(300.0, 24), 37, 3), 36, 3, 3, 0.7, 1.4), None),
    _layer("attention", _att(4, 2, 20, 12, 0.35, _rot(5000.0, 8), kv_from=0), 40),
    _layer("parallel", _par(_left(3, 1, 12, 40, 0.25, _rot(90.0, 6), 70, 5), 50, 1, 4, 1.3, 0.6), 72),
    _layer("gla", _gla(2, 40, 10, 11.0, 9), 64),
], vocab=310, width=80, eps=2e-5, positions=512, mult=0.45, taps=3)

# a width that is no multiple of 4, a window of exactly one page with a pool of 8, two taps in front
# of the sublayers, a gla layer first, two layers that read the keys of the same earlier layer
ODD = _model([
    _layer("gla", _gla(5, 8, 16, 3.0, 3), 50),
    _layer("attention", _att(5, 5, 8, 16, 0.4, _rot(1000.0, 8)), None),
    _layer("parallel", _par(_left(2, 2, 32, 18, 0.2, _rot(40.0, 10), 64, 8), 44, 2, 2, 1.0, 1.0), 30, limit=3.0),
    _layer("attention", _att(10, 5, 8, 16, 0.3, _rot(1000.0, 8), kv_from=1), 44),
    _layer("attention", _att(5, 5, 8, 16, 0.5, _rot(1000.0, 8), kv_from=1), None),
], vocab=131, width=90, eps=3e-6, positions=300, mult=0.8, taps=2)

# nothing is kept per token: gla layers only, one tap in front of the sublayers (the token itself)
NO_KEYS = _model([
    _layer("gla", _gla(2, 16, 8, 2.0, 4), 48),
    _layer("gla", _gla(4, 12, 12, 30.0, 7), None),
], vocab=120, width=48, eps=1e-5, positions=400, mult=1.0, taps=1)

CONFIGS = {"MIXED": MIXED, "ODD": ODD, "NO_KEYS": NO_KEYS}


def single(kind, mixer, ff=None, width=64, vocab=200, positions=700, taps=3, mult=0.5):
    """One layer, for tests of one mechanism and tests that plant a key or a memory."""
    return _model([_layer(kind, mixer, ff)], vocab=vocab, width=width, eps=1e-6, positions=positions,
                  mult=mult, taps=taps)


def write_model(tmp, config: dict, seed: int, dtype=torch.float32, gain: float = 4.0, edit=None) -> str:
    """A random model folder for `config`; every matrix of the layers times `gain` (with the
    library's small random weights a wrong key or a lost state moves nothing), the recurrent unit's
    decays spread so that channels forget at different speeds, the heads' scales away from 1, the
    convolutions strong, the table of positions as large as the token rows; `edit(weights)` may
    change the float64 weights before they are written."""
    import inferllm_amd as I
    from inferllm_amd.weights.safetensors_io import write_safetensors
    from tiny import read_weights
    d = os.path.join(str(tmp), f"dotorax_{seed}_{abs(hash(repr(config))) % 10**8}_{str(dtype)[6:]}")
    I.write_random_model(d, I.config_from_dict(config), seed=seed, dtype=torch.float32)
    w = {}
    g = torch.Generator().manual_seed(seed)
    rnd = lambda shape: torch.randn(shape, generator=g, dtype=torch.float64)
    for n, t in read_weights(d).items():
        t = t.double()
        if n.endswith(".lam"):
            t = rnd(t.shape) * 1.5 - 2.0
        elif n.endswith(".temp"):
            t = 0.5 + torch.rand(t.shape, generator=g, dtype=torch.float64) * 1.5
        elif n.endswith(".a2.b"):
            t = rnd(t.shape) * 2.0 + 2.0
        elif n.endswith(".b"):
            t = rnd(t.shape) * 0.3
        elif ".canon" in n or n.endswith(".conv"):
            t = t * 20
        elif n.endswith(".ra") or n.endswith(".ri"):
            t = t * 8
        elif ".norm" in n and t.dim() == 1 and not n.endswith("mix.norm"):
            t = rnd(t.shape) * 0.3                  # gains 1 + w well away from 1
        elif n in ("embed", "pos"):
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
    """Give `token` alone a large entry in `column` of the embedded rows."""
    for table in ("embed", "pos"):
        w[table][:, column] = 0.0
    w["embed"][token, column] = 3.0


def plant_key(w, config: dict, key_token: int, query_token: int, p: str = "l0.mix.", m: dict = None) -> None:
    """Change layer 0's attention (`p`, `m`: the mixer's tensors and sizes) so that `query_token`'s
    score for `key_token` stands far above every other score, in every head: each of the two tokens
    alone has a large entry in a column of its own of the layer's input (the input convolution is
    switched off so that the mark stays on its token), the last query dim of every head, which is not
    rotated, reads the query token's column and the same dim of every key head the key token's
    column alone (so every other key is blind in it, also after a mean over a block of keys), and
    the key token's values are made large.  Both tokens must occur nowhere else in the sequence."""
    m = m or config["layers"][0]["mixer"]
    _mark(w, key_token, 0)
    _mark(w, query_token, 1)
    w["l0.canon1"][:] = 0.0
    last = m["dim"] - 1
    for hh in range(m["heads"]):
        w[p + "q"][hh * m["dim"] + last, 1] += 8.0
    for g in range(m["kv_heads"]):
        w[p + "k"][g * m["dim"] + last, :] = 0.0
        w[p + "k"][g * m["dim"] + last, 0] = 8.0
    w[p + "v"][:, 0] += 2.0


def plant_memory(w, config: dict, token: int) -> None:
    """Change layer 0's recurrent mixer so that `token` is written into the state with a weight far
    above every other token's and is hardly forgotten afterwards."""
    layer = config["layers"][0]
    _mark(w, token, 0)
    w["l0.canon1"][:] = 0.0
    if layer["type"] == "gla":
        w["l0.mix.k"][:, 0] += 6.0
        w["l0.mix.v"][:, 0] += 2.0
        w["l0.mix.a2.b"][:] = 9.0
    else:
        w["l0.mix.right.x"][:, 0] += 20.0
        w["l0.mix.right.lam"][:] = -9.0


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    return float((got.double().cpu() - want).abs().max() / want.abs().max())
