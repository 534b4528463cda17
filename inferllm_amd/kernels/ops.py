"""The kernel library as Python functions over torch tensors.

Every function checks on the host that shapes, dtypes and devices are what its
kernel and launch grid assume, then launches on torch's current HIP stream.
Tensors must live on the GPU: there is no CPU path, and a missing or unbuildable
library raises (`kernels.build.KernelLibraryError`).  Parts call these through the
module (`ops.add_rmsnorm(...)`).

Matrix products: float32 operands always go to the library's own float32 kernel
(plain fused multiply-adds, fixed summation order).  bfloat16 operands go to the
MFMA kernels of this library when the shape fits them (few rows: decoding), and
to the vendor GEMM through `torch.matmul` otherwise, which is where the reference
uses a vendor GEMM too (cublasSgemm, src/kern/gpu/kernel_gpu.cu:420-435).

Five things ride on the products.  `Weight`: a matrix with a second copy in the
kernels' own tile order (`decode_weight`).  `linear_add` / `NormedRows`: the
residual add in the product's epilogue and the RMS norm that follows it taken by
the next product (up to 16 rows).  `linear_planes`: the product of up to 128 rows (from
17, or from fewer where the plan says that pays) with a long thin matrix, K cut into
ranges whose float32 planes `add_rmsnorm` adds.  `linear_rows`, and `qkv_rope_store` and
`gate_up_silu` from 17 rows on (from fewer where the plan says): products of up to 64 (128)
rows with the wide matrices, X shared by a block's waves through LDS, with the rotation and
cache store or the SiLU-multiply in the same kernel (csrc/gemm_rows.hip).
`_planned_matmul`: products of many rows whole or cut along the output columns, as the
current plan's table says for the shape (`kernels.plan`: fixed tables by default, so that
nothing depends on a stopwatch).
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional

import torch

from . import build
from .plan import NEVER_BELOW, Plan, Rules

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}
_ERRORS = {1: "sizes or dtypes the kernel does not take", 2: "the HIP runtime refused the launch",
           3: "the call needs more of the library's own scratch memory than it holds"}


class KernelError(RuntimeError):
    pass


def _lib():
    return build.library()


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"dtype {t.dtype} is not served (float32 and bfloat16 are)") from None


def _p(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current stream of the current device as a handle for the library (every op calls
    this: the raw lookup costs a fraction of `torch.cuda.current_stream()`)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel operands must be on the GPU (there is no CPU path)")
            _need(t.is_contiguous(), "kernel operands must be contiguous")


def _i32(t: Optional[torch.Tensor], n: Optional[int] = None) -> None:
    if t is not None:
        _need(t.dtype == torch.int32, "index tensors must be int32")
        if n is not None:
            _need(t.numel() >= n, f"index tensor has {t.numel()} entries, {n} needed")


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise KernelError(f"{what}: {_ERRORS.get(rc, rc)}")


# ------------------------------------------------------------------ rows
def embed(tokens: torch.Tensor, table: torch.Tensor, scale: float = 1.0, copies: int = 0) -> torch.Tensor:
    """float32 [T, E] rows of `table` [V, E] at int32 `tokens` [T], times `scale`; with `copies`
    > 0, [T, copies, E]: the row once for every residual stream."""
    _gpu(tokens, table)
    _i32(tokens)
    _need(table.dim() == 2 and tokens.dim() == 1, "embed: tokens [T], table [V, E]")
    T, (V, E) = tokens.numel(), table.shape
    if copies:
        out = torch.empty((T, copies, E), dtype=torch.float32, device=table.device)
        _check(_lib().illm_embed_streams(_p(tokens), _p(table), _code(table), _p(out), T, E, V,
                                         int(copies), ctypes.c_float(scale), _stream()), "embed")
        return out
    out = torch.empty((T, E), dtype=torch.float32, device=table.device)
    _check(_lib().illm_embed_scaled(_p(tokens), _p(table), _code(table), _p(out), T, E, V,
                                    ctypes.c_float(scale), _stream()), "embed")
    return out


def embed_pairs(tokens: torch.Tensor, row_pos: torch.Tensor, row_slot: torch.Tensor,
                table: torch.Tensor, scale: float, pairs: Optional[torch.Tensor], buckets: int,
                mul_prev: int, mul_cur: int, places: Optional[torch.Tensor],
                last_token: Optional[torch.Tensor], remember: bool) -> torch.Tensor:
    """float32 [T, E]: table[token] * scale + pairs[(prev * mul_prev + token * mul_cur) mod buckets]
    + places[position].  prev is the row above if it belongs to the same slot, else
    `last_token[slot]` (int32 [slots]); a row at position 0 takes `pairs[buckets]`.  `pairs`
    [buckets + 1, E] and `places` [positions, E] may be None.  `remember` (every sequence brings one
    row): the row's token is left in `last_token` too; otherwise `remember_last` does that."""
    _gpu(tokens, row_pos, row_slot, table, pairs, places, last_token)
    T = tokens.numel()
    _i32(tokens); _i32(row_pos, T); _i32(row_slot, T); _i32(last_token)
    _need(table.dim() == 2, "embed_pairs: table [V, E]")
    V, E = table.shape
    if pairs is not None:
        _need(pairs.shape == (buckets + 1, E) and last_token is not None,
              f"embed_pairs: pairs [{buckets + 1}, {E}] and the slots' last tokens")
    _need(places is None or (places.dim() == 2 and places.shape[1] == E), "embed_pairs: places [positions, E]")
    out = torch.empty((T, E), dtype=torch.float32, device=table.device)
    _check(_lib().illm_embed_pairs(
        _p(tokens), _p(row_pos), _p(row_slot), _p(table), _code(table), _p(pairs),
        _code(pairs) if pairs is not None else 0, _p(places), _code(places) if places is not None else 0,
        _p(last_token), _p(out), T, E, V, int(buckets), int(mul_prev), int(mul_cur),
        places.shape[0] if places is not None else 1, ctypes.c_float(scale), 1 if remember else 0,
        _stream()), "embed_pairs")
    return out


def remember_last(tokens: torch.Tensor, cu_seqlens: torch.Tensor, seq_slot: torch.Tensor,
                  last_token: torch.Tensor, n_seqs: int) -> None:
    """last_token[seq_slot[b]] = the last of sequence b's tokens in this step."""
    _gpu(tokens, cu_seqlens, seq_slot, last_token)
    _i32(tokens); _i32(cu_seqlens, n_seqs + 1); _i32(seq_slot, n_seqs); _i32(last_token)
    _check(_lib().illm_remember_last(_p(tokens), _p(cu_seqlens), _p(seq_slot), _p(last_token), n_seqs,
                                     _stream()), "remember_last")


def sum_rows(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """float32(a) + float32(b), element by element: what a block whose mixer and feed-forward
    read the same rows leaves for the residual stream."""
    _gpu(a, b)
    _need(a.shape == b.shape, f"sum_rows: {tuple(a.shape)} against {tuple(b.shape)}")
    out = torch.empty(a.shape, dtype=torch.float32, device=a.device)
    _check(_lib().illm_sum_rows(_p(a), _code(a), _p(b), _code(b), _p(out),
                                ctypes.c_size_t(a.numel()), _stream()), "sum_rows")
    return out


class ScaledSum:
    """sa a + sb b of two parts' outputs for the same rows, not yet added: a block that can add it
    in a kernel of its own takes the pieces, any other asks for `tensor()` (float32)."""

    def __init__(self, a: torch.Tensor, sa: float, b: torch.Tensor, sb: float):
        self.a, self.sa, self.b, self.sb = a, float(sa), b, float(sb)

    def tensor(self) -> torch.Tensor:
        a, b = self.a, self.b
        _gpu(a, b)
        _need(a.shape == b.shape, f"ScaledSum: {tuple(a.shape)} against {tuple(b.shape)}")
        out = torch.empty(a.shape, dtype=torch.float32, device=a.device)
        _check(_lib().illm_sum_rows_scaled(_p(a), _code(a), ctypes.c_float(self.sa), _p(b), _code(b),
                                           ctypes.c_float(self.sb), _p(out),
                                           ctypes.c_size_t(a.numel()), _stream()), "sum_rows_scaled")
        return out


def relu_squared(x: torch.Tensor) -> torch.Tensor:
    """max(x, 0)^2, element by element."""
    _gpu(x)
    out = torch.empty_like(x)
    _check(_lib().illm_relu_squared(_p(x), _p(out), _code(x), ctypes.c_size_t(x.numel()), _stream()),
           "relu_squared")
    return out


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """0.5 x (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3))), element by element."""
    _gpu(x)
    out = torch.empty_like(x)
    _check(_lib().illm_gelu_tanh(_p(x), _p(out), _code(x), ctypes.c_size_t(x.numel()), _stream()),
           "gelu_tanh")
    return out


def add_rmsnorm(x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, row_idx: Optional[torch.Tensor] = None,
                weight2: Optional[torch.Tensor] = None):
    """RMS norm of the float32 residual rows `x` [T, E] after adding `delta` to them.
    With `weight2` (of weight's shape and dtype) a pair comes back: the same normed rows under each
    of the two weights, from one pass over x.

    Without `row_idx` the sum is written back to `x`.  With `row_idx` only those
    rows are normed (and `x` is left as it is).  `delta` may be [S, T, E]: the planes of a
    product whose K was split (`linear_planes`), added in order; or a pair of tensors of x's shape
    (the outputs of two parts that read the same rows): x + (first + second).
    """
    delta2 = None
    if isinstance(delta, (tuple, list)):
        delta, delta2 = delta
        _need(delta.shape == x.shape and delta2.shape == x.shape, "add_rmsnorm: a pair needs x's shape")
        _gpu(delta2)
    _gpu(x, delta, weight, row_idx)
    _i32(row_idx)
    _need(x.dtype == torch.float32 and x.dim() == 2, "add_rmsnorm: x must be float32 [T, E]")
    T, E = x.shape
    _need(weight.shape == (E,), f"add_rmsnorm: weight {tuple(weight.shape)} for width {E}")
    planes = 1
    if delta is not None:
        if delta.dim() == 3:
            planes = delta.shape[0]
            _need(planes >= 1 and E % 4 == 0, "add_rmsnorm: planes need a width that is a multiple of 4")
        _need(delta.shape[-2:] == x.shape, "add_rmsnorm: delta must have x's shape")
    rows = T if row_idx is None else row_idx.numel()
    out = torch.empty((rows, E), dtype=out_dtype, device=x.device)
    out2 = None
    if weight2 is not None:
        _gpu(weight2)
        _need(weight2.shape == (E,) and weight2.dtype == weight.dtype, "add_rmsnorm: a second weight like the first")
        out2 = torch.empty((rows, E), dtype=out_dtype, device=x.device)
    _check(_lib().illm_add2_rmsnorm_two(
        _p(x), _p(delta), _code(delta) if delta is not None else 0, planes,
        ctypes.c_size_t(T * E), _p(delta2), _code(delta2) if delta2 is not None else 0,
        _p(weight), _p(weight2), _code(weight),
        _p(out), _p(out2), _code(out), _p(row_idx), rows, E, ctypes.c_float(eps), _stream()), "add_rmsnorm")
    return out if weight2 is None else (out, out2)


class StreamWrite:
    """What a sublayer leaves for several residual streams: its output `y` (or `ya y + yb y2`, the
    outputs of two parts that read the same rows) and how it enters them, x_t <- sum_s mix[s, t]
    x_s + out[t] y (mix float32 [S, S] indexed [from, to], out float32 [S])."""

    def __init__(self, y: torch.Tensor, mix: torch.Tensor, out: torch.Tensor,
                 y2: Optional[torch.Tensor] = None, ya: float = 1.0, yb: float = 1.0):
        self.y, self.mix, self.out, self.y2, self.ya, self.yb = y, mix, out, y2, float(ya), float(yb)


def stream_mix_norm(x: torch.Tensor, write: Optional[StreamWrite], read: Optional[torch.Tensor],
                    weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
                    row_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The write of one sublayer into the float32 residual streams x [T, S, E] (in place unless
    `row_idx` picks rows) and the read and RMS norm of the next: u = sum_s read[s] x_s (no `read`:
    the plain sum of the streams), rows u / sqrt(mean(u^2) + eps) * weight in `out_dtype`."""
    _need(x.dtype == torch.float32 and x.dim() == 3, "stream_mix_norm: x must be float32 [T, S, E]")
    T, S, E = x.shape
    y = y2 = mix = out = None
    ya = yb = 1.0
    if write is not None:
        y, y2, mix, out, ya, yb = write.y, write.y2, write.mix, write.out, write.ya, write.yb
        _need(y.shape == (T, E) and (y2 is None or y2.shape == (T, E)), "stream_mix_norm: y must be [T, E]")
        _need(mix.dtype == torch.float32 and mix.shape == (S, S) and out.dtype == torch.float32
              and out.shape == (S,), "stream_mix_norm: mix float32 [S, S], out float32 [S]")
    _gpu(x, y, y2, mix, out, read, weight, row_idx)
    _i32(row_idx)
    _need(read is None or (read.dtype == torch.float32 and read.shape == (S,)), "stream_mix_norm: read float32 [S]")
    _need(weight.shape == (E,), f"stream_mix_norm: weight {tuple(weight.shape)} for width {E}")
    rows = T if row_idx is None else row_idx.numel()
    h = torch.empty((rows, E), dtype=out_dtype, device=x.device)
    _check(_lib().illm_stream_mix_norm(
        _p(x), S, _p(y), _code(y) if y is not None else 0, ctypes.c_float(ya), _p(y2),
        _code(y2) if y2 is not None else 0, ctypes.c_float(yb), _p(mix), _p(out), _p(read), _p(weight),
        _code(weight), _p(h), _code(h), _p(row_idx), rows, E, ctypes.c_float(eps), _stream()),
        "stream_mix_norm")
    return h


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up from rows [gate (F) | up (F)]."""
    _gpu(gate_up)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "silu_mul: rows of [gate | up]")
    T, F2 = gate_up.shape
    out = torch.empty((T, F2 // 2), dtype=gate_up.dtype, device=gate_up.device)
    _check(_lib().illm_silu_mul(_p(gate_up), _p(out), _code(gate_up), T, F2 // 2, _stream()),
           "silu_mul")
    return out


def rope_store(qkv: torch.Tensor, cos_sin: Optional[torch.Tensor], rot: int, pairing: int,
               row_pos: torch.Tensor, row_slot: Optional[torch.Tensor],
               slot_len: Optional[torch.Tensor], kcache: Optional[torch.Tensor],
               vcache: Optional[torch.Tensor], page_table: Optional[torch.Tensor],
               page_size: int, ring: int, nh: int, nkv: int, hd: int) -> None:
    """Rotate q and k of packed rows in place; store k and v in the paged cache.

    qkv [T, (nh + 2 nkv) hd]; cos_sin float32 [max_pos, rot/2, 2] or None (no rotation);
    kcache / vcache [pages, nkv, page_size, hd] or None (nothing stored);
    page_table int32 [slots, pages per sequence].
    """
    _gpu(qkv, cos_sin, row_pos, row_slot, slot_len, kcache, vcache, page_table)
    _i32(row_pos, qkv.shape[0]); _i32(row_slot, qkv.shape[0]); _i32(slot_len); _i32(page_table)
    T = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] == (nh + 2 * nkv) * hd,
          f"rope_store: rows of {qkv.shape[1]} for {nh}+2*{nkv} heads of {hd}")
    max_pos = 0
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 3 and
              cos_sin.shape[1] * 2 == rot and cos_sin.shape[2] == 2,
              "rope_store: angle table must be float32 [max_pos, rot/2, 2]")
        max_pos = cos_sin.shape[0]
    stride = 1
    if kcache is not None:
        _need(vcache is not None and page_table is not None and row_slot is not None,
              "rope_store: a cache needs vcache, page_table and row_slot")
        _need(kcache.dtype == qkv.dtype and vcache.dtype == qkv.dtype,
              "rope_store: cache dtype differs from the activations'")
        _need(kcache.shape[1:] == (nkv, page_size, hd) and vcache.shape == kcache.shape,
              f"rope_store: cache shape {tuple(kcache.shape)} vs (pages, {nkv}, {page_size}, {hd})")
        _need(page_table.dim() == 2, "rope_store: page_table [slots, pages]")
        stride = page_table.shape[1]
    _check(_lib().illm_rope_store(
        _p(qkv), _code(qkv), _p(cos_sin), max_pos, rot, pairing, _p(row_pos), _p(row_slot),
        _p(slot_len), _p(kcache), _p(vcache), _p(page_table), stride, page_size, ring, T, nh, nkv,
        hd, _stream()), "rope_store")


# ------------------------------------------------------------------ products
def gemm_generic(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """x [M, K] . w [N, K]^T by the library's float32 multiply-add kernel."""
    _gpu(x, w)
    _need(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1],
          f"linear: x {tuple(x.shape)} against w {tuple(w.shape)}")
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _check(_lib().illm_gemm_generic(_p(x), _code(x), _p(w), _code(w), _p(y), _code(y), M, N, K,
                                    _stream()), "gemm_generic")
    return y


def gemm_f32_mfma_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.dtype == torch.float32 and w.dtype == torch.float32 and x.dim() == 2 and w.dim() == 2
            and x.shape[0] >= 1 and x.shape[1] == w.shape[1] and x.shape[1] % 16 == 0
            and x.is_contiguous() and w.is_contiguous())


def gemm_f32_mfma(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """x [M, K] . w [N, K]^T, both float32, on the matrix cores' float32 instruction (float32
    operands, products and sums; no shorter type anywhere).  For many rows."""
    _gpu(x, w)
    _need(gemm_f32_mfma_fits(x, w), "gemm_f32_mfma: operands not taken")
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _check(_lib().illm_gemm_f32_mfma(_p(x), _p(w), _p(y), _code(y), M, N, K, _stream()),
           "gemm_f32_mfma")
    return y


class Weight:
    """A matrix [N, K] of a product with, optionally, a second copy laid out for the few-rows
    kernels (`tile_weight`).  Wherever the ops take a weight they take this or a plain tensor."""
    __slots__ = ("plain", "tiled", "mode")

    def __init__(self, plain: torch.Tensor, tiled: Optional[torch.Tensor] = None, mode: str = "plain"):
        # mode: which kernel's tiles the copy follows (`tile_rows`); only that kernel may read it
        self.plain, self.tiled, self.mode = plain, tiled, mode

    @property
    def shape(self):
        return self.plain.shape

    @property
    def dtype(self):
        return self.plain.dtype


def _w(w, mode: str = "plain"):
    """(plain tensor, pointer of the tiled copy or None) of a weight argument, for the kernel
    whose tiles are `mode`; a copy made for another kernel's tiles is not used."""
    if isinstance(w, Weight):
        return w.plain, (_p(w.tiled) if w.tiled is not None and w.mode == mode else None)
    return w, None


def plain_weight(w) -> torch.Tensor:
    return w.plain if isinstance(w, Weight) else w


def tile_rows(N: int, mode: str = "plain", nh: int = 0, nkv: int = 0, hd: int = 0) -> torch.Tensor:
    """Row numbers (int64 [tiles, 16], -1 = a zero row) of the tiles the few-rows kernels work on.
    "plain": 16 consecutive rows.  "gate_up" (N = 2F rows [gate | up]): 8 gate rows and the same
    8 up rows.  "qkv" (rows [q heads | k heads | v heads]): 8 rows of a q or k head and their
    rotation partners hd/2 further, then 16 consecutive rows of v."""
    if mode == "plain":
        t = torch.arange(((N + 15) // 16) * 16).view(-1, 16)
        return torch.where(t < N, t, torch.full_like(t, -1))
    if mode == "gate_up":
        F = N // 2
        lo = torch.arange(((F + 7) // 8) * 8).view(-1, 8)
        ok = lo < F
        return torch.cat([torch.where(ok, lo, torch.full_like(lo, -1)),
                          torch.where(ok, lo + F, torch.full_like(lo, -1))], dim=1)
    if mode == "qkv":
        heads = torch.arange(nh + nkv).view(-1, 1, 1) * hd
        j = torch.arange(hd // 16).view(1, -1, 1) * 8
        i = torch.arange(8).view(1, 1, -1)
        lo = (heads + j + i).view(-1, 8)
        rot = torch.cat([lo, lo + hd // 2], dim=1)
        v = ((nh + nkv) * hd + torch.arange(nkv * hd)).view(-1, 16)
        return torch.cat([rot, v], dim=0)
    raise ValueError(f"unknown tile mode {mode!r}")


def tile_weight(w: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    """The copy [tiles][K / 32][16][32] of w [N, K] for the given tiles of rows (K % 32 == 0)."""
    N, K = w.shape
    _need(K % 32 == 0 and w.dtype == torch.bfloat16, "tile_weight: bfloat16 with K a multiple of 32")
    rows = rows.to(w.device)
    picked = w[rows.clamp(min=0).view(-1)]
    picked[(rows < 0).view(-1)] = 0
    return picked.view(rows.shape[0], 16, K // 32, 32).permute(0, 2, 1, 3).contiguous()


def decode_weight(w: torch.Tensor, mode: str = "plain", copies=False, **geometry):
    """The weight as the parts keep it: with a tiled copy for the few-rows kernels if the engine
    asked for decode copies and the matrix allows it, else the tensor itself.  `copies`: False,
    True (of every matrix) or "thin" (only of matrices with K >= 2 N, the down projections:
    where the vendor GEMM is weakest at 17 to 64 rows and `linear_planes` needs the copy; for
    models whose copies do not all fit)."""
    if (copies and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] % 32 == 0
            and w.is_cuda and (mode != "qkv" or geometry.get("hd", 0) % 16 == 0)
            and (copies != "thin" or (mode == "plain" and w.shape[1] >= 2 * w.shape[0]))):
        return Weight(w, tile_weight(w, tile_rows(w.shape[0], mode, **geometry)), mode)
    return w


class NormedRows:
    """Residual rows whose RMS norm the next product takes itself (few rows, bfloat16).

    Left by `linear_add(..., norm=)`: `x` the float32 residual rows (the sum already in them),
    `xb` = bfloat16(x * weight), `ssq[m][p]` partial sums of x^2.  A product of few rows reads
    `xb` and scales row m of its result by 1 / sqrt(sum_p ssq[m][p] / K + eps), which is the
    product of the normed rows since the scale is common to a row; anything else asks `rows()`
    for the normed rows."""

    def __init__(self, x: torch.Tensor, weight: torch.Tensor, eps: float, act_dtype: torch.dtype,
                 xb: torch.Tensor, ssq: torch.Tensor):
        self.x, self.weight, self.eps, self.dtype = x, weight, float(eps), act_dtype
        self.xb, self.ssq = xb, ssq
        self.shape = x.shape
        self._rows: Optional[torch.Tensor] = None

    def rows(self) -> torch.Tensor:
        if self._rows is None:
            self._rows = add_rmsnorm(self.x, None, self.weight, self.eps, self.dtype)
        return self._rows

    def made_for(self, weight: torch.Tensor, eps: float) -> bool:
        return weight is self.weight and float(eps) == self.eps


def _operand(x):
    """(tensor the kernel reads, ssq pointer, parts, eps) of a few-rows product's input."""
    if isinstance(x, NormedRows):
        return x.xb, _p(x.ssq), x.ssq.shape[1], ctypes.c_float(x.eps)
    return x, None, 0, ctypes.c_float(0.0)


GEMV_F32_MAX_ROWS = 128    # up to here 16 rows at a time, W read once for each 16, beat the
                           # multiply-add tile, whose blocks each walk all of K (measured at the
                           # 7B shape: a decode step of 64 rows 146 -> 45 ms); where K is a
                           # multiple of 32 `gemm_rows_f32_mfma` takes these rows instead


def gemv_rows_f32_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.dtype == torch.float32 and w.dtype == torch.float32 and x.dim() == 2 and w.dim() == 2
            and 1 <= x.shape[0] <= GEMV_F32_MAX_ROWS and x.shape[1] % 4 == 0
            and x.shape[1] == w.shape[1] and x.is_contiguous() and w.is_contiguous())


def gemv_rows_f32(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """x [M <= 128, K] . w [N, K]^T, both float32, plain float32 multiply-adds, W read once for
    every 16 rows.  A row's sum does not depend on the other rows or on their number."""
    _gpu(x, w)
    _need(gemv_rows_f32_fits(x, w), "gemv_rows_f32: operands not taken")
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    for m0 in range(0, M, 16):
        rows = min(16, M - m0)
        _check(_lib().illm_gemv_rows_f32(_p(x[m0:m0 + rows]), _p(w), _p(y[m0:m0 + rows]), _code(y),
                                         rows, N, K, _stream()), "gemv_rows_f32")
    return y


ROWS_F32_MFMA_FROM = 9     # measured streaming over many matrices of the 7B shapes: up to 8 rows
                           # `gemv_rows_f32` reads W at 4.5 to 5.5 TB/s against 3.2 to 4.0; at 16 rows
                           # it is 2.4 to 2.9 against 3.1 to 3.4, at 64 rows 0.7 against 1.4 to 1.8


def gemm_rows_f32_mfma_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.dtype == torch.float32 and w.dtype == torch.float32 and x.dim() == 2 and w.dim() == 2
            and 1 <= x.shape[0] <= 128 and x.shape[1] % 32 == 0
            and x.shape[1] == w.shape[1] and x.is_contiguous() and w.is_contiguous())


def gemm_rows_f32_mfma(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """x [M <= 128, K] . w [N, K]^T, both float32, W read once, on the matrix cores' float32
    instruction.  A row's sum does not depend on the other rows or on their number."""
    _gpu(x, w)
    _need(gemm_rows_f32_mfma_fits(x, w), "gemm_rows_f32_mfma: operands not taken")
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _check(_lib().illm_gemm_rows_f32_mfma(_p(x), _p(w), _p(y), _code(y), M, N, K, _stream()),
           "gemm_rows_f32_mfma")
    return y


def linear_add_fits(x, w, into: torch.Tensor) -> bool:
    """Whether `linear_add` takes these operands (few bfloat16 rows into float32 rows)."""
    w = plain_weight(w)
    return (isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and x.dim() == 2 and w.dim() == 2 and into.dtype == torch.float32 and
            into.is_contiguous() and 1 <= x.shape[0] <= SKINNY_BEST_ROWS and x.shape[1] % 8 == 0
            and w.shape[1] == x.shape[1] and into.shape == (x.shape[0], w.shape[0]))


def linear_add(x: torch.Tensor, w, into: torch.Tensor, norm=None,
               act_dtype: torch.dtype = torch.bfloat16) -> Optional[NormedRows]:
    """into += x . w^T in the product's kernel: the residual add of a block's output projection,
    each element added by the one thread that owns it.  norm = (weight [N], eps) of the RMS norm
    that follows: the kernel also leaves what the next few-rows product needs to take that norm
    itself, returned as `NormedRows` (only if N % 8 == 0, else None as without `norm`)."""
    _need(linear_add_fits(x, w, into), "linear_add: operands not taken")
    w, wt = _w(w)
    _gpu(x, w, into)
    M, K = x.shape
    N = w.shape[0]
    if norm is not None and (N % 8 or norm[0].dtype not in _CODES or act_dtype != torch.bfloat16
                             or norm[0].shape != (N,)):
        norm = None
    if norm is None:
        _check(_lib().illm_gemm_skinny_add(_p(x), _p(w), wt, _p(into), M, N, K, None, BF16, None,
                                           None, PLAIN_WAVES, _stream()), "linear_add")
        return None
    weight, eps = norm
    _gpu(weight)
    xb = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    ssq = torch.empty((M, (N + 15) // 16), dtype=torch.float32, device=x.device)
    _check(_lib().illm_gemm_skinny_add(_p(x), _p(w), wt, _p(into), M, N, K, _p(weight),
                                       _code(weight), _p(xb), _p(ssq), PLAIN_WAVES, _stream()),
           "linear_add")
    return NormedRows(into, weight, eps, act_dtype, xb, ssq)


MID_MAX_ROWS = 128       # rows a launch of csrc/gemm_mid.hip takes (a limit of the kernel; the break-even
                         # points of the ways are the plan's: `kernels.plan.Rules` and its tables)

# The tables that products with more than one way are dispatched by (`kernels.plan`).  An engine
# makes its own current at the start of each of its steps; nothing is timed unless the plan asks.
_plan: Plan = Plan.fixed()


def use_plan(plan: Plan) -> None:
    global _plan
    _plan = plan


def current_plan() -> Plan:
    return _plan


def linear_planes_fits(x, w) -> bool:
    """Whether `linear_planes` takes these operands: up to 128 bfloat16 rows and a matrix with a
    decode copy in plain tile order that has few rows for its length (K >= 2 N; from 17 rows on
    K >= N)."""
    return (isinstance(w, Weight) and w.tiled is not None and w.mode == "plain"
            and isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16 and x.dim() == 2
            and 1 <= x.shape[0] <= MID_MAX_ROWS and x.shape[1] == w.plain.shape[1]
            and w.plain.shape[0] % 4 == 0 and w.plain.shape[0] <= _plan.rules.planes_most_cols
            and w.plain.shape[1] >= (2 if x.shape[0] <= SKINNY_BEST_ROWS else 1) * w.plain.shape[0])


_flush: Dict[int, torch.Tensor] = {}


def _flush_buffer() -> torch.Tensor:
    """512 MB of zeros on the current device, larger than its last-level cache; kept while the
    process measures (a plan that measures nothing never asks for it)."""
    dev = torch.cuda.current_device()
    if dev not in _flush:
        _flush[dev] = torch.zeros(1 << 28, dtype=torch.int16, device=dev)
    return _flush[dev]


def _cold_time(fn, reps: int = 5) -> float:
    """Median milliseconds of `fn` with the last-level cache flushed before every run: a decode
    step streams gigabytes between two uses of a matrix, so its products always run cold, and a
    matrix of tens of megabytes timed back to back would be served from the cache.  The flush
    reads: after a fill the cache is full of lines to be written back, which costs a kernel
    whose loads allocate in it tens of microseconds that it does not pay in a step (measured
    against streaming over many copies of a matrix, which the reading flush agrees with)."""
    flush = _flush_buffer()
    fn()
    times = []
    for _ in range(reps):
        flush.sum()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        end.synchronize()
        times.append(start.elapsed_time(end))
    return sorted(times)[len(times) // 2]


def measure_planes_from(w: "Weight") -> int:
    """Fewest rows from which `linear_planes` and the norm that adds its planes take less time
    than `linear_add` (whose norm the next product takes), measured at 16, 12, 8 and 4 rows."""
    N, K = w.plain.shape
    if N * K < _plan.rules.planes_min_elements:
        return NEVER_BELOW
    dev = w.plain.device
    x = torch.zeros((SKINNY_BEST_ROWS, K), dtype=torch.bfloat16, device=dev)
    into = torch.zeros((SKINNY_BEST_ROWS, N), dtype=torch.float32, device=dev)
    nw = torch.ones(N, dtype=torch.bfloat16, device=dev)

    timed = _cold_time

    first = NEVER_BELOW
    for rows in (16, 12, 8, 4):
        xs, dst = x[:rows], into[:rows]
        t_add = timed(lambda: linear_add(xs, w, dst, (nw, 1e-5)))
        t_planes = timed(lambda: add_rmsnorm(dst, linear_planes(xs, w), nw, 1e-5, torch.bfloat16))
        if t_planes >= 0.97 * t_add:              # the planes have to pay clearly
            break
        first = rows - 3
    return first


def tune_product(plan: Plan, kind: str, w, votes: int = 1, **geometry) -> Optional[tuple]:
    """Time what the plan's tables lack for one product a part lists (`Part.tunables`) and enter
    it: for a thin "plain" matrix from how few rows the planes pay, for a fused "qkv" or
    "gate_up" matrix from how few rows the kernels that share X do.  The median of `votes`
    measurements.  Returns (table, key, value) of the new entry, or None if nothing was timed
    (no decode copy, a shape the kernels do not take, an entry that is there)."""
    if not (isinstance(w, Weight) and w.tiled is not None and w.mode == kind):
        return None
    N, K = w.shape
    if kind == "plain":
        key, table = (N, K), plan.planes_from
        fits = K >= 2 * N and N <= plan.rules.planes_most_cols and N % 4 == 0
        measure = lambda: measure_planes_from(w)
    elif kind == "qkv":
        key, table = ("qkv", N, K), plan.rows_from
        fits = K % 64 == 0
        measure = lambda: measure_rows_from_qkv(w, geometry["nh"], geometry["nkv"], geometry["hd"])
    elif kind == "gate_up":
        key, table = ("gate_up", N, K), plan.rows_from
        fits = K % 64 == 0
        measure = lambda: measure_rows_from_gate_up(w)
    else:
        raise ValueError(f"unknown kind of product {kind!r}")
    if not fits or key in table:
        return None
    saved, current = _plan, plan
    use_plan(current)
    try:
        runs = sorted(measure() for _ in range(max(1, votes)))
    finally:
        use_plan(saved)
    table[key] = runs[len(runs) // 2]
    return ("planes_from" if kind == "plain" else "rows_from"), key, table[key]


def linear_planes_pays(x, w) -> bool:
    """Whether the planes are the faster way for these operands (which `linear_planes_fits`).
    From 17 to 64 rows always.  Up to 16 rows `linear_add` reads X once per
    block of W rows, so its time grows with the rows, and a matrix whose tiles do not fill the
    chip evenly is slow at any (measured: LLaMA-2-7B's down projection 23.3 against 21.7 us at
    16 rows, the 70B's 105 against 77, a 5120 x 13824 one 34 against 30 at 4 rows): by the
    plan's table; a plan that measures times a shape it lacks once, outside graph capture."""
    rows = x.shape[0]
    if rows > SKINNY_BEST_ROWS:
        # (65 to 128 rows, one launch, product and the norm that adds its planes against the
        # vendor GEMM and its norm: the 7B down projection 28 to 33 us against 38 to 64, the 70B
        # one 86 to 101 against 134 to 221, 4096 x 4096 18 to 22 against 20 to 29; 17 to 64 rows
        # of 4096 x 4096 15 to 18 against 17 to 19, of 5120 x 5120 17 to 22 against 21 to 31)
        return True
    key = tuple(w.plain.shape)
    first = _plan.planes_from.get(key)
    if first is None:
        if not _plan.measure or torch.cuda.is_current_stream_capturing():
            return rows >= NEVER_BELOW
        first = _plan.planes_from[key] = measure_planes_from(w)
    return rows >= first


def linear_planes(x: torch.Tensor, w: "Weight", splits: int = 0) -> torch.Tensor:
    """x . w^T as float32 planes [S, M, N] whose sum over S is the product: K is cut into S
    ranges so that a matrix with few rows fills the chip (csrc/gemm_mid.hip).  The planes go to
    `add_rmsnorm` as `delta`, which adds them in order."""
    _need(linear_planes_fits(x, w), "linear_planes: operands not taken")
    x = x.contiguous()
    _gpu(x, w.plain)
    M, K = x.shape
    N = w.plain.shape[0]
    S = splits or _lib().illm_gemm_mid_splits(N, K)
    y = torch.empty((S, M, N), dtype=torch.float32, device=x.device)
    _check(_lib().illm_gemm_mid_bf16(_p(x), _p(w.tiled), _p(y), F32, M, N, K, S, _stream()),
           "linear_planes")
    return y


def linear(x, w, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """y = x . w^T, w stored [out, in] (src/kern/naive/naive.cpp:363-379).  x may be
    `NormedRows`, w a `Weight`."""
    if isinstance(x, NormedRows):
        if w.dtype == torch.bfloat16:
            return gemm_skinny_bf16(x, w, out_dtype or x.dtype)
        x = x.rows()
    out_dtype = out_dtype or x.dtype
    if (isinstance(w, Weight) and out_dtype == torch.float32 and rows_fits(x, w, "plain")
            and x.shape[0] >= rows_from("plain", w)):
        return linear_rows(x, w, out_dtype)              # logits of 17 to 128 rows
    if isinstance(w, Weight) and not (x.dtype == torch.bfloat16 and 1 <= x.shape[0] <= SKINNY_BEST_ROWS):
        w = w.plain                                      # only the few-rows kernel reads the copy
    if x.dtype == torch.float32 or w.dtype == torch.float32:
        if x.shape[0] >= ROWS_F32_MFMA_FROM and gemm_rows_f32_mfma_fits(x, w):
            return gemm_rows_f32_mfma(x, w, out_dtype)
        if gemv_rows_f32_fits(x, w):
            return gemv_rows_f32(x, w, out_dtype)
        if gemm_f32_mfma_fits(x, w):
            return gemm_f32_mfma(x, w, out_dtype)
        return gemm_generic(x, w, out_dtype)
    M, K = x.shape
    if M == 0:
        return torch.empty((0, w.shape[0]), dtype=out_dtype, device=x.device)
    if skinny_fits(M, w.shape[0], K) and (M <= SKINNY_BEST_ROWS or out_dtype == torch.float32):
        return gemm_skinny_bf16(x, w, out_dtype)
    if out_dtype == torch.float32 and K % 8 == 0:
        # float32 results (logits) keep the accumulator's precision: 64 rows at a time
        return torch.cat([gemm_skinny_bf16(x[i:i + SKINNY_MAX_ROWS], w, out_dtype)
                          for i in range(0, M, SKINNY_MAX_ROWS)], dim=0)
    if out_dtype == torch.float32:
        return gemm_generic(x, w, out_dtype)
    _gpu(x, w)
    return _planned_matmul(x, w)


# The vendor GEMM's own choice of kernel is now and then a poor one for a shape (measured on
# MI355X: 2048 x 22016 x 4096 takes 408 us whole and 253 us as 8192 + 13824 columns; most shapes
# gain nothing).  So products of many rows are planned per shape: the whole product or a cut of
# the output columns, each part written into its slice of one result, as the current plan's
# table says (`kernels.plan`; a plan that measures times the candidates for a shape it lacks).
# Every output element is still one kernel's sum; plans differ in rounding only.
# (from how many rows and columns a cut or a filling-up is a candidate: `kernels.plan.Rules`)


def _split_candidates(N: int, M: int = 0):
    """Plans to measure: () whole, (c,) cut of the output columns at c, ("rows", n) the rows in n
    equal parts (2048 x 12288 x 4096 runs 6 % faster as two products of 1024 rows)."""
    cuts = {(N // 8192) * 8192, (N // 4096) * 4096, (N // 2 // 256) * 256, 8192, 12288, 16384,
            ((2 * N // 3) // 4096) * 4096, ((3 * N // 4) // 4096) * 4096}
    plans = [()] + [(c,) for c in sorted(cuts) if 2048 <= c <= N - 1024]
    if M >= 2048 and M % 512 == 0:
        plans.append(("rows", 2))
    return plans


def _run_plan(x: torch.Tensor, w: torch.Tensor, plan, out: Optional[torch.Tensor] = None):
    if not plan:
        return torch.matmul(x, w.t(), out=out) if out is not None else torch.matmul(x, w.t())
    if plan[0] == "pad":
        # rows filled up to plan[1]; what the added rows hold does not matter, rows are independent
        xp = torch.empty((plan[1], x.shape[1]), dtype=x.dtype, device=x.device)
        xp[:x.shape[0]].copy_(x)
        y = torch.matmul(xp, w.t())[:x.shape[0]]
        if out is not None:
            out.copy_(y)
            return out
        return y
    if out is None:
        out = torch.empty((x.shape[0], w.shape[0]), dtype=x.dtype, device=x.device)
    if plan[0] == "rows":
        step = x.shape[0] // plan[1]
        for a in range(0, x.shape[0], step):
            torch.matmul(x[a:a + step], w.t(), out=out[a:a + step])
        return out
    edges = (0,) + tuple(plan) + (w.shape[0],)
    for a, b in zip(edges[:-1], edges[1:]):
        torch.matmul(x, w[a:b].t(), out=out[:, a:b])
    return out


def measure_plan(x: torch.Tensor, w: torch.Tensor, candidates=None, margin: float = 0.97):
    """The fastest of the candidate plans for x . w^T; a plan replaces the best so far only if
    it takes less than `margin` of its time (a cut has to pay clearly)."""
    out = torch.empty((x.shape[0], w.shape[0]), dtype=x.dtype, device=x.device)
    best, best_t = (), None
    for plan in candidates or _split_candidates(w.shape[0], x.shape[0]):
        # cold, as in a step, where gigabytes pass between two uses of a matrix: run back to
        # back on one matrix the whole product of 2048 x 12288 x 4096 looks as fast as its cut
        # at 8192 columns, over matrices that come from memory it takes 193 against 159 us
        t = _cold_time(lambda: _run_plan(x, w, plan, out), reps=3)
        if best_t is None or t < margin * best_t:
            best, best_t = plan, t
    return best


def _planned_matmul(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    M, K = x.shape
    N = w.shape[0]
    capturing = torch.cuda.is_current_stream_capturing()
    rules = _plan.rules
    if rules.pad_rows_above < M < rules.pad_rows_to:
        # the vendor GEMM takes 65 to 255 rows of some shapes slower than 256 (measured: 4096 x
        # 11008 at 192 rows 82 us, at 256 rows 51): whole or filled up to 256, per shape and
        # 32 rows
        key = ("pad", -(-M // 32), N, K)
        plan = _plan.cuts.get(key)
        if plan is None:
            if not _plan.measure or capturing:
                return torch.matmul(x, w.t())
            plan = _plan.cuts[key] = measure_plan(x, w, [(), ("pad", rules.pad_rows_to)])
        return _run_plan(x, w, plan)
    if M < rules.cut_min_rows or N < rules.cut_min_cols:
        return torch.matmul(x, w.t())
    key = (-(-M // 256), N, K)
    plan = _plan.cuts.get(key)
    if plan is None:
        if not _plan.measure or capturing:
            return torch.matmul(x, w.t())
        plan = _plan.cuts[key] = measure_plan(x, w)
    if plan and plan[0] == "rows" and M % (256 * plan[1]):
        plan = ()                                # measured at the class's full size; M is ragged
    return _run_plan(x, w, plan)


ROWS_MAX = 128           # rows the products of csrc/gemm_rows.hip take, all in one launch (a limit of
                         # the kernel; measured against the vendor GEMM with the elementwise kernel
                         # behind it at 80 / 96 / 128 rows: gate|up of the 7B shape 39 / 40 / 44 against
                         # 50 / 50 / 49 us, of the 8B shape 46 / 48 / 52 against 73 / 59 / 61; in two
                         # launches of 64 rows they lost)


def rows_from(mode: str, w) -> int:
    """Fewest rows from which the product with `w` in tile order `mode` goes to
    csrc/gemm_rows.hip: the plan's entry for the shape, else the plan's rule."""
    return _plan.rows_from.get((mode,) + tuple(w.shape), _plan.rules.rows_from)


def rows_most(mode: str, w) -> int:
    """Most rows for which it does: the plan's entry for the shape, else all a launch takes."""
    return min(ROWS_MAX, _plan.rows_most.get((mode,) + tuple(w.shape), ROWS_MAX))


def rows_fits(x, w, mode: str) -> bool:
    """Whether the products of csrc/gemm_rows.hip take these operands: bfloat16 rows (or
    `NormedRows`, up to 16) and a weight with a decode copy in `mode`'s tile order."""
    xt = x.xb if isinstance(x, NormedRows) else x
    if not (isinstance(w, Weight) and w.tiled is not None and w.mode == mode):
        return False
    most = 16 if isinstance(x, NormedRows) else rows_most(mode, w)
    return (isinstance(w, Weight) and w.tiled is not None and w.mode == mode
            and isinstance(xt, torch.Tensor) and xt.dtype == torch.bfloat16 and xt.dim() == 2
            and 1 <= xt.shape[0] <= most
            and xt.shape[1] == w.plain.shape[1] and xt.shape[1] % 64 == 0)


def linear_rows(x, w: "Weight", out_dtype: torch.dtype) -> torch.Tensor:
    """x [M <= 128, K] . w^T from the plain decode copy, X shared by a block's waves through LDS
    and K cut inside the block: the product of 17 to 128 rows with a wide matrix."""
    _need(rows_fits(x, w, "plain"), "linear_rows: operands not taken")
    xt, ssq, parts, eps = _operand(x)
    xt = xt.contiguous()
    _gpu(xt, w.tiled)
    M, K = xt.shape
    N = w.plain.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=xt.device)
    _check(_lib().illm_gemm_rows_bf16(_p(xt), _p(w.tiled), _p(y), _code(y), M, N, K, ssq, parts,
                                      eps, _stream()), "linear_rows")
    return y


SKINNY_MAX_ROWS = 64     # rows the few-rows kernel takes
SKINNY_BEST_ROWS = 16    # up to here it beats the vendor GEMM (measured at the 7B shapes)


def skinny_fits(M: int, N: int, K: int) -> bool:
    """Shapes the few-rows MFMA kernel takes (csrc/gemm_skinny.hip)."""
    return 1 <= M <= SKINNY_MAX_ROWS and K % 8 == 0


def gemm_skinny_bf16(x, w, out_dtype: torch.dtype) -> torch.Tensor:
    """x [M <= 64, K] . w [N, K]^T, both bfloat16, float32 accumulation on the matrix cores; or
    x `NormedRows`: the product of the normed rows."""
    xt, ssq, parts, eps = _operand(x)
    w, wt = _w(w)
    _gpu(xt, w)
    _need(xt.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny: bfloat16 operands")
    _need(xt.dim() == 2 and w.dim() == 2 and xt.shape[1] == w.shape[1],
          f"linear: x {tuple(xt.shape)} against w {tuple(w.shape)}")
    M, K = xt.shape
    N = w.shape[0]
    _need(skinny_fits(M, N, K), f"gemm_skinny: M={M} K={K} not taken")
    y = torch.empty((M, N), dtype=out_dtype, device=xt.device)
    _check(_lib().illm_gemm_skinny_bf16(_p(xt), _p(w), wt, _p(y), _code(y), M, N, K, ssq, parts,
                                        eps, PLAIN_WAVES, _stream()), "gemm_skinny")
    return y


QKV_ROPE_WAVES = 0       # waves per block of the fused kernel; 0: the kernel's own choice
GATE_UP_WAVES = 0        # the same for the fused gate|up product
PLAIN_WAVES = 0          # and for the plain few-rows product


def qkv_rope_store_fits(x, w_qkv, hd: int) -> bool:
    """Whether the one-kernel q|k|v product + rotation + cache store takes these operands: up to
    16 rows always, up to 128 (96 for small matrices) with a decode copy of the matrix in q|k|v
    tile order."""
    if not (x.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16 and hd % 16 == 0):
        return False
    if 1 <= x.shape[0] <= SKINNY_BEST_ROWS and x.shape[1] % 8 == 0:
        return True
    return rows_fits(x, w_qkv, "qkv")


def measure_rows_from_gate_up(w_gate_up: "Weight") -> int:
    """Fewest rows (1, 5, 9, 13 or 17) from which the fused gate|up product of csrc/gemm_rows.hip
    takes less time than the few-rows one (for the tuner; times both at 16, 12, 8 and 4 rows)."""
    F2, K = w_gate_up.plain.shape
    x = torch.zeros((16, K), dtype=torch.bfloat16, device=w_gate_up.plain.device)
    saved, key = dict(_plan.rows_from), ("gate_up", F2, K)

    def timed(rows: int, threshold: int) -> float:
        _plan.rows_from[key] = threshold
        return _cold_time(lambda: gate_up_silu(x[:rows], w_gate_up))

    first = _plan.rules.rows_from
    try:
        for rows in (16, 12, 8, 4):
            if timed(rows, 1) >= 0.97 * timed(rows, _plan.rules.rows_from):
                break
            first = rows - 3
    finally:
        _plan.rows_from.clear()
        _plan.rows_from.update(saved)
    return first


def measure_rows_from_qkv(w_qkv: "Weight", nh: int, nkv: int, hd: int) -> int:
    """Fewest rows (1, 5, 9, 13 or 17) from which the fused q|k|v product of csrc/gemm_rows.hip
    takes less time than the few-rows one (for the tuner; times both at 16, 12, 8 and 4 rows)."""
    N, K = w_qkv.plain.shape
    dev = w_qkv.plain.device
    x = torch.zeros((16, K), dtype=torch.bfloat16, device=dev)
    table = torch.zeros((16, hd // 2, 2), dtype=torch.float32, device=dev)
    pos = torch.arange(16, dtype=torch.int32, device=dev)
    pages = torch.arange(16, dtype=torch.int32, device=dev).view(16, 1).contiguous()
    kc = torch.zeros((16, nkv, 64, hd), dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    saved, key = dict(_plan.rows_from), ("qkv", N, K)

    def timed(rows: int, threshold: int) -> float:
        _plan.rows_from[key] = threshold
        return _cold_time(lambda: qkv_rope_store(x[:rows], w_qkv, table, pos[:rows], pos[:rows], kc,
                                                 vc, pages, 64, 0, nh, nkv, hd))

    first = _plan.rules.rows_from
    try:
        for rows in (16, 12, 8, 4):
            if timed(rows, 1) >= 0.97 * timed(rows, _plan.rules.rows_from):
                break
            first = rows - 3
    finally:
        _plan.rows_from.clear()
        _plan.rows_from.update(saved)
    return first


def qkv_rope_store(x, w_qkv, cos_sin: torch.Tensor,
                   row_pos: torch.Tensor, row_slot: torch.Tensor, kcache: torch.Tensor,
                   vcache: torch.Tensor, page_table: torch.Tensor, page_size: int, ring: int,
                   nh: int, nkv: int, hd: int) -> torch.Tensor:
    """Decode only: x . Wqkv^T, q and k rotated (pairs (i, i + hd/2), all dims) at row_pos, q
    returned in rows [q | k | v] whose k and v parts are NOT filled, k and v stored in the cache.
    x may be `NormedRows`."""
    xt, ssq, parts, eps = _operand(x)
    _need(qkv_rope_store_fits(x, w_qkv, hd), "qkv_rope_store: operands not taken")
    w_qkv, wt = _w(w_qkv, "qkv")
    _gpu(xt, w_qkv, cos_sin, row_pos, row_slot, kcache, vcache, page_table)
    _i32(row_pos, x.shape[0]); _i32(row_slot, x.shape[0]); _i32(page_table)
    M, K = x.shape
    N = (nh + 2 * nkv) * hd
    _need(w_qkv.shape == (N, K), f"qkv_rope_store: weight {tuple(w_qkv.shape)} vs ({N}, {K})")
    _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 3 and cos_sin.shape[1] * 2 == hd and
          cos_sin.shape[2] == 2, "qkv_rope_store: angle table must be float32 [max_pos, hd/2, 2]")
    _need(kcache.dtype == torch.bfloat16 and kcache.shape[1:] == (nkv, page_size, hd) and
          vcache.shape == kcache.shape and vcache.dtype == torch.bfloat16 and page_table.dim() == 2,
          "qkv_rope_store: cache shape or dtype")
    y = torch.empty((M, N), dtype=torch.bfloat16, device=xt.device)
    if wt is not None and K % 64 == 0 and M >= rows_from("qkv", w_qkv):
        _check(_lib().illm_qkv_rope_store_rows(
            _p(xt), wt, _p(y), M, K, _p(cos_sin), cos_sin.shape[0], _p(row_pos), _p(row_slot),
            _p(kcache), _p(vcache), _p(page_table), page_table.shape[1], page_size, ring, nh, nkv,
            hd, ssq, parts, eps, _stream()), "qkv_rope_store (rows)")
        return y
    _check(_lib().illm_qkv_rope_store_skinny(
        _p(xt), _p(w_qkv), wt, _p(y), M, K, _p(cos_sin), cos_sin.shape[0], _p(row_pos), _p(row_slot),
        _p(kcache), _p(vcache), _p(page_table), page_table.shape[1], page_size, ring, nh, nkv, hd,
        ssq, parts, eps, QKV_ROPE_WAVES, _stream()), "qkv_rope_store")
    return y


def gate_up_silu(x, w_gate_up) -> torch.Tensor:
    """silu(x . Wg^T) * (x . Wu^T) for w_gate_up = [Wg | Wu] stacked as [2F, K].

    Few bfloat16 rows: one fused MFMA kernel.  Otherwise the product and `silu_mul`.
    x may be `NormedRows`."""
    return gate_up_act(x, w_gate_up, 0.0)


def gate_up_act(x, w_gate_up, limit: float = 0.0) -> torch.Tensor:
    """The gate and up products of w_gate_up = [Wg | Wu] ([2F, K]) and their activation: with `limit`
    0 silu(gate) * up, with `limit` > 0 the clamped gate g sigmoid(1.702 g) (u + 1), g = min(gate,
    limit), u = clamp(up, -limit, limit).  Few bfloat16 rows: one fused MFMA kernel (the activation
    acts on the float32 sums).  Otherwise the product and `silu_mul` / `clamped_swish_mul`."""
    limit = float(limit)
    if isinstance(x, NormedRows) and (w_gate_up.dtype != torch.bfloat16 or w_gate_up.shape[0] % 2):
        x = x.rows()
    M, K = x.shape
    F2 = w_gate_up.shape[0]
    if F2 % 2 == 0 and rows_fits(x, w_gate_up, "gate_up") and M >= rows_from("gate_up", w_gate_up):
        xt, ssq, parts, eps = _operand(x)
        xt = xt.contiguous()
        _gpu(xt, w_gate_up.tiled)
        y = torch.empty((M, F2 // 2), dtype=x.dtype, device=xt.device)
        _check(_lib().illm_gemm_rows_gateup_act(_p(xt), _p(w_gate_up.tiled), _p(y), _code(y), M,
                                                F2 // 2, K, ssq, parts, eps, ctypes.c_float(limit),
                                                ctypes.c_float(SWISH_ALPHA), _stream()),
               "gate_up_act (rows)")
        return y
    if (x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and F2 % 2 == 0
            and 1 <= M <= SKINNY_BEST_ROWS and K % 8 == 0):
        xt, ssq, parts, eps = _operand(x)
        wp, wt = _w(w_gate_up, "gate_up")
        _gpu(xt, wp)
        _need(wp.dim() == 2 and wp.shape[1] == K, "gate_up_act: shapes")
        y = torch.empty((M, F2 // 2), dtype=x.dtype, device=xt.device)
        _check(_lib().illm_gemm_skinny_gateup_act(_p(xt), _p(wp), wt, _p(y), _code(y), M,
                                                  F2 // 2, K, ssq, parts, eps, GATE_UP_WAVES,
                                                  ctypes.c_float(limit), ctypes.c_float(SWISH_ALPHA),
                                                  _stream()), "gate_up_act")
        return y
    if isinstance(x, NormedRows):
        x = x.rows()
    both = linear(x, plain_weight(w_gate_up))
    return clamped_swish_mul(both, limit) if limit > 0 else silu_mul(both)


# ------------------------------------------------------------------ attention
def attn_prefill(qkv: torch.Tensor, cu_seqlens: torch.Tensor, n_seqs: int, max_len: int, nh: int,
                 nkv: int, hd: int, scale: float, window: int, softcap: float = 0.0) -> torch.Tensor:
    """Causal attention of whole prompts over packed rows; returns [T, nh * hd].  `softcap` > 0:
    scores softcap * tanh(score / softcap) (the matrix-core kernels only)."""
    _gpu(qkv, cu_seqlens)
    _i32(cu_seqlens, n_seqs + 1)
    T = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] == (nh + 2 * nkv) * hd, "attn_prefill: packed qkv rows")
    _need(nh % nkv == 0, "attn_prefill: heads must be a multiple of kv heads")
    out = torch.empty((T, nh * hd), dtype=qkv.dtype, device=qkv.device)
    if qkv.dtype == torch.bfloat16 and hd % 16 == 0:
        _check(_lib().illm_attn_prefill_bf16_cap(
            _p(qkv), _p(out), _p(cu_seqlens), n_seqs, max_len, nh, nkv, hd,
            ctypes.c_float(scale), ctypes.c_float(softcap), window, _stream()),
            f"attn_prefill_bf16 (head_dim {hd})")
        return out
    _need(not softcap, "attn_prefill: a soft cap needs bfloat16 and a head size in steps of 16")
    _check(_lib().illm_attn_prefill_generic(
        _p(qkv), _p(out), _code(qkv), _p(cu_seqlens), n_seqs, max_len, nh, nkv, hd,
        ctypes.c_float(scale), window, _stream()), f"attn_prefill (head_dim {hd})")
    return out


def attn_prefill_paged(qkv: torch.Tensor, cu_seqlens: torch.Tensor, seq_slot: torch.Tensor,
                       seq_start: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                       page_table: torch.Tensor, page_size: int, ring: int, n_seqs: int,
                       max_len: int, nh: int, nkv: int, hd: int, scale: float,
                       window: int, softcap: float = 0.0) -> torch.Tensor:
    """Causal attention of a step's packed rows that go on from tokens the cache already holds:
    row r of sequence b stands at position seq_start[b] + r and attends over the keys 0 .. its
    position of the paged cache, which must hold the step's own keys and values too by now.
    `max_len`: the most rows a sequence brings.  Returns [T, nh * hd]."""
    _gpu(qkv, cu_seqlens, seq_slot, seq_start, kcache, vcache, page_table)
    _i32(cu_seqlens, n_seqs + 1); _i32(seq_slot, n_seqs); _i32(seq_start, n_seqs); _i32(page_table)
    T = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] >= nh * hd, "attn_prefill_paged: packed rows [q | ...]")
    _need(nh % nkv == 0, "attn_prefill_paged: heads must be a multiple of kv heads")
    _need(kcache.dtype == qkv.dtype and vcache.shape == kcache.shape and
          kcache.shape[1:] == (nkv, page_size, hd) and page_table.dim() == 2,
          "attn_prefill_paged: cache shape or dtype")
    _need(qkv.shape[1] == (nh + 2 * nkv) * hd, "attn_prefill_paged: packed qkv rows")
    out = torch.empty((T, nh * hd), dtype=qkv.dtype, device=qkv.device)
    if qkv.dtype == torch.bfloat16 and hd % 16 == 0 and page_size % 64 == 0:
        _check(_lib().illm_attn_prefill_paged_bf16_cap(
            _p(qkv), _p(out), _p(cu_seqlens), _p(seq_slot), _p(seq_start), _p(kcache), _p(vcache),
            _p(page_table), page_table.shape[1], page_size, ring, n_seqs, max_len, nh, nkv, hd,
            ctypes.c_float(scale), ctypes.c_float(softcap), window, _stream()),
            f"attn_prefill_paged_bf16 (head_dim {hd})")
        return out
    _need(not softcap, "attn_prefill_paged: a soft cap needs bfloat16 and a head size in steps of 16")
    _check(_lib().illm_attn_prefill_paged_generic(
        _p(qkv), _p(out), _code(qkv), _p(cu_seqlens), _p(seq_slot), _p(seq_start), _p(kcache),
        _p(vcache), _p(page_table), page_table.shape[1], page_size, ring, n_seqs, max_len, nh, nkv,
        hd, ctypes.c_float(scale), window, _stream()), f"attn_prefill_paged (head_dim {hd})")
    return out


def decode_splits(B: int, nkv: int, max_len: int, nh: int = 0, hd: int = 0, ragged: bool = False):
    """(nsplit, waves): how to cut the keys of a decode step among blocks (`nsplit` ranges per
    sequence, combined by a merge kernel) and among the waves of a block (combined in LDS).
    Measured on MI355X at head size 128, 32/32, 32/8 and 64/8 heads, 1 to 64 sequences of 650
    to 4000 keys: about as many blocks as the chip has compute units (256) is best or within a
    microsecond of it, in at most 16 ranges; 8 waves a block (idle ones cost nothing) until
    there are 512 blocks, then 4.  `ragged` (the lengths differ widely, the longest has 1,024
    keys or more): every sequence has the same number of ranges, so the long sequences' blocks
    outlast the others'; the ranges are doubled, up to 8, while that makes no more than 1,024
    blocks (16 sequences of 64 to 4,096 keys, 32/8 heads: 30.5 -> 26.3 us, 32/32 heads: 80 -> 74;
    one of 4,000 among 15 of 200: 27.7 -> 21.7 and 51.5 -> 40.7; beyond 1,024 blocks more ranges
    cost more than they even out: one of 2,000 among 63 of 100, 32/32 heads, 34 us whole, 88 in
    8 ranges)."""
    base = max(1, B * nkv)
    if nh > nkv > 0 and hd % 32 == 0 and 0 < hd <= 128:
        base *= -(-(nh // nkv) // 16)          # the grouped kernel takes 16 heads a block
    tiles = max(1, (max_len + 63) // 64)
    nsplit = max(1, min(-(-256 // base), 16, tiles))
    if ragged and tiles >= 16:
        while nsplit < 8 and base * nsplit * 2 <= 1024:
            nsplit *= 2
    return nsplit, (8 if base * nsplit < 512 else 4)


def attn_decode(qkv: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                page_table: torch.Tensor, page_size: int, ring: int, seq_slot: torch.Tensor,
                seq_len: torch.Tensor, nh: int, nkv: int, hd: int, scale: float, window: int,
                nsplit: int, waves: int = 1, softcap: float = 0.0) -> torch.Tensor:
    """One new token per sequence against the paged cache; returns [B, nh * hd].
    seq_len[b]: keys of sequence b, the new one included.  The keys of a sequence are cut
    into `nsplit` ranges (blocks, combined by a merge kernel) and each range is shared by
    `waves` waves of a block (combined in LDS; the bfloat16 kernels only)."""
    _gpu(qkv, kcache, vcache, page_table, seq_slot, seq_len)
    _i32(page_table); _i32(seq_slot, qkv.shape[0]); _i32(seq_len, qkv.shape[0])
    B = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] == (nh + 2 * nkv) * hd, "attn_decode: packed qkv rows")
    _need(kcache.dtype == qkv.dtype and vcache.shape == kcache.shape and
          kcache.shape[1:] == (nkv, page_size, hd), "attn_decode: cache shape or dtype")
    _need(nh % nkv == 0, "attn_decode: heads must be a multiple of kv heads")
    out = torch.empty((B, nh * hd), dtype=qkv.dtype, device=qkv.device)
    if qkv.dtype == torch.bfloat16 and hd % 8 == 0 and page_size % 64 == 0:
        partial = (torch.empty((B, nh, nsplit, hd + 2), dtype=torch.float32, device=qkv.device)
                   if nsplit > 1 else None)
        _check(_lib().illm_attn_decode_bf16_cap(
            _p(qkv), _p(out), _p(kcache), _p(vcache), _p(page_table), page_table.shape[1],
            page_size, ring, _p(seq_slot), _p(seq_len), _p(partial), nsplit, waves, B, nh, nkv, hd,
            ctypes.c_float(scale), ctypes.c_float(softcap), window, _stream()),
            f"attn_decode_bf16 (head_dim {hd})")
        return out
    _need(not softcap, "attn_decode: a soft cap needs bfloat16 and a head size in steps of 8")
    partial = torch.empty((B, nh, nsplit, hd + 2), dtype=torch.float32, device=qkv.device)
    _check(_lib().illm_attn_decode_generic(
        _p(qkv), _p(out), _code(qkv), _p(kcache), _p(vcache), _p(page_table), page_table.shape[1],
        page_size, ring, _p(seq_slot), _p(seq_len), _p(partial), nsplit, B, nh, nkv, hd,
        ctypes.c_float(scale), window, _stream()), f"attn_decode (head_dim {hd})")
    return out


# ------------------------------------------------------------------ latent attention
def latent_rope_store(y: torch.Tensor, H: int, dn: int, dr: int, R: int, rot: int,
                      cos_sin: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                      row_pos: torch.Tensor, row_slot: torch.Tensor,
                      slot_len: Optional[torch.Tensor], cache: Optional[torch.Tensor],
                      page_table: Optional[torch.Tensor], page_size: int, ring: int,
                      want_rows: bool, cache_t: Optional[torch.Tensor] = None):
    """Rows y [T, >= H (dn + dr) + R + dr] = [q | down | ...]: the latent (first R of `down`) is
    RMS-normed, the key part (last dr) and every q head's last dr dims are rotated (pairs
    (2i, 2i+1), i < rot/2) at row_pos, q in place; latent and key part are stored in the paged
    cache [pages, page_size, R + dr] (and the latent alone a second time, transposed, in
    cache_t [pages, R, page_size, 1] if given).  `want_rows`: also return them as (c [T, R],
    kr [T, dr])."""
    _gpu(y, cos_sin, norm_w, row_pos, row_slot, slot_len, cache, page_table, cache_t)
    _need(cache_t is None or (cache is not None and cache_t.dtype == y.dtype and
                              cache_t.shape == (cache.shape[0], R, page_size, 1)),
          "latent_rope_store: the transposed copy must be [pages, R, page_size, 1]")
    T, ncols = y.shape
    _i32(row_pos, T); _i32(row_slot, T); _i32(slot_len); _i32(page_table)
    _need(ncols >= H * (dn + dr) + R + dr, "latent_rope_store: rows too short")
    _need(norm_w.shape == (R,), "latent_rope_store: norm weight [R]")
    max_pos = 0
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 3 and cos_sin.shape[1] * 2 == rot
              and cos_sin.shape[2] == 2 and rot <= dr,
              "latent_rope_store: angle table must be float32 [max_pos, rot/2, 2], rot <= dr")
        max_pos = cos_sin.shape[0]
    stride = 1
    if cache is not None:
        _need(cache.dtype == y.dtype and cache.dim() == 3 and cache.shape[1:] == (page_size, R + dr)
              and page_table is not None and page_table.dim() == 2,
              f"latent_rope_store: cache {tuple(cache.shape)} vs (pages, {page_size}, {R + dr})")
        stride = page_table.shape[1]
    c = torch.empty((T, R), dtype=y.dtype, device=y.device) if want_rows else None
    kr = torch.empty((T, dr), dtype=y.dtype, device=y.device) if want_rows else None
    _check(_lib().illm_latent_rope_store(
        _p(y), _code(y), ncols, T, H, dn, dr, R, rot, _p(cos_sin), max_pos, _p(norm_w),
        _code(norm_w), ctypes.c_float(eps), _p(row_pos), _p(row_slot), _p(slot_len), _p(cache),
        _p(page_table), stride, page_size, ring, _p(c), _p(kr), _p(cache_t), _stream()),
        "latent_rope_store")
    return c, kr


def latent_pack(y: torch.Tensor, kvu: torch.Tensor, kr: torch.Tensor, H: int, dn: int, dr: int,
                dv: int, P: int) -> torch.Tensor:
    """Packed rows [q | k | v] of H heads, each P wide, for `attn_prefill`: q heads from y, key
    heads [kvu's key part | kr], value heads from kvu's value part, zeros beyond a head's dims."""
    _gpu(y, kvu, kr)
    T = y.shape[0]
    _need(kvu.shape == (T, H * (dn + dv)) and kr.shape == (T, dr) and kvu.dtype == y.dtype
          and kr.dtype == y.dtype, "latent_pack: shapes or dtypes")
    out = torch.empty((T, 3 * H * P), dtype=y.dtype, device=y.device)
    _check(_lib().illm_latent_pack(_p(y), _code(y), y.shape[1], _p(kvu), _p(kr), _p(out), T, H, dn,
                                   dr, dv, P, _stream()), "latent_pack")
    return out


def latent_gate(attn: torch.Tensor, y: torch.Tensor, gate_off: int, H: int, dv: int, P: int) -> torch.Tensor:
    """[T, H dv]: the first dv dims of every head of attn [T, H P] times sigmoid(y[:, gate_off + h])."""
    _gpu(attn, y)
    T = y.shape[0]
    _need(attn.shape == (T, H * P) and attn.dtype == y.dtype, "latent_gate: shapes or dtypes")
    out = torch.empty((T, H * dv), dtype=y.dtype, device=y.device)
    _check(_lib().illm_latent_gate(_p(attn), _p(y), _code(y), y.shape[1], gate_off, _p(out), T, H,
                                   dv, P, _stream()), "latent_gate")
    return out


def latent_decode_splits(B: int, H: int, longest: int, mfma: bool = False) -> int:
    """Ranges the keys of a one-token step are cut into: about as many blocks as the chip has
    compute units, at most 16 ranges, none shorter than 64 keys; for the matrix-core kernel, whose
    blocks are single waves, about four waves a compute unit, at most 64 ranges of 32 keys or more."""
    if mfma:
        return max(1, min(-(-1024 // max(1, B * -(-H // 16))), 64, (longest + 31) // 32))
    groups = -(-H // (16 if H >= 16 else 8 if H >= 8 else 4))
    return max(1, min(-(-256 // max(1, B * groups)), 16, (longest + 63) // 64))


def latent_decode_mfma_fits(cache: torch.Tensor, cache_t: Optional[torch.Tensor], R: int, dr: int,
                            page_size: int) -> bool:
    return (cache_t is not None and cache.dtype == torch.bfloat16 and R % 16 == 0 and R <= 512
            and (R + dr) % 8 == 0 and page_size % 32 == 0)


def latent_absorb_q(y: torch.Tensor, w_uk: torch.Tensor, H: int, dn: int, dr: int, R: int,
                    out_dtype: torch.dtype) -> torch.Tensor:
    """qa [B, H, R + dr] = [W_uk,h^T q_h | q_h's rot part] of the (already rotated) queries in y:
    what a head's query looks like against latent rows.  float32 sums; bfloat16 for the
    matrix-core kernel, of whose product it is an operand."""
    _gpu(y, w_uk)
    B = y.shape[0]
    _need(w_uk.shape == (H * dn, R), "latent_absorb_q: W_uk [H dn, R]")
    qa = torch.empty((B, H, R + dr), dtype=out_dtype, device=y.device)
    _check(_lib().illm_latent_absorb_q(_p(y), _code(y), y.shape[1], _p(w_uk), _code(w_uk), _p(qa),
                                       _code(qa), B, H, dn, dr, R, _stream()), "latent_absorb_q")
    return qa


def latent_store_absorb(y: torch.Tensor, H: int, dn: int, dr: int, R: int, rot: int,
                        cos_sin: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                        row_pos: torch.Tensor, row_slot: torch.Tensor, cache: torch.Tensor,
                        page_table: torch.Tensor, page_size: int, ring: int, w_uk: torch.Tensor,
                        out_dtype: torch.dtype, cache_t: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`latent_rope_store` (without the rows' copies) and `latent_absorb_q` in one launch, for rows
    that will walk the cache: the latent and key part of every row are normed, rotated and stored,
    and qa is made from the queries with their rot part rotated on the way (y keeps them unrotated)."""
    _gpu(y, cos_sin, norm_w, row_pos, row_slot, cache, page_table, w_uk, cache_t)
    B, ncols = y.shape
    _i32(row_pos, B); _i32(row_slot, B); _i32(page_table)
    _need(ncols >= H * (dn + dr) + R + dr and norm_w.shape == (R,) and w_uk.shape == (H * dn, R),
          "latent_store_absorb: shapes")
    max_pos = 0
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 3 and cos_sin.shape[1] * 2 == rot
              and cos_sin.shape[2] == 2 and rot <= dr,
              "latent_store_absorb: angle table must be float32 [max_pos, rot/2, 2], rot <= dr")
        max_pos = cos_sin.shape[0]
    _need(cache.dtype == y.dtype and cache.dim() == 3 and cache.shape[1:] == (page_size, R + dr)
          and page_table.dim() == 2, "latent_store_absorb: cache shape or dtype")
    _need(cache_t is None or (cache_t.dtype == y.dtype and cache_t.shape == (cache.shape[0], R, page_size, 1)),
          "latent_store_absorb: the transposed copy must be [pages, R, page_size, 1]")
    qa = torch.empty((B, H, R + dr), dtype=out_dtype, device=y.device)
    _check(_lib().illm_latent_store_absorb(
        _p(y), _code(y), ncols, B, H, dn, dr, R, rot, _p(cos_sin), max_pos, _p(norm_w), _code(norm_w),
        ctypes.c_float(eps), _p(row_pos), _p(row_slot), _p(cache), _p(page_table), page_table.shape[1],
        page_size, ring, _p(cache_t), _p(w_uk), _code(w_uk), _p(qa), _code(qa), _stream()),
        "latent_store_absorb")
    return qa


def latent_attn_decode(qa: torch.Tensor, y: torch.Tensor, w_uv: torch.Tensor, gate_off: int,
                       cache: torch.Tensor, page_table: torch.Tensor, page_size: int, ring: int,
                       seq_slot: torch.Tensor, seq_len: torch.Tensor, len_more: int, H: int, dr: int,
                       R: int, dv: int, scale: float, window: int, nsplit: int,
                       cache_t: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per sequence over the latent cache, never building a head's keys or values: the
    queries qa [B, H, R + dr] have been taken through W_uk (`latent_absorb_q`), the weighted sums of
    latent rows go through W_uv after, then the head's output gate (y[:, gate_off + h]).  Token b
    sees seq_len[b] + len_more keys of the sequence in seq_slot[b], itself included.  With the
    transposed copy `cache_t` (and qa in bfloat16) both products run on the matrix cores.
    Returns [B, H dv]."""
    _gpu(qa, y, w_uv, cache, page_table, seq_slot, seq_len, cache_t)
    B = y.shape[0]
    _i32(page_table); _i32(seq_slot, B); _i32(seq_len, B)
    _need(w_uv.shape == (H * dv, R) and qa.shape == (B, H, R + dr), "latent_attn_decode: W_uv or qa")
    _need(cache.dim() == 3 and cache.shape[1:] == (page_size, R + dr) and cache.dtype == y.dtype,
          "latent_attn_decode: cache shape or dtype")
    partial = torch.empty((B, H, nsplit, R + 4), dtype=torch.float32, device=y.device)
    if cache_t is not None:
        _need(latent_decode_mfma_fits(cache, cache_t, R, dr, page_size) and qa.dtype == torch.bfloat16 and
              cache_t.shape == (cache.shape[0], R, page_size, 1) and cache_t.is_contiguous(),
              "latent_attn_decode: the transposed copy is not taken")
        _check(_lib().illm_latent_attn_decode_mfma(
            _p(qa), _p(cache), _p(cache_t), _p(page_table), page_table.shape[1], page_size, ring,
            _p(seq_slot), _p(seq_len), len_more, _p(partial), nsplit, B, H, R, dr,
            ctypes.c_float(scale), window, _stream()), f"latent_attn_decode_mfma (latent {R}+{dr})")
    else:
        _need(qa.dtype == torch.float32, "latent_attn_decode: float32 queries")
        _check(_lib().illm_latent_attn_decode(
            _p(qa), _p(cache), _code(cache), _p(page_table), page_table.shape[1], page_size, ring,
            _p(seq_slot), _p(seq_len), len_more, _p(partial), nsplit, B, H, R, dr, ctypes.c_float(scale),
            window, _stream()), f"latent_attn_decode (latent {R}+{dr})")
    out = torch.empty((B, H * dv), dtype=y.dtype, device=y.device)
    _check(_lib().illm_latent_merge_up(_p(partial), nsplit, _p(w_uv), _code(w_uv), _p(y), _code(y),
                                       y.shape[1], gate_off, _p(out), B, H, R, dv, _stream()),
           "latent_merge_up")
    return out


# ------------------------------------------------------------------ routed feed-forward
def few_outputs_f32(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """float32 x . w^T for a float32 matrix w [outputs, K] of few rows (a router's) and rows x of
    either type; products and sums in float32."""
    _gpu(x, w)
    _need(w.dtype == torch.float32 and x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1],
          f"few_outputs_f32: x {tuple(x.shape)} against float32 w {tuple(w.shape)}")
    T, K = x.shape
    z = torch.empty((T, w.shape[0]), dtype=torch.float32, device=x.device)
    _check(_lib().illm_few_outputs_f32(_p(x), _code(x), _p(w), _p(z), T, w.shape[0], K, _stream()),
           "few_outputs_f32")
    return z


MOE_SCORES = {"softmax": 0, "sigmoid": 1}            # a router's scores: over all outputs, or each its own
MOE_ACTIVATIONS = {"silu": 0, "clamped_swish": 1}    # see `moe_experts`


def moe_route(z: torch.Tensor, correction: Optional[torch.Tensor], top: int, score: str = "softmax"):
    """(idx int32 [T, top], weight float32 [T, top]): per row of the router's float32 outputs z
    the `top` largest score(z) + correction, and their scores (`score`: "softmax" over all
    outputs, or "sigmoid" of each)."""
    _need(score in MOE_SCORES, f"moe_route: score {score!r}; known: {sorted(MOE_SCORES)}")
    _gpu(z, correction)
    _need(z.dtype == torch.float32 and z.dim() == 2, "moe_route: float32 [T, outputs]")
    T, NE = z.shape
    _need(correction is None or correction.shape == (NE,), "moe_route: correction [outputs]")
    idx = torch.empty((T, top), dtype=torch.int32, device=z.device)
    wt = torch.empty((T, top), dtype=torch.float32, device=z.device)
    _check(_lib().illm_moe_route(_p(z), _p(correction),
                                 _code(correction) if correction is not None else 0, T, NE, top,
                                 _p(idx), _p(wt), MOE_SCORES[score], _stream()), "moe_route")
    return idx, wt


MOE_MFMA_FROM = 0        # (token, choice) pairs an expert on average from which the experts' products
                         # run on the matrix cores where the shape allows (measured on MI355X, 64
                         # experts of 1408 x 2048, 6 of them a token: a wave a column with lanes over
                         # K took 253 + 166 us for 64 tokens, bound by its sums across lanes)


def _moe_tiling(dtype: torch.dtype, E: int, F: int, NP: int, n_exp: int):
    """(on the matrix cores?, rows a tile, upper bound of tiles) for NP (token, choice) pairs."""
    # many pairs an expert (prompts): tiles of up to 64 rows; few (single tokens): tiles of 16 rows
    # on the matrix cores, or of 8 rows with a wave a column (float32, odd sizes)
    per_expert = NP / max(1, n_exp)
    mfma = dtype == torch.bfloat16 and E % 32 == 0 and F % 32 == 0 and per_expert >= MOE_MFMA_FROM
    rows = (64 if per_expert >= 48 else 32 if per_expert >= 24 else 16) if mfma else _lib().illm_moe_tile_rows()
    return mfma, rows, max(1, min(NP, NP // rows + n_exp))


def _moe_group(idx: torch.Tensor, n_exp: int, dtype: torch.dtype, E: int, F: int):
    NP = idx.numel()
    mfma, rows, max_tiles = _moe_tiling(dtype, E, F, NP, n_exp)
    order = torch.empty((NP,), dtype=torch.int32, device=idx.device)
    tiles = torch.empty((3 * max_tiles + 1,), dtype=torch.int32, device=idx.device)
    _check(_lib().illm_moe_group(_p(idx), NP, n_exp, _p(order), _p(tiles), max_tiles, rows,
                                 _stream()), "moe_group")
    return order, tiles, max_tiles, rows, mfma


def moe_plan(h: torch.Tensor, w_router: torch.Tensor, correction: Optional[torch.Tensor], top: int,
             w_gate_up: Optional[torch.Tensor], score: str = "softmax"):
    """A routed layer's plan for the rows h: (idx, weight, grouped).  idx, weight [T, top] as
    `moe_route` gives them for the router's float32 outputs h . w_router^T; grouped: the pairs
    grouped by expert for `moe_experts` (None without stacked experts)."""
    E = h.shape[1]
    n_exp = w_gate_up.shape[0] if w_gate_up is not None else 0
    idx, wt = moe_route(few_outputs_f32(h, w_router), correction, top, score)
    grouped = _moe_group(idx, n_exp, h.dtype, E, w_gate_up.shape[1] // 2) if n_exp else None
    return idx, wt, grouped


def moe_experts(h: torch.Tensor, idx: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor,
                grouped=None, activation: str = "silu", limit: float = 0.0,
                input_weight: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Y [T * top, E]: for every (token, choice) pair whose choice is one of the stacked experts
    (w_gate_up [experts, 2 F, E] = [gate | up], w_down [experts, E, F]) the expert's
    down(act(gate h, up h)); rows of other pairs are not written.  `activation` "silu":
    silu(g) * u; "clamped_swish": with g = min(g, limit) and u = clamp(u, -limit, limit),
    g * sigmoid(1.702 g) * (u + 1).  `input_weight` float32 [T, top]: the pair's expert sees
    weight * h instead of h.  `grouped`: the pairs by expert as `moe_plan` left them (else they
    are grouped here)."""
    _need(activation in MOE_ACTIVATIONS, f"moe_experts: activation {activation!r}; known: {sorted(MOE_ACTIVATIONS)}")
    act_kind, lim = MOE_ACTIVATIONS[activation], ctypes.c_float(limit)
    _need(input_weight is None or (input_weight.dtype == torch.float32 and input_weight.numel() == idx.numel()),
          "moe_experts: input weights are float32 [T, top]")
    _gpu(input_weight)
    _gpu(h, idx, w_gate_up, w_down)
    _i32(idx)
    T, E = h.shape
    top = idx.shape[1]
    n_exp, F2, _ = w_gate_up.shape
    _need(w_gate_up.shape[2] == E and w_down.shape == (n_exp, E, F2 // 2) and F2 % 2 == 0
          and w_gate_up.dtype == h.dtype and w_down.dtype == h.dtype and idx.shape[0] == T,
          "moe_experts: shapes or dtypes")
    NP = T * top
    F = F2 // 2
    order, tiles, max_tiles, rows, mfma = grouped if grouped is not None else _moe_group(idx, n_exp, h.dtype, E, F)
    act = torch.empty((NP, F), dtype=h.dtype, device=h.device)
    y = torch.empty((NP, E), dtype=h.dtype, device=h.device)
    if mfma:
        _check(_lib().illm_moe_rows_mfma(_p(h), top, _p(w_gate_up), 1, rows, _p(order), _p(tiles),
                                         max_tiles, _p(act), F, E, act_kind, lim, _p(input_weight),
                                         _stream()), "moe_rows_mfma (gate|up)")
        _check(_lib().illm_moe_rows_mfma(_p(act), 1, _p(w_down), 0, rows, _p(order), _p(tiles),
                                         max_tiles, _p(y), E, F, 0, ctypes.c_float(0.0), _p(None),
                                         _stream()), "moe_rows_mfma (down)")
        return y
    _check(_lib().illm_moe_rows(_p(h), top, _p(w_gate_up), _code(h), 1, _p(order), _p(tiles),
                                max_tiles, _p(act), F, E, act_kind, lim, _p(input_weight), _stream()),
           "moe_rows (gate|up)")
    _check(_lib().illm_moe_rows(_p(act), 1, _p(w_down), _code(h), 0, _p(order), _p(tiles),
                                max_tiles, _p(y), E, F, 0, ctypes.c_float(0.0), _p(None), _stream()),
           "moe_rows (down)")
    return y


def moe_combine(h: torch.Tensor, idx: torch.Tensor, wt: Optional[torch.Tensor], y: Optional[torch.Tensor],
                n_real: int, shared: Optional[torch.Tensor] = None,
                shared_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 [T, E]: sum over a token's choices of weight * (the expert's row of y, or h itself
    for a choice >= n_real), plus sigmoid(h . shared_gate) * shared.  `wt` None: every weight 1."""
    _gpu(h, idx, wt, y, shared, shared_gate)
    T, E = h.shape
    top = idx.shape[1]
    _need(y is not None or n_real == 0, "moe_combine: expert rows are needed")
    _need(y is None or (y.shape == (T * top, E) and y.dtype == h.dtype), "moe_combine: expert rows")
    _need(shared is None or (shared.shape == (T, E) and shared.dtype == h.dtype), "moe_combine: shared rows")
    _need(shared_gate is None or shared_gate.numel() == E, "moe_combine: shared gate [E]")
    out = torch.empty((T, E), dtype=torch.float32, device=h.device)
    _check(_lib().illm_moe_combine(_p(h), _code(h), _p(idx), _p(wt), _p(y), _p(shared),
                                   _p(shared_gate),
                                   _code(shared_gate) if shared_gate is not None else 0, _p(out), T,
                                   E, top, n_real, _stream()), "moe_combine")
    return out


# ------------------------------------------------------------------ attention with a soft cap
def kv_store2(rows: torch.Tensor, k_off: int, v_off: int, row_pos: torch.Tensor,
              row_slot: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
              page_table: torch.Tensor, page_size: int, ring: int, nkv: int, dk: int, dv: int) -> None:
    """Store the keys (columns k_off .. of width nkv dk) and values (v_off .. of width nkv dv) of
    packed rows into the paged cache, K [pages, nkv, page_size, dk], V [pages, nkv, page_size, dv]."""
    _gpu(rows, row_pos, row_slot, kcache, vcache, page_table)
    T = rows.shape[0]
    _i32(row_pos, T); _i32(row_slot, T); _i32(page_table)
    _need(rows.dim() == 2 and kcache.dtype == rows.dtype and vcache.dtype == rows.dtype,
          "kv_store2: rows [T, n] and a cache of their dtype")
    _need(kcache.shape[1:] == (nkv, page_size, dk) and vcache.shape[1:] == (nkv, page_size, dv)
          and kcache.shape[0] == vcache.shape[0] and page_table.dim() == 2, "kv_store2: cache shapes")
    _check(_lib().illm_kv_store2(_p(rows), _code(rows), rows.shape[1], k_off, v_off, _p(row_pos),
                                 _p(row_slot), _p(kcache), _p(vcache), _p(page_table),
                                 page_table.shape[1], page_size, ring, T, nkv, dk, dv, _stream()),
           "kv_store2")


def _cap_cache_ok(q, kcache, vcache, page_table, page_size, nh, nkv, dk, dv, what):
    _need(q.dim() == 2 and q.shape[1] >= nh * dk, f"{what}: rows [q | ...]")
    _need(nh % nkv == 0, f"{what}: heads must be a multiple of kv heads")
    _need(kcache.dtype == q.dtype and vcache.dtype == q.dtype
          and kcache.shape[1:] == (nkv, page_size, dk) and vcache.shape[1:] == (nkv, page_size, dv)
          and page_table.dim() == 2, f"{what}: cache shape or dtype")


def _cap_extras_ok(q, slopes, gate, gate_off, nh, dv, what, gate_heads=False):
    _gpu(slopes, gate)
    if gate_heads:
        dv = 1
    _need(slopes is None or (slopes.dtype == torch.float32 and slopes.shape == (nh,)),
          f"{what}: slopes float32 [{nh}]")
    _need(gate is None or (gate.dim() == 2 and gate.dtype == q.dtype and gate.shape[0] == q.shape[0]
                           and 0 <= gate_off and gate_off + nh * dv <= gate.shape[1]),
          f"{what}: gate rows of the queries' dtype with {nh * dv} columns from {gate_off}")


def _lse_ok(lse, rows, nh, what):
    if lse is not None:
        _gpu(lse)
        _need(lse.dtype == torch.float32 and lse.shape == (rows, nh), f"{what}: lse float32 [{rows}, {nh}]")


def qkv_norm_mix_store(rows: torch.Tensor, k_off: int, v_off: int, q_weight: Optional[torch.Tensor],
                       k_weight: Optional[torch.Tensor], eps: float, lam: Optional[torch.Tensor],
                       first: Optional[torch.Tensor], first_off: int, row_pos: torch.Tensor,
                       row_slot: torch.Tensor, kcache: Optional[torch.Tensor],
                       vcache: Optional[torch.Tensor], page_table: Optional[torch.Tensor],
                       page_size: int, ring: int, nh: int, nkv: int, dk: int, dv: int) -> None:
    """In place on packed rows [q (nh dk) | .. k at k_off (nkv dk) | v at v_off (nkv dv)], in float32:
    q and k each divided by the root mean square over all their heads at once and multiplied by
    `q_weight` [nh dk], `k_weight` [nkv dk] (None: untouched); v <- (1 - lam) v + lam first[:,
    first_off ..] with `lam` one float32 on the device (None: untouched); then k and v are stored in
    the paged cache K [pages, nkv, page_size, dk], V [pages, nkv, page_size, dv] (None: not stored)."""
    _gpu(rows, q_weight, k_weight, lam, first, row_pos, row_slot, kcache, vcache, page_table)
    T = rows.shape[0]
    _i32(row_pos, T); _i32(row_slot, T); _i32(page_table)
    _need(rows.dim() == 2, "qkv_norm_mix_store: rows [T, n]")
    _need((q_weight is None) == (k_weight is None), "qkv_norm_mix_store: both norm weights or none")
    if q_weight is not None:
        _need(q_weight.shape == (nh * dk,) and k_weight.shape == (nkv * dk,) and q_weight.dtype == k_weight.dtype,
              "qkv_norm_mix_store: norm weights over all heads")
    if lam is not None:
        _need(lam.dtype == torch.float32 and lam.numel() == 1 and first is not None and first.dim() == 2
              and first.dtype == rows.dtype and first.shape[0] == T and first_off + nkv * dv <= first.shape[1],
              "qkv_norm_mix_store: lam float32 [1] and the first layer's rows")
    if kcache is not None:
        _need(kcache.dtype == rows.dtype and vcache.dtype == rows.dtype
              and kcache.shape[1:] == (nkv, page_size, dk) and vcache.shape[1:] == (nkv, page_size, dv)
              and page_table is not None and page_table.dim() == 2, "qkv_norm_mix_store: cache shapes")
    _check(_lib().illm_qkv_norm_mix_store(
        _p(rows), _code(rows), rows.shape[1], k_off, v_off, _p(q_weight), _p(k_weight),
        _code(q_weight) if q_weight is not None else 0, ctypes.c_float(eps), _p(lam), _p(first),
        first.shape[1] if first is not None else 0, first_off, _p(row_pos), _p(row_slot), _p(kcache),
        _p(vcache), _p(page_table), page_table.shape[1] if page_table is not None else 0, page_size, ring,
        T, nh, nkv, dk, dv, _stream()), "qkv_norm_mix_store")


def attn_cap_rows(q: torch.Tensor, cu_seqlens: torch.Tensor, seq_slot: torch.Tensor,
                  seq_start: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                  page_table: torch.Tensor, page_size: int, ring: int, n_seqs: int, max_rows: int,
                  nh: int, nkv: int, dk: int, dv: int, scale: float, cap: float,
                  window: int, slopes: Optional[torch.Tensor] = None, chunk: int = 0,
                  gate: Optional[torch.Tensor] = None, gate_off: int = 0,
                  gate_heads: bool = False, lse: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of a step's packed rows over the paged cache (which holds the step's own
    keys and values by now): row r of sequence b stands at position seq_start[b] + r; scores
    cap tanh(q . k scale / cap) (cap 0: none); queries and keys of width dk, values of dv.
    `slopes` float32 [nh]: score -= slopes[h] (i - j).  `chunk` > 0: a row sees only the keys of its
    own chunk of positions.  `gate` [T, n] (columns gate_off ..): out *= sigmoid(gate), one
    number a head and value dim, or with `gate_heads` one a head.  `lse` float32 [T, nh] takes
    max + log(sum) of every row's and head's softmax.  Returns [T, nh dv]."""
    _cap_extras_ok(q, slopes, gate, gate_off, nh, dv, "attn_cap_rows", gate_heads)
    _lse_ok(lse, q.shape[0], nh, "attn_cap_rows")
    _gpu(q, cu_seqlens, seq_slot, seq_start, kcache, vcache, page_table)
    _i32(cu_seqlens, n_seqs + 1); _i32(seq_slot, n_seqs); _i32(seq_start, n_seqs); _i32(page_table)
    _cap_cache_ok(q, kcache, vcache, page_table, page_size, nh, nkv, dk, dv, "attn_cap_rows")
    out = torch.empty((q.shape[0], nh * dv), dtype=q.dtype, device=q.device)
    _check(_lib().illm_attn_cap_rows(
        _p(q), q.shape[1], _p(out), _code(q), _p(cu_seqlens), _p(seq_slot), _p(seq_start), _p(kcache),
        _p(vcache), _p(page_table), page_table.shape[1], page_size, ring, n_seqs, max_rows, nh, nkv,
        dk, dv, ctypes.c_float(scale), ctypes.c_float(cap), window, _p(slopes), int(chunk), _p(gate),
        gate.shape[1] if gate is not None else 0, gate_off, 1 if gate_heads else 0, _p(lse), _stream()),
        f"attn_cap_rows (sizes {dk}, {dv})")
    return out


def attn_cap_decode(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                    page_table: torch.Tensor, page_size: int, ring: int, seq_slot: torch.Tensor,
                    seq_len: torch.Tensor, nh: int, nkv: int, dk: int, dv: int, scale: float,
                    cap: float, window: int, nsplit: int, slopes: Optional[torch.Tensor] = None,
                    chunk: int = 0, gate: Optional[torch.Tensor] = None, gate_off: int = 0,
                    gate_heads: bool = False, lse: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The same attention for one new token per sequence: row b of q against the seq_len[b] keys
    (the new one included) of its slot, the keys cut into `nsplit` ranges.  Returns [B, nh dv]."""
    _cap_extras_ok(q, slopes, gate, gate_off, nh, dv, "attn_cap_decode", gate_heads)
    _lse_ok(lse, q.shape[0], nh, "attn_cap_decode")
    _need(lse is None or nsplit >= 2, "attn_cap_decode: lse comes from the merge of two or more ranges")
    _gpu(q, kcache, vcache, page_table, seq_slot, seq_len)
    B = q.shape[0]
    _i32(page_table); _i32(seq_slot, B); _i32(seq_len, B)
    _cap_cache_ok(q, kcache, vcache, page_table, page_size, nh, nkv, dk, dv, "attn_cap_decode")
    out = torch.empty((B, nh * dv), dtype=q.dtype, device=q.device)
    partial = torch.empty((B, nh, nsplit, dv + 2), dtype=torch.float32, device=q.device)
    _check(_lib().illm_attn_cap_decode(
        _p(q), q.shape[1], _p(out), _code(q), _p(kcache), _p(vcache), _p(page_table),
        page_table.shape[1], page_size, ring, _p(seq_slot), _p(seq_len), _p(partial), nsplit, B, nh,
        nkv, dk, dv, ctypes.c_float(scale), ctypes.c_float(cap), window, _p(slopes), int(chunk),
        _p(gate), gate.shape[1] if gate is not None else 0, gate_off, 1 if gate_heads else 0, _p(lse),
        _stream()), f"attn_cap_decode (sizes {dk}, {dv})")
    return out


# ------------------------------------------------------------------ the gated delta rule
def delta_prepare(P: torch.Tensor, b_off: int, A: torch.Tensor, a_off: int, conv_w: torch.Tensor,
                  tail: torch.Tensor, row_slot: torch.Tensor, a_log: torch.Tensor,
                  dt_bias: torch.Tensor, G: int, H: int, dk: int, dv: int, per_channel: bool,
                  update_tail: bool = False):
    """From the projections P [T, n] = [q (G dk) | k (G dk) | v (H dv) | ...] the recurrence's
    float32 inputs: q and k after the short convolution (conv_w float32 [C, taps], the inputs
    before a step's first row from `tail` [slots, taps - 1, C]), SiLU and the unit norm per head
    (q also times dk^-1/2), v after convolution and SiLU, beta = sigmoid(P[:, b_off + h]) and the
    decays exp(-exp(a_log[h]) softplus(A[:, a_off + i] + dt_bias[i])), one a head or, with
    `per_channel`, one a head and key channel.  `update_tail` (every sequence brings exactly one
    row): the tail is also moved on by that row here, and `delta_conv_tail` is not needed.
    Returns (q [T, G, dk], k, v [T, H, dv], beta [T, H], decay [T, H, 1 or dk])."""
    _gpu(P, A, conv_w, tail, row_slot, a_log, dt_bias)
    T = P.shape[0]
    _i32(row_slot, T)
    C = 2 * G * dk + H * dv
    DW = dk if per_channel else 1
    _need(P.dim() == 2 and P.shape[1] >= max(C, b_off + H) and A.dim() == 2 and A.shape[0] == T
          and A.shape[1] >= a_off + H * DW, "delta_prepare: projections too narrow")
    _need(conv_w.dtype == torch.float32 and conv_w.dim() == 2 and conv_w.shape[0] == C,
          "delta_prepare: conv_w float32 [C, taps]")
    taps = conv_w.shape[1]
    _need(tail.dim() == 3 and tail.shape[1:] == (max(taps - 1, 1), C), "delta_prepare: tail [slots, taps - 1, C]")
    _need(A.dtype == P.dtype and tail.dtype == P.dtype, "delta_prepare: P, A and the tail share one dtype")
    _need(a_log.dtype == torch.float32 and a_log.shape == (H,) and dt_bias.dtype == torch.float32
          and dt_bias.numel() == H * DW, "delta_prepare: a_log float32 [H], dt_bias float32 [H (dk)]")
    dev = P.device
    qn = torch.empty((T, G, dk), dtype=torch.float32, device=dev)
    kn = torch.empty((T, G, dk), dtype=torch.float32, device=dev)
    vv = torch.empty((T, H, dv), dtype=torch.float32, device=dev)
    beta = torch.empty((T, H), dtype=torch.float32, device=dev)
    dec = torch.empty((T, H, DW), dtype=torch.float32, device=dev)
    _check(_lib().illm_delta_prepare(
        _p(P), _code(P), P.shape[1], b_off, _p(A), _code(A), A.shape[1], a_off, _p(conv_w), taps,
        _p(tail), _code(tail), _p(row_slot), _p(a_log), _p(dt_bias), _p(qn), _p(kn), _p(vv), _p(beta),
        _p(dec), T, G, H, dk, dv, DW, 1 if update_tail else 0, _stream()), "delta_prepare")
    return qn, kn, vv, beta, dec


def delta_conv_tail(P: torch.Tensor, tail: torch.Tensor, cu_seqlens: torch.Tensor,
                    seq_slot: torch.Tensor, n_seqs: int, taps: int, col_off: int = 0) -> None:
    """Keep the last taps - 1 convolution inputs of every sequence of the step in `tail`; the
    convolution's channels are P's columns from `col_off` on."""
    _gpu(P, tail, cu_seqlens, seq_slot)
    _i32(cu_seqlens, n_seqs + 1); _i32(seq_slot, n_seqs)
    C = tail.shape[2]
    _need(P.dim() == 2 and col_off >= 0 and P.shape[1] >= col_off + C
          and tail.shape[1] == max(taps - 1, 1), "delta_conv_tail: shapes")
    first = ctypes.c_void_p(P.data_ptr() + col_off * P.element_size())
    _check(_lib().illm_delta_conv_tail(first, _code(P), P.shape[1], _p(tail), _code(tail),
                                       _p(cu_seqlens), _p(seq_slot), n_seqs, C, taps, _stream()),
           "delta_conv_tail")


def delta_scan(qn, kn, vv, beta, dec, state: torch.Tensor, cu_seqlens: torch.Tensor,
               seq_slot: torch.Tensor, n_seqs: int, max_rows: int, correct: bool = True) -> torch.Tensor:
    """The recurrence S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q over every
    sequence's rows in order, from `state` float32 [slots, H, dk, dv] and back into it.  With
    `correct` False the plain gated rule, u = beta v: S <- diag(g) S + k (beta v)^T.
    `max_rows`: the most rows a sequence brings (long sequences are laid out for their chain of
    tokens, short steps for the state's bytes).  Returns o float32 [T, H, dv]."""
    _gpu(qn, kn, vv, beta, dec, state, cu_seqlens, seq_slot)
    _i32(cu_seqlens, n_seqs + 1); _i32(seq_slot, n_seqs)
    T, G, dk = qn.shape
    _, H, dv = vv.shape
    _need(all(t.dtype == torch.float32 for t in (qn, kn, vv, beta, dec, state)), "delta_scan: float32")
    _need(kn.shape == qn.shape and beta.shape == (T, H) and dec.shape[:2] == (T, H)
          and dec.shape[2] in (1, dk) and state.shape[1:] == (H, dk, dv), "delta_scan: shapes")
    o = torch.empty((T, H, dv), dtype=torch.float32, device=qn.device)
    _check(_lib().illm_gated_scan(_p(qn), _p(kn), _p(vv), _p(beta), _p(dec), dec.shape[2], _p(state),
                                  _p(cu_seqlens), _p(seq_slot), _p(o), n_seqs, max_rows, G, H, dk, dv,
                                  1 if correct else 0, _stream()),
           "delta_scan")
    return o


# ------------------------------------------------------------------ around the plain gated rule
def ssm_prepare(U: torch.Tensor, x_off: int, dt_off: int, conv_w: torch.Tensor, conv_b: torch.Tensor,
                tail: torch.Tensor, row_slot: torch.Tensor, a_log: torch.Tensor,
                dt_bias: torch.Tensor, G: int, H: int, N: int, dv: int, update_tail: bool = False):
    """A state-space mixer's float32 inputs for the plain gated rule, from the input projection U
    [T, n]: columns x_off .. = x (H dv) | B (G N) | C (G N) go through the short convolution with
    bias (conv_w float32 [C, taps], conv_b [C]; the inputs before a step's first row from `tail`
    [slots, taps - 1, C]) and SiLU; step = softplus(U[:, dt_off + h] + dt_bias[h]) is the token's
    weight and exp(-exp(a_log[h]) step) its decay.  `update_tail` as in `delta_prepare`.
    Returns (q = C [T, G, N], k = B [T, G, N], v = x [T, H, dv], weight [T, H], decay [T, H, 1])."""
    _gpu(U, conv_w, conv_b, tail, row_slot, a_log, dt_bias)
    T = U.shape[0]
    _i32(row_slot, T)
    C = H * dv + 2 * G * N
    _need(U.dim() == 2 and U.shape[1] >= max(x_off + C, dt_off + H), "ssm_prepare: projection too narrow")
    _need(conv_w.dtype == torch.float32 and conv_w.dim() == 2 and conv_w.shape[0] == C
          and conv_b.dtype == torch.float32 and conv_b.shape == (C,), "ssm_prepare: conv_w float32 [C, taps], conv_b [C]")
    taps = conv_w.shape[1]
    _need(tail.dim() == 3 and tail.shape[1:] == (max(taps - 1, 1), C) and tail.dtype == U.dtype,
          "ssm_prepare: tail [slots, taps - 1, C] of the projection's dtype")
    _need(all(t.dtype == torch.float32 and t.shape == (H,) for t in (a_log, dt_bias)),
          "ssm_prepare: a_log, dt_bias float32 [H]")
    dev = U.device
    qn = torch.empty((T, G, N), dtype=torch.float32, device=dev)
    kn = torch.empty((T, G, N), dtype=torch.float32, device=dev)
    vv = torch.empty((T, H, dv), dtype=torch.float32, device=dev)
    beta = torch.empty((T, H), dtype=torch.float32, device=dev)
    dec = torch.empty((T, H, 1), dtype=torch.float32, device=dev)
    _check(_lib().illm_ssm_prepare(
        _p(U), _code(U), U.shape[1], x_off, dt_off, _p(conv_w), _p(conv_b), taps, _p(tail), _p(row_slot),
        _p(a_log), _p(dt_bias), _p(qn), _p(kn), _p(vv), _p(beta), _p(dec), T, G, H, N, dv,
        1 if update_tail else 0, _stream()), "ssm_prepare")
    return qn, kn, vv, beta, dec


def ssm_finish(o: torch.Tensor, x: torch.Tensor, D: torch.Tensor, Z: torch.Tensor, z_off: int,
               weight: torch.Tensor, norm_groups: int, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """[T, H dv] rows y = (o + D[h] x) silu(Z[:, z_off ..]), RMS-normed in `norm_groups` equal parts
    of the row (each by its own root mean square), times weight [H dv]."""
    _gpu(o, x, D, Z, weight)
    T, H, dv = o.shape
    _need(o.dtype == torch.float32 and x.dtype == torch.float32 and x.shape == o.shape
          and D.dtype == torch.float32 and D.shape == (H,) and weight.shape == (H * dv,)
          and Z.dim() == 2 and Z.shape[0] == T and Z.shape[1] >= z_off + H * dv
          and norm_groups >= 1 and (H * dv) % norm_groups == 0, "ssm_finish: shapes")
    out = torch.empty((T, H * dv), dtype=out_dtype, device=o.device)
    _check(_lib().illm_ssm_finish(_p(o), _p(x), _p(D), _p(Z), _code(Z), Z.shape[1], z_off, _p(weight),
                                  _code(weight), _p(out), _code(out), T, H, dv, int(norm_groups),
                                  ctypes.c_float(eps), _stream()), "ssm_finish")
    return out


def memory_prepare(U: torch.Tensor, i_off: int, f_off: int, i_bias: torch.Tensor, f_bias: torch.Tensor,
                   cap: float, m_state: torch.Tensor, cu_seqlens: torch.Tensor, seq_slot: torch.Tensor,
                   n_seqs: int, H: int, dk: int, dv: int):
    """A matrix memory's float32 inputs for the plain gated rule, from U [T, n] = [q (H dk) | k (H dk)
    | v (H dv) | ..]: q dk^-1/2, k, and v with a column of ones behind it (so the state's last
    column sums the weighted keys); the gates i = cap tanh((U[:, i_off + h] + i_bias) / cap) and
    f = logsigmoid(cap tanh((U[:, f_off + h] + f_bias) / cap)) against the running maximum
    m_t = max(f + m_(t-1), i), token after token from `m_state` float32 [slots, H] and back into it:
    decay exp(f + m_(t-1) - m_t), weight exp(i - m_t).
    Returns (q [T, H, dk], k, v [T, H, dv + 1], weight [T, H], decay [T, H, 1], exp(-m) [T, H])."""
    _gpu(U, i_bias, f_bias, m_state, cu_seqlens, seq_slot)
    _i32(cu_seqlens, n_seqs + 1); _i32(seq_slot, n_seqs)
    T = U.shape[0]
    _need(U.dim() == 2 and U.shape[1] >= max(2 * H * dk + H * dv, i_off + H, f_off + H),
          "memory_prepare: projection too narrow")
    _need(all(t.dtype == torch.float32 and t.shape == (H,) for t in (i_bias, f_bias))
          and m_state.dtype == torch.float32 and m_state.dim() == 2 and m_state.shape[1] == H,
          "memory_prepare: biases float32 [H], m_state float32 [slots, H]")
    dev = U.device
    qn = torch.empty((T, H, dk), dtype=torch.float32, device=dev)
    kn = torch.empty((T, H, dk), dtype=torch.float32, device=dev)
    vv = torch.empty((T, H, dv + 1), dtype=torch.float32, device=dev)
    beta = torch.empty((T, H), dtype=torch.float32, device=dev)
    dec = torch.empty((T, H, 1), dtype=torch.float32, device=dev)
    em = torch.empty((T, H), dtype=torch.float32, device=dev)
    _check(_lib().illm_memory_prepare(
        _p(U), _code(U), U.shape[1], i_off, f_off, _p(i_bias), _p(f_bias), ctypes.c_float(cap),
        _p(m_state), _p(cu_seqlens), _p(seq_slot), _p(qn), _p(kn), _p(vv), _p(beta), _p(dec), _p(em), T,
        n_seqs, H, dk, dv, _stream()), "memory_prepare")
    return qn, kn, vv, beta, dec, em


def memory_finish(o: torch.Tensor, em: torch.Tensor, weight: torch.Tensor, Z: torch.Tensor, z_off: int,
                  eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """o float32 [T, H, dv + 1] (the last column n . q): y = o[..., :dv] / (max(|n . q|, em) + 1e-6),
    then per head y / sqrt(mean y^2 + eps) * weight[h dv + j] * sigmoid(Z[:, z_off + h dv + j])."""
    _gpu(o, em, weight, Z)
    T, H, dv1 = o.shape
    dv = dv1 - 1
    _need(o.dtype == torch.float32 and em.dtype == torch.float32 and em.shape == (T, H)
          and weight.shape == (H * dv,) and Z.dim() == 2 and Z.shape[0] == T
          and Z.shape[1] >= z_off + H * dv, "memory_finish: shapes")
    out = torch.empty((T, H * dv), dtype=out_dtype, device=o.device)
    _check(_lib().illm_memory_finish(_p(o), _p(em), _p(weight), _code(weight), _p(Z), _code(Z), Z.shape[1],
                                     z_off, _p(out), _code(out), T, H, dv, ctypes.c_float(eps), _stream()),
           "memory_finish")
    return out


DELTA_GATES = {"silu": 0, "sigmoid": 1}


def delta_finish(o: torch.Tensor, weight: torch.Tensor, Z: torch.Tensor, z_off: int, gate: str,
                 eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """[T, H dv] rows o / sqrt(mean over dv of o^2 + eps) * weight [dv] * act(Z[:, z_off + ...]),
    act "silu" or "sigmoid", per head."""
    _gpu(o, weight, Z)
    T, H, dv = o.shape
    _need(o.dtype == torch.float32 and weight.shape == (dv,) and Z.dim() == 2 and Z.shape[0] == T
          and Z.shape[1] >= z_off + H * dv and gate in DELTA_GATES, "delta_finish: shapes or gate")
    out = torch.empty((T, H * dv), dtype=out_dtype, device=o.device)
    _check(_lib().illm_delta_finish(_p(o), _p(weight), _code(weight), _p(Z), _code(Z), Z.shape[1], z_off,
                                    DELTA_GATES[gate], _p(out), _code(out), T, H, dv,
                                    ctypes.c_float(eps), _stream()), "delta_finish")
    return out


# ------------------------------------------------------------------ short convolutions, a sublayer's own norm
def short_conv(X: torch.Tensor, x_off: int, C: int, weight: torch.Tensor, tail: torch.Tensor,
               row_slot: torch.Tensor, out_dtype: torch.dtype, bias: Optional[torch.Tensor] = None,
               in_bias: Optional[torch.Tensor] = None, add_input: bool = False,
               update_tail: bool = False) -> torch.Tensor:
    """A causal convolution over time on `C` channels of packed rows X [T, n] (columns x_off ..):
    y(t) = (in(t) if add_input) + bias + sum_j weight[:, j] in(t - (taps - 1 - j)), in = X (+ in_bias);
    the inputs before a step's first row come from `tail` [slots, taps - 1, C] (zeros in a fresh
    slot).  weight float32 [C, taps].  `update_tail` (every sequence brings exactly one row): the
    tail is moved on by that row in the same launch; otherwise `short_conv_tail` does that."""
    _gpu(X, weight, tail, row_slot, bias, in_bias)
    T = X.shape[0]
    _i32(row_slot, T)
    _need(X.dim() == 2 and 0 <= x_off and x_off + C <= X.shape[1], "short_conv: rows [T, n] with the channels inside")
    _need(weight.dtype == torch.float32 and weight.dim() == 2 and weight.shape[0] == C
          and 1 <= weight.shape[1] <= 8, "short_conv: weight float32 [C, taps] with 1 to 8 taps")
    taps = weight.shape[1]
    _need(tail.dim() == 3 and tail.shape[1:] == (max(taps - 1, 1), C), "short_conv: tail [slots, taps - 1, C]")
    for b in (bias, in_bias):
        _need(b is None or (b.dtype == torch.float32 and b.shape == (C,)), "short_conv: biases float32 [C]")
    out = torch.empty((T, C), dtype=out_dtype, device=X.device)
    _check(_lib().illm_short_conv(_p(X), _code(X), X.shape[1], x_off, _p(in_bias), _p(weight), _p(bias),
                                  taps, _p(tail), _code(tail), _p(row_slot), 1 if add_input else 0,
                                  _p(out), _code(out), C, T, C, 1 if update_tail else 0, _stream()),
           "short_conv")
    return out


def short_conv_tail(X: torch.Tensor, x_off: int, tail: torch.Tensor, cu_seqlens: torch.Tensor,
                    seq_slot: torch.Tensor, n_seqs: int, taps: int,
                    in_bias: Optional[torch.Tensor] = None) -> None:
    """Keep the last taps - 1 inputs (X's columns from x_off on, + in_bias) of every sequence of the
    step in `tail` [slots, taps - 1, C]."""
    _gpu(X, tail, cu_seqlens, seq_slot, in_bias)
    _i32(cu_seqlens, n_seqs + 1); _i32(seq_slot, n_seqs)
    C = tail.shape[2]
    _need(X.dim() == 2 and x_off >= 0 and X.shape[1] >= x_off + C and tail.shape[1] == max(taps - 1, 1),
          "short_conv_tail: shapes")
    _need(in_bias is None or (in_bias.dtype == torch.float32 and in_bias.shape == (C,)),
          "short_conv_tail: in_bias float32 [C]")
    _check(_lib().illm_short_conv_tail(_p(X), _code(X), X.shape[1], x_off, _p(in_bias), _p(tail),
                                       _code(tail), _p(cu_seqlens), _p(seq_slot), n_seqs, C, taps,
                                       _stream()), "short_conv_tail")


def rms_rows_gain(a: torch.Tensor, weight: torch.Tensor, eps: float, gain: float) -> torch.Tensor:
    """float32 [T, E]: gain * a / sqrt(mean(a^2) + eps) * weight, the norm of a sublayer's own output
    before it is added to the residual stream."""
    _gpu(a, weight)
    _need(a.dim() == 2 and weight.shape == (a.shape[1],), "rms_rows_gain: rows [T, E], weight [E]")
    out = torch.empty(a.shape, dtype=torch.float32, device=a.device)
    _check(_lib().illm_rms_rows_gain(_p(a), _code(a), _p(weight), _code(weight), _p(out), a.shape[0],
                                     a.shape[1], ctypes.c_float(eps), ctypes.c_float(gain), _stream()),
           "rms_rows_gain")
    return out


class PostNormed:
    """gain * a / sqrt(mean(a^2) + eps) * weight, not yet formed: what a sublayer with a norm of its
    own behind it leaves to be added to the residual stream.  A norm that adds it in its own kernel
    (`post_add_rmsnorm`) takes the pieces, any other asks for `tensor()` (float32)."""

    def __init__(self, a: torch.Tensor, weight: torch.Tensor, eps: float, gain: float):
        self.a, self.weight, self.eps, self.gain = a, weight, float(eps), float(gain)

    def tensor(self) -> torch.Tensor:
        return rms_rows_gain(self.a, self.weight, self.eps, self.gain)


POST_ADD_MAX_WIDTH = 16384


def post_add_rmsnorm(x: torch.Tensor, post: Optional[PostNormed], weight: torch.Tensor, eps: float,
                     out_dtype: torch.dtype, row_idx: Optional[torch.Tensor] = None, conv=None) -> torch.Tensor:
    """One pass between two sublayers: x += `post` (its norm formed here; None: nothing), then the
    RMS norm of x under `weight` in `out_dtype`, then, with `conv` = (weight float32 [E, taps], tail
    [slots, taps - 1, E], row_slot), the normed row plus its short convolution over time, the tail
    moved on (for steps of one row a sequence).  With `row_idx` only those rows, and x stays."""
    _gpu(x, weight, row_idx)
    _i32(row_idx)
    _need(x.dtype == torch.float32 and x.dim() == 2, "post_add_rmsnorm: x must be float32 [T, E]")
    T, E = x.shape
    _need(weight.shape == (E,) and E <= POST_ADD_MAX_WIDTH, f"post_add_rmsnorm: weight [{E}], width up to {POST_ADD_MAX_WIDTH}")
    a = pw = None
    if post is not None:
        a, pw = post.a, post.weight
        _gpu(a, pw)
        _need(a.shape == x.shape and pw.shape == (E,), "post_add_rmsnorm: the sublayer's output has x's shape")
    rows = T if row_idx is None else row_idx.numel()
    cw = tail = slots = None
    taps = 0
    if conv is not None:
        cw, tail, slots = conv
        _gpu(cw, tail, slots)
        _i32(slots, T)
        taps = cw.shape[1]
        _need(row_idx is None and cw.dtype == torch.float32 and cw.shape == (E, taps) and 2 <= taps <= 8
              and tail.dim() == 3 and tail.shape[1:] == (taps - 1, E), "post_add_rmsnorm: convolution shapes")
    out = torch.empty((rows, E), dtype=out_dtype, device=x.device)
    _check(_lib().illm_post_add_rmsnorm(
        _p(x), _p(a), _code(a) if a is not None else 0, _p(pw), _code(pw) if pw is not None else 0,
        ctypes.c_float(post.eps if post is not None else 0.0), ctypes.c_float(post.gain if post is not None else 0.0),
        _p(weight), _code(weight), _p(out), _code(out), _p(row_idx), rows, E, ctypes.c_float(eps), _p(cw), taps,
        _p(tail), _code(tail) if tail is not None else 0, _p(slots), _stream()), "post_add_rmsnorm")
    return out


SWISH_ALPHA = 1.702


def clamped_swish_mul(gate_up: torch.Tensor, limit: float) -> torch.Tensor:
    """[T, 2F] = [gate | up] -> [T, F]: g sigmoid(1.702 g) (u + 1) with g = min(gate, limit) and
    u = clamp(up, -limit, limit)."""
    _gpu(gate_up)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "clamped_swish_mul: rows [T, 2F]")
    T, F = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((T, F), dtype=gate_up.dtype, device=gate_up.device)
    _check(_lib().illm_clamped_swish_mul(_p(gate_up), _p(out), _code(gate_up), T, F, ctypes.c_float(limit),
                                         ctypes.c_float(SWISH_ALPHA), _stream()), "clamped_swish_mul")
    return out


# ------------------------------------------------------------------ attention over a window and pooled blocks
def qk_rotate_store(rows: torch.Tensor, k_off: int, v_off: int, cos_sin: Optional[torch.Tensor],
                    rot: int, pairing: int, unit_norm: bool, eps: float, row_pos: torch.Tensor,
                    row_slot: torch.Tensor, kcache: Optional[torch.Tensor],
                    vcache: Optional[torch.Tensor], page_table: Optional[torch.Tensor], page_size: int,
                    ring: int, nh: int, nkv: int, dk: int, dv: int,
                    q_scale: Optional[torch.Tensor] = None) -> None:
    """In place on packed rows [q (nh dk) | .. k at k_off (nkv dk) | v at v_off (nkv dv)], in float32:
    the first `rot` dims of every q and k head turned by the row's position (cos_sin float32
    [positions, rot / 2, 2]; pairing 0: i with i + rot / 2, 1: 2i with 2i + 1), then with `unit_norm`
    every head divided by its root mean square, then query head h times `q_scale`[h] (float32 [nh]:
    a scale of the scores that differs by head, taken into the queries); k and v stored in the paged
    cache K [pages, nkv, page_size, dk], V [pages, nkv, page_size, dv] (None: not stored; nkv 0: rows
    of queries alone)."""
    _gpu(rows, cos_sin, row_pos, row_slot, kcache, vcache, page_table, q_scale)
    _need(q_scale is None or (q_scale.dtype == torch.float32 and q_scale.shape == (nh,)),
          f"qk_rotate_store: q_scale float32 [{nh}]")
    T = rows.shape[0]
    _i32(row_pos, T); _i32(row_slot, T); _i32(page_table)
    _need(rows.dim() == 2, "qk_rotate_store: rows [T, n]")
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 3 and cos_sin.shape[1:] == (rot // 2, 2),
              "qk_rotate_store: cos_sin float32 [positions, rot / 2, 2]")
    if kcache is not None:
        _need(kcache.dtype == rows.dtype and vcache.dtype == rows.dtype
              and kcache.shape[1:] == (nkv, page_size, dk) and vcache.shape[1:] == (nkv, page_size, dv)
              and page_table is not None and page_table.dim() == 2, "qk_rotate_store: cache shapes")
    _check(_lib().illm_qk_rotate_store(
        _p(rows), _code(rows), rows.shape[1], k_off, v_off, _p(cos_sin), rot if cos_sin is not None else 0,
        pairing, cos_sin.shape[0] if cos_sin is not None else 0, 1 if unit_norm else 0, ctypes.c_float(eps),
        _p(q_scale), _p(row_pos), _p(row_slot), _p(kcache), _p(vcache), _p(page_table),
        page_table.shape[1] if page_table is not None else 0, page_size, ring, T, nh, nkv, dk, dv,
        _stream()), "qk_rotate_store")


def pool_store(row_pos: torch.Tensor, row_slot: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
               kpool: torch.Tensor, vpool: torch.Tensor, page_table: torch.Tensor, page_size: int,
               nkv: int, dk: int, dv: int, pool: int) -> None:
    """For every row of the step whose position p ends a block of `pool` tokens ((p + 1) % pool == 0):
    the mean of the block's keys and of its values, as the cache holds them, into row p // pool of
    the row's sequence in kpool, vpool (laid out and paged like the cache)."""
    _gpu(row_pos, row_slot, kcache, vcache, kpool, vpool, page_table)
    T = row_pos.numel()
    _i32(row_pos); _i32(row_slot, T); _i32(page_table)
    _need(kcache.shape[1:] == (nkv, page_size, dk) and vcache.shape[1:] == (nkv, page_size, dv)
          and kpool.shape == kcache.shape and vpool.shape == vcache.shape
          and len({t.dtype for t in (kcache, vcache, kpool, vpool)}) == 1 and page_table.dim() == 2,
          "pool_store: cache shapes")
    _check(_lib().illm_pool_store(_p(row_pos), _p(row_slot), _p(kcache), _p(vcache), _p(kpool), _p(vpool),
                                  _code(kcache), _p(page_table), page_table.shape[1], page_size, T, nkv, dk,
                                  dv, int(pool), _stream()), "pool_store")


def _pooled_ok(q, kcache, vcache, kpool, vpool, page_table, page_size, nh, nkv, dk, dv, head_scale, pool, what):
    _gpu(q, kcache, vcache, kpool, vpool, page_table, head_scale)
    _i32(page_table)
    _cap_cache_ok(q, kcache, vcache, page_table, page_size, nh, nkv, dk, dv, what)
    _need(head_scale is None or (head_scale.dtype == torch.float32 and head_scale.shape == (nh,)),
          f"{what}: head_scale float32 [{nh}]")
    if pool:
        _need(kpool is not None and vpool is not None and kpool.shape == kcache.shape
              and vpool.shape == vcache.shape and kpool.dtype == q.dtype and vpool.dtype == q.dtype,
              f"{what}: pooled rows laid out like the cache")


def _pooled_out(q, nh, dv, pool, out, lse, what):
    if lse is None:
        _need(out is None, f"{what}: `out` is given together with `lse`")
        return torch.empty((q.shape[0], nh * dv), dtype=q.dtype, device=q.device)
    _gpu(out)
    _lse_ok(lse, q.shape[0], nh, what)
    _need(pool > 0 and out is not None and out.dtype == q.dtype and out.shape == (q.shape[0], nh * dv),
          f"{what}: with `lse`, `out` [{q.shape[0]}, {nh * dv}] of the queries' dtype and pooled blocks")
    return out


def attn_pooled_rows(q: torch.Tensor, cu_seqlens: torch.Tensor, seq_slot: torch.Tensor,
                     seq_start: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                     kpool: Optional[torch.Tensor], vpool: Optional[torch.Tensor],
                     page_table: torch.Tensor, page_size: int, n_seqs: int, max_rows: int, nh: int,
                     nkv: int, dk: int, dv: int, scale: float, head_scale: Optional[torch.Tensor],
                     window: int, pool: int, out: Optional[torch.Tensor] = None,
                     lse: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of a step's packed rows over the paged cache (which holds the step's own keys and
    values, and the pooled rows of the blocks it completed, by now): the row at position i sees
    tokens j with 0 <= i - j < window and pooled block b if b pool + pool - 1 <= i - window, in one
    softmax; score = q . k scale head_scale[h].  Returns [T, nh dv].  With `out` and `lse` (what
    `attn_cap_rows` with that window left: the tokens' normalised sums and max + log(sum) of their
    softmax) only the pooled blocks are gone through and merged into `out` in place."""
    _pooled_ok(q, kcache, vcache, kpool, vpool, page_table, page_size, nh, nkv, dk, dv, head_scale, pool,
               "attn_pooled_rows")
    _gpu(cu_seqlens, seq_slot, seq_start)
    _i32(cu_seqlens, n_seqs + 1); _i32(seq_slot, n_seqs); _i32(seq_start, n_seqs)
    out = _pooled_out(q, nh, dv, pool, out, lse, "attn_pooled_rows")
    _check(_lib().illm_attn_pooled_rows(
        _p(q), q.shape[1], _p(out), _code(q), _p(cu_seqlens), _p(seq_slot), _p(seq_start), _p(kcache),
        _p(vcache), _p(kpool), _p(vpool), _p(page_table), page_table.shape[1], page_size, n_seqs, max_rows,
        nh, nkv, dk, dv, ctypes.c_float(scale), _p(head_scale), int(window), int(pool), _p(lse), _stream()),
        f"attn_pooled_rows (sizes {dk}, {dv})")
    return out


def attn_pooled_decode(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                       kpool: Optional[torch.Tensor], vpool: Optional[torch.Tensor],
                       page_table: torch.Tensor, page_size: int, seq_slot: torch.Tensor,
                       seq_len: torch.Tensor, nh: int, nkv: int, dk: int, dv: int, scale: float,
                       head_scale: Optional[torch.Tensor], window: int, pool: int,
                       out: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The same attention for one new token per sequence, at position seq_len[b] - 1 (`out` and `lse`
    as above, from `attn_cap_decode`).  Returns [B, nh dv]."""
    _pooled_ok(q, kcache, vcache, kpool, vpool, page_table, page_size, nh, nkv, dk, dv, head_scale, pool,
               "attn_pooled_decode")
    _gpu(seq_slot, seq_len)
    B = q.shape[0]
    _i32(seq_slot, B); _i32(seq_len, B)
    out = _pooled_out(q, nh, dv, pool, out, lse, "attn_pooled_decode")
    _check(_lib().illm_attn_pooled_decode(
        _p(q), q.shape[1], _p(out), _code(q), _p(kcache), _p(vcache), _p(kpool), _p(vpool), _p(page_table),
        page_table.shape[1], page_size, _p(seq_slot), _p(seq_len), B, nh, nkv, dk, dv, ctypes.c_float(scale),
        _p(head_scale), int(window), int(pool), _p(lse), _stream()), f"attn_pooled_decode (sizes {dk}, {dv})")
    return out


# ------------------------------------------------------------------ gated linear attention, a gated linear recurrent unit
def gla_prepare(U: torch.Tensor, q_off: int, k_off: int, v_off: int, Z: torch.Tensor,
                z_bias: torch.Tensor, tau: float, H: int, dk: int, dv: int):
    """Gated linear attention's float32 inputs for the plain gated rule with a decay per key channel,
    from the projections U [T, n] (q at q_off and k at k_off, H dk wide; v at v_off, H dv wide) and
    the decays' pre-activations Z [T, H dk] with their bias: q dk^-1/2, k, v, weight 1 and
    decay = sigmoid(Z + z_bias)^(1 / tau).
    Returns (q [T, H, dk], k, v [T, H, dv], weight [T, H], decay [T, H, dk])."""
    _gpu(U, Z, z_bias)
    T = U.shape[0]
    _need(U.dim() == 2 and Z.dim() == 2 and Z.shape == (T, H * dk) and max(q_off, k_off) + H * dk <= U.shape[1]
          and v_off + H * dv <= U.shape[1], "gla_prepare: projections too narrow")
    _need(z_bias.dtype == torch.float32 and z_bias.shape == (H * dk,), "gla_prepare: z_bias float32 [H dk]")
    dev = U.device
    qn = torch.empty((T, H, dk), dtype=torch.float32, device=dev)
    kn = torch.empty((T, H, dk), dtype=torch.float32, device=dev)
    vv = torch.empty((T, H, dv), dtype=torch.float32, device=dev)
    beta = torch.empty((T, H), dtype=torch.float32, device=dev)
    dec = torch.empty((T, H, dk), dtype=torch.float32, device=dev)
    _check(_lib().illm_gla_prepare(_p(U), _code(U), U.shape[1], q_off, k_off, v_off, _p(Z), _code(Z),
                                   Z.shape[1], _p(z_bias), ctypes.c_float(tau), _p(qn), _p(kn), _p(vv),
                                   _p(beta), _p(dec), T, H, dk, dv, _stream()), "gla_prepare")
    return qn, kn, vv, beta, dec


def lru_gates(u: torch.Tensor, w_t: torch.Tensor, r_bias: torch.Tensor, i_bias: torch.Tensor,
              lam: torch.Tensor, rate: float):
    """The gates of a gated linear recurrent unit from its input u float32 [T, C]: with the two
    block-diagonal maps `w_t` float32 [2, blocks, C / blocks (in), C / blocks (out)],
    r = sigmoid(Wr u + r_bias), i = sigmoid(Wi u + i_bias), a = exp(-rate r softplus(lam)) and
    x = sqrt(1 - a^2) i u.  Returns (a, x), float32 [T, C]."""
    _gpu(u, w_t, r_bias, i_bias, lam)
    T, C = u.shape
    _need(u.dtype == torch.float32 and w_t.dtype == torch.float32 and w_t.dim() == 4 and w_t.shape[0] == 2
          and w_t.shape[2] == w_t.shape[3] and w_t.shape[1] * w_t.shape[2] == C, "lru_gates: shapes")
    _need(all(t.dtype == torch.float32 and t.shape == (C,) for t in (r_bias, i_bias, lam)),
          "lru_gates: biases and lam float32 [C]")
    a = torch.empty((T, C), dtype=torch.float32, device=u.device)
    x = torch.empty((T, C), dtype=torch.float32, device=u.device)
    _check(_lib().illm_lru_gates(_p(u), _p(w_t), _p(r_bias), _p(i_bias), _p(lam), ctypes.c_float(rate),
                                 _p(a), _p(x), T, C, w_t.shape[1], _stream()), "lru_gates")
    return a, x


def lru_scan(a: torch.Tensor, x: torch.Tensor, state: torch.Tensor, Y: torch.Tensor, y_off: int,
             y_bias: Optional[torch.Tensor], cu_seqlens: torch.Tensor, seq_slot: torch.Tensor,
             n_seqs: int, max_rows: int, out_dtype: torch.dtype) -> torch.Tensor:
    """S <- a S + x per channel over every sequence's rows in order, from `state` float32 [slots, C]
    and back into it; returns S gelu_tanh(Y[:, y_off ..] + y_bias) as [T, C].  `max_rows`: the most
    rows a sequence brings; from 64 on the rows are gone through in chunks of 32 in parallel (a chunk's
    product of decays and sum first, then the chunks' start states in order, then the rows), which
    sums a row's state in another order than token by token."""
    _gpu(a, x, state, Y, y_bias, cu_seqlens, seq_slot)
    _i32(cu_seqlens, n_seqs + 1); _i32(seq_slot, n_seqs)
    T, C = a.shape
    _need(a.dtype == torch.float32 and x.dtype == torch.float32 and x.shape == a.shape
          and state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] == C
          and Y.dim() == 2 and Y.shape[0] == T and y_off + C <= Y.shape[1], "lru_scan: shapes")
    _need(y_bias is None or (y_bias.dtype == torch.float32 and y_bias.shape == (C,)), "lru_scan: y_bias float32 [C]")
    out = torch.empty((T, C), dtype=out_dtype, device=a.device)
    scratch = None
    if max_rows >= 64:
        scratch = torch.empty((2, n_seqs, -(-max_rows // 32), C), dtype=torch.float32, device=a.device)
    _check(_lib().illm_lru_scan(_p(a), _p(x), _p(state), _p(Y), _code(Y), Y.shape[1], y_off, _p(y_bias),
                                _p(out), _code(out), _p(cu_seqlens), _p(seq_slot), n_seqs, int(max_rows), C,
                                _p(scratch), _stream()), "lru_scan")
    return out


# ------------------------------------------------------------------ sampling
def argmax(logits: torch.Tensor) -> torch.Tensor:
    _gpu(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "argmax: float32 [B, V]")
    B, V = logits.shape
    out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    # a row in parts of 2,048 ids or more, about 512 blocks in all: one block a row walks a long
    # row alone (128,256 ids: 56 us whatever the batch)
    parts = max(1, min(64, V // 2048, 512 // max(B, 1)))
    scratch = torch.empty((2, B, parts), dtype=torch.int32, device=logits.device) if parts > 1 else None
    _check(_lib().illm_argmax(_p(logits), _p(out), _p(scratch), B, V, parts, _stream()), "argmax")
    return out


SAMPLE_LONG_FROM = 16384          # ids from which a row without top_k is sampled by several blocks
_sample_long_row_bytes = 0        # ILLM_SAMPLE_LONG_ROW_BYTES of csrc/api.h, asked of the library at first use


def sample(logits: torch.Tensor, temperature: float, top_k: int, top_p: float,
           repeat_penalty: float, last_tokens: Optional[torch.Tensor], seeds: torch.Tensor,
           counters: torch.Tensor) -> torch.Tensor:
    """One draw per row; see csrc/sampling.hip.  seeds: int64 [B] (bit pattern used), counters int32 [B]."""
    _gpu(logits, last_tokens, seeds, counters)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "sample: float32 [B, V]")
    B, V = logits.shape
    _need(seeds.dtype == torch.int64 and seeds.numel() >= B, "sample: seeds int64 [B]")
    _i32(counters, B); _i32(last_tokens)
    n_last = 0
    if last_tokens is not None:
        _need(last_tokens.dim() == 2 and last_tokens.shape[0] == B, "sample: last_tokens [B, n]")
        n_last = last_tokens.shape[1]
    _need(temperature > 0 and top_p > 0 and repeat_penalty > 0 and n_last <= 256,
          "sample: temperature, top_p and repeat_penalty must be positive, window <= 256")
    out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    scratch = torch.empty((2, B, V), dtype=torch.float32, device=logits.device)
    if (top_k <= 0 or top_k >= V) and V >= SAMPLE_LONG_FROM and B <= 65535:
        # a long row without top_k: several blocks a row (one block walks 32,000 ids in 54 us for
        # temperature alone and 109 us with top_p, 128,256 in 134 and 395 us)
        global _sample_long_row_bytes
        if not _sample_long_row_bytes:
            _sample_long_row_bytes = int(_lib().illm_sample_long_row_bytes())
        rows = torch.empty((B, (_sample_long_row_bytes + 7) // 8), dtype=torch.int64, device=logits.device)
        _check(_lib().illm_sample_long(
            _p(logits), _p(scratch), _p(rows), _p(out), B, V, ctypes.c_float(temperature),
            ctypes.c_float(top_p), ctypes.c_float(repeat_penalty), _p(last_tokens), n_last, _p(seeds),
            _p(counters), _stream()), "sample_long")
        return out
    _check(_lib().illm_sample(
        _p(logits), _p(scratch), _p(out), B, V, ctypes.c_float(temperature), int(top_k),
        ctypes.c_float(top_p), ctypes.c_float(repeat_penalty), _p(last_tokens), n_last, _p(seeds),
        _p(counters), _stream()), "sample")
    return out
