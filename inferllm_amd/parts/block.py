"""Arrangements of mixer, feed-forward and norms around the residual stream."""
from __future__ import annotations

import torch

from ..cache.manager import StateSpec
from ..kernels import ops
from ..weights.loader import TensorWant
from .base import Block, StepContext, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    """x1 = x + mixer(norm(x)); x2 = x1 + feed_forward(norm(x1)).

    src/graph/llama_like.cpp:66-105.  The residual stream stays float32; each add is
    fused into the norm that follows it, so the block returns its feed-forward
    output for the next norm (the next block's, or the model's last) to add.  For steps of
    few rows, parts that say so (`Part.adds_residual`, `takes_normed_rows`) shorten this: a
    part adds its output to the stream in its last kernel, which also prepares the norm that
    follows for the next part's first kernel; what the block hands on is then None (nothing
    left to add) or `ops.NormedRows`.
    """

    graph_safe_prompts = True

    takes_next_norm = True
    takes_prepared_rows = True

    @staticmethod
    def _enter(norm, part, x, pending, ctx):
        """The input of `part`: the normed rows of x (+ pending), by a kernel or prepared."""
        if isinstance(pending, ops.NormedRows):
            params = norm.rms_params()
            if params is not None and pending.made_for(*params):
                return pending if part.takes_normed_rows else pending.rows()
            pending = None                       # the sum is in x already; another norm follows
        return norm.forward(x, pending, ctx)

    def forward(self, x, pending, ctx: StepContext, line, writes_cache, next_norm=None):
        h = self._enter(self.mixer_norm, self.mixer, x, pending, ctx)
        if self.mixer.adds_residual:
            d = self.mixer.forward(h, ctx, line, writes_cache, self.position, residual=x,
                                   next_norm=self.feed_forward_norm)
        else:
            d = self.mixer.forward(h, ctx, line, writes_cache, self.position)
        h2 = self._enter(self.feed_forward_norm, self.feed_forward, x, d, ctx)
        if self.feed_forward.adds_residual:
            return self.feed_forward.forward(h2, ctx, residual=x, next_norm=next_norm)
        return self.feed_forward.forward(h2, ctx)


@register_part("block", "parallel")
class ParallelBlock(Block):
    """x <- x + (mixer(h) + feed_forward(h)) with h = norm(x): one norm, both parts read its rows.
    With a second norm (`feed_forward_norm`) the feed-forward reads rows of its own,
    x <- x + (mixer(norm1(x)) + feed_forward(norm2(x))), both norms of the same x.

    The two outputs are left for the next norm to add to the stream as (mixer + feed-forward) in
    float32: as a pair, if that norm says it adds pairs in its own kernel (`Norm.adds_pairs`), else
    as their float32 sum (`ops.sum_rows`).  A feed-forward that returns None (a layer without one)
    leaves the mixer's output alone.
    """

    graph_safe_prompts = True

    takes_next_norm = True           # to know whether the norm that follows adds a pair itself
    takes_prepared_rows = True       # (prepared rows mean: the sum is in x already)

    def forward(self, x, pending, ctx: StepContext, line, writes_cache, next_norm=None):
        if isinstance(pending, ops.NormedRows):
            pending = None                       # its sum is in x already
        if isinstance(pending, tuple) and not getattr(self.mixer_norm, "adds_pairs", False):
            pending = ops.sum_rows(*pending)
        h2 = None
        if self.feed_forward_norm is not None and hasattr(self.mixer_norm, "forward_with"):
            both = self.mixer_norm.forward_with(self.feed_forward_norm, x, pending, ctx)   # one pass over x
            if both is not None:
                h, h2 = both
        if h2 is None:
            h = self.mixer_norm.forward(x, pending, ctx)
            # a second norm reads the same x, which holds the sum by now
            h2 = self.feed_forward_norm.forward(x, None, ctx) if self.feed_forward_norm is not None else h
        a = self.mixer.forward(h, ctx, line, writes_cache, self.position)
        f = self.feed_forward.forward(h2, ctx)
        if f is None:
            return a
        if next_norm is not None and getattr(next_norm, "adds_pairs", False):
            return (a, f)
        return ops.sum_rows(a, f)


@register_part("block", "sandwich")
class SandwichBlock(Block):
    """Sublayers with a norm in front and a norm of their own behind, a gain on what they add, and
    a short convolution over time in front of what they read:

        x <- x + gain * post1(mixer(c1(norm1(x))));   x <- x + gain * post2(feed_forward(c2(norm2(x))))
        c(h)_t = h_t + sum_j w[:, j] h_(t - taps + 1 + j)       (zeros before the sequence; taps 0: c(h) = h)

    The post norms are RMS norms over the width with gain `weight_offset` + stored weight, like the
    norms in front (which are parts of their own).  The last taps - 1 normed rows of either sublayer
    are part of a sequence's state, which the arrangement keeps itself ("tail1", "tail2").  What a
    sublayer adds is formed in float32 and handed to the next norm, which adds it to the stream.
    A layer whose feed-forward is "none" has the first sublayer alone.
    """

    graph_safe_prompts = True

    takes_next_norm = True           # to hand a norm that forms a sublayer's own norm the pieces
    takes_prepared_rows = True       # (prepared rows mean: the sum is in x already)

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm, position, size: int,
                 eps: float, gain: float = 1.0, taps: int = 0, weight_offset: float = 0.0, tensors=None):
        super().__init__(mixer, feed_forward, mixer_norm, feed_forward_norm, position, tensors)
        self.size, self.eps, self.gain = int(size), float(eps), float(gain)
        self.taps, self.weight_offset = int(taps), float(weight_offset)
        if not 0 <= self.taps <= 8:
            raise ValueError(f"sandwich block: {taps} taps; the kernels take up to 8")
        self.has_ff = feed_forward_norm is not None
        self.post = [None, None]
        self.conv = [None, None]

    def _sublayers(self):
        return (1, 2) if self.has_ff else (1,)

    def shapes(self):
        out = {}
        for q in self._sublayers():
            out[f"post{q}"] = TensorWant((self.size,), init="normal" if self.weight_offset else "ones_normal",
                                         keep_stored=True)
            if self.taps:
                out[f"conv{q}"] = TensorWant((self.size, self.taps), keep_stored=True)
        return out

    def state_spec(self):
        if self.taps < 2:
            return None
        return {f"tail{q}": StateSpec((self.taps - 1, self.size), None) for q in self._sublayers()}

    def load_own(self, tensors) -> None:
        for q in self._sublayers():
            w = self._take(tensors, f"post{q}")
            self.post[q - 1] = ((w.to(torch.float32) + self.weight_offset) if self.weight_offset else w).contiguous()
            if self.taps:
                self.conv[q - 1] = self._take(tensors, f"conv{q}").to(torch.float32).contiguous()

    def _tail(self, q: int, ctx: StepContext):
        return ctx.cache.state_line(("block", ctx.run))[f"tail{q}"]

    def _read(self, h, q: int, ctx: StepContext):
        """What sublayer q reads: the normed rows plus their convolution over time."""
        if not self.taps:
            return h
        tail = self._tail(q, ctx) if self.taps > 1 else h.new_zeros((1, 1, self.size))
        out = ops.short_conv(h, 0, self.size, self.conv[q - 1], tail, ctx.row_slot, h.dtype,
                             add_input=True, update_tail=not ctx.prefill)
        if ctx.prefill and self.taps > 1:
            ops.short_conv_tail(h, 0, tail, ctx.cu_seqlens, ctx.seq_slot, ctx.n_seqs, self.taps)
        return out

    def _enter(self, norm, q: int, x, pending, ctx: StepContext):
        """Sublayer q's input: `pending` added to x, the norm, the convolution.  A plain RMS norm
        and a step of single tokens make that one kernel."""
        if isinstance(pending, ops.NormedRows):
            pending = None                       # its sum is in x already
        params = norm.rms_params()
        plain = pending is None or isinstance(pending, ops.PostNormed)
        if (params is not None and plain and not ctx.prefill and self.taps > 1
                and self.size <= ops.POST_ADD_MAX_WIDTH):
            return ops.post_add_rmsnorm(x, pending, params[0], params[1], ctx.act_dtype,
                                        conv=(self.conv[q - 1], self._tail(q, ctx), ctx.row_slot))
        if isinstance(pending, ops.PostNormed) and not getattr(norm, "adds_post_normed", False):
            pending = pending.tensor()
        return self._read(norm.forward(x, pending, ctx), q, ctx)

    def _leave(self, y, q: int, next_norm):
        """What sublayer q leaves to be added: its output under its own norm, times the gain; as
        pieces if the norm that follows forms them in its own pass."""
        post = ops.PostNormed(y, self.post[q - 1], self.eps, self.gain)
        return post if next_norm is not None and getattr(next_norm, "adds_post_normed", False) else post.tensor()

    def forward(self, x, pending, ctx: StepContext, line, writes_cache, next_norm=None):
        h = self._enter(self.mixer_norm, 1, x, pending, ctx)
        a = self.mixer.forward(h, ctx, line, writes_cache, self.position)
        if not self.has_ff:
            return self._leave(a, 1, next_norm)
        h2 = self._enter(self.feed_forward_norm, 2, x, self._leave(a, 1, self.feed_forward_norm), ctx)
        return self._leave(self.feed_forward.forward(h2, ctx), 2, next_norm)


@register_part("block", "hyper_connections")
class HyperConnectionBlock(Block):
    """Pre-norm sublayers over `streams` residual streams x_1 .. x_s in place of one.

    For each sublayer q (the mixer, then the feed-forward): u = sum_s read_q[s] x_s,
    y = sublayer(norm_q(u)), then for all streams at once x_t <- sum_s mix_q[s, t] x_s + out_q[t] y.
    The reads belong to the norms (`stream_rms_norm`, whose kernel also does the write of the
    sublayer before it); the block owns mix_q [streams, streams] (indexed [from, to]) and out_q
    [streams] and hands each sublayer's output on as `ops.StreamWrite`, the last one to whatever
    norm comes next.  A layer whose feed-forward is "none" has the mixer's sublayer alone; if it is
    given the second sublayer's mix matrix all the same (`mix2` among its tensors), the streams are
    still mixed by it, with nothing added: folded at load into the first sublayer's write,
    x <- M2^T (M1^T x + out1 y) = (M1 M2)^T x + (M2^T out1) y.
    """

    graph_safe_prompts = True

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm, position, streams: int,
                 tensors=None):
        super().__init__(mixer, feed_forward, mixer_norm, feed_forward_norm, position, tensors)
        self.streams = int(streams)
        self.has_ff = feed_forward_norm is not None
        if hasattr(mixer, "takes_scaled_sums"):
            mixer.takes_scaled_sums = True       # the streams' kernel adds sa a + sb b itself
        self.mix = [None, None]
        self.out = [None, None]

    def shapes(self):
        S = self.streams
        mix = lambda: TensorWant((S, S), init="eye_normal", keep_stored=True)
        out = lambda: TensorWant((S,), init="ones_normal", keep_stored=True)
        out = {"mix1": mix(), "out1": out()} | ({"mix2": mix(), "out2": out()} if self.has_ff else {})
        if not self.has_ff and "mix2" in self.tensors:
            out["mix2"] = mix()
        return out

    def load_own(self, tensors) -> None:
        for q in range(2 if self.has_ff else 1):
            self.mix[q] = self._take(tensors, f"mix{q + 1}").to(torch.float32).contiguous()
            self.out[q] = self._take(tensors, f"out{q + 1}").to(torch.float32).contiguous()
        if not self.has_ff and "mix2" in self.tensors:
            second = self._take(tensors, "mix2").to(torch.float32)
            self.out[0] = (self.out[0] @ second).contiguous()
            self.mix[0] = (self.mix[0] @ second).contiguous()

    def _write(self, y, q: int) -> ops.StreamWrite:
        if isinstance(y, ops.ScaledSum):
            return ops.StreamWrite(y.a, self.mix[q], self.out[q], y2=y.b, ya=y.sa, yb=y.sb)
        return ops.StreamWrite(y, self.mix[q], self.out[q])

    def forward(self, x, pending, ctx: StepContext, line, writes_cache):
        h = self.mixer_norm.forward(x, pending, ctx)
        first = self._write(self.mixer.forward(h, ctx, line, writes_cache, self.position), 0)
        if not self.has_ff:
            return first
        h2 = self.feed_forward_norm.forward(x, first, ctx)
        return self._write(self.feed_forward.forward(h2, ctx), 1)
