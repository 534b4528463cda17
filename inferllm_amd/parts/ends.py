"""The two ends of a decoder: token embedding and the head that gives logits."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.manager import StateSpec
from ..kernels import ops
from ..weights.loader import TensorWant
from .base import Embedding, Head, StepContext, register_part


@register_part("embedding", "token_embedding")
class TokenEmbedding(Embedding):
    """Row copy (src/kern/naive/naive.cpp:43-54); rows become float32 and are multiplied by
    `scale` (1: the reference's plain copy).  `streams` > 0: a model with several residual
    streams; the rows come out as [rows, streams, hidden], every stream the embedded row."""

    graph_safe_prompts = True

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, streams: int = 0,
                 tensors=None):
        super().__init__(tensors)
        self.V, self.E = int(vocab_size), int(hidden_size)
        self.scale, self.streams = float(scale), int(streams)
        self.weight: Optional[torch.Tensor] = None

    def shapes(self) -> Dict[str, TensorWant]:
        return {"weight": TensorWant((self.V, self.E))}

    def load(self, tensors) -> None:
        self.weight = self._take(tensors, "weight").contiguous()

    def forward(self, ctx: StepContext):
        if self.streams:
            return ops.embed(ctx.tokens, self.weight, self.scale, self.streams)
        return ops.embed(ctx.tokens, self.weight, self.scale)


@register_part("embedding", "token_pair_embedding")
class TokenPairEmbedding(Embedding):
    """The token's row times `scale`, plus a row of a table hashed by the pair (previous token, token),
    plus a learned row of the position:

        x = table[t] * scale + pairs[(t_before * mul_prev + t * mul_cur) mod buckets] + places[p]

    A sequence's first token takes the pair table's last row (number `buckets`).  The token before
    a step's first row is part of the sequence's state: one int per slot, kept by the cache manager
    under the line `STATE_LINE` like a mixer's state.  `buckets` 0: no pair table; `positions` 0: no
    position table.  All sums are float32."""

    graph_safe_prompts = True
    STATE_LINE = "embedding"

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, buckets: int = 0,
                 mul_prev: int = 1, mul_cur: int = 1, positions: int = 0, tensors=None):
        super().__init__(tensors)
        self.V, self.E, self.scale = int(vocab_size), int(hidden_size), float(scale)
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        self.positions = int(positions)
        if self.buckets < 0 or self.mul_prev < 0 or self.mul_cur < 0 or self.positions < 0:
            raise ValueError("token_pair_embedding: buckets, multipliers and positions are not negative")
        self.weight = self.pairs = self.places = None

    def shapes(self) -> Dict[str, TensorWant]:
        out = {"weight": TensorWant((self.V, self.E))}
        if self.buckets:
            out["pairs"] = TensorWant((self.buckets + 1, self.E))
        if self.positions:
            out["places"] = TensorWant((self.positions, self.E))
        return out

    def state_spec(self):
        """The last token of every sequence (int32), if there is a pair table."""
        return StateSpec((), torch.int32) if self.buckets else None

    def load(self, tensors) -> None:
        self.weight = self._take(tensors, "weight").contiguous()
        self.pairs = self._take(tensors, "pairs").contiguous() if self.buckets else None
        self.places = self._take(tensors, "places").contiguous() if self.positions else None

    def forward(self, ctx: StepContext):
        last = ctx.cache.state_line(self.STATE_LINE) if self.buckets else None
        x = ops.embed_pairs(ctx.tokens, ctx.row_pos, ctx.row_slot, self.weight, self.scale, self.pairs,
                            self.buckets, self.mul_prev, self.mul_cur, self.places, last,
                            remember=not ctx.prefill)
        if ctx.prefill and last is not None:
            ops.remember_last(ctx.tokens, ctx.cu_seqlens, ctx.seq_slot, last, ctx.n_seqs)
        return x


@register_part("head", "lm_head")
class LMHead(Head):
    """logits = h . W^T in float32, for the rows asked for only.

    src/core/graph.cpp:117-141 and src/core/op.cpp:230-274 (the reference takes the
    last row only).  `tied_fallback` names the tensor used when the head's own is
    absent from the checkpoint (tied embeddings).
    """

    graph_safe_prompts = True

    def __init__(self, hidden_size: int, vocab_size: int, tied_fallback: Optional[str] = None,
                 tensors=None):
        super().__init__(tensors)
        self.E, self.V = int(hidden_size), int(vocab_size)
        self.tied_fallback = tied_fallback
        self.weight: Optional[torch.Tensor] = None

    def wants(self) -> Dict[str, TensorWant]:
        out = {self.tensors["weight"]: TensorWant((self.V, self.E),
                                                  optional=self.tied_fallback is not None)}
        if self.tied_fallback is not None:
            out[self.tied_fallback] = TensorWant((self.V, self.E))
        return out

    def load(self, tensors) -> None:
        own = self.tensors["weight"]
        self.weight = ops.decode_weight(
            (tensors[own] if own in tensors else tensors[self.tied_fallback]).contiguous(),
            "plain", self.decode_copies)

    def forward(self, h, ctx: StepContext):
        return ops.linear(h, self.weight, out_dtype=torch.float32)
