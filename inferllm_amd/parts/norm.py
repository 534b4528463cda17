"""RMS norm fused with the residual add that precedes it."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import TensorWant
from .base import Norm, StepContext, register_part


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    """y = x / sqrt(mean(x^2) + eps) * weight, statistics in float32.

    src/kern/naive/naive.cpp:186-207 and src/core/op.cpp:37-47; eps is a parameter
    (the reference fixes 1e-6 / 1e-5 at src/graph/llama_like.cpp:78 and src/core/graph.h:163).
    `weight_offset` c: the stored tensor lies around zero and the gain is c + stored (formed once,
    in float32, as the tensor is taken).
    """

    graph_safe_prompts = True

    adds_planes = True
    # `forward` also takes `delta` as a pair of tensors (two parts' outputs for the same rows),
    # added as x + (first + second) in the norm's own kernel
    adds_pairs = True

    def __init__(self, size: int, eps: float, weight_offset: float = 0.0, tensors=None):
        super().__init__(tensors)
        self.size, self.eps, self.weight_offset = int(size), float(eps), float(weight_offset)
        self.weight: Optional[torch.Tensor] = None

    def shapes(self) -> Dict[str, TensorWant]:
        return {"weight": TensorWant((self.size,), init="normal" if self.weight_offset else "ones_normal",
                                     keep_stored=True)}

    def load(self, tensors) -> None:
        self.weight = self._take(tensors, "weight").contiguous()
        if self.weight_offset:
            self.weight = (self.weight.to(torch.float32) + self.weight_offset).contiguous()

    def rms_params(self):
        return self.weight, self.eps

    # `forward` also takes `delta` as `ops.PostNormed` (a sublayer's output whose own norm is still
    # to be formed) and forms it in the same pass
    adds_post_normed = True

    def forward(self, x, delta, ctx: StepContext, row_idx=None):
        if isinstance(delta, ops.PostNormed):
            if self.size <= ops.POST_ADD_MAX_WIDTH:
                return ops.post_add_rmsnorm(x, delta, self.weight, self.eps, ctx.act_dtype, row_idx)
            delta = delta.tensor()
        return ops.add_rmsnorm(x, delta, self.weight, self.eps, ctx.act_dtype, row_idx)

    def forward_with(self, other: "RMSNorm", x, delta, ctx: StepContext):
        """(this norm's rows, `other`'s rows) of the same x (+ delta) in one pass, or None if the two
        norms cannot share one (another eps, another precision of the weights)."""
        if (type(other) is not RMSNorm or other.eps != self.eps or other.size != self.size
                or other.weight.dtype != self.weight.dtype):
            return None
        return ops.add_rmsnorm(x, delta, self.weight, self.eps, ctx.act_dtype, weight2=other.weight)


@register_part("norm", "stream_rms_norm")
class StreamRMSNorm(Norm):
    """The norm in front of a sublayer of a model with several residual streams: the write of the
    sublayer before (`ops.StreamWrite`: x_t <- sum_s mix[s, t] x_s + out[t] y for all streams at
    once), the read u = sum_s read[s] x_s and y = u / sqrt(mean(u^2) + eps) * weight, in one kernel.
    x is float32 [rows, streams, size].  Without a `read` tensor the streams are summed as they
    are (the model's last norm)."""

    graph_safe_prompts = True

    def __init__(self, size: int, eps: float, streams: int, tensors=None):
        super().__init__(tensors)
        self.size, self.eps, self.streams = int(size), float(eps), int(streams)
        if not 1 <= self.streams <= 8:
            raise ValueError(f"{streams} residual streams: the kernels take 1 to 8")
        self.weight: Optional[torch.Tensor] = None
        self.read: Optional[torch.Tensor] = None

    def shapes(self) -> Dict[str, TensorWant]:
        out = {"weight": TensorWant((self.size,), init="ones_normal", keep_stored=True)}
        if "read" in self.tensors:
            out["read"] = TensorWant((self.streams,), init="ones_normal", keep_stored=True)
        return out

    def load(self, tensors) -> None:
        self.weight = self._take(tensors, "weight").contiguous()
        if "read" in self.tensors:
            self.read = self._take(tensors, "read").to(torch.float32).contiguous()

    def forward(self, x, delta, ctx: StepContext, row_idx=None):
        if delta is not None and not isinstance(delta, ops.StreamWrite):
            raise TypeError("stream_rms_norm adds what a block of several streams leaves "
                            "(ops.StreamWrite), not plain rows")
        return ops.stream_mix_norm(x, delta, self.read, self.weight, self.eps, ctx.act_dtype, row_idx)
