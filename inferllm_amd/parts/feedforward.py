"""Feed-forward parts."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import TensorWant
from .attention import _fuse
from .base import FeedForward, StepContext, register_part


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """down( silu(h gate^T) * (h up^T) ), gate and up as one fused product.

    src/core/graph.cpp:57-79 (w1 = gate, w3 = up, w2 = down); silu(x) = x / (1 + exp(-x))
    (src/kern/naive/naive.cpp:80-89).  The reference runs silu and the multiply as two
    elementwise kernels (src/kern/gpu/kernel_gpu.cu:183-258).
    """

    graph_safe_prompts = True

    adds_residual = True
    takes_normed_rows = True

    def __init__(self, hidden_size: int, intermediate_size: int, tensors=None):
        super().__init__(tensors)
        self.E, self.F = int(hidden_size), int(intermediate_size)
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def shapes(self) -> Dict[str, TensorWant]:
        return {"gate": TensorWant((self.F, self.E)), "up": TensorWant((self.F, self.E)),
                "down": TensorWant((self.E, self.F))}

    def load(self, tensors) -> None:
        self.w_gate_up = ops.decode_weight(_fuse([self._take(tensors, "gate"), self._take(tensors, "up")]),
                                           "gate_up", self.decode_copies)
        self.w_down = ops.decode_weight(self._take(tensors, "down").contiguous(), "plain",
                                        self.decode_copies)

    def tunables(self):
        return (("gate_up", self.w_gate_up, {}), ("plain", self.w_down, {}))

    def forward(self, h, ctx: StepContext, residual=None, next_norm=None):
        a = ops.gate_up_silu(h, self.w_gate_up)
        if (next_norm is not None and getattr(next_norm, "adds_planes", False)
                and ops.linear_planes_fits(a, self.w_down) and ops.linear_planes_pays(a, self.w_down)):
            return ops.linear_planes(a, self.w_down)
        if residual is not None and ops.linear_add_fits(a, self.w_down, residual):
            return ops.linear_add(a, self.w_down, residual,
                                  next_norm.rms_params() if next_norm is not None else None,
                                  ctx.act_dtype)
        return ops.linear(a, self.w_down)


@register_part("feed_forward", "none")
class NoFeedForward(FeedForward):
    """A layer without a feed-forward: nothing is added (blocks that take None say so)."""

    graph_safe_prompts = True

    def __init__(self, tensors=None):
        super().__init__(tensors)

    def forward(self, h, ctx: StepContext):
        return None


# activation -> the op that computes it
_ACTIVATIONS = {"relu_squared": "relu_squared", "gelu_tanh": "gelu_tanh"}


@register_part("feed_forward", "dense_activation")
class DenseActivation(FeedForward):
    """down(act(up h)) without a gate; `activation` "relu_squared": max(z, 0)^2, or "gelu_tanh":
    0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))."""

    graph_safe_prompts = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "relu_squared",
                 tensors=None):
        super().__init__(tensors)
        if activation not in _ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {sorted(_ACTIVATIONS)}")
        self.E, self.F, self.activation = int(hidden_size), int(intermediate_size), activation
        self.w_up = self.w_down = None

    def shapes(self) -> Dict[str, TensorWant]:
        return {"up": TensorWant((self.F, self.E)), "down": TensorWant((self.E, self.F))}

    def load(self, tensors) -> None:
        self.w_up = ops.decode_weight(self._take(tensors, "up").contiguous(), "plain", self.decode_copies)
        self.w_down = ops.decode_weight(self._take(tensors, "down").contiguous(), "plain", self.decode_copies)

    def tunables(self):
        return (("plain", self.w_down, {}),)

    def forward(self, h, ctx: StepContext):
        act = getattr(ops, _ACTIVATIONS[self.activation])
        return ops.linear(act(ops.linear(h, self.w_up)), self.w_down)


@register_part("feed_forward", "clamped_gated")
class ClampedGated(FeedForward):
    """down(g sigmoid(1.702 g) (u + 1)) with g = min(gate h, limit) and u = clamp(up h, -limit, limit):
    the clamped activation of the routed experts as a dense feed-forward; gate and up are one
    fused product, which in steps of few bfloat16 rows also applies the activation."""

    graph_safe_prompts = True

    def __init__(self, hidden_size: int, intermediate_size: int, limit: float, tensors=None):
        super().__init__(tensors)
        if not float(limit) > 0:
            raise ValueError("clamped gated feed-forward: the limit must be positive")
        self.E, self.F, self.limit = int(hidden_size), int(intermediate_size), float(limit)
        self.w_gate_up = self.w_down = None

    def shapes(self) -> Dict[str, TensorWant]:
        return {"gate": TensorWant((self.F, self.E)), "up": TensorWant((self.F, self.E)),
                "down": TensorWant((self.E, self.F))}

    def load(self, tensors) -> None:
        self.w_gate_up = ops.decode_weight(_fuse([self._take(tensors, "gate"), self._take(tensors, "up")]),
                                           "gate_up", self.decode_copies)
        self.w_down = ops.decode_weight(self._take(tensors, "down").contiguous(), "plain", self.decode_copies)

    def tunables(self):
        return (("gate_up", self.w_gate_up, {}), ("plain", self.w_down, {}))

    def forward(self, h, ctx: StepContext):
        return ops.linear(ops.gate_up_act(h, self.w_gate_up, self.limit), self.w_down)


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    """A mixture of gated experts, of which every token uses `top`.

        s = softmax(W_router h) over `num_experts` real experts followed by `num_identity`
            identity experts (float32)
        chosen = the `top` largest of s (+ `correction`, a stored vector that moves the choice
                 and not the weights)
        out = sum over chosen e of s_e * (expert_e(h) if e is real, else h)
              (+ sigmoid(w_sg . h) * shared(h))
        expert(h) = W_down (silu(W_gate h) * (W_up h))

    The weights are the chosen scores as they are (no renormalisation).  `shared_size` > 0 adds
    an expert that every token uses, scaled per token by a sigmoid gate if `shared_gate`.
    `score` "sigmoid" scores every router output by its own sigmoid instead of the softmax over
    all.  `activation` "clamped_swish" with `limit`: g = min(W_gate h, limit), u = clamp(W_up h,
    -limit, limit), expert(h) = W_down (g sigmoid(1.702 g) (u + 1)).  `weight_on` "input": the
    weight multiplies what the expert reads, out = sum over chosen e of expert_e(s_e h).
    Tensor parameters: "router", "correction", "e<i>.gate" / ".up" / ".down", "shared.gate" /
    ".up" / ".down", "shared.sg".  The result is float32.
    """

    graph_safe_prompts = True

    def __init__(self, hidden_size: int, expert_size: int, num_experts: int, top: int,
                 num_identity: int = 0, correction: bool = True, shared_size: int = 0,
                 shared_gate: bool = True, score: str = "softmax", activation: str = "silu",
                 limit: float = 0.0, weight_on: str = "output", tensors=None):
        super().__init__(tensors)
        if score not in ops.MOE_SCORES or activation not in ops.MOE_ACTIVATIONS:
            raise ValueError(f"routed experts: score {score!r} or activation {activation!r} is unknown; "
                             f"known: {sorted(ops.MOE_SCORES)}, {sorted(ops.MOE_ACTIVATIONS)}")
        if weight_on not in ("output", "input"):
            raise ValueError(f"routed experts: weight_on {weight_on!r} is neither 'output' nor 'input'")
        if activation == "clamped_swish" and not float(limit) > 0:
            raise ValueError("routed experts: the clamped activation needs a positive limit")
        if weight_on == "input" and int(num_identity):
            raise ValueError("routed experts: identity experts take their weight on the output")
        self.score, self.activation, self.limit, self.weight_on = score, activation, float(limit), weight_on
        self.E, self.F = int(hidden_size), int(expert_size)
        self.n_real, self.n_id, self.top = int(num_experts), int(num_identity), int(top)
        self.has_correction, self.Fs = bool(correction), int(shared_size)
        self.has_shared_gate = bool(shared_gate) and self.Fs > 0
        n_all = self.n_real + self.n_id
        if self.n_real < 0 or self.n_id < 0 or n_all <= 0 or not 0 < self.top <= n_all:
            raise ValueError(f"routed experts: {self.top} of {self.n_real} + {self.n_id} cannot be chosen")
        if n_all > 512:
            raise ValueError("routed experts: more than 512 router outputs are beyond the kernels")
        if self.n_real and self.F <= 0:
            raise ValueError("routed experts: the experts need a size")
        self.w_router = self.correction = self.w_gate_up = self.w_down = None
        self.w_shared_gate_up = self.w_shared_down = self.w_sg = None

    def shapes(self) -> Dict[str, TensorWant]:
        out = {"router": TensorWant((self.n_real + self.n_id, self.E))}
        if self.has_correction:
            out["correction"] = TensorWant((self.n_real + self.n_id,), keep_stored=True)
        for i in range(self.n_real):
            out[f"e{i}.gate"] = TensorWant((self.F, self.E))
            out[f"e{i}.up"] = TensorWant((self.F, self.E))
            out[f"e{i}.down"] = TensorWant((self.E, self.F))
        if self.Fs:
            out["shared.gate"] = TensorWant((self.Fs, self.E))
            out["shared.up"] = TensorWant((self.Fs, self.E))
            out["shared.down"] = TensorWant((self.E, self.Fs))
            if self.has_shared_gate:
                out["shared.sg"] = TensorWant((1, self.E))
        return out

    def load(self, tensors) -> None:
        take = lambda n: self._take(tensors, n)
        self.w_router = take("router").to(torch.float32).contiguous()      # the router runs in float32
        self.correction = take("correction").contiguous() if self.has_correction else None
        if self.n_real:
            self.w_gate_up = torch.stack([torch.cat([take(f"e{i}.gate"), take(f"e{i}.up")], dim=0)
                                          for i in range(self.n_real)]).contiguous()
            self.w_down = torch.stack([take(f"e{i}.down") for i in range(self.n_real)]).contiguous()
        if self.Fs:
            self.w_shared_gate_up = ops.decode_weight(_fuse([take("shared.gate"), take("shared.up")]),
                                                      "gate_up", self.decode_copies)
            self.w_shared_down = ops.decode_weight(take("shared.down").contiguous(), "plain",
                                                   self.decode_copies)
            if self.has_shared_gate:
                self.w_sg = take("shared.sg").reshape(-1).contiguous()

    def forward(self, h, ctx: StepContext):
        idx, weight, grouped = ops.moe_plan(h, self.w_router, self.correction, self.top,
                                            self.w_gate_up, self.score)
        on_input = self.weight_on == "input"
        y = (ops.moe_experts(h, idx, self.w_gate_up, self.w_down, grouped, self.activation, self.limit,
                             weight if on_input else None) if self.n_real else None)
        if on_input:
            weight = None                        # the experts' rows are summed as they are
        shared = None
        if self.Fs:
            shared = ops.linear(ops.gate_up_silu(h, self.w_shared_gate_up), self.w_shared_down)
        return ops.moe_combine(h, idx, weight, y, self.n_real, shared, self.w_sg)
