"""Mixers that keep a matrix of state per head and update it by the plain gated rule
S <- g S + k (w v)^T, o = S^T q: a state-space mixer with a scalar decay a head, and a matrix
memory with exponential gates; gated linear attention, which is that rule with a decay per key
channel; and a gated linear recurrent unit, whose state is one number a channel."""
from __future__ import annotations

from typing import Dict

import torch

from ..cache.manager import StateSpec
from ..kernels import ops
from ..weights.loader import TensorWant
from .attention import _fuse
from .base import Mixer, StepContext, register_part


@register_part("mixer", "state_space_duality")
class StateSpaceDuality(Mixer):
    """A selective state-space mixer with one decay a head.  The input projection gives, side by
    side, [z: H dv | x: H dv | B: G N | C: G N | dt: H].  x, B and C pass a short causal
    convolution per channel (`conv` taps with a bias, the last tap on the token itself, zeros ahead
    of the sequence) and SiLU.  With step = softplus(dt + dt_bias), per head h of group
    h / (H / G):

        S <- exp(-exp(A_log[h]) step) S + step B x^T      (S is N x dv)
        y = S^T C + D[h] x

    y (heads side by side) times silu(z), then an RMS norm in `norm_groups` equal parts of the row
    (each by its own root mean square, `eps`), times `norm`, then the output projection.

    Kept per sequence: S (float32) and the convolution's last conv - 1 inputs.  A step goes on from
    whatever the slot holds, by one token or by many.  Everything that enters the recurrence is
    float32; the projections take the engine's dtype.
    """

    graph_safe_prompts = True
    takes_continuations = True

    def __init__(self, hidden_size: int, num_heads: int, groups: int, state_size: int, value_dim: int,
                 conv: int, norm_groups: int, eps: float, tensors=None):
        super().__init__(tensors)
        if num_heads % groups:
            raise ValueError(f"{num_heads} heads are not a multiple of {groups} groups")
        if not 1 <= int(conv) <= 8:
            raise ValueError(f"state-space mixer: {conv} taps; the kernels take 1 to 8")
        if state_size > 256:
            raise ValueError(f"state-space mixer: a state of {state_size} rows is beyond the kernels' limit of 256")
        if (num_heads * value_dim) % norm_groups:
            raise ValueError(f"{num_heads * value_dim} columns do not split into {norm_groups} equal parts")
        self.E, self.H, self.G = int(hidden_size), int(num_heads), int(groups)
        self.N, self.dv, self.taps = int(state_size), int(value_dim), int(conv)
        self.norm_groups, self.eps = int(norm_groups), float(eps)
        self.inner = self.H * self.dv
        self.C = self.inner + 2 * self.G * self.N                # channels of the convolution

    def shapes(self) -> Dict[str, TensorWant]:
        keep = dict(keep_stored=True)
        return {"in": TensorWant((2 * self.inner + 2 * self.G * self.N + self.H, self.E)),
                "conv": TensorWant((self.C, self.taps), **keep), "conv_bias": TensorWant((self.C,), **keep),
                "dt_bias": TensorWant((self.H,), **keep), "A_log": TensorWant((self.H,), **keep),
                "D": TensorWant((self.H,), init="ones_normal", **keep),
                "norm": TensorWant((self.inner,), init="ones_normal", **keep),
                "o": TensorWant((self.E, self.inner))}

    def state_spec(self):
        return {"S": StateSpec((self.H, self.N, self.dv), torch.float32),
                "tail": StateSpec((max(self.taps - 1, 1), self.C), None)}

    def load(self, tensors) -> None:
        take = lambda n: self._take(tensors, n)
        f32 = lambda n: take(n).to(torch.float32).contiguous()
        self.w_in = ops.decode_weight(take("in").contiguous(), "plain", self.decode_copies)
        self.w_o = ops.decode_weight(take("o").contiguous(), "plain", self.decode_copies)
        self.conv_w, self.conv_b = f32("conv"), f32("conv_bias")
        self.dt_bias, self.a_log, self.D = f32("dt_bias"), f32("A_log"), f32("D")
        self.norm_w = take("norm").contiguous()

    def tunables(self):
        return (("plain", self.w_o, {}),)

    def forward(self, h, ctx: StepContext, line, writes_cache, position):
        U = ops.linear(h, self.w_in)
        state = ctx.cache.state_line(line)
        S, tail = state["S"], state["tail"]
        qn, kn, vv, step, dec = ops.ssm_prepare(
            U, self.inner, 2 * self.inner + 2 * self.G * self.N, self.conv_w, self.conv_b, tail,
            ctx.row_slot, self.a_log, self.dt_bias, self.G, self.H, self.N, self.dv,
            update_tail=not ctx.prefill)
        if ctx.prefill:
            ops.delta_conv_tail(U, tail, ctx.cu_seqlens, ctx.seq_slot, ctx.n_seqs, self.taps,
                                col_off=self.inner)
        o = ops.delta_scan(qn, kn, vv, step, dec, S, ctx.cu_seqlens, ctx.seq_slot, ctx.n_seqs,
                           ctx.max_rows if ctx.prefill else 1, correct=False)
        y = ops.ssm_finish(o, vv, self.D, U, 0, self.norm_w, self.norm_groups, self.eps, ctx.act_dtype)
        return ops.linear(y, self.w_o)


@register_part("mixer", "matrix_memory")
class MatrixMemory(Mixer):
    """A matrix memory with exponential gates (the mLSTM cell).  q = W_q h dk^-1/2, k = W_k h, v = W_v h
    per head; per head a log input gate i = cap tanh((W_i h + b_i) / cap) and a log forget gate
    f = logsigmoid(cap tanh((W_f h + b_f) / cap)).  With a running maximum m that starts at 0:

        m_t = max(f + m_(t-1), i)
        S <- exp(f + m_(t-1) - m_t) S + exp(i - m_t) k v^T,   n likewise with k alone
        o = S^T q / (max(|n . q|, exp(-m_t)) + 1e-6)

    Each head's o is divided by its root mean square (`eps`); the heads side by side times `norm`
    (all heads' width), times sigmoid(W_g h), then the output projection.

    Kept per sequence, float32: S with n as one more column ([H, dk, dv + 1]) and m [H].  A step
    goes on from whatever the slot holds.  Gates, maxima, decays and the state are float32; the
    projections take the engine's dtype.
    """

    graph_safe_prompts = True
    takes_continuations = True

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, gate_cap: float,
                 eps: float, tensors=None):
        super().__init__(tensors)
        if key_dim > 256:
            raise ValueError(f"matrix memory: a key size of {key_dim} is beyond the kernels' limit of 256")
        if not float(gate_cap) > 0:
            raise ValueError(f"matrix memory: the gates' cap must be positive, got {gate_cap!r}")
        self.E, self.H, self.dk, self.dv = int(hidden_size), int(num_heads), int(key_dim), int(value_dim)
        self.cap, self.eps = float(gate_cap), float(eps)

    def shapes(self) -> Dict[str, TensorWant]:
        E, H, dk, dv = self.E, self.H, self.dk, self.dv
        keep = dict(keep_stored=True)
        return {"q": TensorWant((H * dk, E)), "k": TensorWant((H * dk, E)), "v": TensorWant((H * dv, E)),
                "g": TensorWant((H * dv, E)), "i": TensorWant((H, E)), "f": TensorWant((H, E)),
                "i_bias": TensorWant((H,), **keep), "f_bias": TensorWant((H,), **keep),
                "norm": TensorWant((H * dv,), init="ones_normal", **keep), "o": TensorWant((E, H * dv))}

    def state_spec(self):
        return {"S": StateSpec((self.H, self.dk, self.dv + 1), torch.float32),
                "m": StateSpec((self.H,), torch.float32)}

    def load(self, tensors) -> None:
        take = lambda n: self._take(tensors, n)
        H, dk, dv = self.H, self.dk, self.dv
        # one product for everything that reads h: [q | k | v | i | f | g]
        self.w_in = ops.decode_weight(_fuse([take(n) for n in ("q", "k", "v", "i", "f", "g")]), "plain",
                                      self.decode_copies)
        self.i_off = 2 * H * dk + H * dv
        self.f_off, self.z_off = self.i_off + H, self.i_off + 2 * H
        self.i_bias = take("i_bias").to(torch.float32).contiguous()
        self.f_bias = take("f_bias").to(torch.float32).contiguous()
        self.norm_w = take("norm").contiguous()
        self.w_o = ops.decode_weight(take("o").contiguous(), "plain", self.decode_copies)

    def tunables(self):
        return (("plain", self.w_o, {}),)

    def forward(self, h, ctx: StepContext, line, writes_cache, position):
        U = ops.linear(h, self.w_in)
        state = ctx.cache.state_line(line)
        qn, kn, vv, weight, dec, em = ops.memory_prepare(
            U, self.i_off, self.f_off, self.i_bias, self.f_bias, self.cap, state["m"], ctx.cu_seqlens,
            ctx.seq_slot, ctx.n_seqs, self.H, self.dk, self.dv)
        o = ops.delta_scan(qn, kn, vv, weight, dec, state["S"], ctx.cu_seqlens, ctx.seq_slot, ctx.n_seqs,
                           ctx.max_rows if ctx.prefill else 1, correct=False)
        y = ops.memory_finish(o, em, self.norm_w, U, self.z_off, self.eps, ctx.act_dtype)
        return ops.linear(y, self.w_o)


@register_part("mixer", "gated_linear_attention")
class GatedLinearAttention(Mixer):
    """Per head a matrix of state S [key_dim, value_dim] with a decay per key channel:

        q = W_q h key_dim^-1/2,  k = W_k h,  v = W_v h
        alpha = sigmoid(W_a2 (W_a1 h) + b)^(1 / tau)             one a head and key channel
        S <- diag(alpha) S + k v^T;   o = S^T q
        out = W_o (o / rms(o) * norm * silu(W_g h))

    rms over a head's value dims with `eps`; `norm` [value_dim] is shared by the heads.  Kept per
    sequence: S (float32).  A step goes on from whatever the slot holds.  Decays, their logarithms
    and the state are float32; the projections take the engine's dtype.
    """

    graph_safe_prompts = True
    takes_continuations = True

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, decay_rank: int,
                 tau: float, eps: float, tensors=None):
        super().__init__(tensors)
        if key_dim > 256 or value_dim > 256:
            raise ValueError(f"gated linear attention: head sizes {key_dim}, {value_dim} are beyond the kernels' limit of 256")
        if not float(tau) > 0 or int(decay_rank) <= 0:
            raise ValueError("gated linear attention: tau and the decays' rank must be positive")
        self.E, self.H, self.dk, self.dv = int(hidden_size), int(num_heads), int(key_dim), int(value_dim)
        self.ra, self.tau, self.eps = int(decay_rank), float(tau), float(eps)

    def shapes(self) -> Dict[str, TensorWant]:
        E, H, dk, dv = self.E, self.H, self.dk, self.dv
        keep = dict(keep_stored=True)
        return {"q": TensorWant((H * dk, E)), "k": TensorWant((H * dk, E)), "v": TensorWant((H * dv, E)),
                "g": TensorWant((H * dv, E)), "a1": TensorWant((self.ra, E)), "a2": TensorWant((H * dk, self.ra)),
                "a2_bias": TensorWant((H * dk,), **keep), "norm": TensorWant((dv,), init="ones_normal", **keep),
                "o": TensorWant((E, H * dv))}

    def state_spec(self):
        return {"S": StateSpec((self.H, self.dk, self.dv), torch.float32)}

    def load(self, tensors) -> None:
        take = lambda n: self._take(tensors, n)
        H, dk, dv = self.H, self.dk, self.dv
        # one product for everything that reads h: [q | k | v | g | a1]
        self.w_in = ops.decode_weight(_fuse([take(n) for n in ("q", "k", "v", "g", "a1")]), "plain",
                                      self.decode_copies)
        self.g_off = 2 * H * dk + H * dv
        self.a_off = self.g_off + H * dv
        self.w_a2 = ops.decode_weight(take("a2").contiguous(), "plain", self.decode_copies)
        self.a2_bias = take("a2_bias").to(torch.float32).contiguous()
        self.norm_w = take("norm").contiguous()
        self.w_o = ops.decode_weight(take("o").contiguous(), "plain", self.decode_copies)

    def tunables(self):
        return (("plain", self.w_o, {}),)

    def forward(self, h, ctx: StepContext, line, writes_cache, position):
        H, dk, dv = self.H, self.dk, self.dv
        U = ops.linear(h, self.w_in)
        Z = ops.linear(U[:, self.a_off:].contiguous(), self.w_a2)
        qn, kn, vv, weight, dec = ops.gla_prepare(U, 0, H * dk, 2 * H * dk, Z, self.a2_bias, self.tau, H, dk, dv)
        S = ctx.cache.state_line(line)["S"]
        o = ops.delta_scan(qn, kn, vv, weight, dec, S, ctx.cu_seqlens, ctx.seq_slot, ctx.n_seqs,
                           ctx.max_rows if ctx.prefill else 1, correct=False)
        y = ops.delta_finish(o, self.norm_w, U, self.g_off, "silu", self.eps, ctx.act_dtype)
        return ops.linear(y, self.w_o)


# a = exp(-rate r softplus(lam)): the unit fixes the rate
LRU_RATE = 8.0


@register_part("mixer", "gated_linear_recurrence")
class GatedLinearRecurrence(Mixer):
    """A recurrent block with a real-gated linear recurrent unit.  Two branches `channels` wide:

        y = gelu_tanh(W_y h + b_y)
        u = conv(W_x h + b_x)           a short causal convolution per channel, `conv` taps with a bias,
                                        the last tap on the token itself, zeros ahead of the sequence
        r = sigmoid(R_b u_b + b_r),  i = sigmoid(I_b u_b + b_i)      in `blocks` equal parts b of the
                                        channels, R_b and I_b square [out, in]
        a = exp(-8 r softplus(lam)),   S <- a S + sqrt(1 - a^2) (i u)      from S = 0, one number a channel
        out = W_o (S y)

    Kept per sequence: S (float32) and the convolution's last conv - 1 inputs.  A step goes on from
    whatever the slot holds.  Gates, decays and the state are float32; the projections take the
    engine's dtype.
    """

    graph_safe_prompts = True
    takes_continuations = True

    def __init__(self, hidden_size: int, channels: int, blocks: int, conv: int, tensors=None):
        super().__init__(tensors)
        if int(channels) % int(blocks):
            raise ValueError(f"gated linear recurrence: {channels} channels do not split into {blocks} equal blocks")
        if not 1 <= int(conv) <= 8:
            raise ValueError(f"gated linear recurrence: {conv} taps; the kernels take 1 to 8")
        if int(channels) // int(blocks) > 4096:
            raise ValueError("gated linear recurrence: blocks of more than 4096 channels are beyond the gates' kernel")
        self.E, self.C, self.nb, self.taps = int(hidden_size), int(channels), int(blocks), int(conv)

    def shapes(self) -> Dict[str, TensorWant]:
        E, C, nb = self.E, self.C, self.nb
        cb = C // nb
        keep = dict(keep_stored=True)
        return {"y": TensorWant((C, E)), "y_bias": TensorWant((C,), **keep), "x": TensorWant((C, E)),
                "x_bias": TensorWant((C,), **keep), "conv": TensorWant((C, self.taps), **keep),
                "conv_bias": TensorWant((C,), **keep), "ra": TensorWant((nb, cb, cb), **keep),
                "ra_bias": TensorWant((nb, cb), **keep), "ri": TensorWant((nb, cb, cb), **keep),
                "ri_bias": TensorWant((nb, cb), **keep), "lam": TensorWant((C,), **keep),
                "o": TensorWant((E, C))}

    def state_spec(self):
        return {"S": StateSpec((self.C,), torch.float32),
                "tail": StateSpec((max(self.taps - 1, 1), self.C), None)}

    def load(self, tensors) -> None:
        take = lambda n: self._take(tensors, n)
        f32 = lambda n: take(n).to(torch.float32).contiguous()
        self.w_in = ops.decode_weight(_fuse([take("y"), take("x")]), "plain", self.decode_copies)   # [y | x]
        self.y_bias, self.x_bias = f32("y_bias"), f32("x_bias")
        self.conv_w, self.conv_b = f32("conv"), f32("conv_bias")
        # the gates' maps transposed ([in, out] per block), so that neighbouring threads read
        # neighbouring outputs
        self.w_gates = torch.stack([f32("ra").transpose(1, 2), f32("ri").transpose(1, 2)]).contiguous()
        self.r_bias, self.i_bias = f32("ra_bias").reshape(-1), f32("ri_bias").reshape(-1)
        self.lam = f32("lam")
        self.w_o = ops.decode_weight(take("o").contiguous(), "plain", self.decode_copies)

    def tunables(self):
        return (("plain", self.w_o, {}),)

    def forward(self, h, ctx: StepContext, line, writes_cache, position):
        C = self.C
        U = ops.linear(h, self.w_in)
        state = ctx.cache.state_line(line)
        S, tail = state["S"], state["tail"]
        u = ops.short_conv(U, C, C, self.conv_w, tail, ctx.row_slot, torch.float32, bias=self.conv_b,
                           in_bias=self.x_bias, update_tail=not ctx.prefill)
        if ctx.prefill:
            ops.short_conv_tail(U, C, tail, ctx.cu_seqlens, ctx.seq_slot, ctx.n_seqs, self.taps,
                                in_bias=self.x_bias)
        a, x = ops.lru_gates(u, self.w_gates, self.r_bias, self.i_bias, self.lam, LRU_RATE)
        y = ops.lru_scan(a, x, S, U, 0, self.y_bias, ctx.cu_seqlens, ctx.seq_slot, ctx.n_seqs,
                         ctx.max_rows if ctx.prefill else 1, ctx.act_dtype)
        return ops.linear(y, self.w_o)
