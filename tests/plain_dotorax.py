"""Dotorax, plainly: one function per mechanism, float64 on the CPU, token by token where the
design is recurrent.  It shares no code with the library; the tests compare the engine with it.

Notation: h holds a sublayer's input rows [T, E]; a matrix W [out, in] acts on a row as W h, which
for all rows at once is h @ W.T.  Positions count from 0.
"""
from __future__ import annotations

import math

import torch


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight lies around zero: the gain is 1 + w."""
    return unit_rms(x, eps) * (1 + w)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def silu(x):
    return x * torch.sigmoid(x)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def causal_conv(x, w, b=None):
    """x [T, C], w [C, taps]: y[t] = sum_j w[:, j] x[t - (taps - 1 - j)] (+ b), zeros before 0."""
    T, taps = x.shape[0], w.shape[1]
    y = torch.zeros_like(x) if b is None else b.expand(T, -1).clone()
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            y[back:] += w[:, j] * x[:T - back]
    return y


def input_conv(h, w):
    """What a sublayer reads: its normed rows plus their short causal convolution."""
    return h + causal_conv(h, w)


def rotate(x, base, dims, layout, first_pos=0):
    """x [T, heads, d]: the first `dims` of every head turned by position; "half" pairs i with
    i + dims / 2, "interleaved" pairs 2i with 2i + 1."""
    T = x.shape[0]
    half = dims // 2
    f = torch.tensor(base, dtype=torch.float64) ** (-2.0 * torch.arange(half, dtype=torch.float64) / dims)
    a = (torch.arange(T, dtype=torch.float64) + first_pos)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :].to(x.dtype), torch.sin(a)[:, None, :].to(x.dtype)
    out = x.clone()
    if layout == "half":
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half], out[..., half:dims] = u * c - v * s, v * c + u * s
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2], out[..., 1:dims:2] = u * c - v * s, v * c + u * s
    return out


def softmax_attention(q, k, v, scale, visible, pooled=None):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv]; scale a number or one per head [H];
    visible [T, T] bool.  `pooled` = (keys [B, G, dk], values [B, G, dv], seen [T, B] bool):
    further keys that share the softmax.  Returns [T, H, dv]."""
    T, H, _ = q.shape
    rep = H // k.shape[1]
    scale = torch.as_tensor(scale, dtype=q.dtype).expand(H)
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for hh in range(H):
        g = hh // rep
        s = (q[:, hh] @ k[:, g].T) * scale[hh]
        s = s.masked_fill(~visible, float("-inf"))
        vals = v[:, g]
        if pooled is not None and pooled[0].shape[0]:
            pk, pv, seen = pooled
            sp = ((q[:, hh] @ pk[:, g].T) * scale[hh]).masked_fill(~seen, float("-inf"))
            s, vals = torch.cat([s, sp], 1), torch.cat([vals, pv[:, g]], 0)
        out[:, hh] = torch.softmax(s, 1) @ vals
    return out


def attention(h, w, p, m, shared=None):
    """Causal attention with rotated q and k and one sigmoid gate a head.  `shared` = (k, v) of the
    layer whose keys and values this one reads.  Returns (output, (k, v))."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    rot = m["rot"]
    q = rotate((h @ w[p + "q"].T).view(T, H, dk), rot["base"], rot["dims"], "half")
    if shared is None:
        k = rotate((h @ w[p + "k"].T).view(T, G, dk), rot["base"], rot["dims"], "half")
        v = (h @ w[p + "v"].T).view(T, G, dv)
    else:
        k, v = shared
    i = torch.arange(T)
    o = softmax_attention(q, k, v, m["scale"], i[None, :] <= i[:, None])
    o = o * torch.sigmoid(h @ w[p + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ w[p + "o"].T, (k, v)


def pooled_window_attention(h, w, p, m, eps, edge_shift=0, pool_shift=0):
    """Attention over the last `size` tokens and, before them, one mean key and value for every
    block of `pool` tokens that lies wholly before the window.  `edge_shift` and `pool_shift` move
    the window's far edge and the blocks' condition by that many positions: what an implementation
    that is off by one there would compute."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T, rot, size, P = h.shape[0], m["rot"], m["mask"]["size"], m["mask"]["pool"]
    q = unit_rms(rotate((h @ w[p + "q"].T).view(T, H, dk), rot["base"], rot["dims"], "interleaved"), eps)
    k = unit_rms(rotate((h @ w[p + "k"].T).view(T, G, dk), rot["base"], rot["dims"], "interleaved"), eps)
    v = (h @ w[p + "v"].T).view(T, G, dv)
    i = torch.arange(T)
    dist = i[:, None] - i[None, :]
    visible = (dist >= 0) & (dist < size + edge_shift)
    B = T // P
    pk = k[:B * P].view(B, P, G, dk).mean(1)
    pv = v[:B * P].view(B, P, G, dv).mean(1)
    last = torch.arange(B) * P + P - 1
    seen = last[None, :] <= (i[:, None] - size + pool_shift)
    o = softmax_attention(q, k, v, m["scale"] * w[p + "temp"], visible, (pk, pv, seen))
    return o.reshape(T, H * dv) @ w[p + "o"].T


def gated_recurrent_unit(h, w, p, m):
    """Two branches: y = gelu(W_y h + b), u = conv(W_x h + b); per channel a state
    S <- a S + sqrt(1 - a^2) (i u) with a = exp(-8 r softplus(lam)), r and i sigmoids of
    block-diagonal maps of u; output W_o (S y)."""
    T, C, nb = h.shape[0], m["width"], m["blocks"]
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = causal_conv(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"], w[p + "conv.b"])
    ub = u.view(T, nb, C // nb)
    r = torch.sigmoid(torch.einsum("boi,tbi->tbo", w[p + "ra"], ub) + w[p + "ra.b"]).reshape(T, C)
    i = torch.sigmoid(torch.einsum("boi,tbi->tbo", w[p + "ri"], ub) + w[p + "ri.b"]).reshape(T, C)
    log_a = -8.0 * r * softplus(w[p + "lam"])
    a = torch.exp(log_a)
    S = torch.zeros(C, dtype=h.dtype)
    out = torch.zeros(T, C, dtype=h.dtype)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1 - a[t] * a[t]) * (i[t] * u[t])
        out[t] = S
    return (out * y) @ w[p + "o"].T


def gated_linear_attention(h, w, p, m, eps):
    """Per head a matrix S <- diag(alpha) S + k v^T with a decay per key channel,
    alpha = sigmoid(W_a2 W_a1 h + b)^(1 / tau); o = S^T q; norm over a head's values, silu gate."""
    H, dk, dv, tau = m["heads"], m["dim"], m["vdim"], m["tau"]
    T = h.shape[0]
    q = (h @ w[p + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, dk)
    v = (h @ w[p + "v"].T).view(T, H, dv)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = torch.exp(-softplus(-z) / tau).view(T, H, dk)
    S = torch.zeros(H, dk, dv, dtype=h.dtype)
    o = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = unit_rms(o, eps) * w[p + "norm"]
    return (o.reshape(T, H * dv) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def clamped_feed_forward(h, w, p, limit):
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w[p + "down"].T


def forward(config, w, ids, layers_out=None, edge_shift=0, pool_shift=0):
    """float64 logits [T, vocab] of one sequence from its first token on."""
    eps, mult = config["norm"]["eps"], config["residual_mult"]
    ids = torch.as_tensor(ids, dtype=torch.long)
    x = w["embed"][ids] + w["pos"][: len(ids)]
    kept = {}
    for i, layer in enumerate(config["layers"]):
        L, p, m = f"l{i}.", f"l{i}.mix.", layer["mixer"]
        h = input_conv(offset_norm(x, w[L + "norm1"], eps), w[L + "canon1"])
        if layer["type"] == "attention":
            a, kept[i] = attention(h, w, p, m, kept[m["kv_from"]] if "kv_from" in m else None)
        elif layer["type"] == "parallel":
            a = (m["left_scale"] * pooled_window_attention(h, w, p + "left.", m["left"], eps, edge_shift, pool_shift)
                 + m["right_scale"] * gated_recurrent_unit(h, w, p + "right.", m["right"]))
        elif layer["type"] == "gla":
            a = gated_linear_attention(h, w, p, m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + mult * offset_norm(a, w[L + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = input_conv(offset_norm(x, w[L + "norm2"], eps), w[L + "canon2"])
            x = x + mult * offset_norm(clamped_feed_forward(h, w, L + "mlp.", mlp["limit"]), w[L + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return offset_norm(x, w["final.norm"], eps) @ w["head"].T


def generate_greedy(config, w, prompt, n_new):
    ids, out = list(prompt), []
    for _ in range(n_new):
        t = int(torch.argmax(forward(config, w, ids)[-1]))
        ids.append(t)
        out.append(t)
    return out
