"""Sabipel, plainly: one function per mechanism, float64 on the CPU, token by token where the
design is recurrent.  It shares no code with the library; the tests compare the engine with it.

Notation: h holds a sublayer's input rows [T, E]; a matrix W [out, in] acts on a row as W h, which
for all rows at once is h @ W.T.
"""
from __future__ import annotations

import math

import torch


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def log_sigmoid(x):
    return -softplus(-x)


def silu(x):
    return x * torch.sigmoid(x)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def embed(w, emb, ids):
    """Token row times a scale, plus a row of a hashed table of (previous, current) pairs (its
    last row for a sequence's first token), plus a learned row per position."""
    big = emb["bigram"]
    n, a, b = big["buckets"], big["mul_prev"], big["mul_cur"]
    rows = []
    for p, t in enumerate(ids):
        r = n if p == 0 else (ids[p - 1] * a + t * b) % n
        rows.append(w["embed"][t] * emb["scale"] + w["bigram"][r] + w["pos"][p])
    return torch.stack(rows)


def causal_conv(x, w, b):
    """x [T, C], w [C, taps], b [C]: y[t] = b + sum_j w[:, j] x[t - (taps - 1 - j)], zeros before 0."""
    T, taps = x.shape[0], w.shape[1]
    y = b.expand(T, -1).clone()
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            y[back:] += w[:, j] * x[:T - back]
    return y


def mamba2(h, w, p, m, eps):
    H, dv, N, G, NG = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    T, inner = h.shape[0], H * dv
    u = h @ w[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].view(T, H, dv)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w[p + "dt_bias"])
    rate = torch.exp(w[p + "A_log"])
    S = torch.zeros(H, N, dv, dtype=h.dtype)
    y = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        for hh in range(H):
            g = hh // (H // G)
            S[hh] = torch.exp(-rate[hh] * dt[t, hh]) * S[hh] + dt[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S[hh].T @ C[t, g] + w[p + "D"][hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)
    y = y.view(T, NG, inner // NG)
    y = y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)
    return (y.reshape(T, inner) * w[p + "norm"]) @ w[p + "o"].T


def mlstm(h, w, p, m, eps):
    H, dk, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    T = h.shape[0]
    q = (h @ w[p + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, dk)
    v = (h @ w[p + "v"].T).view(T, H, dv)
    ig = cap * torch.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)
    fg = log_sigmoid(cap * torch.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))
    S = torch.zeros(H, dk, dv, dtype=h.dtype)
    n = torch.zeros(H, dk, dtype=h.dtype)
    mx = torch.zeros(H, dtype=h.dtype)
    o = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        for hh in range(H):
            new = torch.maximum(fg[t, hh] + mx[hh], ig[t, hh])
            keep, take = torch.exp(fg[t, hh] + mx[hh] - new), torch.exp(ig[t, hh] - new)
            S[hh] = keep * S[hh] + take * torch.outer(k[t, hh], v[t, hh])
            n[hh] = keep * n[hh] + take * k[t, hh]
            mx[hh] = new
            o[t, hh] = S[hh].T @ q[t, hh] / (torch.maximum((n[hh] @ q[t, hh]).abs(), torch.exp(-new)) + 1e-6)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps)
    o = o.reshape(T, H * dv) * w[p + "norm"] * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def attention(h, w, p, m, eps, first_values, is_first, edge_shift=0):
    """Returns (output, the values this layer would hand on as the first layer's).  `edge_shift`
    moves every chunk's first visible key by that many positions: what an implementation that is
    off by one at the edge would compute (for tests that show a fault there would be seen)."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T, rep = h.shape[0], m["heads"] // m["kv_heads"]
    q = rms_norm(h @ w[p + "q"].T, w[p + "q.norm"], eps).view(T, H, dk)
    k = rms_norm(h @ w[p + "k"].T, w[p + "k.norm"], eps).view(T, G, dk)
    v = h @ w[p + "v"].T
    handed = v
    if m.get("v_mix") and not is_first:
        lam = w[p + "vmix"]
        v = (1 - lam) * v + lam * first_values
    v = v.view(T, G, dv)
    chunk = (m.get("mask") or {}).get("size")
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    j = torch.arange(T)
    for i in range(T):
        lo = (i // chunk) * chunk if chunk else 0
        lo = min(max(lo + edge_shift, 0), i)
        for hh in range(H):
            slope = 2.0 ** (-8.0 * (hh + 1) / H)
            s = (k[lo:i + 1, hh // rep] @ q[i, hh]) * m["scale"] - slope * (i - j[lo:i + 1])
            out[i, hh] = torch.softmax(s, 0) @ v[lo:i + 1, hh // rep]
    out = out.reshape(T, H * dv) * torch.sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T, handed


def dense(h, w, p):
    return gelu_tanh(h @ w[p + "up"].T) @ w[p + "down"].T


def forward(config, w, ids, layers_out=None, edge_shift=0):
    """float64 logits [T, vocab] of one sequence from its first token on."""
    eps = config["norm"]["eps"]
    x = embed(w, config["embedding"], ids)
    first_values = None
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]
        h = rms_norm(x, w[f"l{i}.norm1"], eps)
        if layer["type"] == "mamba2":
            a = mamba2(h, w, p, m, eps)
        elif layer["type"] == "mlstm":
            a = mlstm(h, w, p, m, eps)
        else:
            is_first = bool(m.get("v_mix")) and first_values is None
            a, handed = attention(h, w, p, m, eps, first_values, is_first, edge_shift)
            if is_first:
                first_values = handed
        if layer.get("mlp") is not None:
            a = a + dense(rms_norm(x, w[f"l{i}.norm2"], eps), w, f"l{i}.mlp.")
        x = x + a
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T


def generate_greedy(config, w, prompt, n_new):
    ids, out = list(prompt), []
    for _ in range(n_new):
        t = int(torch.argmax(forward(config, w, ids)[-1]))
        ids.append(t)
        out.append(t)
    return out
