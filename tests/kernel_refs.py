"""Plain torch versions of every kernel's contract (float64 inside).

Two uses: the expected side of each kernel's own test on the GPU, and, patched
over `inferllm_amd.kernels.ops` on the CPU, a stand-in that lets the step
function, the cache and the generation loop run without a GPU so that their
bookkeeping is tested where there is none.  They share no code with the kernels.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

F64 = torch.float64


def embed(tokens, table, scale=1.0, copies=0):
    rows = _embed_rows(tokens, table, scale)
    return rows[:, None, :].repeat(1, copies, 1).contiguous() if copies else rows


def _embed_rows(tokens, table, scale=1.0):
    return table[tokens.long()].to(torch.float32) * scale


def add_rmsnorm(x, delta, weight, eps, out_dtype, row_idx=None, weight2=None):
    if weight2 is not None:
        first = add_rmsnorm(x, delta, weight, eps, out_dtype, row_idx)
        return first, add_rmsnorm(x, None, weight2, eps, out_dtype, row_idx)
    if isinstance(delta, (tuple, list)):               # two parts' outputs for the same rows
        delta = delta[0].to(F64) + delta[1].to(F64)
    if delta is not None:
        if delta.dim() == 3:                           # planes of a split product
            delta = delta.to(F64).sum(0)
        s = (x.to(F64) + delta.to(F64)).to(torch.float32)
        if row_idx is None:
            x.copy_(s)
    else:
        s = x
    if row_idx is not None:
        s = s[row_idx.long()]
    v = s.to(F64)
    scale = 1.0 / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)
    return ((v * scale) * weight.to(F64)).to(out_dtype)


def silu_mul(gate_up):
    F = gate_up.shape[1] // 2
    g, u = gate_up[:, :F].to(F64), gate_up[:, F:].to(F64)
    return (g / (1.0 + torch.exp(-g)) * u).to(gate_up.dtype)


def cache_offsets(page_table, slot, pos, page_size, ring):
    lp = pos // page_size
    if ring > 0:
        lp = lp % ring
    return int(page_table[slot, lp]), pos % page_size


def rope_store(qkv, cos_sin, rot, pairing, row_pos, row_slot, slot_len, kcache, vcache,
               page_table, page_size, ring, nh, nkv, hd):
    T = qkv.shape[0]
    view = qkv.view(T, nh + 2 * nkv, hd)
    if cos_sin is not None:
        heads = view[:, : nh + nkv, :].to(F64)
        cs = cos_sin[row_pos.long()].to(F64)          # [T, rot/2, 2]
        c, s = cs[:, None, :, 0], cs[:, None, :, 1]
        half = rot // 2
        if pairing == 0:
            a = heads[:, :, :half].clone()
            b = heads[:, :, hd // 2: hd // 2 + half].clone()
            heads[:, :, :half] = a * c - b * s
            heads[:, :, hd // 2: hd // 2 + half] = a * s + b * c
        else:
            a = heads[:, :, 0:rot:2].clone()
            b = heads[:, :, 1:rot:2].clone()
            heads[:, :, 0:rot:2] = a * c - b * s
            heads[:, :, 1:rot:2] = a * s + b * c
        view[:, : nh + nkv, :] = heads.to(qkv.dtype)
    if kcache is None:
        return
    for t in range(T):
        slot, pos = int(row_slot[t]), int(row_pos[t])
        if ring > 0 and slot_len is not None:
            last_page = (int(slot_len[slot]) - 1) // page_size
            if pos // page_size + ring <= last_page:
                continue
        page, r = cache_offsets(page_table, slot, pos, page_size, ring)
        kcache[page, :, r, :] = view[t, nh: nh + nkv, :]
        vcache[page, :, r, :] = view[t, nh + nkv:, :]


def linear(x, w, out_dtype=None):
    return (x.to(F64) @ w.to(F64).t()).to(out_dtype or x.dtype)


def qkv_rope_store_fits(x, w_qkv, hd):
    return False        # the CPU stand-in goes through linear + rope_store


def linear_add_fits(x, w, into):
    return False


def gate_up_silu(x, w_gate_up):
    return silu_mul(linear(x, w_gate_up))


def gate_up_act(x, w_gate_up, limit=0.0):
    both = linear(x, w_gate_up)
    return clamped_swish_mul(both, limit) if limit > 0 else silu_mul(both)


def gemm_generic(x, w, out_dtype):
    return linear(x, w, out_dtype)


def _attend(q, k, v, scale, visible):
    """q [nh, hd], k/v [L, nkv, hd], visible: bool [L]."""
    nh, nkv = q.shape[0], k.shape[1]
    per = nh // nkv
    out = torch.zeros(nh, q.shape[1], dtype=F64)
    for h in range(nh):
        s = (k[:, h // per, :].to(F64) @ q[h].to(F64)) * scale
        s = s.masked_fill(~visible, -math.inf)
        p = torch.softmax(s, dim=0)
        out[h] = p @ v[:, h // per, :].to(F64)
    return out


def attn_prefill(qkv, cu_seqlens, n_seqs, max_len, nh, nkv, hd, scale, window, softcap=0.0):
    assert not softcap
    T = qkv.shape[0]
    view = qkv.view(T, nh + 2 * nkv, hd)
    out = torch.zeros(T, nh * hd, dtype=qkv.dtype, device=qkv.device)
    for b in range(n_seqs):
        s0, s1 = int(cu_seqlens[b]), int(cu_seqlens[b + 1])
        k, v = view[s0:s1, nh: nh + nkv], view[s0:s1, nh + nkv:]
        idx = torch.arange(s1 - s0)
        for a in range(s1 - s0):
            vis = idx <= a
            if window and window > 0:
                vis = vis & (idx > a - window)
            out[s0 + a] = _attend(view[s0 + a, :nh], k, v, scale, vis).reshape(-1).to(qkv.dtype)
    return out


def attn_prefill_paged(qkv, cu_seqlens, seq_slot, seq_start, kcache, vcache, page_table, page_size,
                       ring, n_seqs, max_len, nh, nkv, hd, scale, window):
    """Rows that go on from tokens the cache holds: row r of sequence b stands at position
    seq_start[b] + r and sees the keys 0 .. its position, all read from the paged cache."""
    T = qkv.shape[0]
    view = qkv.view(T, nh + 2 * nkv, hd)
    out = torch.zeros(T, nh * hd, dtype=qkv.dtype, device=qkv.device)
    for b in range(n_seqs):
        s0, s1 = int(cu_seqlens[b]), int(cu_seqlens[b + 1])
        if s1 == s0:
            continue
        slot, p0 = int(seq_slot[b]), int(seq_start[b])
        total = p0 + (s1 - s0)
        first = max(0, p0 - window + 1) if window and window > 0 else 0
        ks, vs = [], []
        for pos in range(first, total):
            page, r = cache_offsets(page_table, slot, pos, page_size, ring)
            ks.append(kcache[page, :, r, :])
            vs.append(vcache[page, :, r, :])
        k, v = torch.stack(ks), torch.stack(vs)
        idx = torch.arange(first, total)
        for a in range(s1 - s0):
            vis = idx <= p0 + a
            if window and window > 0:
                vis = vis & (idx > p0 + a - window)
            out[s0 + a] = _attend(view[s0 + a, :nh], k, v, scale, vis).reshape(-1).to(qkv.dtype)
    return out


def decode_splits(B, nkv, max_len, nh=0, hd=0, ragged=False):
    return 2, 1


def attn_decode(qkv, kcache, vcache, page_table, page_size, ring, seq_slot, seq_len, nh, nkv, hd,
                scale, window, nsplit, waves=1):
    B = qkv.shape[0]
    view = qkv.view(B, nh + 2 * nkv, hd)
    out = torch.zeros(B, nh * hd, dtype=qkv.dtype, device=qkv.device)
    for b in range(B):
        slot = int(seq_slot[b])
        n = int(seq_len[b])
        first = max(0, n - window) if window and window > 0 else 0
        ks, vs = [], []
        for pos in range(first, n):
            page, r = cache_offsets(page_table, slot, pos, page_size, ring)
            ks.append(kcache[page, :, r, :])
            vs.append(vcache[page, :, r, :])
        if not ks:
            continue
        k, v = torch.stack(ks), torch.stack(vs)
        vis = torch.ones(k.shape[0], dtype=torch.bool)
        out[b] = _attend(view[b, :nh], k, v, scale, vis).reshape(-1).to(qkv.dtype)
    return out


def argmax(logits):
    return torch.argmax(logits, dim=-1).to(torch.int32)   # first index on ties


def kept_distribution(logits_row, temperature, top_k, top_p, repeat_penalty, last_tokens):
    """ids kept by the sampler and their probabilities (float64), in descending order."""
    V = logits_row.numel()
    s = logits_row.to(F64) / temperature
    if last_tokens is not None:
        for t in set(int(x) for x in last_tokens if int(x) >= 0):
            s[t] = s[t] * repeat_penalty if float(logits_row[t]) < 0 else s[t] / repeat_penalty
    order = sorted(range(V), key=lambda i: (-float(s[i]), i))
    if 0 < top_k < V:
        order = order[:top_k]
    sc = torch.tensor([float(s[i]) for i in order], dtype=F64)
    p = torch.exp(sc - sc.max())
    p = p / p.sum()
    if top_p < 1.0:
        cum = torch.cumsum(p, 0)
        n = int((cum >= top_p).nonzero()[0]) + 1 if bool((cum >= top_p).any()) else len(order)
        order, p = order[:n], p[:n] / p[:n].sum()
    return order, p


_M64 = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15


def mix64(z):
    """The output function of the splitmix64 generator (public domain, Vigna): its published
    first outputs from state 0 are mix64(1 * golden), mix64(2 * golden), ... =
    0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F (pinned in the kernel tests)."""
    z &= _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def uniform(seed, counter):
    """The sampler's contract, restated here and shared with nothing of the product: draw
    `counter` of a request with 64-bit `seed` uses the top 24 bits of
    mix64(seed + golden * (counter + 1)) as a number in [0, 1)."""
    return (mix64((seed + _GOLDEN * (counter + 1)) & _M64) >> 40) / 16777216.0


def sample(logits, temperature, top_k, top_p, repeat_penalty, last_tokens, seeds, counters):
    out = []
    for b in range(logits.shape[0]):
        ids, p = kept_distribution(logits[b], temperature, top_k, top_p, repeat_penalty,
                                   last_tokens[b] if last_tokens is not None else None)
        pairs = sorted(zip(ids, p.tolist()))              # inverse CDF in ascending id order
        u = uniform(int(seeds[b]) & ((1 << 64) - 1), int(counters[b]))
        cum, pick = 0.0, pairs[-1][0]
        for i, pi in pairs:
            cum += pi
            if u < cum:
                pick = i
                break
        out.append(pick)
    return torch.tensor(out, dtype=torch.int32)



# ---------------------------------------------------------------- latent attention
def sum_rows(a, b):
    return (a.to(F64) + b.to(F64)).to(torch.float32)


def relu_squared(x):
    return (torch.relu(x.to(F64)) ** 2).to(x.dtype)


def _rotate_pairs(v, cc, ss, rot):
    """Pairs (2i, 2i+1), i < rot/2, of the last axis of v (float64, changed in place)."""
    a, b = v[..., 0:rot:2].clone(), v[..., 1:rot:2].clone()
    v[..., 0:rot:2] = a * cc - b * ss
    v[..., 1:rot:2] = b * cc + a * ss


def latent_rope_store(y, H, dn, dr, R, rot, cos_sin, norm_w, eps, row_pos, row_slot, slot_len,
                      cache, page_table, page_size, ring, want_rows, cache_t=None):
    T, q_cols = y.shape[0], H * (dn + dr)
    down = y[:, q_cols:q_cols + R + dr].to(F64)
    c = down[:, :R]
    c = c / torch.sqrt((c * c).mean(dim=-1, keepdim=True) + eps) * norm_w.to(F64)
    kr = down[:, R:].clone()
    if cos_sin is not None:
        cs = cos_sin[row_pos.long()].to(F64)                      # [T, rot/2, 2]
        _rotate_pairs(kr, cs[..., 0], cs[..., 1], rot)
        q = y[:, :q_cols].to(F64).reshape(T, H, dn + dr)
        tail = q[:, :, dn:].clone()
        _rotate_pairs(tail, cs[:, None, :, 0], cs[:, None, :, 1], rot)
        q[:, :, dn:] = tail
        y[:, :q_cols] = q.reshape(T, q_cols).to(y.dtype)
    c, kr = c.to(y.dtype), kr.to(y.dtype)
    if cache is not None:
        for t in range(T):
            slot, pos = int(row_slot[t]), int(row_pos[t])
            if ring > 0 and slot_len is not None:
                if pos // page_size + ring <= (int(slot_len[slot]) - 1) // page_size:
                    continue
            page, r = cache_offsets(page_table, slot, pos, page_size, ring)
            cache[page, r, :R] = c[t]
            cache[page, r, R:] = kr[t]
            if cache_t is not None:
                cache_t[page, :, r, 0] = c[t]
    return (c, kr) if want_rows else (None, None)


def latent_pack(y, kvu, kr, H, dn, dr, dv, P):
    T = y.shape[0]
    out = torch.zeros((T, 3, H, P), dtype=y.dtype)
    out[:, 0, :, :dn + dr] = y[:, :H * (dn + dr)].reshape(T, H, dn + dr)
    out[:, 1, :, :dn] = kvu[:, :H * dn].reshape(T, H, dn)
    out[:, 1, :, dn:dn + dr] = kr[:, None, :]
    out[:, 2, :, :dv] = kvu[:, H * dn:].reshape(T, H, dv)
    return out.reshape(T, 3 * H * P)


def latent_gate(attn, y, gate_off, H, dv, P):
    T = y.shape[0]
    g = torch.sigmoid(y[:, gate_off:gate_off + H].to(F64))
    return (attn.to(F64).reshape(T, H, P)[:, :, :dv] * g[:, :, None]).reshape(T, H * dv).to(y.dtype)


def latent_decode_splits(B, H, longest, mfma=False):
    return 1


def latent_decode_mfma_fits(cache, cache_t, R, dr, page_size):
    return False


def latent_absorb_q(y, w_uk, H, dn, dr, R, out_dtype):
    B = y.shape[0]
    q = y[:, :H * (dn + dr)].to(F64).reshape(B, H, dn + dr)
    wk = w_uk.to(F64).reshape(H, dn, R)
    return torch.cat([torch.einsum("bhd,hdr->bhr", q[:, :, :dn], wk), q[:, :, dn:]], dim=-1).to(out_dtype)


def latent_store_absorb(y, H, dn, dr, R, rot, cos_sin, norm_w, eps, row_pos, row_slot, cache, page_table,
                        page_size, ring, w_uk, out_dtype, cache_t=None):
    rotated = y.clone()                                # y itself keeps the unrotated queries
    latent_rope_store(rotated, H, dn, dr, R, rot, cos_sin, norm_w, eps, row_pos, row_slot, None, cache,
                      page_table, page_size, ring, False, cache_t)
    if y.dtype != torch.float32:
        # the rotated part is not rounded on its way: take it from the unrounded rotation
        wide = y.to(F64)
        latent_rope_store(wide, H, dn, dr, R, rot, cos_sin, norm_w, eps, row_pos, row_slot, None, None,
                          page_table, page_size, ring, False)
        rotated = wide
    return latent_absorb_q(rotated, w_uk, H, dn, dr, R, out_dtype)


def latent_attn_decode(qa, y, w_uv, gate_off, cache, page_table, page_size, ring, seq_slot, seq_len,
                       len_more, H, dr, R, dv, scale, window, nsplit, cache_t=None):
    B = y.shape[0]
    out = torch.zeros((B, H * dv), dtype=y.dtype)
    wv = w_uv.to(F64).reshape(H, dv, R)
    for b in range(B):
        slot, L = int(seq_slot[b]), int(seq_len[b]) + len_more
        lo = max(0, L - window) if window and window > 0 else 0
        rows = torch.stack([cache[cache_offsets(page_table, slot, p, page_size, ring)] for p in range(lo, L)]).to(F64)
        gate = torch.sigmoid(y[b, gate_off:gate_off + H].to(F64))
        for h in range(H):
            p = torch.softmax((rows @ qa[b, h].to(F64)) * scale, dim=0)
            out[b, h * dv:(h + 1) * dv] = ((wv[h] @ (p @ rows[:, :R])) * gate[h]).to(y.dtype)
    return out


# ---------------------------------------------------------------- routed feed-forward
def few_outputs_f32(x, w):
    return (x.to(F64) @ w.to(F64).t()).to(torch.float32)


def moe_route(z, correction, top, score="softmax"):
    s = torch.softmax(z.to(F64), dim=-1) if score == "softmax" else torch.sigmoid(z.to(F64))
    pick = s + correction.to(F64) if correction is not None else s
    idx = torch.topk(pick, top, dim=-1).indices
    return idx.to(torch.int32), torch.gather(s, 1, idx).to(torch.float32)


def moe_plan(h, w_router, correction, top, w_gate_up, score="softmax"):
    idx, wt = moe_route(few_outputs_f32(h, w_router), correction, top, score)
    return idx, wt, None


def moe_experts(h, idx, w_gate_up, w_down, grouped=None, activation="silu", limit=0.0, input_weight=None):
    T, top = idx.shape
    F = w_gate_up.shape[1] // 2
    y = torch.zeros((T * top, h.shape[1]), dtype=h.dtype)
    for t in range(T):
        for k in range(top):
            e = int(idx[t, k])
            if e < w_gate_up.shape[0]:
                x = h[t].to(F64) * (input_weight[t, k].to(F64) if input_weight is not None else 1.0)
                gu = w_gate_up[e].to(F64) @ x
                if activation == "silu":
                    a = torch.nn.functional.silu(gu[:F]) * gu[F:]
                else:
                    g, u = torch.clamp(gu[:F], max=limit), torch.clamp(gu[F:], -limit, limit)
                    a = g * torch.sigmoid(1.702 * g) * (u + 1)
                y[t * top + k] = (w_down[e].to(F64) @ a).to(h.dtype)
    return y


def moe_combine(h, idx, wt, y, n_real, shared=None, shared_gate=None):
    T, top = idx.shape
    out = torch.zeros(h.shape, dtype=F64)
    for t in range(T):
        for k in range(top):
            v = y[t * top + k] if int(idx[t, k]) < n_real else h[t]
            out[t] += (wt[t, k].to(F64) if wt is not None else 1.0) * v.to(F64)
    if shared is not None:
        g = torch.sigmoid(h.to(F64) @ shared_gate.to(F64))[:, None] if shared_gate is not None else 1.0
        out = out + g * shared.to(F64)
    return out.to(torch.float32)


# ---------------------------------------------------------------- several residual streams
def stream_mix_norm(x, write, read, weight, eps, out_dtype, row_idx=None):
    T, S, E = x.shape
    xn = x.to(F64)
    if write is not None:
        y = write.ya * write.y.to(F64) + (write.yb * write.y2.to(F64) if write.y2 is not None else 0.0)
        xn = torch.stack([sum(write.mix[s, t].to(F64) * xn[:, s] for s in range(S)) + write.out[t].to(F64) * y
                          for t in range(S)], dim=1)
        if row_idx is None:
            x.copy_(xn.to(torch.float32))
    u = sum((read[s].to(F64) if read is not None else 1.0) * xn[:, s] for s in range(S))
    if row_idx is not None:
        u = u[row_idx.long()]
    return (u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps) * weight.to(F64)).to(out_dtype)


def scaled_sum_tensor(self):
    return (self.sa * self.a.to(F64) + self.sb * self.b.to(F64)).to(torch.float32)


# ---------------------------------------------------------------- attention with a soft cap
def kv_store2(rows, k_off, v_off, row_pos, row_slot, kcache, vcache, page_table, page_size, ring, nkv, dk, dv):
    for r in range(rows.shape[0]):
        page, at = cache_offsets(page_table, int(row_slot[r]), int(row_pos[r]), page_size, ring)
        kcache[page, :, at, :] = rows[r, k_off:k_off + nkv * dk].view(nkv, dk)
        vcache[page, :, at, :] = rows[r, v_off:v_off + nkv * dv].view(nkv, dv)


def _attend_capped(q, k, v, scale, cap, slopes=None, lse=None):
    """q [nh, dk], k [L, nkv, dk], v [L, nkv, dv]: every key visible, the last one the query's own.
    `lse` [nh] takes log(sum(exp(score))) of every head."""
    nh, per, L = q.shape[0], q.shape[0] // k.shape[1], k.shape[0]
    out = torch.zeros(nh, v.shape[2], dtype=F64)
    for h in range(nh):
        s = (k[:, h // per, :].to(F64) @ q[h].to(F64)) * scale
        if cap:
            s = cap * torch.tanh(s / cap)
        if slopes is not None:
            s = s - slopes[h].to(F64) * torch.arange(L - 1, -1, -1, dtype=F64)
        out[h] = torch.softmax(s, dim=0) @ v[:, h // per, :].to(F64)
        if lse is not None:
            lse[h] = torch.logsumexp(s, dim=0).to(lse.dtype)
    return out


def _first_seen(pos, window, chunk):
    first = max(0, pos - window + 1) if window and window > 0 else 0
    return max(first, pos // chunk * chunk) if chunk and chunk > 0 else first


def _gated(out_row, gate, r, gate_off, heads=0):
    if gate is None:
        return out_row
    if heads:                                         # one number a head
        g = torch.sigmoid(gate[r, gate_off:gate_off + heads].to(F64))
        return (out_row.view(heads, -1) * g[:, None]).reshape(-1)
    return out_row * torch.sigmoid(gate[r, gate_off:gate_off + out_row.numel()].to(F64))


def qkv_norm_mix_store(rows, k_off, v_off, q_weight, k_weight, eps, lam, first, first_off, row_pos, row_slot,
                       kcache, vcache, page_table, page_size, ring, nh, nkv, dk, dv):
    def normed(x, w):
        x = x.to(F64)
        return (x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.to(F64)).to(rows.dtype)
    if q_weight is not None:
        rows[:, :nh * dk] = normed(rows[:, :nh * dk], q_weight)
        rows[:, k_off:k_off + nkv * dk] = normed(rows[:, k_off:k_off + nkv * dk], k_weight)
    if lam is not None:
        l = lam.to(F64)[0]
        rows[:, v_off:v_off + nkv * dv] = ((1 - l) * rows[:, v_off:v_off + nkv * dv].to(F64)
                                           + l * first[:, first_off:first_off + nkv * dv].to(F64)).to(rows.dtype)
    if kcache is not None:
        kv_store2(rows, k_off, v_off, row_pos, row_slot, kcache, vcache, page_table, page_size, ring, nkv, dk, dv)


def _cached(kcache, vcache, page_table, slot, first, total, page_size, ring):
    at = [cache_offsets(page_table, slot, pos, page_size, ring) for pos in range(first, total)]
    return (torch.stack([kcache[p, :, r, :] for p, r in at]), torch.stack([vcache[p, :, r, :] for p, r in at]))


def attn_cap_rows(q, cu_seqlens, seq_slot, seq_start, kcache, vcache, page_table, page_size, ring,
                  n_seqs, max_rows, nh, nkv, dk, dv, scale, cap, window, slopes=None, chunk=0, gate=None,
                  gate_off=0, gate_heads=False, lse=None):
    out = torch.zeros(q.shape[0], nh * dv, dtype=q.dtype)
    for b in range(n_seqs):
        s0, s1 = int(cu_seqlens[b]), int(cu_seqlens[b + 1])
        for a in range(s1 - s0):
            pos = int(seq_start[b]) + a
            first = _first_seen(pos, window, chunk)
            k, v = _cached(kcache, vcache, page_table, int(seq_slot[b]), first, pos + 1, page_size, ring)
            row = _attend_capped(q[s0 + a, :nh * dk].view(nh, dk), k, v, scale, cap, slopes,
                                 lse[s0 + a] if lse is not None else None).reshape(-1)
            out[s0 + a] = _gated(row, gate, s0 + a, gate_off, nh if gate_heads else 0).to(q.dtype)
    return out


def attn_cap_decode(q, kcache, vcache, page_table, page_size, ring, seq_slot, seq_len, nh, nkv, dk, dv,
                    scale, cap, window, nsplit, slopes=None, chunk=0, gate=None, gate_off=0, gate_heads=False,
                    lse=None):
    out = torch.zeros(q.shape[0], nh * dv, dtype=q.dtype)
    for b in range(q.shape[0]):
        n = int(seq_len[b])
        first = _first_seen(n - 1, window, chunk)
        k, v = _cached(kcache, vcache, page_table, int(seq_slot[b]), first, n, page_size, ring)
        row = _attend_capped(q[b, :nh * dk].view(nh, dk), k, v, scale, cap, slopes,
                             lse[b] if lse is not None else None).reshape(-1)
        out[b] = _gated(row, gate, b, gate_off, nh if gate_heads else 0).to(q.dtype)
    return out


# ---------------------------------------------------------------- the gated delta rule
def delta_prepare(P, b_off, A, a_off, conv_w, tail, row_slot, a_log, dt_bias, G, H, dk, dv, per_channel,
                  update_tail=False):
    T, C, taps = P.shape[0], conv_w.shape[0], conv_w.shape[1]
    K, DW = taps - 1, dk if per_channel else 1
    y = torch.zeros(T, C, dtype=F64)
    for r in range(T):
        slot, before = int(row_slot[r]), 0
        while before < K and r - before - 1 >= 0 and int(row_slot[r - before - 1]) == slot:
            before += 1
        for j in range(taps):
            d = K - j
            src = P[r - d, :C] if d <= before else tail[slot, K - (d - before)]
            y[r] += conv_w[:, j].to(F64) * src.to(F64)
    y = y * torch.sigmoid(y)
    unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    qn = unit(y[:, :G * dk].view(T, G, dk)) * dk ** -0.5
    kn = unit(y[:, G * dk:2 * G * dk].view(T, G, dk))
    vv = y[:, 2 * G * dk:].view(T, H, dv)
    beta = torch.sigmoid(P[:, b_off:b_off + H].to(F64))
    a = A[:, a_off:a_off + H * DW].to(F64) + dt_bias.to(F64)
    sp = torch.where(a > 30, a, torch.log1p(torch.exp(torch.clamp(a, max=30))))
    dec = torch.exp(-torch.exp(a_log.to(F64)).repeat_interleave(DW) * sp).view(T, H, DW)
    if update_tail:                                   # one row a sequence: its tail moves on by that row
        for r in range(T if K else 0):
            slot = int(row_slot[r])
            tail[slot] = torch.cat([tail[slot, 1:], P[r:r + 1, :C].to(tail.dtype)])
    return tuple(t.to(torch.float32).contiguous() for t in (qn, kn, vv, beta, dec))


def delta_conv_tail(P, tail, cu_seqlens, seq_slot, n_seqs, taps, col_off=0):
    K, C = taps - 1, tail.shape[2]
    P = P[:, col_off:]
    for b in range(n_seqs if K else 0):
        r0, n, slot = int(cu_seqlens[b]), int(cu_seqlens[b + 1]) - int(cu_seqlens[b]), int(seq_slot[b])
        if n <= 0:
            continue
        old = tail[slot].clone()
        for j in range(K):
            at = n - K + j
            tail[slot, j] = P[r0 + at, :C].to(tail.dtype) if at >= 0 else old[j + n]


def delta_scan(qn, kn, vv, beta, dec, state, cu_seqlens, seq_slot, n_seqs, max_rows, correct=True):
    T, G, dk = qn.shape
    H, dv = vv.shape[1], vv.shape[2]
    o = torch.zeros(T, H, dv, dtype=torch.float32)
    for b in range(n_seqs):
        slot = int(seq_slot[b])
        for r in range(int(cu_seqlens[b]), int(cu_seqlens[b + 1])):
            for h in range(H):
                g = h // (H // G)
                S = state[slot, h].to(F64) * dec[r, h].to(F64).expand(dk)[:, None]
                u = beta[r, h].to(F64) * (vv[r, h].to(F64) - (S.t() @ kn[r, g].to(F64) if correct else 0.0))
                S = S + torch.outer(kn[r, g].to(F64), u)
                o[r, h] = (S.t() @ qn[r, g].to(F64)).to(torch.float32)
                state[slot, h] = S.to(torch.float32)
    return o


def delta_finish(o, weight, Z, z_off, gate, eps, out_dtype):
    T, H, dv = o.shape
    z = Z[:, z_off:z_off + H * dv].to(F64).view(T, H, dv)
    act = torch.sigmoid(z) if gate == "sigmoid" else z * torch.sigmoid(z)
    x = o.to(F64)
    return (x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight.to(F64) * act).reshape(T, H * dv).to(out_dtype)


# ---------------------------------------------------------------- around the plain gated rule
def _softplus(a):
    return torch.where(a > 30, a, torch.log1p(torch.exp(torch.clamp(a, max=30))))


def ssm_prepare(U, x_off, dt_off, conv_w, conv_b, tail, row_slot, a_log, dt_bias, G, H, N, dv, update_tail=False):
    T, C, taps = U.shape[0], conv_w.shape[0], conv_w.shape[1]
    K, inner, GN = taps - 1, H * dv, G * N
    X = U[:, x_off:x_off + C]
    y = conv_b.to(F64).expand(T, C).clone()
    for r in range(T):
        slot, before = int(row_slot[r]), 0
        while before < K and r - before - 1 >= 0 and int(row_slot[r - before - 1]) == slot:
            before += 1
        for j in range(taps):
            d = K - j
            src = X[r - d] if d <= before else tail[slot, K - (d - before)]
            y[r] += conv_w[:, j].to(F64) * src.to(F64)
    y = y * torch.sigmoid(y)
    vv, kn, qn = y[:, :inner].view(T, H, dv), y[:, inner:inner + GN].view(T, G, N), y[:, inner + GN:].view(T, G, N)
    step = _softplus(U[:, dt_off:dt_off + H].to(F64) + dt_bias.to(F64))
    dec = torch.exp(-torch.exp(a_log.to(F64)) * step).view(T, H, 1)
    if update_tail:
        for r in range(T if K else 0):
            slot = int(row_slot[r])
            tail[slot] = torch.cat([tail[slot, 1:], X[r:r + 1].to(tail.dtype)])
    return tuple(t.to(torch.float32).contiguous() for t in (qn, kn, vv, step, dec))


def ssm_finish(o, x, D, Z, z_off, weight, norm_groups, eps, out_dtype):
    T, H, dv = o.shape
    z = Z[:, z_off:z_off + H * dv].to(F64)
    y = (o.to(F64) + D.to(F64)[None, :, None] * x.to(F64)).reshape(T, H * dv) * (z * torch.sigmoid(z))
    y = y.view(T, norm_groups, -1)
    y = y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)
    return (y.reshape(T, H * dv) * weight.to(F64)).to(out_dtype)


def memory_prepare(U, i_off, f_off, i_bias, f_bias, cap, m_state, cu_seqlens, seq_slot, n_seqs, H, dk, dv):
    T = U.shape[0]
    qn = U[:, :H * dk].to(F64).view(T, H, dk) * dk ** -0.5
    kn = U[:, H * dk:2 * H * dk].to(F64).view(T, H, dk)
    vv = torch.cat([U[:, 2 * H * dk:2 * H * dk + H * dv].to(F64).view(T, H, dv), torch.ones(T, H, 1, dtype=F64)], dim=2)
    ig = cap * torch.tanh((U[:, i_off:i_off + H].to(F64) + i_bias.to(F64)) / cap)
    fg = -_softplus(-(cap * torch.tanh((U[:, f_off:f_off + H].to(F64) + f_bias.to(F64)) / cap)))
    beta, dec, em = (torch.zeros(T, H, dtype=F64) for _ in range(3))
    for b in range(n_seqs):
        slot = int(seq_slot[b])
        m = m_state[slot].to(F64)
        for r in range(int(cu_seqlens[b]), int(cu_seqlens[b + 1])):
            new = torch.maximum(fg[r] + m, ig[r])
            dec[r], beta[r], em[r] = torch.exp(fg[r] + m - new), torch.exp(ig[r] - new), torch.exp(-new)
            m = new
        if int(cu_seqlens[b + 1]) > int(cu_seqlens[b]):
            m_state[slot] = m.to(torch.float32)
    return tuple(t.to(torch.float32).contiguous() for t in (qn, kn, vv, beta, dec.view(T, H, 1), em))


def memory_finish(o, em, weight, Z, z_off, eps, out_dtype):
    T, H, dv1 = o.shape
    dv = dv1 - 1
    x = o.to(F64)
    den = torch.maximum(x[:, :, dv].abs(), em.to(F64)) + 1e-6
    y = x[:, :, :dv] / den[:, :, None]
    y = y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)
    z = Z[:, z_off:z_off + H * dv].to(F64)
    return (y.reshape(T, H * dv) * weight.to(F64) * torch.sigmoid(z)).to(out_dtype)


def embed_pairs(tokens, row_pos, row_slot, table, scale, pairs, buckets, mul_prev, mul_cur, places, last_token,
                remember):
    T = tokens.numel()
    out = torch.zeros(T, table.shape[1], dtype=torch.float32)
    for t in range(T):
        tok, pos, slot = int(tokens[t]), int(row_pos[t]), int(row_slot[t])
        v = table[tok].to(F64) * scale
        if pairs is not None:
            if pos == 0:
                at = buckets
            else:
                prev = int(tokens[t - 1]) if t > 0 and int(row_slot[t - 1]) == slot else int(last_token[slot])
                at = (prev * mul_prev + tok * mul_cur) % buckets
            v = v + pairs[at].to(F64)
        if places is not None:
            v = v + places[pos].to(F64)
        out[t] = v.to(torch.float32)
        if remember and last_token is not None:
            last_token[slot] = tok
    return out


def remember_last(tokens, cu_seqlens, seq_slot, last_token, n_seqs):
    for b in range(n_seqs):
        if int(cu_seqlens[b + 1]) > int(cu_seqlens[b]):
            last_token[int(seq_slot[b])] = int(tokens[int(cu_seqlens[b + 1]) - 1])


def gelu_tanh(x):
    z = x.to(F64)
    return (0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))).to(x.dtype)


# ---------------------------------------------------------------- short convolutions, a sublayer's own norm
def _rows_above(row_slot, r, most):
    n = 0
    while n < most and r - n - 1 >= 0 and int(row_slot[r - n - 1]) == int(row_slot[r]):
        n += 1
    return n


def short_conv(X, x_off, C, weight, tail, row_slot, out_dtype, bias=None, in_bias=None, add_input=False,
               update_tail=False):
    T, taps = X.shape[0], weight.shape[1]
    K = taps - 1
    x = X[:, x_off:x_off + C].to(F64)
    if in_bias is not None:
        x = (x + in_bias.to(F64)).to(tail.dtype).to(F64)      # as the tail would hold them
    out = torch.zeros(T, C, dtype=F64)
    for r in range(T):
        slot, n = int(row_slot[r]), _rows_above(row_slot, r, K)
        ins = []
        for j in range(taps):
            back = K - j
            ins.append(x[r - back] if back <= n else tail[slot, K - (back - n)].to(F64))
        y = bias.to(F64).clone() if bias is not None else torch.zeros(C, dtype=F64)
        for j in range(taps):
            y = y + weight[:, j].to(F64) * ins[j]
        out[r] = y + (ins[K] if add_input else 0.0)
        if update_tail and K:
            tail[slot] = torch.stack(ins[1:]).to(tail.dtype)
    return out.to(out_dtype)


def short_conv_tail(X, x_off, tail, cu_seqlens, seq_slot, n_seqs, taps, in_bias=None):
    K, C = taps - 1, tail.shape[2]
    x = X[:, x_off:x_off + C].to(F64)
    if in_bias is not None:
        x = x + in_bias.to(F64)
    for b in range(n_seqs if K else 0):
        r0, n, slot = int(cu_seqlens[b]), int(cu_seqlens[b + 1]) - int(cu_seqlens[b]), int(seq_slot[b])
        if n <= 0:
            continue
        old = tail[slot].clone()
        for j in range(K):
            at = n - K + j
            tail[slot, j] = x[r0 + at].to(tail.dtype) if at >= 0 else old[j + n]


def rms_rows_gain(a, weight, eps, gain):
    x = a.to(F64)
    return (gain * (x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight.to(F64))).to(torch.float32)


def post_add_rmsnorm(x, post, weight, eps, out_dtype, row_idx=None, conv=None):
    delta = rms_rows_gain(post.a, post.weight, post.eps, post.gain) if post is not None else None
    h = add_rmsnorm(x, delta, weight, eps, out_dtype, row_idx)
    if conv is None:
        return h
    cw, tail, slots = conv
    return short_conv(h, 0, h.shape[1], cw, tail, slots, out_dtype, add_input=True, update_tail=True)


def clamped_swish_mul(gate_up, limit):
    F = gate_up.shape[1] // 2
    g = torch.clamp(gate_up[:, :F].to(F64), max=limit)
    u = torch.clamp(gate_up[:, F:].to(F64), -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)).to(gate_up.dtype)


# ---------------------------------------------------------------- attention over a window and pooled blocks
def qk_rotate_store(rows, k_off, v_off, cos_sin, rot, pairing, unit_norm, eps, row_pos, row_slot, kcache,
                    vcache, page_table, page_size, ring, nh, nkv, dk, dv, q_scale=None):
    half = rot // 2
    for r in range(rows.shape[0]):
        for off, heads in ((0, nh), (k_off, nkv)):
            if not heads:
                continue
            x = rows[r, off:off + heads * dk].to(F64).view(heads, dk).clone()
            if cos_sin is not None and rot:
                c, s = cos_sin[int(row_pos[r]), :, 0].to(F64), cos_sin[int(row_pos[r]), :, 1].to(F64)
                ia = torch.arange(half) if pairing == 0 else 2 * torch.arange(half)
                ib = ia + half if pairing == 0 else ia + 1
                u, v = x[:, ia].clone(), x[:, ib].clone()
                x[:, ia], x[:, ib] = u * c - v * s, v * c + u * s
            if unit_norm:
                x = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
            if q_scale is not None and off == 0:
                x = x * q_scale.to(F64)[:, None]
            rows[r, off:off + heads * dk] = x.reshape(-1).to(rows.dtype)
    if kcache is not None:
        kv_store2(rows, k_off, v_off, row_pos, row_slot, kcache, vcache, page_table, page_size, ring, nkv, dk, dv)


def pool_store(row_pos, row_slot, kcache, vcache, kpool, vpool, page_table, page_size, nkv, dk, dv, pool):
    for r in range(row_pos.numel()):
        pos, slot = int(row_pos[r]), int(row_slot[r])
        if (pos + 1) % pool:
            continue
        b = pos // pool
        k, v = _cached(kcache, vcache, page_table, slot, b * pool, b * pool + pool, page_size, 0)
        page, at = cache_offsets(page_table, slot, b, page_size, 0)
        kpool[page, :, at, :] = k.to(F64).mean(0).to(kpool.dtype)
        vpool[page, :, at, :] = v.to(F64).mean(0).to(vpool.dtype)


def _attend_pooled(q, pos, slot, kcache, vcache, kpool, vpool, page_table, page_size, nh, nkv, dk, dv, scale,
                   head_scale, window, pool):
    first = max(0, pos - window + 1)
    k, v = _cached(kcache, vcache, page_table, slot, first, pos + 1, page_size, 0)
    seen = (pos - window + 1) // pool if pool and pos - window + 1 >= pool else 0
    if seen:
        pk, pv = _cached(kpool, vpool, page_table, slot, 0, seen, page_size, 0)
        k, v = torch.cat([pk, k]), torch.cat([pv, v])
    per = nh // nkv
    out = torch.zeros(nh, dv, dtype=F64)
    for h in range(nh):
        s = (k[:, h // per, :].to(F64) @ q[h].to(F64)) * scale * (head_scale[h].to(F64) if head_scale is not None else 1.0)
        out[h] = torch.softmax(s, dim=0) @ v[:, h // per, :].to(F64)
    return out.reshape(-1)


def attn_pooled_rows(q, cu_seqlens, seq_slot, seq_start, kcache, vcache, kpool, vpool, page_table, page_size,
                     n_seqs, max_rows, nh, nkv, dk, dv, scale, head_scale, window, pool, out=None, lse=None):
    # (with `out` and `lse`, what the window's kernel left, the kernel merges the pooled blocks in;
    # the result is the whole attention either way)
    out = torch.zeros(q.shape[0], nh * dv, dtype=q.dtype) if out is None else out
    for b in range(n_seqs):
        s0, s1 = int(cu_seqlens[b]), int(cu_seqlens[b + 1])
        for a in range(s1 - s0):
            out[s0 + a] = _attend_pooled(q[s0 + a, :nh * dk].view(nh, dk), int(seq_start[b]) + a, int(seq_slot[b]),
                                         kcache, vcache, kpool, vpool, page_table, page_size, nh, nkv, dk, dv,
                                         scale, head_scale, window, pool).to(q.dtype)
    return out


def attn_pooled_decode(q, kcache, vcache, kpool, vpool, page_table, page_size, seq_slot, seq_len, nh, nkv, dk,
                       dv, scale, head_scale, window, pool, out=None, lse=None):
    out = torch.zeros(q.shape[0], nh * dv, dtype=q.dtype) if out is None else out
    for b in range(q.shape[0]):
        out[b] = _attend_pooled(q[b, :nh * dk].view(nh, dk), int(seq_len[b]) - 1, int(seq_slot[b]), kcache,
                                vcache, kpool, vpool, page_table, page_size, nh, nkv, dk, dv, scale, head_scale,
                                window, pool).to(q.dtype)
    return out


# ---------------------------------------------------------------- gated linear attention, a gated linear recurrent unit
def gla_prepare(U, q_off, k_off, v_off, Z, z_bias, tau, H, dk, dv):
    T = U.shape[0]
    u = U.to(F64)
    qn = (u[:, q_off:q_off + H * dk] * dk ** -0.5).view(T, H, dk)
    kn = u[:, k_off:k_off + H * dk].view(T, H, dk)
    vv = u[:, v_off:v_off + H * dv].view(T, H, dv)
    z = Z.to(F64) + z_bias.to(F64)
    dec = torch.exp(-_softplus(-z) / tau).view(T, H, dk)
    beta = torch.ones(T, H, dtype=F64)
    return tuple(t.to(torch.float32).contiguous() for t in (qn, kn, vv, beta, dec))


def lru_gates(u, w_t, r_bias, i_bias, lam, rate):
    T, C = u.shape
    nb, cb = w_t.shape[1], w_t.shape[2]
    ub = u.to(F64).view(T, nb, cb)
    r = torch.sigmoid(torch.einsum("bio,tbi->tbo", w_t[0].to(F64), ub).reshape(T, C) + r_bias.to(F64))
    i = torch.sigmoid(torch.einsum("bio,tbi->tbo", w_t[1].to(F64), ub).reshape(T, C) + i_bias.to(F64))
    a = torch.exp(-rate * r * _softplus(lam.to(F64)))
    x = torch.sqrt(torch.clamp(1 - a * a, min=0)) * i * u.to(F64)
    return a.to(torch.float32), x.to(torch.float32)


def lru_scan(a, x, state, Y, y_off, y_bias, cu_seqlens, seq_slot, n_seqs, max_rows, out_dtype):
    T, C = a.shape
    out = torch.zeros(T, C, dtype=F64)
    y = Y[:, y_off:y_off + C].to(F64) + (y_bias.to(F64) if y_bias is not None else 0.0)
    y = 0.5 * y * (1 + torch.tanh(math.sqrt(2 / math.pi) * (y + 0.044715 * y ** 3)))
    for b in range(n_seqs):
        slot = int(seq_slot[b])
        S = state[slot].to(F64)
        for r in range(int(cu_seqlens[b]), int(cu_seqlens[b + 1])):
            S = (a[r].to(F64) * S + x[r].to(F64)).to(torch.float32).to(F64)
            out[r] = S * y[r]
        state[slot] = S.to(torch.float32)
    return out.to(out_dtype)


def patch(monkeypatch):
    """Put these functions in place of the GPU ops (CPU tests only)."""
    from inferllm_amd.kernels import ops
    for name in ("embed", "add_rmsnorm", "silu_mul", "rope_store", "linear", "gemm_generic", "gate_up_silu", "qkv_rope_store_fits",
                 "linear_add_fits",
                 "attn_prefill", "attn_prefill_paged", "decode_splits", "attn_decode", "argmax", "sample",
                 "sum_rows", "relu_squared", "latent_rope_store", "latent_pack", "latent_gate",
                 "latent_decode_splits", "latent_decode_mfma_fits", "latent_attn_decode", "latent_absorb_q",
                 "latent_store_absorb",
                 "few_outputs_f32", "moe_route", "moe_plan", "moe_experts", "moe_combine",
                 "stream_mix_norm", "kv_store2", "attn_cap_rows", "attn_cap_decode", "delta_prepare",
                 "delta_conv_tail", "delta_scan", "delta_finish", "qkv_norm_mix_store", "ssm_prepare",
                 "ssm_finish", "memory_prepare", "memory_finish", "embed_pairs", "remember_last", "gelu_tanh",
                 "short_conv", "short_conv_tail", "rms_rows_gain", "post_add_rmsnorm", "gate_up_act", "clamped_swish_mul", "qk_rotate_store",
                 "pool_store", "attn_pooled_rows", "attn_pooled_decode", "gla_prepare", "lru_gates", "lru_scan"):
        monkeypatch.setattr(ops, name, globals()[name])
    monkeypatch.setattr(ops.ScaledSum, "tensor", scaled_sum_tensor)
