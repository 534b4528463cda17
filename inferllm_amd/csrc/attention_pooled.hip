// Attention over a sliding window of tokens and, before the window, one pooled key and value for
// every block of `pool` tokens that lies wholly before it:
//   position i sees token j with 0 <= i - j < window, and block b (positions b pool .. b pool +
//   pool - 1) if b pool + pool - 1 <= i - window; tokens and blocks share one softmax.
// A block's key is the mean of its keys as the cache holds them, its value the mean of its values.
// The pooled rows live in the same paged cache line as the tokens, under the same page table: block
// b is row b of the sequence ("kp", "vp" beside "k", "v"), so it is there as soon as its last token
// is and is read densely.  score = (q . k) scale head_scale[h] (`head_scale` null: 1).
// The attention kernels do both parts themselves, or, given `lse`, the pooled part alone on top of
// what a kernel for windows left: `out` holds the window's normalised sums and `lse` [rows][heads]
// max + log(sum) of its softmax (attention_capped.hip writes both), and the pooled rows are merged
// into `out` in place.
// Float32 arithmetic over float32 or bfloat16 storage; key and value widths of up to 256.
//
// Beside the attention: `qk_rotate_store` turns q and k of packed rows by their positions (either
// pairing, the first `rot` dims of a head), optionally divides every head by its root mean square
// and multiplies query head h by q_scale[h] (a scale of the scores that differs by head, taken into
// the queries), and stores k and v (widths of their own) in the cache; `pool_store` forms the pooled rows of the
// blocks that a step completes.
#include <math.h>

#include "api.h"
#include "common.h"

#define PQ 32  // query rows of a block
#define PK 32  // keys of a tile
#define NEG_INF (-INFINITY)

// ---------------------------------------------------------------- rotation, unit norm, store
// grid (rows, nh + nkv); 64 threads.  Block (t, h): h < nh is query head h (columns h dk ..), else
// key head h - nh (columns k_off ..), whose block also stores the value head (columns v_off ..).
__global__ void __launch_bounds__(64)
qk_rotate_store_kernel(void* __restrict__ rows, int dt, int row_len, int k_off, int v_off,
                       const float* __restrict__ cos_sin, int rot, int pairing, int unit_norm, float eps,
                       const float* __restrict__ q_scale, const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
                       void* __restrict__ kcache, void* __restrict__ vcache,
                       const int32_t* __restrict__ page_table, int table_stride, int page_size, int ring,
                       int nh, int nkv, int dk, int dv) {
    __shared__ float x[256];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int pos = row_pos[t];
    const bool is_k = h >= nh;
    const size_t base = (size_t)t * row_len + (is_k ? k_off + (size_t)(h - nh) * dk : (size_t)h * dk);
    for (int d = lane; d < dk; d += 64) x[d] = ld_f(rows, dt, base + d);
    __syncthreads();
    if (cos_sin && rot > 0) {
        const float* cs = cos_sin + (size_t)pos * rot;              // [rot / 2][2]
        const int half = rot / 2;
        for (int i = lane; i < half; i += 64) {
            const int a = pairing == 0 ? i : 2 * i, b = pairing == 0 ? i + half : 2 * i + 1;
            const float c = cs[2 * i], s = cs[2 * i + 1];
            const float u = x[a], v = x[b];
            x[a] = u * c - v * s;
            x[b] = v * c + u * s;
        }
        __syncthreads();
    }
    float inv = 1.f;
    if (unit_norm) {
        float ss = 0.f;
        for (int d = lane; d < dk; d += 64) ss = fmaf(x[d], x[d], ss);
        ss = wave_sum(ss);
        inv = 1.0f / sqrtf(ss / (float)dk + eps);
    }
    if (q_scale && !is_k) inv *= q_scale[h];
    size_t kat = 0, vat = 0;
    const bool store = is_k && kcache != nullptr;
    if (store) {
        const int slot = row_slot[t];
        kat = cache_row_offset(page_table, table_stride, slot, pos, page_size, ring, nkv, h - nh, dk);
        vat = cache_row_offset(page_table, table_stride, slot, pos, page_size, ring, nkv, h - nh, dv);
    }
    for (int d = lane; d < dk; d += 64) {
        const float y = x[d] * inv;
        st_f(rows, dt, base + d, y);
        if (store) st_f(kcache, dt, kat + d, y);
    }
    if (store) {
        const size_t vb = (size_t)t * row_len + v_off + (size_t)(h - nh) * dv;
        for (int d = lane; d < dv; d += 64) {
            if (dt == ILLM_BF16) ((bf16_t*)vcache)[vat + d] = ((const bf16_t*)rows)[vb + d];
            else ((float*)vcache)[vat + d] = ((const float*)rows)[vb + d];
        }
    }
}

extern "C" int illm_qk_rotate_store(void* rows, int dt, int row_len, int k_off, int v_off,
                                    const float* cos_sin, int rot, int pairing, int n_positions,
                                    int unit_norm, float eps, const float* q_scale, const int32_t* row_pos,
                                    const int32_t* row_slot, void* kcache, void* vcache,
                                    const int32_t* page_table, int table_stride, int page_size, int ring,
                                    int T, int nh, int nkv, int dk, int dv, void* stream) {
    if (T < 0 || nh < 0 || nkv < 0 || nh + nkv <= 0 || nh + nkv > 65535 || dk <= 0 || dk > 256 || dv < 0 ||
        dv > 256 || !illm_dtype_ok(dt) || rot < 0 || rot % 2 || rot > dk || (pairing != 0 && pairing != 1) ||
        nh * dk > row_len || (nkv > 0 && (k_off + nkv * dk > row_len || v_off + nkv * dv > row_len)) ||
        (cos_sin && rot > 0 && n_positions <= 0) || (kcache && (!vcache || !page_table || page_size <= 0)))
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(qk_rotate_store_kernel, dim3(T, nh + nkv), dim3(64), 0, (hipStream_t)stream, rows,
                       dt, row_len, k_off, v_off, cos_sin, rot, pairing, unit_norm, eps, q_scale, row_pos, row_slot,
                       kcache, vcache, page_table, table_stride, page_size, ring, nh, nkv, dk, dv);
    return illm_launch_status();
}

// ---------------------------------------------------------------- pooled rows of completed blocks
// grid (rows, nkv); 256 threads.  The row at position p completes block p / pool if (p + 1) % pool
// == 0: its block's keys and values, which the cache holds by now, are averaged in position order.
__global__ void __launch_bounds__(256)
pool_store_kernel(const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
                  const void* __restrict__ kcache, const void* __restrict__ vcache,
                  void* __restrict__ kpool, void* __restrict__ vpool, int dt,
                  const int32_t* __restrict__ page_table, int table_stride, int page_size, int nkv,
                  int dk, int dv, int pool) {
    const int t = blockIdx.x, g = blockIdx.y, d = threadIdx.x;
    const int pos = row_pos[t];
    if ((pos + 1) % pool != 0) return;
    const int slot = row_slot[t], b = pos / pool;
    const float inv = 1.0f / (float)pool;
    if (d < dk) {
        float s = 0.f;
        for (int j = 0; j < pool; ++j)
            s += ld_f(kcache, dt, cache_row_offset(page_table, table_stride, slot, b * pool + j, page_size, 0, nkv, g, dk) + d);
        st_f(kpool, dt, cache_row_offset(page_table, table_stride, slot, b, page_size, 0, nkv, g, dk) + d, s * inv);
    }
    if (d < dv) {
        float s = 0.f;
        for (int j = 0; j < pool; ++j)
            s += ld_f(vcache, dt, cache_row_offset(page_table, table_stride, slot, b * pool + j, page_size, 0, nkv, g, dv) + d);
        st_f(vpool, dt, cache_row_offset(page_table, table_stride, slot, b, page_size, 0, nkv, g, dv) + d, s * inv);
    }
}

extern "C" int illm_pool_store(const int32_t* row_pos, const int32_t* row_slot, const void* kcache,
                               const void* vcache, void* kpool, void* vpool, int dt,
                               const int32_t* page_table, int table_stride, int page_size, int T,
                               int nkv, int dk, int dv, int pool, void* stream) {
    if (T < 0 || nkv <= 0 || nkv > 65535 || dk <= 0 || dk > 256 || dv <= 0 || dv > 256 || pool <= 0 ||
        page_size <= 0 || !illm_dtype_ok(dt))
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(pool_store_kernel, dim3(T, nkv), dim3(256), 0, (hipStream_t)stream, row_pos,
                       row_slot, kcache, vcache, kpool, vpool, dt, page_table, table_stride, page_size, nkv,
                       dk, dv, pool);
    return illm_launch_status();
}

// blocks that position `pos` sees: those whose last token is at most pos - window
__device__ __forceinline__ int blocks_seen(int pos, int window, int pool) {
    const int n = pos - window + 1;
    return n >= pool ? n / pool : 0;
}

// ---------------------------------------------------------------- rows of a step over the cache
// grid (query tiles, heads, sequences); 256 threads: 8 a query row.  Row r of sequence b stands at
// position seq_start[b] + r.  Two passes over tiles of 32 keys with one running softmax: the pooled
// rows that the tile's last row sees, then the tokens from the first row's window on.  Dynamic LDS:
// (PQ + PK) (dk + 1) + PK (dv + 1) + PQ (PK + 1) floats.
__global__ void __launch_bounds__(256)
attn_pooled_rows_kernel(const void* __restrict__ q, int q_stride, void* __restrict__ out, int dt,
                        const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_slot,
                        const int32_t* __restrict__ seq_start, const void* __restrict__ kcache,
                        const void* __restrict__ vcache, const void* __restrict__ kpool,
                        const void* __restrict__ vpool, const int32_t* __restrict__ page_table,
                        int table_stride, int page_size, int nh, int nkv, int dk, int dv, float scale,
                        const float* __restrict__ head_scale, int window, int pool,
                        const float* __restrict__ lse) {
    extern __shared__ float smem[];
    const int kp = dk + 1, vp = dv + 1;
    float* qs = smem;               // [PQ][kp]
    float* ks = qs + PQ * kp;       // [PK][kp]
    float* vs = ks + PK * kp;       // [PK][vp]
    float* ps = vs + PK * vp;       // [PQ][PK + 1]
    const int b = blockIdx.z, h = blockIdx.y;
    const int start = cu[b], len = cu[b + 1] - start;
    const int q0 = blockIdx.x * PQ;
    if (q0 >= len) return;
    const int pos0 = seq_start[b], slot = seq_slot[b];
    const int total = pos0 + len;
    const int kvh = h / (nh / nkv);
    const int tid = threadIdx.x, i = tid >> 3, g = tid & 7;
    const float sc = scale * (head_scale ? head_scale[h] : 1.f);

    for (int e = tid; e < PQ * dk; e += 256) {
        const int r = e / dk, d = e - r * dk;
        qs[r * kp + d] = (q0 + r < len) ? ld_f(q, dt, (size_t)(start + q0 + r) * q_stride + (size_t)h * dk + d) : 0.f;
    }
    float m_i = NEG_INF, l_i = 0.f;
    float acc[32];
#pragma unroll
    for (int k = 0; k < 32; ++k) acc[k] = 0.f;
    const int qrow = q0 + i, qpos = pos0 + qrow;
    const int last_pos = min(total, pos0 + q0 + PQ) - 1;
    const int seen_i = pool > 0 ? blocks_seen(qpos, window, pool) : 0;
    if (lse) {
        // the tokens of the window are done: `out` holds their normalised sums and `lse` max +
        // log(sum) of their softmax, which is a running softmax with that max and a sum of 1
        if (blocks_seen(last_pos, window, pool) == 0) return;       // no row of the tile sees a block
        if (qrow < len) {
            m_i = lse[(size_t)(start + qrow) * nh + h];
            l_i = 1.f;
            const size_t ob = (size_t)(start + qrow) * nh * dv + (size_t)h * dv;
#pragma unroll
            for (int k = 0; k < 32; ++k) {
                const int d = g + 8 * k;
                if (d < dv) acc[k] = ld_f(out, dt, ob + d);
            }
        }
    }

    for (int pass = 0; pass < (lse ? 1 : 2); ++pass) {
        const void* kc = pass == 0 ? kpool : kcache;
        const void* vc = pass == 0 ? vpool : vcache;
        int lo, hi;
        if (pass == 0) {
            lo = 0;
            hi = pool > 0 ? blocks_seen(last_pos, window, pool) : 0;
        } else {
            lo = (max(0, pos0 + q0 - window + 1) / PK) * PK;
            hi = last_pos + 1;
        }
        for (int k0 = lo; k0 < hi; k0 += PK) {
            __syncthreads();
            for (int e = tid; e < PK * dk; e += 256) {
                const int r = e / dk, d = e - r * dk;
                ks[r * kp + d] = k0 + r < hi
                    ? ld_f(kc, dt, cache_row_offset(page_table, table_stride, slot, k0 + r, page_size, 0, nkv, kvh, dk) + d)
                    : 0.f;
            }
            for (int e = tid; e < PK * dv; e += 256) {
                const int r = e / dv, d = e - r * dv;
                vs[r * vp + d] = k0 + r < hi
                    ? ld_f(vc, dt, cache_row_offset(page_table, table_stride, slot, k0 + r, page_size, 0, nkv, kvh, dv) + d)
                    : 0.f;
            }
            __syncthreads();
            float s[4];
            float tm = NEG_INF;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int j = g + 8 * c, kj = k0 + j;
                float a = 0.f;
                for (int d = 0; d < dk; ++d) a = fmaf(qs[i * kp + d], ks[j * kp + d], a);
                const bool ok = qrow < len && (pass == 0 ? kj < seen_i : (kj <= qpos && kj > qpos - window));
                s[c] = ok ? a * sc : NEG_INF;
                tm = fmaxf(tm, s[c]);
            }
            tm = fmaxf(tm, __shfl_xor(tm, 1, ILLM_WAVE));
            tm = fmaxf(tm, __shfl_xor(tm, 2, ILLM_WAVE));
            tm = fmaxf(tm, __shfl_xor(tm, 4, ILLM_WAVE));
            const float m_new = fmaxf(m_i, tm);
            const float alpha = (m_new == NEG_INF) ? 1.f : expf(m_i - m_new);
            float psum = 0.f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float p = (s[c] == NEG_INF) ? 0.f : expf(s[c] - m_new);
                ps[i * (PK + 1) + g + 8 * c] = p;
                psum += p;
            }
            psum += __shfl_xor(psum, 1, ILLM_WAVE);
            psum += __shfl_xor(psum, 2, ILLM_WAVE);
            psum += __shfl_xor(psum, 4, ILLM_WAVE);
            l_i = l_i * alpha + psum;
            m_i = m_new;
            __syncthreads();
#pragma unroll
            for (int k = 0; k < 32; ++k) {
                const int d = g + 8 * k;
                if (d < dv) {
                    float a = acc[k] * alpha;
                    for (int j = 0; j < PK; ++j) a = fmaf(ps[i * (PK + 1) + j], vs[j * vp + d], a);
                    acc[k] = a;
                }
            }
        }
    }
    if (qrow < len) {
        const float inv = 1.0f / l_i;
        const size_t ob = (size_t)(start + qrow) * nh * dv + (size_t)h * dv;
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            const int d = g + 8 * k;
            if (d < dv) st_f(out, dt, ob + d, acc[k] * inv);
        }
    }
}

extern "C" int illm_attn_pooled_rows(const void* q, int q_stride, void* out, int dt, const int32_t* cu,
                                     const int32_t* seq_slot, const int32_t* seq_start,
                                     const void* kcache, const void* vcache, const void* kpool,
                                     const void* vpool, const int32_t* page_table, int table_stride,
                                     int page_size, int n_seqs, int max_rows, int nh, int nkv, int dk,
                                     int dv, float scale, const float* head_scale, int window, int pool,
                                     const float* lse, void* stream) {
    if (n_seqs < 0 || max_rows < 0 || nh <= 0 || nkv <= 0 || nh % nkv || dk <= 0 || dk > 256 || dv <= 0 ||
        dv > 256 || page_size <= 0 || !illm_dtype_ok(dt) || nh > 65535 || n_seqs > 65535 || window <= 0 ||
        pool < 0 || (pool > 0 && (!kpool || !vpool)) || nh * dk > q_stride || (lse && pool <= 0))
        return ILLM_ERR_ARG;
    if (n_seqs == 0 || max_rows == 0) return ILLM_OK;
    const size_t lds = ((size_t)(PQ + PK) * (dk + 1) + (size_t)PK * (dv + 1) + PQ * (PK + 1)) * sizeof(float);
    if (lds > 48 * 1024 &&
        hipFuncSetAttribute((const void*)attn_pooled_rows_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
        return ILLM_ERR_LAUNCH;
    hipLaunchKernelGGL(attn_pooled_rows_kernel, dim3((max_rows + PQ - 1) / PQ, nh, n_seqs), dim3(256), lds,
                       (hipStream_t)stream, q, q_stride, out, dt, cu, seq_slot, seq_start, kcache, vcache,
                       kpool, vpool, page_table, table_stride, page_size, nh, nkv, dk, dv, scale, head_scale,
                       window, pool, lse);
    return illm_launch_status();
}

// ---------------------------------------------------------------- single tokens
// grid (heads, sequences); 256 threads.  The new token at position len - 1 sees `seen` pooled rows
// and the last min(window, len) tokens: one list of seen + tokens keys, of which a wave takes four
// at a time in turn with the block's other waves, lane l holding dims l, l + 64, ... of the query
// and of its sums.  The waves' (sums, max, weight) are combined in wave order.
__global__ void __launch_bounds__(256)
attn_pooled_decode_kernel(const void* __restrict__ q, int q_stride, void* __restrict__ out, int dt,
                          const void* __restrict__ kcache, const void* __restrict__ vcache,
                          const void* __restrict__ kpool, const void* __restrict__ vpool,
                          const int32_t* __restrict__ page_table, int table_stride, int page_size,
                          const int32_t* __restrict__ seq_slot, const int32_t* __restrict__ seq_len,
                          int nh, int nkv, int dk, int dv, float scale,
                          const float* __restrict__ head_scale, int window, int pool,
                          const float* __restrict__ lse) {
    __shared__ float wacc[4][256];
    __shared__ float wm[4], wl[4];
    const int h = blockIdx.x, b = blockIdx.y;
    const int w = wave_index(), lane = threadIdx.x & 63;
    const int len = seq_len[b], slot = seq_slot[b];
    const int kvh = h / (nh / nkv);
    const int seen = pool > 0 ? blocks_seen(len - 1, window, pool) : 0;
    const int lo = max(0, len - window);
    // with `lse` the window's tokens are done (`out` and `lse` hold their softmax): the pooled rows alone
    if (lse && seen == 0) return;
    const int n_keys = lse ? seen : seen + (len - lo);
    const float sc = scale * (head_scale ? head_scale[h] : 1.f);
    float qv[4], acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int d = lane + 64 * c;
        qv[c] = d < dk ? ld_f(q, dt, (size_t)b * q_stride + (size_t)h * dk + d) * sc : 0.f;
        acc[c] = 0.f;
    }
    float m = NEG_INF, l = 0.f;
    for (int k0 = 4 * w; k0 < n_keys; k0 += 16) {
        float s[4];
        size_t vat[4];
        const void* vsrc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int kj = min(k0 + j, n_keys - 1);
            const bool pooled = kj < seen;
            const int row = pooled ? kj : lo + (kj - seen);
            const void* kc = pooled ? kpool : kcache;
            vsrc[j] = pooled ? vpool : vcache;
            const size_t kat = cache_row_offset(page_table, table_stride, slot, row, page_size, 0, nkv, kvh, dk);
            vat[j] = cache_row_offset(page_table, table_stride, slot, row, page_size, 0, nkv, kvh, dv);
            float a = 0.f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int d = lane + 64 * c;
                if (d < dk) a = fmaf(qv[c], ld_f(kc, dt, kat + d), a);
            }
            s[j] = a;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
#pragma unroll
            for (int j = 0; j < 4; ++j) s[j] += __shfl_xor(s[j], o, 64);
        }
        float tm = NEG_INF;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (k0 + j >= n_keys) s[j] = NEG_INF;
            tm = fmaxf(tm, s[j]);
        }
        const float m_new = fmaxf(m, tm);
        const float alpha = expf(m - m_new);             // m_new is finite: key k0 is in range
        l *= alpha;
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[c] *= alpha;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float p = s[j] == NEG_INF ? 0.f : expf(s[j] - m_new);
            l += p;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int d = lane + 64 * c;
                if (d < dv) acc[c] = fmaf(p, ld_f(vsrc[j], dt, vat[j] + d), acc[c]);
            }
        }
        m = m_new;
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) wacc[w][lane + 64 * c] = acc[c];
    if (lane == 0) { wm[w] = m; wl[w] = l; }
    __syncthreads();
    float mm = wm[0];
    for (int i = 1; i < 4; ++i) mm = fmaxf(mm, wm[i]);
    const float m0 = lse ? lse[(size_t)b * nh + h] : NEG_INF;       // the window's softmax: max m0, sum 1
    mm = fmaxf(mm, m0);
    float f[4], lt = 0.f;
    for (int i = 0; i < 4; ++i) {
        f[i] = wm[i] == NEG_INF ? 0.f : expf(wm[i] - mm);
        lt += f[i] * wl[i];
    }
    const float f0 = lse ? expf(m0 - mm) : 0.f;
    lt += f0;
    const float inv = 1.0f / lt;
    for (int d = threadIdx.x; d < dv; d += 256) {
        const size_t at = ((size_t)b * nh + h) * dv + d;
        float a = f[0] * wacc[0][d] + f[1] * wacc[1][d] + f[2] * wacc[2][d] + f[3] * wacc[3][d];
        if (lse) a += f0 * ld_f(out, dt, at);
        st_f(out, dt, at, a * inv);
    }
}

extern "C" int illm_attn_pooled_decode(const void* q, int q_stride, void* out, int dt,
                                       const void* kcache, const void* vcache, const void* kpool,
                                       const void* vpool, const int32_t* page_table, int table_stride,
                                       int page_size, const int32_t* seq_slot, const int32_t* seq_len,
                                       int B, int nh, int nkv, int dk, int dv, float scale,
                                       const float* head_scale, int window, int pool, const float* lse,
                                       void* stream) {
    if (B < 0 || nh <= 0 || nkv <= 0 || nh % nkv || dk <= 0 || dk > 256 || dv <= 0 || dv > 256 ||
        page_size <= 0 || !illm_dtype_ok(dt) || B > 65535 || window <= 0 || pool < 0 ||
        (pool > 0 && (!kpool || !vpool)) || nh * dk > q_stride || (lse && pool <= 0))
        return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
    hipLaunchKernelGGL(attn_pooled_decode_kernel, dim3(nh, B), dim3(256), 0, (hipStream_t)stream, q,
                       q_stride, out, dt, kcache, vcache, kpool, vpool, page_table, table_stride, page_size,
                       seq_slot, seq_len, nh, nkv, dk, dv, scale, head_scale, window, pool, lse);
    return illm_launch_status();
}
