// Causal attention whose scores pass a soft cap and whose keys and values have sizes of their own:
//     score = cap * tanh((q . k) * scale / cap)     (cap <= 0: no cap)
// softmax over the visible keys (all j <= i, or the last `window`), context = sum p_j v_j with
// values of width dv where queries and keys have width dk.  Three more things a caller may ask for:
// a bias by distance, score -= slopes[h] (i - j) (`slopes` null: none); chunks, position i sees only
// the keys of its own chunk, floor(j / chunk) = floor(i / chunk), counted from the sequence's
// position 0 (`chunk` <= 0: none); an output gate, out *= sigmoid(gate[row, gate_off + h dv + d])
// (`gate` null: none).  Positions enter through the bias and the chunks alone.
// Keys and values live in the paged cache, K [page][kv head][row][dk], V [page][kv head][row][dv],
// under one page table; a step first stores its rows (`kv_store2`) and then every row attends over
// the cache at absolute positions, so whole prompts, portions of prompts and single tokens take
// the same path.  Float32 arithmetic over float32 or bfloat16 storage; bfloat16 prompts with sizes
// in steps of 16 take the matrix-core kernel below.
#include <math.h>

#include "api.h"
#include "common.h"

#define CQ 32  // query rows of a block
#define CK 32  // keys of a tile
#define NEG_INF (-INFINITY)

__device__ __forceinline__ float soft_cap(float s, float cap, float inv_cap) {
    return cap > 0.f ? cap * tanhf(s * inv_cap) : s;
}

// ---------------------------------------------------------------- store
// rows [T, row_len]: k at k_off (nkv dk), v at v_off (nkv dv).  grid (rows); 256 threads.
__global__ void __launch_bounds__(256)
kv_store2_kernel(const void* __restrict__ rows, int dt, int row_len, int k_off, int v_off,
                 const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
                 void* __restrict__ kcache, void* __restrict__ vcache,
                 const int32_t* __restrict__ page_table, int table_stride, int page_size, int ring,
                 int nkv, int dk, int dv) {
    const size_t r = blockIdx.x;
    const int pos = row_pos[r], slot = row_slot[r];
    for (int e = threadIdx.x; e < nkv * dk; e += 256) {
        const int kvh = e / dk, d = e - kvh * dk;
        const size_t at = cache_row_offset(page_table, table_stride, slot, pos, page_size, ring, nkv, kvh, dk) + d;
        if (dt == ILLM_BF16) ((bf16_t*)kcache)[at] = ((const bf16_t*)rows)[r * row_len + k_off + e];
        else ((float*)kcache)[at] = ((const float*)rows)[r * row_len + k_off + e];
    }
    for (int e = threadIdx.x; e < nkv * dv; e += 256) {
        const int kvh = e / dv, d = e - kvh * dv;
        const size_t at = cache_row_offset(page_table, table_stride, slot, pos, page_size, ring, nkv, kvh, dv) + d;
        if (dt == ILLM_BF16) ((bf16_t*)vcache)[at] = ((const bf16_t*)rows)[r * row_len + v_off + e];
        else ((float*)vcache)[at] = ((const float*)rows)[r * row_len + v_off + e];
    }
}

extern "C" int illm_kv_store2(const void* rows, int dt, int row_len, int k_off, int v_off,
                              const int32_t* row_pos, const int32_t* row_slot, void* kcache,
                              void* vcache, const int32_t* page_table, int table_stride,
                              int page_size, int ring, int T, int nkv, int dk, int dv, void* stream) {
    if (T < 0 || nkv <= 0 || dk <= 0 || dv <= 0 || page_size <= 0 || !illm_dtype_ok(dt) ||
        k_off < 0 || v_off < 0 || k_off + nkv * dk > row_len || v_off + nkv * dv > row_len)
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(kv_store2_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, rows, dt, row_len,
                       k_off, v_off, row_pos, row_slot, kcache, vcache, page_table, table_stride,
                       page_size, ring, nkv, dk, dv);
    return illm_launch_status();
}

// ---------------------------------------------------------------- norms, value mixing and the store
// rows [T, row_len] = [q (nh dk) | ... k at k_off (nkv dk) | v at v_off (nkv dv)].  In place and in
// float32: q and k each divided by the root mean square over ALL their heads at once and multiplied
// by a weight of that whole width (`qw`, `kw`; null: left as they are), v <- (1 - lam) v + lam first
// with `first` [T, first_stride] + first_off the values another layer made of the same rows (`lam`
// one float on the device; null: no mixing).  Then k and v go into the paged cache (if given).
// grid (rows); 256 threads.
__global__ void __launch_bounds__(256)
qkv_norm_mix_store_kernel(void* __restrict__ rows, int dt, int row_len, int k_off, int v_off,
                          const void* __restrict__ qw, const void* __restrict__ kw, int w_dt, float eps,
                          const float* __restrict__ lam, const void* __restrict__ first, int first_stride,
                          int first_off, const int32_t* __restrict__ row_pos,
                          const int32_t* __restrict__ row_slot, void* __restrict__ kcache,
                          void* __restrict__ vcache, const int32_t* __restrict__ page_table,
                          int table_stride, int page_size, int ring, int nh, int nkv, int dk, int dv) {
    __shared__ float red[16];
    const size_t r = blockIdx.x, base = r * row_len;
    const int pos = row_pos[r], slot = row_slot[r];
    if (qw) {
        const int n = nh * dk;
        float ss = 0.f;
        for (int e = threadIdx.x; e < n; e += 256) { const float x = ld_f(rows, dt, base + e); ss += x * x; }
        ss = block_sum(ss, red);
        const float inv = 1.0f / sqrtf(ss / (float)n + eps);
        for (int e = threadIdx.x; e < n; e += 256)
            st_f(rows, dt, base + e, (ld_f(rows, dt, base + e) * inv) * ld_f(qw, w_dt, e));
    }
    float kinv = 1.0f;
    if (kw) {
        const int n = nkv * dk;
        float ss = 0.f;
        for (int e = threadIdx.x; e < n; e += 256) { const float x = ld_f(rows, dt, base + k_off + e); ss += x * x; }
        ss = block_sum(ss, red);
        kinv = 1.0f / sqrtf(ss / (float)n + eps);
    }
    for (int e = threadIdx.x; e < nkv * dk; e += 256) {
        float x = ld_f(rows, dt, base + k_off + e);
        if (kw) {
            x = (x * kinv) * ld_f(kw, w_dt, e);
            st_f(rows, dt, base + k_off + e, x);
        }
        if (kcache) {
            const int kvh = e / dk, d = e - kvh * dk;
            st_f(kcache, dt, cache_row_offset(page_table, table_stride, slot, pos, page_size, ring, nkv, kvh, dk) + d, x);
        }
    }
    const float l = lam ? lam[0] : 0.f;
    for (int e = threadIdx.x; e < nkv * dv; e += 256) {
        float x = ld_f(rows, dt, base + v_off + e);
        if (lam) {
            x = (1.0f - l) * x + l * ld_f(first, dt, r * first_stride + first_off + e);
            st_f(rows, dt, base + v_off + e, x);
        }
        if (vcache) {
            const int kvh = e / dv, d = e - kvh * dv;
            st_f(vcache, dt, cache_row_offset(page_table, table_stride, slot, pos, page_size, ring, nkv, kvh, dv) + d, x);
        }
    }
}

extern "C" int illm_qkv_norm_mix_store(void* rows, int dt, int row_len, int k_off, int v_off,
                                       const void* qw, const void* kw, int w_dt, float eps,
                                       const float* lam, const void* first, int first_stride,
                                       int first_off, const int32_t* row_pos, const int32_t* row_slot,
                                       void* kcache, void* vcache, const int32_t* page_table,
                                       int table_stride, int page_size, int ring, int T, int nh, int nkv,
                                       int dk, int dv, void* stream) {
    if (T < 0 || nh <= 0 || nkv <= 0 || dk <= 0 || dv <= 0 || page_size <= 0 || !illm_dtype_ok(dt) ||
        !illm_dtype_ok(w_dt) || k_off < nh * dk || v_off < 0 || k_off + nkv * dk > row_len ||
        v_off + nkv * dv > row_len || (lam && (!first || first_off < 0 || first_off + nkv * dv > first_stride)) ||
        ((kcache == nullptr) != (vcache == nullptr)))
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(qkv_norm_mix_store_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, rows, dt,
                       row_len, k_off, v_off, qw, kw, w_dt, eps, lam, first, first_stride, first_off, row_pos,
                       row_slot, kcache, vcache, page_table, table_stride, page_size, ring, nh, nkv, dk, dv);
    return illm_launch_status();
}

// ---------------------------------------------------------------- rows of a step over the cache
// grid (query tiles, heads, sequences); 256 threads: 8 a query row.  Row r of sequence b stands at
// position seq_start[b] + r.  q [T, q_stride] with head h at h dk.  Dynamic LDS:
// (CQ + CK) (dk + 1) + CK (dv + 1) + CQ (CK + 1) floats.
__global__ void __launch_bounds__(256)
attn_cap_rows_kernel(const void* __restrict__ q, int q_stride, void* __restrict__ out, int dt,
                     const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_slot,
                     const int32_t* __restrict__ seq_start, const void* __restrict__ kcache,
                     const void* __restrict__ vcache, const int32_t* __restrict__ page_table,
                     int table_stride, int page_size, int ring, int nh, int nkv, int dk, int dv,
                     float scale, float cap, int window, const float* __restrict__ slopes, int chunk,
                     const void* __restrict__ gate, int gate_stride, int gate_off) {
    extern __shared__ float smem[];
    const int kp = dk + 1, vp = dv + 1;
    float* qs = smem;               // [CQ][kp]
    float* ks = qs + CQ * kp;       // [CK][kp]
    float* vs = ks + CK * kp;       // [CK][vp]
    float* ps = vs + CK * vp;       // [CQ][CK + 1]
    const int b = blockIdx.z, h = blockIdx.y;
    const int start = cu[b], len = cu[b + 1] - start;
    const int q0 = blockIdx.x * CQ;
    if (q0 >= len) return;
    const int pos0 = seq_start[b], slot = seq_slot[b];
    const int total = pos0 + len;
    const int kvh = h / (nh / nkv);
    const int tid = threadIdx.x, i = tid >> 3, g = tid & 7;
    const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;

    for (int e = tid; e < CQ * dk; e += 256) {
        const int r = e / dk, d = e - r * dk;
        qs[r * kp + d] = (q0 + r < len) ? ld_f(q, dt, (size_t)(start + q0 + r) * q_stride + (size_t)h * dk + d) : 0.f;
    }
    float m_i = NEG_INF, l_i = 0.f;
    float acc[32];
#pragma unroll
    for (int k = 0; k < 32; ++k) acc[k] = 0.f;
    const int qrow = q0 + i, qpos = pos0 + qrow;
    const int k_hi = min(total, pos0 + q0 + CQ);
    int k_lo = window > 0 ? max(0, pos0 + q0 - window + 1) : 0;
    if (chunk > 0) k_lo = max(k_lo, ((pos0 + q0) / chunk) * chunk);     // the block's first row sees farthest back
    k_lo = (k_lo / CK) * CK;
    const float slope = slopes ? slopes[h] : 0.f;
    const int c_lo = chunk > 0 ? (qpos / chunk) * chunk : 0;            // first key of this row's chunk

    for (int k0 = k_lo; k0 < k_hi; k0 += CK) {
        __syncthreads();
        for (int e = tid; e < CK * dk; e += 256) {
            const int r = e / dk, d = e - r * dk;
            ks[r * kp + d] = k0 + r < total
                ? ld_f(kcache, dt, cache_row_offset(page_table, table_stride, slot, k0 + r, page_size, ring, nkv, kvh, dk) + d)
                : 0.f;
        }
        for (int e = tid; e < CK * dv; e += 256) {
            const int r = e / dv, d = e - r * dv;
            vs[r * vp + d] = k0 + r < total
                ? ld_f(vcache, dt, cache_row_offset(page_table, table_stride, slot, k0 + r, page_size, ring, nkv, kvh, dv) + d)
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
            const bool ok = qrow < len && kj <= qpos && kj >= c_lo && (window <= 0 || kj > qpos - window);
            s[c] = ok ? soft_cap(a * scale, cap, inv_cap) - slope * (float)(qpos - kj) : NEG_INF;
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
            ps[i * (CK + 1) + g + 8 * c] = p;
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
                for (int j = 0; j < CK; ++j) a = fmaf(ps[i * (CK + 1) + j], vs[j * vp + d], a);
                acc[k] = a;
            }
        }
    }
    if (qrow < len) {
        const float inv = 1.0f / l_i;
        const size_t ob = (size_t)(start + qrow) * nh * dv + (size_t)h * dv;
        const size_t gb = (size_t)(start + qrow) * gate_stride + gate_off + (size_t)h * dv;
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            const int d = g + 8 * k;
            if (d < dv) {
                float y = acc[k] * inv;
                if (gate) y *= 1.0f / (1.0f + expf(-ld_f(gate, dt, gb + d)));
                st_f(out, dt, ob + d, y);
            }
        }
    }
}

extern "C" int illm_attn_cap_rows(const void* q, int q_stride, void* out, int dt, const int32_t* cu,
                                  const int32_t* seq_slot, const int32_t* seq_start,
                                  const void* kcache, const void* vcache, const int32_t* page_table,
                                  int table_stride, int page_size, int ring, int n_seqs, int max_rows,
                                  int nh, int nkv, int dk, int dv, float scale, float cap, int window,
                                  const float* slopes, int chunk, const void* gate, int gate_stride,
                                  int gate_off, void* stream) {
    if (gate && (gate_off < 0 || gate_off + nh * dv > gate_stride)) return ILLM_ERR_ARG;
    if (n_seqs < 0 || max_rows < 0 || nh <= 0 || nkv <= 0 || nh % nkv || dk <= 0 || dk > 256 ||
        dv <= 0 || dv > 256 || page_size <= 0 || !illm_dtype_ok(dt) || nh > 65535 || n_seqs > 65535)
        return ILLM_ERR_ARG;
    if (n_seqs == 0 || max_rows == 0) return ILLM_OK;
    const size_t lds = ((size_t)(CQ + CK) * (dk + 1) + (size_t)CK * (dv + 1) + CQ * (CK + 1)) * sizeof(float);
    if (lds > 48 * 1024 &&
        hipFuncSetAttribute((const void*)attn_cap_rows_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
        return ILLM_ERR_LAUNCH;
    hipLaunchKernelGGL(attn_cap_rows_kernel, dim3((max_rows + CQ - 1) / CQ, nh, n_seqs), dim3(256), lds,
                       (hipStream_t)stream, q, q_stride, out, dt, cu, seq_slot, seq_start, kcache, vcache,
                       page_table, table_stride, page_size, ring, nh, nkv, dk, dv, scale, cap, window, slopes,
                       chunk, gate, gate_stride, gate_off);
    return illm_launch_status();
}

// ---------------------------------------------------------------- single tokens
// grid (heads, sequences, splits); 256 threads.  A split takes a range of whole tiles of 64 keys;
// a wave takes four keys at a time in turn with the block's other waves, lane l holding dims l,
// l + 64, ... of the query and of its sums (rows are read whole lines an instruction).  The waves'
// (sums, max, weight) are combined in wave order; each block leaves (acc[dv], max, sum) in
// `partial` [B][nh][nsplit][dv + 2], which the merge kernel combines in split order.
template <int DT>
__global__ void __launch_bounds__(256)
attn_cap_decode_kernel(const void* __restrict__ q, int q_stride, const void* __restrict__ kcache,
                       const void* __restrict__ vcache, const int32_t* __restrict__ page_table,
                       int table_stride, int page_size, int ring, const int32_t* __restrict__ seq_slot,
                       const int32_t* __restrict__ seq_len, float* __restrict__ partial, int nsplit,
                       int nh, int nkv, int dk, int dv, float scale, float cap, int window,
                       const float* __restrict__ slopes, int chunk) {
    __shared__ float wacc[4][256];
    __shared__ float wm[4], wl[4];
    const int h = blockIdx.x, b = blockIdx.y, sp = blockIdx.z;
    const int w = wave_index(), lane = threadIdx.x & 63;
    const int len = seq_len[b], slot = seq_slot[b];
    const int kvh = h / (nh / nkv);
    int lo_all = window > 0 ? max(0, len - window) : 0;
    if (chunk > 0) lo_all = max(lo_all, ((len - 1) / chunk) * chunk);   // the new token's own chunk
    const float slope = slopes ? slopes[h] : 0.f;
    const int tiles = (len + 63) / 64, t0 = lo_all / 64;
    const int per = (tiles - t0 + nsplit - 1) / nsplit;
    const int k_lo = max(lo_all, (t0 + sp * per) * 64), k_hi = min(len, (t0 + (sp + 1) * per) * 64);
    const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;
    float qv[4], acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int d = lane + 64 * c;
        qv[c] = d < dk ? (DT == ILLM_BF16 ? bf16_to_f32(((const bf16_t*)q)[(size_t)b * q_stride + (size_t)h * dk + d])
                                          : ((const float*)q)[(size_t)b * q_stride + (size_t)h * dk + d]) * scale
                       : 0.f;
        acc[c] = 0.f;
    }
    float m = NEG_INF, l = 0.f;
    for (int k0 = k_lo + 4 * w; k0 < k_hi; k0 += 16) {
        float s[4];
        size_t vat[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int kj = min(k0 + j, k_hi - 1);
            const size_t kat = cache_row_offset(page_table, table_stride, slot, kj, page_size, ring, nkv, kvh, dk);
            vat[j] = cache_row_offset(page_table, table_stride, slot, kj, page_size, ring, nkv, kvh, dv);
            float a = 0.f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int d = lane + 64 * c;
                if (d < dk)
                    a = fmaf(qv[c], DT == ILLM_BF16 ? bf16_to_f32(((const bf16_t*)kcache)[kat + d])
                                                    : ((const float*)kcache)[kat + d], a);
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
            s[j] = k0 + j < k_hi ? soft_cap(s[j], cap, inv_cap) - slope * (float)(len - 1 - (k0 + j)) : NEG_INF;
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
                if (d < dv)
                    acc[c] = fmaf(p, DT == ILLM_BF16 ? bf16_to_f32(((const bf16_t*)vcache)[vat[j] + d])
                                                     : ((const float*)vcache)[vat[j] + d], acc[c]);
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
    float f[4], lt = 0.f;
    for (int i = 0; i < 4; ++i) {
        f[i] = wm[i] == NEG_INF ? 0.f : expf(wm[i] - mm);
        lt += f[i] * wl[i];
    }
    float* pp = partial + (((size_t)b * nh + h) * nsplit + sp) * (dv + 2);
    for (int d = threadIdx.x; d < dv; d += 256)
        pp[d] = f[0] * wacc[0][d] + f[1] * wacc[1][d] + f[2] * wacc[2][d] + f[3] * wacc[3][d];
    if (threadIdx.x == 0) { pp[dv] = mm; pp[dv + 1] = lt; }
}

// grid (heads, sequences): combine the splits' partial results in split order.
__global__ void attn_cap_merge_kernel(const float* __restrict__ partial, void* __restrict__ out,
                                      int dt, int nsplit, int nh, int dv, const void* __restrict__ gate,
                                      int gate_stride, int gate_off) {
    const int h = blockIdx.x, b = blockIdx.y;
    const float* pp = partial + ((size_t)b * nh + h) * nsplit * (dv + 2);
    float mm = NEG_INF;
    for (int s = 0; s < nsplit; ++s) mm = fmaxf(mm, pp[(size_t)s * (dv + 2) + dv]);
    float lt = 0.f;
    for (int s = 0; s < nsplit; ++s) {
        const float ms = pp[(size_t)s * (dv + 2) + dv];
        lt += (ms == NEG_INF ? 0.f : expf(ms - mm)) * pp[(size_t)s * (dv + 2) + dv + 1];
    }
    const float inv = 1.0f / lt;
    for (int d = threadIdx.x; d < dv; d += blockDim.x) {
        float a = 0.f;
        for (int s = 0; s < nsplit; ++s) {
            const float ms = pp[(size_t)s * (dv + 2) + dv];
            a += (ms == NEG_INF ? 0.f : expf(ms - mm)) * pp[(size_t)s * (dv + 2) + d];
        }
        float y = a * inv;
        if (gate) y *= 1.0f / (1.0f + expf(-ld_f(gate, dt, (size_t)b * gate_stride + gate_off + (size_t)h * dv + d)));
        st_f(out, dt, ((size_t)b * nh + h) * dv + d, y);
    }
}

extern "C" int illm_attn_cap_decode(const void* q, int q_stride, void* out, int dt,
                                    const void* kcache, const void* vcache,
                                    const int32_t* page_table, int table_stride, int page_size,
                                    int ring, const int32_t* seq_slot, const int32_t* seq_len,
                                    float* partial, int nsplit, int B, int nh, int nkv, int dk, int dv,
                                    float scale, float cap, int window, const float* slopes, int chunk,
                                    const void* gate, int gate_stride, int gate_off, void* stream) {
    if (gate && (gate_off < 0 || gate_off + nh * dv > gate_stride)) return ILLM_ERR_ARG;
    if (B < 0 || nh <= 0 || nkv <= 0 || nh % nkv || dk <= 0 || dk > 256 || dv <= 0 || dv > 256 ||
        page_size <= 0 || nsplit < 1 || nsplit > 65535 || B > 65535 || !illm_dtype_ok(dt) || !partial)
        return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dt == ILLM_BF16)
        hipLaunchKernelGGL(attn_cap_decode_kernel<ILLM_BF16>, dim3(nh, B, nsplit), dim3(256), 0, st, q,
                           q_stride, kcache, vcache, page_table, table_stride, page_size, ring, seq_slot,
                           seq_len, partial, nsplit, nh, nkv, dk, dv, scale, cap, window, slopes, chunk);
    else
        hipLaunchKernelGGL(attn_cap_decode_kernel<ILLM_F32>, dim3(nh, B, nsplit), dim3(256), 0, st, q,
                           q_stride, kcache, vcache, page_table, table_stride, page_size, ring, seq_slot,
                           seq_len, partial, nsplit, nh, nkv, dk, dv, scale, cap, window, slopes, chunk);
    if (hipGetLastError() != hipSuccess) return ILLM_ERR_LAUNCH;
    hipLaunchKernelGGL(attn_cap_merge_kernel, dim3(nh, B), dim3(64), 0, st, partial, out, dt, nsplit, nh, dv,
                       gate, gate_stride, gate_off);
    return illm_launch_status();
}
