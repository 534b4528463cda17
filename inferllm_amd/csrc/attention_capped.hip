// Causal attention whose scores pass a soft cap and whose keys and values have sizes of their own:
//     score = cap * tanh((q . k) * scale / cap)     (cap <= 0: no cap)
// softmax over the visible keys (all j <= i, or the last `window`), context = sum p_j v_j with
// values of width dv where queries and keys have width dk.  Three more things a caller may ask for:
// a bias by distance, score -= slopes[h] (i - j) (`slopes` null: none); chunks, position i sees only
// the keys of its own chunk, floor(j / chunk) = floor(i / chunk), counted from the sequence's
// position 0 (`chunk` <= 0: none); an output gate, out *= sigmoid(gate[row, gate_off + h dv + d])
// (`gate` null: none; with `gate_heads` one number a head, gate[row, gate_off + h]).  Positions enter
// through the bias and the chunks alone.  `lse` (null: none) takes max + log(sum) of every row's and
// head's softmax, [rows][heads], for whoever goes on with further keys.
// Keys and values live in the paged cache, K [page][kv head][row][dk], V [page][kv head][row][dv],
// under one page table; a step first stores its rows (`kv_store2`) and then every row attends over
// the cache at absolute positions, so whole prompts, portions of prompts and single tokens take
// the same path.  Float32 arithmetic over float32 or bfloat16 storage: widths of up to 128 in steps
// of 4 (single tokens: of 16 bytes) take the kernels on the matrix cores' float32 instruction and
// with eight lanes a key, every other width the plain ones on the vector units.
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
                     const void* __restrict__ gate, int gate_stride, int gate_off, int gate_heads,
                     float* __restrict__ lse) {
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
        if (lse && g == 0) lse[(size_t)(start + qrow) * nh + h] = m_i + logf(l_i);
        const size_t ob = (size_t)(start + qrow) * nh * dv + (size_t)h * dv;
        const size_t gb = (size_t)(start + qrow) * gate_stride + gate_off + (size_t)h * (gate_heads ? 1 : dv);
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            const int d = g + 8 * k;
            if (d < dv) {
                float y = acc[k] * inv;
                if (gate) y *= 1.0f / (1.0f + expf(-ld_f(gate, dt, gb + (gate_heads ? 0 : d))));
                st_f(out, dt, ob + d, y);
            }
        }
    }
}

// ---------------------------------------------------------------- the same rows on the matrix cores
// Key and value widths of up to 128 in steps of 4: both products on the float32 instruction of the
// matrix cores (MFMA 32x32x2: float32 operands, products and sums), so scores and weights stay
// float32 whatever the storage.  grid (tiles of 128 queries, heaviest first; heads; sequences); a
// wave takes 32 queries.  Both products are kept transposed so that a lane's column is its query:
// scores^T = K . Q^T puts the 16 scores of query (lane % 32) into a lane and its partner 32 lanes on
// (max and sum: one exchange), and in context^T = V^T . P^T the lane's own 16 weights are the second
// operand as they stand.  Keys and values go through LDS 32 keys at a time as float32, widths filled
// up with zeros to whole tiles of 32 (KT, VT); the next tile's loads are in flight while this one is
// multiplied.  A wave leaves out tiles that none of its rows sees (after them, before their window or
// before their chunk).
typedef float cap_f32x16_t __attribute__((ext_vector_type(16)));
#define MQ 128  // query rows of a block
#define MK 32   // keys of a tile

// Four elements as they are stored (8 bytes of bfloat16 or 16 of float32), kept raw while the load
// is in flight: whoever turns them into floats waits for the load, so that is left to the user.
typedef uint32_t cap_u32x2_t __attribute__((ext_vector_type(2)));
template <int DT> struct Raw4;
template <> struct Raw4<ILLM_BF16> {
    cap_u32x2_t r;
    __device__ __forceinline__ void zero() { r.x = r.y = 0u; }
    __device__ __forceinline__ void load(const void* p, size_t at) { r = *(const cap_u32x2_t*)((const bf16_t*)p + at); }
    __device__ __forceinline__ void floats(float* x) const {
        x[0] = __uint_as_float(r.x << 16); x[1] = __uint_as_float(r.x & 0xffff0000u);
        x[2] = __uint_as_float(r.y << 16); x[3] = __uint_as_float(r.y & 0xffff0000u);
    }
};
template <> struct Raw4<ILLM_F32> {
    illm_u32x4_t r;
    __device__ __forceinline__ void zero() { r.x = r.y = r.z = r.w = 0u; }
    __device__ __forceinline__ void load(const void* p, size_t at) { r = *(const illm_u32x4_t*)((const float*)p + at); }
    __device__ __forceinline__ void floats(float* x) const {
        x[0] = __uint_as_float(r.x); x[1] = __uint_as_float(r.y); x[2] = __uint_as_float(r.z); x[3] = __uint_as_float(r.w);
    }
};

template <int DT>
__device__ __forceinline__ void ld4(const void* p, size_t at, float* x) {
    if (DT == ILLM_BF16) {
        const uint2 r = *(const uint2*)((const bf16_t*)p + at);
        x[0] = __uint_as_float(r.x << 16); x[1] = __uint_as_float(r.x & 0xffff0000u);
        x[2] = __uint_as_float(r.y << 16); x[3] = __uint_as_float(r.y & 0xffff0000u);
    } else {
        const float4 r = *(const float4*)((const float*)p + at);
        x[0] = r.x; x[1] = r.y; x[2] = r.z; x[3] = r.w;
    }
}

template <int DT, int KT, int VT>
__global__ void __launch_bounds__(256, 2)
attn_cap_rows_mfma_kernel(const void* __restrict__ q, int q_stride, void* __restrict__ out,
                          const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_slot,
                          const int32_t* __restrict__ seq_start, const void* __restrict__ kcache,
                          const void* __restrict__ vcache, const int32_t* __restrict__ page_table,
                          int table_stride, int page_size, int ring, int nh, int nkv, int dk, int dv,
                          float scale, float cap, int window, const float* __restrict__ slopes, int chunk,
                          const void* __restrict__ gate, int gate_stride, int gate_off, int gate_heads,
                          float* __restrict__ lse) {
    constexpr int DKP = 32 * KT, DVP = 32 * VT, KLD = DKP + 1;
    __shared__ float ks[MK * KLD];
    __shared__ float vs[MK * DVP];
    const int b = blockIdx.z, h = blockIdx.y;
    const int start = cu[b], len = cu[b + 1] - start;
    const int q0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * MQ;
    if (q0 >= len) return;
    const int pos0 = seq_start[b], slot = seq_slot[b];
    const int total = pos0 + len;
    const int kvh = h / (nh / nkv);
    const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
    const int col = lane & 31, half = lane >> 5;
    const int qrow = q0 + 32 * wave + col;                 // row within the step's rows of the sequence
    const int qpos = pos0 + qrow;
    const bool wave_has_rows = q0 + 32 * wave < len;
    const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;
    const float slope = slopes ? slopes[h] : 0.f;

    // the query row: dims 2 s + half (zeros beyond dk)
    float qr[DKP / 2];
    {
        const size_t at = (size_t)(start + min(qrow, len - 1)) * q_stride + (size_t)h * dk;
#pragma unroll
        for (int j = 0; j < DKP / 4; ++j) {
            float x[4] = {0.f, 0.f, 0.f, 0.f};
            if (4 * j < dk) ld4<DT>(q, at + 4 * j, x);
            qr[2 * j] = half ? x[1] : x[0];
            qr[2 * j + 1] = half ? x[3] : x[2];
        }
    }
    // a thread's share of a tile: quads e = tid + 256 i of [32 keys][DKP / 4] and of [32 keys][DVP / 4]
    Raw4<DT> kreg[KT], vreg[VT];                   // (raw: turned into floats when they are staged)
    auto fetch = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < KT; ++i) {
            const int e = tid + 256 * i, row = e / (DKP / 4), d = 4 * (e % (DKP / 4));
            const int kj = min(k0 + row, total - 1);       // keys past the end: a valid row, masked below
            kreg[i].zero();
            if (d < dk)
                kreg[i].load(kcache, cache_row_offset(page_table, table_stride, slot, kj, page_size, ring, nkv, kvh, dk) + d);
        }
#pragma unroll
        for (int i = 0; i < VT; ++i) {
            const int e = tid + 256 * i, row = e / (DVP / 4), d = 4 * (e % (DVP / 4));
            const int kj = min(k0 + row, total - 1);
            vreg[i].zero();
            if (d < dv)
                vreg[i].load(vcache, cache_row_offset(page_table, table_stride, slot, kj, page_size, ring, nkv, kvh, dv) + d);
        }
    };
    auto stage = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < KT; ++i) {
            const int e = tid + 256 * i, row = e / (DKP / 4), d = 4 * (e % (DKP / 4));
            kreg[i].floats(ks + row * KLD + d);
        }
#pragma unroll
        for (int i = 0; i < VT; ++i) {
            const int e = tid + 256 * i, row = e / (DVP / 4), d = 4 * (e % (DVP / 4));
            vreg[i].floats(vs + row * DVP + d);
        }
    };
    cap_f32x16_t o[VT];
#pragma unroll
    for (int t = 0; t < VT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[t][v] = 0.f;
    float m_i = NEG_INF, l_i = 0.f;

    const int k_hi = min(total, pos0 + q0 + MQ);
    int k_lo = window > 0 ? max(0, pos0 + q0 - window + 1) : 0;
    if (chunk > 0) k_lo = max(k_lo, ((pos0 + q0) / chunk) * chunk);
    k_lo = (k_lo / MK) * MK;
    const int wq_lo = pos0 + q0 + 32 * wave, wq_hi = wq_lo + 31;
    const int wc_lo = chunk > 0 ? (wq_lo / chunk) * chunk : 0;     // the wave's first row sees farthest back
    const int c_lo = chunk > 0 ? (qpos / chunk) * chunk : 0;
    const int k_last = k_lo + ((k_hi - 1 - k_lo) / MK) * MK;
    fetch(k_lo);
    for (int k0 = k_lo; k0 < k_hi; k0 += MK) {
        __syncthreads();
        stage();
        __syncthreads();
        fetch(min(k0 + MK, k_last));              // (unconditional: the last tile is asked for twice)
        if (!wave_has_rows || k0 > wq_hi || k0 + MK - 1 < wc_lo || (window > 0 && k0 + MK - 1 <= wq_lo - window))
            continue;
        cap_f32x16_t sc;
#pragma unroll
        for (int v = 0; v < 16; ++v) sc[v] = 0.f;
        const float* kr = ks + col * KLD + half;
#pragma unroll
        for (int s2 = 0; s2 < DKP / 2; ++s2)
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(kr[2 * s2], qr[s2], sc, 0, 0, 0);
        float tm = NEG_INF;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int kj = k0 + 8 * (v >> 2) + 4 * half + (v & 3);
            const bool ok = qrow < len && kj <= qpos && kj >= c_lo && (window <= 0 || kj > qpos - window);
            sc[v] = ok ? soft_cap(sc[v] * scale, cap, inv_cap) - slope * (float)(qpos - kj) : NEG_INF;
            tm = fmaxf(tm, sc[v]);
        }
        tm = fmaxf(tm, __shfl_xor(tm, 32, ILLM_WAVE));
        const float m_new = fmaxf(m_i, tm);
        const float alpha = (m_new == NEG_INF) ? 1.f : expf(m_i - m_new);
        float psum = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            sc[v] = (sc[v] == NEG_INF) ? 0.f : expf(sc[v] - m_new);
            psum += sc[v];
        }
        psum += __shfl_xor(psum, 32, ILLM_WAVE);
        l_i = l_i * alpha + psum;
        m_i = m_new;
#pragma unroll
        for (int t = 0; t < VT; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) o[t][v] *= alpha;
        const float* vr = vs + 4 * half * DVP + col;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = 8 * (v >> 2) + (v & 3);         // + 4 * half, in vr
#pragma unroll
            for (int t = 0; t < VT; ++t)
                o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(vr[key * DVP + 32 * t], sc[v], o[t], 0, 0, 0);
        }
    }
    if (qrow < len) {
        const float inv = 1.0f / l_i;
        if (lse && half == 0) lse[(size_t)(start + qrow) * nh + h] = m_i + logf(l_i);
        const size_t ob = (size_t)(start + qrow) * nh * dv + (size_t)h * dv;
        const size_t gb = (size_t)(start + qrow) * gate_stride + gate_off + (size_t)h * (gate_heads ? 1 : dv);
#pragma unroll
        for (int t = 0; t < VT; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int d = 32 * t + 8 * (v >> 2) + 4 * half + (v & 3);
                if (d < dv) {
                    float y = o[t][v] * inv;
                    if (gate) y *= 1.0f / (1.0f + expf(-ld_f(gate, DT, gb + (gate_heads ? 0 : d))));
                    st_f(out, DT, ob + d, y);
                }
            }
    }
}

static int g_attn_cap_mfma = 1;
extern "C" void illm_set_attn_cap_mfma(int on) { g_attn_cap_mfma = on ? 1 : 0; }
static int g_attn_cap_heads = 4;
extern "C" void illm_set_attn_cap_heads(int n) { g_attn_cap_heads = n == 2 ? 2 : 4; }

extern "C" int illm_attn_cap_rows(const void* q, int q_stride, void* out, int dt, const int32_t* cu,
                                  const int32_t* seq_slot, const int32_t* seq_start,
                                  const void* kcache, const void* vcache, const int32_t* page_table,
                                  int table_stride, int page_size, int ring, int n_seqs, int max_rows,
                                  int nh, int nkv, int dk, int dv, float scale, float cap, int window,
                                  const float* slopes, int chunk, const void* gate, int gate_stride,
                                  int gate_off, int gate_heads, float* lse, void* stream) {
    if (gate && (gate_off < 0 || gate_off + nh * (gate_heads ? 1 : dv) > gate_stride)) return ILLM_ERR_ARG;
    if (n_seqs < 0 || max_rows < 0 || nh <= 0 || nkv <= 0 || nh % nkv || dk <= 0 || dk > 256 ||
        dv <= 0 || dv > 256 || page_size <= 0 || !illm_dtype_ok(dt) || nh > 65535 || n_seqs > 65535)
        return ILLM_ERR_ARG;
    if (n_seqs == 0 || max_rows == 0) return ILLM_OK;
    if (g_attn_cap_mfma && dk <= 128 && dv <= 128 && dk % 4 == 0 && dv % 4 == 0 && q_stride % 4 == 0) {
        const dim3 grid((max_rows + MQ - 1) / MQ, nh, n_seqs);
        const int kt = (dk + 31) / 32, vt = (dv + 31) / 32;
#define GO(DT_, KT_, VT_)                                                                          \
    hipLaunchKernelGGL((attn_cap_rows_mfma_kernel<DT_, KT_, VT_>), grid, dim3(256), 0, (hipStream_t)stream, \
                       q, q_stride, out, cu, seq_slot, seq_start, kcache, vcache, page_table, table_stride, \
                       page_size, ring, nh, nkv, dk, dv, scale, cap, window, slopes, chunk, gate, gate_stride, gate_off, gate_heads, lse)
#define GO_V(DT_, KT_)                                                                             \
    switch (vt) { case 1: GO(DT_, KT_, 1); break; case 2: GO(DT_, KT_, 2); break;                  \
                  case 3: GO(DT_, KT_, 3); break; default: GO(DT_, KT_, 4); break; }
#define GO_K(DT_)                                                                                  \
    switch (kt) { case 1: GO_V(DT_, 1) break; case 2: GO_V(DT_, 2) break;                          \
                  case 3: GO_V(DT_, 3) break; default: GO_V(DT_, 4) break; }
        if (dt == ILLM_BF16) { GO_K(ILLM_BF16) } else { GO_K(ILLM_F32) }
#undef GO_K
#undef GO_V
#undef GO
        return illm_launch_status();
    }
    const size_t lds = ((size_t)(CQ + CK) * (dk + 1) + (size_t)CK * (dv + 1) + CQ * (CK + 1)) * sizeof(float);
    if (lds > 48 * 1024 &&
        hipFuncSetAttribute((const void*)attn_cap_rows_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
        return ILLM_ERR_LAUNCH;
    hipLaunchKernelGGL(attn_cap_rows_kernel, dim3((max_rows + CQ - 1) / CQ, nh, n_seqs), dim3(256), lds,
                       (hipStream_t)stream, q, q_stride, out, dt, cu, seq_slot, seq_start, kcache, vcache,
                       page_table, table_stride, page_size, ring, nh, nkv, dk, dv, scale, cap, window, slopes,
                       chunk, gate, gate_stride, gate_off, gate_heads, lse);
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

// Single tokens with key and value widths of up to 128 in steps of 4 (float32) or 8 (bfloat16).
// grid (kv heads x groups of up to 4 query heads that share them, sequences, splits); 256 threads.
// Eight lanes take a key, each 16 bytes of a row at a time (a unit: 4 floats or 8 bfloat16), so a
// wave reads 8 rows of keys (and of values) an instruction, a whole 128-byte line a row, for all
// the block's query heads at once; a score is 3 exchanges among the eight lanes.  Every group of
// eight keeps its own running max, sum and weighted values (lane s of a group holds dims U s + 8 U j
// ..), the next round's rows are asked for before this round's arithmetic, and the groups, then the
// waves, are combined at the end in a fixed order.  `partial` as above.
template <int CTRL>
__device__ __forceinline__ float cap_dpp(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xf, 0xf, true));
}

template <int DT>
__device__ __forceinline__ void ld_unit(const void* p, size_t at, float* x) {
    if (DT == ILLM_BF16) {
        const uint4 r = *(const uint4*)((const bf16_t*)p + at);
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            x[2 * k] = __uint_as_float(w[k] << 16);
            x[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
        }
    } else {
        const float4 r = *(const float4*)((const float*)p + at);
        x[0] = r.x; x[1] = r.y; x[2] = r.z; x[3] = r.w;
    }
}

template <int DT, int KQ, int VQ, int DH>        // DH: query heads a block takes at most
__global__ void __launch_bounds__(256)
attn_cap_decode_rows8_kernel(const void* __restrict__ q, int q_stride, const void* __restrict__ kcache,
                             const void* __restrict__ vcache, const int32_t* __restrict__ page_table,
                             int table_stride, int page_size, int ring, const int32_t* __restrict__ seq_slot,
                             const int32_t* __restrict__ seq_len, float* __restrict__ partial, int nsplit,
                             int nh, int nkv, int dk, int dv, float scale, float cap, int window,
                             const float* __restrict__ slopes, int chunk, void* __restrict__ out,
                             const void* __restrict__ gate, int gate_stride, int gate_off, int gate_heads) {
    constexpr int U = DT == ILLM_BF16 ? 8 : 4;          // elements of a unit
    constexpr int NK = U * KQ, NV = U * VQ;             // dims of a key, of a value, a lane holds
    __shared__ float wacc[4][DH][8 * NV];
    __shared__ float wm[4][DH], wl[4][DH];
    const int rep = nh / nkv, per_kv = (rep + DH - 1) / DH;
    const int kvh = blockIdx.x / per_kv, h0 = kvh * rep + (blockIdx.x % per_kv) * DH;
    const int hb = min(DH, (kvh + 1) * rep - h0);
    const int b = blockIdx.y, sp = blockIdx.z;
    const int w = wave_index(), lane = threadIdx.x & 63, grp = lane >> 3, sub = lane & 7;
    const int len = seq_len[b], slot = seq_slot[b];
    int lo_all = window > 0 ? max(0, len - window) : 0;
    if (chunk > 0) lo_all = max(lo_all, ((len - 1) / chunk) * chunk);
    const int tiles = (len + 63) / 64, t0 = lo_all / 64;
    const int per = (tiles - t0 + nsplit - 1) / nsplit;
    const int k_lo = max(lo_all, (t0 + sp * per) * 64), k_hi = min(len, (t0 + (sp + 1) * per) * 64);
    const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;
    float qv[DH][NK], acc[DH][NV], m[DH], l[DH], slope[DH];
#pragma unroll
    for (int i = 0; i < DH; ++i) {
        m[i] = NEG_INF; l[i] = 0.f;
        slope[i] = (slopes && i < hb) ? slopes[h0 + i] : 0.f;
#pragma unroll
        for (int c = 0; c < NV; ++c) acc[i][c] = 0.f;
#pragma unroll
        for (int j = 0; j < KQ; ++j) {
            const int d = U * sub + 8 * U * j;
#pragma unroll
            for (int c = 0; c < U; ++c) qv[i][U * j + c] = 0.f;
            if (i < hb && d < dk) ld_unit<DT>(q, (size_t)b * q_stride + (size_t)(h0 + i) * dk + d, &qv[i][U * j]);
        }
    }
    illm_u32x4_t kn[KQ], vn[VQ];                   // (raw: turned into floats when the round begins)
    auto unit_floats = [&](const illm_u32x4_t r, float* x) __attribute__((always_inline)) {
        if (DT == ILLM_BF16) {
            const uint32_t wd[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                x[2 * k] = __uint_as_float(wd[k] << 16);
                x[2 * k + 1] = __uint_as_float(wd[k] & 0xffff0000u);
            }
        } else {
            x[0] = __uint_as_float(r.x); x[1] = __uint_as_float(r.y);
            x[2] = __uint_as_float(r.z); x[3] = __uint_as_float(r.w);
        }
    };
    // the page of a round's key is looked up a round before its rows are asked for, so that a round
    // waits for one trip to memory, not for two in a row
    auto page_of = [&](int base) __attribute__((always_inline)) {
        int lp = min(base + grp, k_hi - 1) / page_size;
        if (ring > 0) lp %= ring;
        return page_table[(size_t)slot * table_stride + lp];
    };
    auto fetch = [&](int base, int page) __attribute__((always_inline)) {
        const int kj = min(base + grp, k_hi - 1);
        const size_t row = ((size_t)page * nkv + kvh) * page_size + (kj % page_size);
        const size_t kat = row * dk, vat = row * dv;
        const size_t esz = DT == ILLM_BF16 ? 2 : 4;
#pragma unroll
        for (int j = 0; j < KQ; ++j) {
            const int d = U * sub + 8 * U * j;
            kn[j] = illm_u32x4_t{0u, 0u, 0u, 0u};
            if (d < dk) kn[j] = *(const illm_u32x4_t*)((const char*)kcache + (kat + d) * esz);
        }
#pragma unroll
        for (int j = 0; j < VQ; ++j) {
            const int d = U * sub + 8 * U * j;
            vn[j] = illm_u32x4_t{0u, 0u, 0u, 0u};
            if (d < dv) vn[j] = *(const illm_u32x4_t*)((const char*)vcache + (vat + d) * esz);
        }
    };
    int page_next = 0;
    if (k_lo + 8 * w < k_hi) {
        fetch(k_lo + 8 * w, page_of(k_lo + 8 * w));
        page_next = page_of(k_lo + 8 * w + 32);
    }
    for (int base = k_lo + 8 * w; base < k_hi; base += 32) {
        float kc[NK], vc[NV];
#pragma unroll
        for (int j = 0; j < KQ; ++j) unit_floats(kn[j], &kc[U * j]);
#pragma unroll
        for (int j = 0; j < VQ; ++j) unit_floats(vn[j], &vc[U * j]);
        if (base + 32 < k_hi) {
            fetch(base + 32, page_next);
            page_next = page_of(base + 64);
        }
        const int kj = base + grp;
        const bool valid = kj < k_hi;
#pragma unroll
        for (int i = 0; i < DH; ++i) {
            if (i >= hb) continue;
            float a0 = 0.f, a1 = 0.f;
#pragma unroll
            for (int c = 0; c < NK; c += 2) {
                a0 = fmaf(qv[i][c], kc[c], a0);
                a1 = fmaf(qv[i][c + 1], kc[c + 1], a1);
            }
            // the sum over the group's eight lanes by data-parallel moves (no trip through LDS):
            // lanes 1 0 3 2 of every four, lanes 2 3 0 1, then the other four of the eight (mirrored)
            float d = a0 + a1;
            d += cap_dpp<0xB1>(d);
            d += cap_dpp<0x4E>(d);
            d += cap_dpp<0x141>(d);
            const float sc = valid ? soft_cap(d * scale, cap, inv_cap) - slope[i] * (float)(len - 1 - kj) : NEG_INF;
            const float m_new = fmaxf(m[i], sc);
            const float alpha = m_new == NEG_INF ? 1.f : expf(m[i] - m_new);
            const float p = valid ? expf(sc - m_new) : 0.f;
            l[i] = l[i] * alpha + p;
            m[i] = m_new;
#pragma unroll
            for (int c = 0; c < NV; ++c) acc[i][c] = fmaf(p, vc[c], acc[i][c] * alpha);
        }
    }
    // the wave's eight groups into one (every lane of a group holds the same m and l)
#pragma unroll
    for (int i = 0; i < DH; ++i) {
        if (i >= hb) continue;
        float mm = m[i];
        mm = fmaxf(mm, __shfl_xor(mm, 8, ILLM_WAVE));
        mm = fmaxf(mm, __shfl_xor(mm, 16, ILLM_WAVE));
        mm = fmaxf(mm, __shfl_xor(mm, 32, ILLM_WAVE));
        const float f = m[i] == NEG_INF ? 0.f : expf(m[i] - mm);
        float lt = f * l[i];
        lt += __shfl_xor(lt, 8, ILLM_WAVE);
        lt += __shfl_xor(lt, 16, ILLM_WAVE);
        lt += __shfl_xor(lt, 32, ILLM_WAVE);
#pragma unroll
        for (int c = 0; c < NV; ++c) {
            float a = f * acc[i][c];
            a += __shfl_xor(a, 8, ILLM_WAVE);
            a += __shfl_xor(a, 16, ILLM_WAVE);
            a += __shfl_xor(a, 32, ILLM_WAVE);
            if (grp == 0) wacc[w][i][U * sub + 8 * U * (c / U) + (c % U)] = a;
        }
        if (lane == 0) { wm[w][i] = mm; wl[w][i] = lt; }
    }
    __syncthreads();
    for (int i = 0; i < hb; ++i) {
        float mm = wm[0][i];
        for (int x = 1; x < 4; ++x) mm = fmaxf(mm, wm[x][i]);
        float f[4], lt = 0.f;
        for (int x = 0; x < 4; ++x) {
            f[x] = wm[x][i] == NEG_INF ? 0.f : expf(wm[x][i] - mm);
            lt += f[x] * wl[x][i];
        }
        if (nsplit == 1) {                              // the one range is the whole result: no merge
            const float inv = 1.0f / lt;
            for (int d = threadIdx.x; d < dv; d += 256) {
                float y = (f[0] * wacc[0][i][d] + f[1] * wacc[1][i][d] + f[2] * wacc[2][i][d] + f[3] * wacc[3][i][d]) * inv;
                if (gate)
                    y *= 1.0f / (1.0f + expf(-ld_f(gate, DT, (size_t)b * gate_stride + gate_off + (gate_heads ? (size_t)(h0 + i) : (size_t)(h0 + i) * dv + d))));
                st_f(out, DT, ((size_t)b * nh + h0 + i) * dv + d, y);
            }
            continue;
        }
        float* pp = partial + (((size_t)b * nh + h0 + i) * nsplit + sp) * (dv + 2);
        for (int d = threadIdx.x; d < dv; d += 256)
            pp[d] = f[0] * wacc[0][i][d] + f[1] * wacc[1][i][d] + f[2] * wacc[2][i][d] + f[3] * wacc[3][i][d];
        if (threadIdx.x == 0) { pp[dv] = mm; pp[dv + 1] = lt; }
    }
}

// grid (heads, sequences): combine the splits' partial results in split order.
__global__ void attn_cap_merge_kernel(const float* __restrict__ partial, void* __restrict__ out,
                                      int dt, int nsplit, int nh, int dv, const void* __restrict__ gate,
                                      int gate_stride, int gate_off, int gate_heads, float* __restrict__ lse) {
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
    if (lse && threadIdx.x == 0) lse[(size_t)b * nh + h] = mm + logf(lt);
    for (int d = threadIdx.x; d < dv; d += blockDim.x) {
        float a = 0.f;
        for (int s = 0; s < nsplit; ++s) {
            const float ms = pp[(size_t)s * (dv + 2) + dv];
            a += (ms == NEG_INF ? 0.f : expf(ms - mm)) * pp[(size_t)s * (dv + 2) + d];
        }
        float y = a * inv;
        if (gate) y *= 1.0f / (1.0f + expf(-ld_f(gate, dt, (size_t)b * gate_stride + gate_off + (gate_heads ? (size_t)h : (size_t)h * dv + d))));
        st_f(out, dt, ((size_t)b * nh + h) * dv + d, y);
    }
}

extern "C" int illm_attn_cap_decode(const void* q, int q_stride, void* out, int dt,
                                    const void* kcache, const void* vcache,
                                    const int32_t* page_table, int table_stride, int page_size,
                                    int ring, const int32_t* seq_slot, const int32_t* seq_len,
                                    float* partial, int nsplit, int B, int nh, int nkv, int dk, int dv,
                                    float scale, float cap, int window, const float* slopes, int chunk,
                                    const void* gate, int gate_stride, int gate_off, int gate_heads, float* lse, void* stream) {
    if (gate && (gate_off < 0 || gate_off + nh * (gate_heads ? 1 : dv) > gate_stride)) return ILLM_ERR_ARG;
    if (B < 0 || nh <= 0 || nkv <= 0 || nh % nkv || dk <= 0 || dk > 256 || dv <= 0 || dv > 256 ||
        page_size <= 0 || nsplit < 1 || nsplit > 65535 || B > 65535 || !illm_dtype_ok(dt) || !partial ||
        (lse && nsplit < 2))                       // the kernel that merges the ranges writes it
        return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
    hipStream_t st = (hipStream_t)stream;
    const int unit = dt == ILLM_BF16 ? 8 : 4;
    if (g_attn_cap_mfma && dk <= 128 && dv <= 128 && dk % unit == 0 && dv % unit == 0 && q_stride % unit == 0) {
        // four query heads of a kv head a block (their keys and values are read once), or two where
        // that is asked for: half the registers, twice the waves a SIMD, the rows read twice
        const int rep = nh / nkv, dh = g_attn_cap_heads == 2 ? 2 : 4;
        const dim3 grid(nkv * ((rep + dh - 1) / dh), B, nsplit);
        const int kq = (dk + 8 * unit - 1) / (8 * unit), vq = (dv + 8 * unit - 1) / (8 * unit);
#define GO(DT_, KQ_, VQ_)                                                                          \
    if (dh == 2)                                                                                   \
        hipLaunchKernelGGL((attn_cap_decode_rows8_kernel<DT_, KQ_, VQ_, 2>), grid, dim3(256), 0, st, q, q_stride, \
                           kcache, vcache, page_table, table_stride, page_size, ring, seq_slot, seq_len, partial, \
                           nsplit, nh, nkv, dk, dv, scale, cap, window, slopes, chunk, out, gate, gate_stride, gate_off, gate_heads); \
    else                                                                                           \
        hipLaunchKernelGGL((attn_cap_decode_rows8_kernel<DT_, KQ_, VQ_, 4>), grid, dim3(256), 0, st, q, q_stride, \
                           kcache, vcache, page_table, table_stride, page_size, ring, seq_slot, seq_len, partial, \
                           nsplit, nh, nkv, dk, dv, scale, cap, window, slopes, chunk, out, gate, gate_stride, gate_off, gate_heads)
#define GO_V(DT_, KQ_)                                                                             \
    switch (vq) { case 1: { GO(DT_, KQ_, 1); } break; case 2: { GO(DT_, KQ_, 2); } break;          \
                  case 3: { GO(DT_, KQ_, 3); } break; default: { GO(DT_, KQ_, 4); } break; }
#define GO_K(DT_)                                                                                  \
    switch (kq) { case 1: GO_V(DT_, 1) break; case 2: GO_V(DT_, 2) break;                          \
                  case 3: GO_V(DT_, 3) break; default: GO_V(DT_, 4) break; }
        if (dt == ILLM_BF16) { GO_K(ILLM_BF16) } else { GO_K(ILLM_F32) }
#undef GO_K
#undef GO_V
#undef GO
        if (nsplit == 1) return illm_launch_status();    // written whole by the kernel itself
    } else if (dt == ILLM_BF16)
        hipLaunchKernelGGL(attn_cap_decode_kernel<ILLM_BF16>, dim3(nh, B, nsplit), dim3(256), 0, st, q,
                           q_stride, kcache, vcache, page_table, table_stride, page_size, ring, seq_slot,
                           seq_len, partial, nsplit, nh, nkv, dk, dv, scale, cap, window, slopes, chunk);
    else
        hipLaunchKernelGGL(attn_cap_decode_kernel<ILLM_F32>, dim3(nh, B, nsplit), dim3(256), 0, st, q,
                           q_stride, kcache, vcache, page_table, table_stride, page_size, ring, seq_slot,
                           seq_len, partial, nsplit, nh, nkv, dk, dv, scale, cap, window, slopes, chunk);
    if (hipGetLastError() != hipSuccess) return ILLM_ERR_LAUNCH;
    hipLaunchKernelGGL(attn_cap_merge_kernel, dim3(nh, B), dim3(64), 0, st, partial, out, dt, nsplit, nh, dv,
                       gate, gate_stride, gate_off, gate_heads, lse);
    return illm_launch_status();
}
