// What stands around the plain gated recurrence (illm_gated_scan with `correct` 0,
//     S <- g S + k (beta v)^T;   o = S^T q,   S [key dim, value dim] float32 per head)
// for two mixers that keep such a state.
//
// A state-space mixer with a scalar decay a head (state-space duality):
//   ssm_prepare   short causal convolution with bias over time of the x | B | C columns of the input
//                 projection (the taps before a step's first row from the kept tail), SiLU;
//                 dt = softplus(dt + dt_bias), g = exp(-exp(A_log) dt), beta = dt; k = B, q = C of the
//                 head's group, v = x
//   ssm_finish    y = (o + D x) silu(z), RMS norm in `norm_groups` equal parts of the row, weight
//
// A matrix memory with exponential gates held in range by a running maximum m (from 0):
//   memory_rows   q dim^-1/2, k, and v with a column of ones behind it as float32 (the state's
//                 last column is then the normaliser n = sum of the weighted keys)
//   memory_gates  i = cap tanh((i + b_i) / cap), f = logsigmoid(cap tanh((f + b_f) / cap)),
//                 m_t = max(f + m_(t-1), i), g = exp(f + m_(t-1) - m_t), beta = exp(i - m_t), token
//                 after token per sequence and head, m kept per sequence
//   memory_finish o / (max(|n . q|, exp(-m)) + 1e-6), RMS norm per head, weight, sigmoid gate
//
// Everything but the stored projections is float32.  A sequence's rows in a step are consecutive.
#include <math.h>

#include "api.h"
#include "common.h"

#define SCAN_MAX_TAPS 8

__device__ __forceinline__ float ls_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float ls_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float ls_log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// ---------------------------------------------------------------- state-space mixer
// grid (rows, NB); 256 threads over the convolution's channels.  U [T, u_stride]: columns
// [x_off, x_off + C) = x (H dv) | B (G N) | C (G N) before the convolution, dt_off: H columns.
// `update_tail`: every sequence brings one row, and the thread that has read a channel's taps also
// writes its tail for the next step.
__global__ void __launch_bounds__(256)
ssm_prepare_kernel(const void* __restrict__ U, int dt, int u_stride, int x_off, int dt_off,
                   const float* __restrict__ conv_w, const float* __restrict__ conv_b, int taps,
                   void* __restrict__ tail, const int32_t* __restrict__ row_slot,
                   const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                   float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ vv,
                   float* __restrict__ beta, float* __restrict__ dec, int G, int H, int N, int dv,
                   int update_tail) {
    const int r = blockIdx.x, NB = gridDim.y;
    const int inner = H * dv, GN = G * N, C = inner + 2 * GN, K = taps - 1;
    const int slot = row_slot[r];
    int before = 0;                                     // rows of this sequence ahead of r in the step, up to K
    while (before < K && r - before - 1 >= 0 && row_slot[r - before - 1] == slot) ++before;
    for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += 256 * NB) {
        float x[SCAN_MAX_TAPS], cw[SCAN_MAX_TAPS];
#pragma unroll
        for (int j = 0; j < SCAN_MAX_TAPS; ++j) {
            x[j] = cw[j] = 0.f;
            if (j < taps) {
                const int d = K - j;                    // tap j looks d tokens back
                x[j] = d <= before ? ld_f(U, dt, (size_t)(r - d) * u_stride + x_off + c)
                                   : ld_f(tail, dt, ((size_t)slot * K + (K - (d - before))) * C + c);
                cw[j] = conv_w[(size_t)c * taps + j];
            }
        }
        float a = conv_b[c];
#pragma unroll
        for (int j = 0; j < SCAN_MAX_TAPS; ++j) {
            if (j < taps) {
                a = fmaf(cw[j], x[j], a);
                if (update_tail && j > 0) st_f(tail, dt, ((size_t)slot * K + (j - 1)) * C + c, x[j]);
            }
        }
        const float y = a * ls_sigmoid(a);
        if (c < inner) vv[(size_t)r * inner + c] = y;
        else if (c < inner + GN) kn[(size_t)r * GN + (c - inner)] = y;
        else qn[(size_t)r * GN + (c - inner - GN)] = y;
    }
    for (int i = blockIdx.y * 256 + threadIdx.x; i < H; i += 256 * NB) {
        const float step = ls_softplus(ld_f(U, dt, (size_t)r * u_stride + dt_off + i) + dt_bias[i]);
        beta[(size_t)r * H + i] = step;
        dec[(size_t)r * H + i] = expf(-expf(a_log[i]) * step);
    }
}

extern "C" int illm_ssm_prepare(const void* U, int dt, int u_stride, int x_off, int dt_off,
                                const float* conv_w, const float* conv_b, int taps, void* tail,
                                const int32_t* row_slot, const float* a_log, const float* dt_bias,
                                float* qn, float* kn, float* vv, float* beta, float* dec, int T, int G,
                                int H, int N, int dv, int update_tail, void* stream) {
    if (T < 0 || G <= 0 || H <= 0 || H % G || N <= 0 || dv <= 0 || taps < 1 || taps > SCAN_MAX_TAPS ||
        !illm_dtype_ok(dt) || x_off < 0 || dt_off < 0 || x_off + H * dv + 2 * G * N > u_stride ||
        dt_off + H > u_stride)
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    const int C = H * dv + 2 * G * N, most = (C + 255) / 256;
    int nb = T >= 2048 ? 1 : (2048 + T - 1) / T;        // enough blocks to fill the chip when the rows are few
    nb = nb > most ? most : nb;
    hipLaunchKernelGGL(ssm_prepare_kernel, dim3(T, nb), dim3(256), 0, (hipStream_t)stream, U, dt, u_stride,
                       x_off, dt_off, conv_w, conv_b, taps, tail, row_slot, a_log, dt_bias, qn, kn, vv,
                       beta, dec, G, H, N, dv, update_tail);
    return illm_launch_status();
}

// grid (rows, norm groups); 256 threads.  y_j = (o_j + D[head of j] x_j) silu(z_j) over the part's
// columns, out = y / sqrt(mean over the part of y^2 + eps) * w.  Z [T, z_stride] + z_off.
__global__ void __launch_bounds__(256)
ssm_finish_kernel(const float* __restrict__ o, const float* __restrict__ x,
                  const float* __restrict__ D, const void* __restrict__ Z, int z_dt, int z_stride,
                  int z_off, const void* __restrict__ w, int w_dt, void* __restrict__ out, int out_dt,
                  int inner, int dv, int part, float eps) {
    __shared__ float red[16];
    const size_t r = blockIdx.x;
    const int j0 = blockIdx.y * part;
    float ss = 0.f;
    for (int j = j0 + threadIdx.x; j < j0 + part; j += 256) {
        const float z = ld_f(Z, z_dt, r * z_stride + z_off + j);
        const float y = fmaf(D[j / dv], x[r * inner + j], o[r * inner + j]) * (z * ls_sigmoid(z));
        ss += y * y;
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)part + eps);
    for (int j = j0 + threadIdx.x; j < j0 + part; j += 256) {
        const float z = ld_f(Z, z_dt, r * z_stride + z_off + j);
        const float y = fmaf(D[j / dv], x[r * inner + j], o[r * inner + j]) * (z * ls_sigmoid(z));
        st_f(out, out_dt, r * inner + j, (y * inv) * ld_f(w, w_dt, j));
    }
}

extern "C" int illm_ssm_finish(const float* o, const float* x, const float* D, const void* Z, int z_dt,
                               int z_stride, int z_off, const void* w, int w_dt, void* out, int out_dt,
                               int T, int H, int dv, int norm_groups, float eps, void* stream) {
    if (T < 0 || H <= 0 || dv <= 0 || norm_groups <= 0 || norm_groups > 65535 ||
        (H * dv) % norm_groups || !illm_dtype_ok(z_dt) || !illm_dtype_ok(w_dt) || !illm_dtype_ok(out_dt) ||
        z_off < 0 || z_off + H * dv > z_stride)
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(ssm_finish_kernel, dim3(T, norm_groups), dim3(256), 0, (hipStream_t)stream, o, x, D,
                       Z, z_dt, z_stride, z_off, w, w_dt, out, out_dt, H * dv, dv, (H * dv) / norm_groups, eps);
    return illm_launch_status();
}

// ---------------------------------------------------------------- matrix memory
// grid (rows); 256 threads.  U [T, u_stride] = [q (H dk) | k (H dk) | v (H dv) | ...].
__global__ void __launch_bounds__(256)
memory_rows_kernel(const void* __restrict__ U, int dt, int u_stride, float* __restrict__ qn,
                   float* __restrict__ kn, float* __restrict__ vv, int H, int dk, int dv, float qscale) {
    const size_t r = blockIdx.x;
    const int nq = H * dk, nv = H * (dv + 1);
    for (int i = threadIdx.x; i < nq; i += 256) {
        qn[r * nq + i] = ld_f(U, dt, r * u_stride + i) * qscale;
        kn[r * nq + i] = ld_f(U, dt, r * u_stride + nq + i);
    }
    for (int i = threadIdx.x; i < nv; i += 256) {
        const int h = i / (dv + 1), j = i - h * (dv + 1);
        vv[r * nv + i] = j < dv ? ld_f(U, dt, r * u_stride + 2 * nq + h * dv + j) : 1.0f;
    }
}

// grid (sequences, H); one wave.  64 tokens at a time: every lane forms its token's two gates, then
// the running maximum goes through the 64 tokens in order (the lanes' values are read one after the
// other as scalars), and every lane leaves its token's decay, weight and exp(-m).
__global__ void __launch_bounds__(64)
memory_gates_kernel(const void* __restrict__ U, int dt, int u_stride, int i_off, int f_off,
                    const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap,
                    float* __restrict__ m_state, const int32_t* __restrict__ cu,
                    const int32_t* __restrict__ seq_slot, float* __restrict__ beta,
                    float* __restrict__ dec, float* __restrict__ em, int H) {
    const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int r0 = cu[b], n = cu[b + 1] - r0;
    if (n <= 0) return;
    const int slot = seq_slot[b];
    const float bi = i_bias[h], bf = f_bias[h], inv_cap = 1.0f / cap;
    float m = m_state[(size_t)slot * H + h];
    for (int t0 = 0; t0 < n; t0 += 64) {
        const bool ok = t0 + lane < n;
        const size_t row = (size_t)(r0 + (ok ? t0 + lane : n - 1));
        const float ig = ok ? cap * tanhf((ld_f(U, dt, row * u_stride + i_off + h) + bi) * inv_cap) : -INFINITY;
        const float fg = ok ? ls_log_sigmoid(cap * tanhf((ld_f(U, dt, row * u_stride + f_off + h) + bf) * inv_cap)) : 0.f;
        float m_before = 0.f, m_mine = 0.f;
#pragma unroll
        for (int l = 0; l < 64; ++l) {
            const float fl = __shfl(fg, l, 64), il = __shfl(ig, l, 64);
            const float m_new = fmaxf(fl + m, il);      // a lane beyond the sequence leaves m as it is
            if (lane == l) { m_before = m; m_mine = m_new; }
            m = m_new;
        }
        if (ok) {
            dec[row * H + h] = expf(fg + m_before - m_mine);
            beta[row * H + h] = expf(ig - m_mine);
            em[row * H + h] = expf(-m_mine);
        }
    }
    if (lane == 0) m_state[(size_t)slot * H + h] = m;
}

extern "C" int illm_memory_prepare(const void* U, int dt, int u_stride, int i_off, int f_off,
                                   const float* i_bias, const float* f_bias, float cap, float* m_state,
                                   const int32_t* cu, const int32_t* seq_slot, float* qn, float* kn,
                                   float* vv, float* beta, float* dec, float* em, int T, int n_seqs,
                                   int H, int dk, int dv, void* stream) {
    if (T < 0 || n_seqs < 0 || n_seqs > 65535 || H <= 0 || H > 65535 || dk <= 0 || dv <= 0 ||
        !illm_dtype_ok(dt) || !(cap > 0.f) || 2 * H * dk + H * dv > u_stride || i_off < 0 || f_off < 0 ||
        i_off + H > u_stride || f_off + H > u_stride)
        return ILLM_ERR_ARG;
    if (T == 0 || n_seqs == 0) return ILLM_OK;
    hipLaunchKernelGGL(memory_rows_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, U, dt, u_stride, qn,
                       kn, vv, H, dk, dv, 1.0f / sqrtf((float)dk));
    if (hipGetLastError() != hipSuccess) return ILLM_ERR_LAUNCH;
    hipLaunchKernelGGL(memory_gates_kernel, dim3(n_seqs, H), dim3(64), 0, (hipStream_t)stream, U, dt,
                       u_stride, i_off, f_off, i_bias, f_bias, cap, m_state, cu, seq_slot, beta, dec, em, H);
    return illm_launch_status();
}

// grid (rows, H); one wave.  o [T, H, dv + 1]: the last column is n . q.
//   y_j = o_j / (max(|n . q|, exp(-m)) + 1e-6);  out = y / sqrt(mean_j y^2 + eps) * w[h dv + j] * sigmoid(z)
__global__ void __launch_bounds__(64)
memory_finish_kernel(const float* __restrict__ o, const float* __restrict__ em,
                     const void* __restrict__ w, int w_dt, const void* __restrict__ Z, int z_dt,
                     int z_stride, int z_off, void* __restrict__ out, int out_dt, int H, int dv, float eps) {
    const size_t r = blockIdx.x;
    const int h = blockIdx.y, lane = threadIdx.x;
    const float* op = o + (r * H + h) * (dv + 1);
    const float den = fmaxf(fabsf(op[dv]), em[r * H + h]) + 1e-6f;
    float ss = 0.f;
    for (int j = lane; j < dv; j += 64) {
        const float y = op[j] / den;
        ss += y * y;
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
    for (int j = lane; j < dv; j += 64) {
        const float z = ld_f(Z, z_dt, r * z_stride + z_off + (size_t)h * dv + j);
        st_f(out, out_dt, (r * H + h) * dv + j,
             ((op[j] / den) * inv) * ld_f(w, w_dt, (size_t)h * dv + j) * ls_sigmoid(z));
    }
}

extern "C" int illm_memory_finish(const float* o, const float* em, const void* w, int w_dt, const void* Z,
                                  int z_dt, int z_stride, int z_off, void* out, int out_dt, int T, int H,
                                  int dv, float eps, void* stream) {
    if (T < 0 || H <= 0 || H > 65535 || dv <= 0 || !illm_dtype_ok(w_dt) || !illm_dtype_ok(z_dt) ||
        !illm_dtype_ok(out_dt) || z_off < 0 || z_off + H * dv > z_stride)
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(memory_finish_kernel, dim3(T, H), dim3(64), 0, (hipStream_t)stream, o, em, w, w_dt, Z,
                       z_dt, z_stride, z_off, out, out_dt, H, dv, eps);
    return illm_launch_status();
}

// ---------------------------------------------------------------- gated linear attention
// The plain gated rule with a decay per key channel: from the projections U [T, u_stride] (q at
// q_off, k at k_off, both H dk wide, v at v_off, H dv wide) and the decays' pre-activations
// Z [T, z_stride] (H dk wide) with their bias zb:
//   q dk^-1/2, k, v as float32; decay = sigmoid(Z + zb)^(1 / tau) = exp(logsigmoid(Z + zb) / tau);
//   the token's weight is 1.
// grid (rows); 256 threads.
__global__ void __launch_bounds__(256)
gla_prepare_kernel(const void* __restrict__ U, int dt, int u_stride, int q_off, int k_off, int v_off,
                   const void* __restrict__ Z, int z_dt, int z_stride, const float* __restrict__ zb,
                   float inv_tau, float* __restrict__ qn, float* __restrict__ kn,
                   float* __restrict__ vv, float* __restrict__ beta, float* __restrict__ dec, int H,
                   int dk, int dv) {
    const size_t t = blockIdx.x;
    const float qs = 1.0f / sqrtf((float)dk);
    for (int e = threadIdx.x; e < H * dk; e += 256) {
        qn[t * H * dk + e] = ld_f(U, dt, t * u_stride + q_off + e) * qs;
        kn[t * H * dk + e] = ld_f(U, dt, t * u_stride + k_off + e);
        dec[t * H * dk + e] = expf(ls_log_sigmoid(ld_f(Z, z_dt, t * z_stride + e) + zb[e]) * inv_tau);
    }
    for (int e = threadIdx.x; e < H * dv; e += 256) vv[t * H * dv + e] = ld_f(U, dt, t * u_stride + v_off + e);
    for (int e = threadIdx.x; e < H; e += 256) beta[t * H + e] = 1.0f;
}

extern "C" int illm_gla_prepare(const void* U, int dt, int u_stride, int q_off, int k_off, int v_off,
                                const void* Z, int z_dt, int z_stride, const float* zb, float tau,
                                float* qn, float* kn, float* vv, float* beta, float* dec, int T, int H,
                                int dk, int dv, void* stream) {
    if (T < 0 || H <= 0 || dk <= 0 || dv <= 0 || !illm_dtype_ok(dt) || !illm_dtype_ok(z_dt) || !(tau > 0.f) ||
        q_off < 0 || k_off < 0 || v_off < 0 || q_off + H * dk > u_stride || k_off + H * dk > u_stride ||
        v_off + H * dv > u_stride || H * dk > z_stride)
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(gla_prepare_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, U, dt, u_stride,
                       q_off, k_off, v_off, Z, z_dt, z_stride, zb, 1.0f / tau, qn, kn, vv, beta, dec, H, dk, dv);
    return illm_launch_status();
}

// ---------------------------------------------------------------- a gated linear recurrent unit
// Per channel c of `C`, in `nb` equal blocks of cb channels: with u the recurrence's input,
//   r = sigmoid(Wr[b] u_b + br),  i = sigmoid(Wi[b] u_b + bi)        (square maps within a block)
//   a = exp(-rate r softplus(lam)),  x = sqrt(1 - a^2) i u
//   S <- a S + x,   out = S gelu_tanh(Y + yb)
// lru_gates gives a and x; lru_scan runs the recurrence from the kept state [slots][C] and back
// into it and multiplies by the other branch.  All float32 but the stored Y and the output.
//
// grid (ceil(T / ROWS), nb); 256 threads over a block's outputs; the rows' inputs go through LDS, laid
// out [input][row] so that a thread reads one input of all its rows in 16-byte pieces.  Steps of few
// rows take tiles of 4 rows (more blocks), longer ones tiles of 16.  Wt [2][nb][cb in][cb out] float32:
// the two maps transposed, so that the threads of a wave read neighbouring outputs of one input.
template <int ROWS>
__global__ void __launch_bounds__(256)
lru_gates_kernel(const float* __restrict__ u, const float* __restrict__ Wt, const float* __restrict__ br,
                 const float* __restrict__ bi, const float* __restrict__ lam, float rate,
                 float* __restrict__ a_out, float* __restrict__ x_out, int T, int C, int cb) {
    extern __shared__ float us[];                   // [cb][ROWS], then the slices' partial sums
    const int t0 = blockIdx.x * ROWS, b = blockIdx.y, nb = C / cb;
    const int rows = min(ROWS, T - t0);
    for (int e = threadIdx.x; e < ROWS * cb; e += 256) {
        const int r = e / cb, i = e - r * cb;
        us[i * ROWS + r] = r < rows ? u[(size_t)(t0 + r) * C + (size_t)b * cb + i] : 0.f;
    }
    __syncthreads();
    const float* wr = Wt + (size_t)b * cb * cb;
    const float* wi = Wt + ((size_t)nb + b) * cb * cb;
    // a block narrower than the thread block cuts its inputs into S slices, one a group of cb
    // threads, whose sums are added in slice order
    const int S = cb < 256 ? 256 / cb : 1;
    const int per = (cb + S - 1) / S;
    float* part = us + (size_t)cb * ROWS;           // [S][cb][2 ROWS]
    for (int o0 = 0; o0 < cb; o0 += 256) {
        const int o = S > 1 ? (int)threadIdx.x % cb : o0 + (int)threadIdx.x;
        const int sl = S > 1 ? (int)threadIdx.x / cb : 0;
        const bool live = o < cb && sl < S;
        float ar[ROWS], ai[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) ar[r] = ai[r] = 0.f;
        if (live) {
            const int i_lo = sl * per, i_hi = min(cb, i_lo + per);
#pragma unroll 8
            for (int i = i_lo; i < i_hi; ++i) {
                const float w1 = wr[(size_t)i * cb + o], w2 = wi[(size_t)i * cb + o];
                const float4* xr = (const float4*)(us + i * ROWS);
#pragma unroll
                for (int r4 = 0; r4 < ROWS / 4; ++r4) {
                    const float4 x = xr[r4];
                    ar[4 * r4 + 0] = fmaf(w1, x.x, ar[4 * r4 + 0]); ai[4 * r4 + 0] = fmaf(w2, x.x, ai[4 * r4 + 0]);
                    ar[4 * r4 + 1] = fmaf(w1, x.y, ar[4 * r4 + 1]); ai[4 * r4 + 1] = fmaf(w2, x.y, ai[4 * r4 + 1]);
                    ar[4 * r4 + 2] = fmaf(w1, x.z, ar[4 * r4 + 2]); ai[4 * r4 + 2] = fmaf(w2, x.z, ai[4 * r4 + 2]);
                    ar[4 * r4 + 3] = fmaf(w1, x.w, ar[4 * r4 + 3]); ai[4 * r4 + 3] = fmaf(w2, x.w, ai[4 * r4 + 3]);
                }
            }
        }
        if (S > 1) {
            if (live) {
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    part[((size_t)sl * cb + o) * 2 * ROWS + r] = ar[r];
                    part[((size_t)sl * cb + o) * 2 * ROWS + ROWS + r] = ai[r];
                }
            }
            __syncthreads();
            if (live && sl == 0) {
                for (int s2 = 1; s2 < S; ++s2) {
#pragma unroll
                    for (int r = 0; r < ROWS; ++r) {
                        ar[r] += part[((size_t)s2 * cb + o) * 2 * ROWS + r];
                        ai[r] += part[((size_t)s2 * cb + o) * 2 * ROWS + ROWS + r];
                    }
                }
            }
        }
        if (!live || sl != 0) continue;
        const int c = b * cb + o;
        const float sp = ls_softplus(lam[c]), b1 = br[c], b2 = bi[c];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            if (r >= rows) continue;
            const float rg = ls_sigmoid(ar[r] + b1), ig = ls_sigmoid(ai[r] + b2);
            const float log_a = -rate * rg * sp;
            a_out[(size_t)(t0 + r) * C + c] = expf(log_a);
            // 1 - a^2 as -expm1(2 log a): a decay close to 1 keeps its digits
            x_out[(size_t)(t0 + r) * C + c] = sqrtf(fmaxf(-expm1f(2.0f * log_a), 0.f)) * ig * us[o * ROWS + r];
        }
    }
}

template <int ROWS>
static int lru_gates_launch(const float* u, const float* Wt, const float* br, const float* bi,
                            const float* lam, float rate, float* a_out, float* x_out, int T, int C,
                            int nb, hipStream_t st) {
    const int cb = C / nb;
    const int slices = cb < 256 ? 256 / cb : 1;
    const size_t lds = ((size_t)ROWS * cb + (slices > 1 ? (size_t)slices * cb * 2 * ROWS : 0)) * sizeof(float);
    if (lds > 64 * 1024) return ILLM_ERR_ARG;
    if (lds > 48 * 1024 &&
        hipFuncSetAttribute((const void*)lru_gates_kernel<ROWS>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
        return ILLM_ERR_LAUNCH;
    hipLaunchKernelGGL(lru_gates_kernel<ROWS>, dim3((T + ROWS - 1) / ROWS, nb), dim3(256), lds, st, u, Wt, br,
                       bi, lam, rate, a_out, x_out, T, C, cb);
    return illm_launch_status();
}

extern "C" int illm_lru_gates(const float* u, const float* Wt, const float* br, const float* bi,
                              const float* lam, float rate, float* a_out, float* x_out, int T, int C,
                              int nb, void* stream) {
    if (T < 0 || C <= 0 || nb <= 0 || C % nb || nb > 65535) return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    // tiles of 16 rows where a block's inputs of 16 rows fit LDS (blocks of up to 1,024 channels)
    if (T <= 128 || C / nb > 1024)
        return lru_gates_launch<4>(u, Wt, br, bi, lam, rate, a_out, x_out, T, C, nb, (hipStream_t)stream);
    return lru_gates_launch<16>(u, Wt, br, bi, lam, rate, a_out, x_out, T, C, nb, (hipStream_t)stream);
}

__device__ __forceinline__ float ls_gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// grid (sequences, ceil(C / 256)); a thread walks its channel through the sequence's rows.
__global__ void __launch_bounds__(256)
lru_scan_kernel(const float* __restrict__ a, const float* __restrict__ x, float* __restrict__ state,
                const void* __restrict__ Y, int y_dt, int y_stride, int y_off,
                const float* __restrict__ yb, void* __restrict__ out, int out_dt,
                const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_slot, int C) {
    const int b = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int r0 = cu[b], n = cu[b + 1] - r0;
    if (n <= 0) return;
    const int slot = seq_slot[b];
    float S = state[(size_t)slot * C + c];
    const float bias = yb ? yb[c] : 0.f;
    for (int t = 0; t < n; ++t) {
        const size_t at = (size_t)(r0 + t) * C + c;
        S = fmaf(a[at], S, x[at]);
        const float y = ls_gelu_tanh(ld_f(Y, y_dt, (size_t)(r0 + t) * y_stride + y_off + c) + bias);
        st_f(out, out_dt, at, S * y);
    }
    state[(size_t)slot * C + c] = S;
}

// The same recurrence for long steps, in three launches over chunks of LRU_CHUNK rows:
//   lru_chunk_sums   per (sequence, chunk, channel): the chunk's product of decays P and its sum B
//                    from a state of zero (S_end = P S_start + B)
//   lru_chunk_carry  per (sequence, channel): the state at every chunk's start, chunk after chunk
//                    (and the sequence's last state back into the slot)
//   lru_chunk_apply  per (sequence, chunk, channel): the recurrence again from the chunk's start
//                    state, with the other branch multiplied in
// A row's state is then summed in another order than token by token: it differs in rounding only.
#define LRU_CHUNK 32
__global__ void __launch_bounds__(256)
lru_chunk_sums_kernel(const float* __restrict__ a, const float* __restrict__ x, float* __restrict__ P,
                      float* __restrict__ B, const int32_t* __restrict__ cu, int C, int max_chunks) {
    const int b = blockIdx.z, ch = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int r0 = cu[b], n = cu[b + 1] - r0;
    const int t0 = ch * LRU_CHUNK;
    if (t0 >= n) return;
    const int t1 = min(n, t0 + LRU_CHUNK);
    float p = 1.f, s = 0.f;
    for (int t = t0; t < t1; ++t) {
        const size_t at = (size_t)(r0 + t) * C + c;
        const float av = a[at];
        s = fmaf(av, s, x[at]);
        p *= av;
    }
    const size_t o = ((size_t)b * max_chunks + ch) * C + c;
    P[o] = p;
    B[o] = s;
}

__global__ void __launch_bounds__(256)
lru_chunk_carry_kernel(const float* __restrict__ P, float* __restrict__ B, float* __restrict__ state,
                       const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_slot, int C,
                       int max_chunks) {
    const int b = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int n = cu[b + 1] - cu[b];
    if (n <= 0) return;
    const int chunks = (n + LRU_CHUNK - 1) / LRU_CHUNK, slot = seq_slot[b];
    float S = state[(size_t)slot * C + c];
    for (int ch = 0; ch < chunks; ++ch) {
        const size_t o = ((size_t)b * max_chunks + ch) * C + c;
        const float next = fmaf(P[o], S, B[o]);
        B[o] = S;                                   // the chunk's start state, for lru_chunk_apply
        S = next;
    }
    state[(size_t)slot * C + c] = S;
}

__global__ void __launch_bounds__(256)
lru_chunk_apply_kernel(const float* __restrict__ a, const float* __restrict__ x,
                       const float* __restrict__ S0, const void* __restrict__ Y, int y_dt, int y_stride,
                       int y_off, const float* __restrict__ yb, void* __restrict__ out, int out_dt,
                       const int32_t* __restrict__ cu, int C, int max_chunks) {
    const int b = blockIdx.z, ch = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int r0 = cu[b], n = cu[b + 1] - r0;
    const int t0 = ch * LRU_CHUNK;
    if (t0 >= n) return;
    const int t1 = min(n, t0 + LRU_CHUNK);
    float S = S0[((size_t)b * max_chunks + ch) * C + c];
    const float bias = yb ? yb[c] : 0.f;
    for (int t = t0; t < t1; ++t) {
        const size_t at = (size_t)(r0 + t) * C + c;
        S = fmaf(a[at], S, x[at]);
        const float y = ls_gelu_tanh(ld_f(Y, y_dt, (size_t)(r0 + t) * y_stride + y_off + c) + bias);
        st_f(out, out_dt, at, S * y);
    }
}

// `scratch`: 2 * n_seqs * ceil(max_rows / 32) * C floats for steps of 64 rows a sequence or more
// (null, or fewer rows: a thread walks its channel through the whole sequence).
extern "C" int illm_lru_scan(const float* a, const float* x, float* state, const void* Y, int y_dt,
                             int y_stride, int y_off, const float* yb, void* out, int out_dt,
                             const int32_t* cu, const int32_t* seq_slot, int n_seqs, int max_rows, int C,
                             float* scratch, void* stream) {
    if (n_seqs < 0 || C <= 0 || !illm_dtype_ok(y_dt) || !illm_dtype_ok(out_dt) || y_off < 0 ||
        y_off + C > y_stride || n_seqs > 65535 || max_rows < 0)
        return ILLM_ERR_ARG;
    if (n_seqs == 0) return ILLM_OK;
    hipStream_t st = (hipStream_t)stream;
    const int cblocks = (C + 255) / 256;
    if (scratch && max_rows >= 2 * LRU_CHUNK) {
        const int chunks = (max_rows + LRU_CHUNK - 1) / LRU_CHUNK;
        if (chunks > 65535) return ILLM_ERR_ARG;
        float* P = scratch;
        float* B = scratch + (size_t)n_seqs * chunks * C;
        hipLaunchKernelGGL(lru_chunk_sums_kernel, dim3(cblocks, chunks, n_seqs), dim3(256), 0, st, a, x, P, B, cu,
                           C, chunks);
        hipLaunchKernelGGL(lru_chunk_carry_kernel, dim3(cblocks, n_seqs), dim3(256), 0, st, P, B, state, cu,
                           seq_slot, C, chunks);
        hipLaunchKernelGGL(lru_chunk_apply_kernel, dim3(cblocks, chunks, n_seqs), dim3(256), 0, st, a, x, B, Y,
                           y_dt, y_stride, y_off, yb, out, out_dt, cu, C, chunks);
        return illm_launch_status();
    }
    hipLaunchKernelGGL(lru_scan_kernel, dim3(n_seqs, cblocks), dim3(256), 0, st, a, x, state, Y, y_dt,
                       y_stride, y_off, yb, out, out_dt, cu, seq_slot, C);
    return illm_launch_status();
}
