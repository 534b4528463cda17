// The gated delta rule: a recurrent mixer whose state per head is a matrix S [key dim, value dim]
// (float32) that every token decays, corrects and reads:
//     S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// with g in (0, 1) one decay a head or one a key channel.  Three kernels around it:
//   delta_prepare   short causal convolution over time of the q|k|v projections (per channel,
//                   `taps` taps, the taps before a step's first row from the kept tail), SiLU, unit
//                   norm of q and k per head (q also times dim^-1/2), beta = sigmoid(b),
//                   g = exp(-exp(A_log) softplus(a + dt_bias))
//   delta_conv_tail the last taps - 1 inputs of every sequence, kept for the next step
//   delta_scan      the recurrence, token after token, from the kept state and back into it
//   delta_finish    o / rms(o) * weight * gate, gate = silu(z) or sigmoid(z)
// The scan also runs the plain gated rule without the correction (`correct` 0),
//     S <- diag(g) S + k (beta v)^T;   o = S^T q
// which is the recurrence of state-space and matrix-memory mixers (linear_scan.hip prepares their
// inputs): beta is then the weight of the token's outer product.
// Everything but the stored projections is float32.  A sequence's rows in a step are consecutive;
// a step may go on from any state (single tokens, portions of a prompt) or start from the zeros a
// fresh slot holds.  Sums run in an order fixed by the sizes alone.
#include <math.h>

#include "api.h"
#include "common.h"

#define DELTA_MAX_TAPS 8

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// grid (rows, NB); 256 threads.  A wave takes a head's vector at a time (q heads, k heads, v heads:
// vector 4 y + w, then every 4 NB-th), lanes over its channels: convolution, SiLU, and for q and k the
// unit norm, all in the wave.  beta and the decays are spread over all threads of the row's blocks.
// P [T, p_stride]: columns [0, C) = q (G dk) | k (G dk) | v (H dv) before the convolution, b_off: H
// columns of b.  A [T, a_stride] + a_off: the decays' pre-activations, DW a head (1 or dk).
// `update_tail`: every sequence brings one row, and the lane that has read a channel's taps also
// writes its tail for the next step (no other row reads that tail in this step).
#define DELTA_VEC_MAX 4                                 // channels a lane holds: head sizes up to 256
template <int DT>
__device__ __forceinline__ float ld_t(const void* p, size_t i) {
    return DT == ILLM_BF16 ? bf16_to_f32(((const bf16_t*)p)[i]) : ((const float*)p)[i];
}
template <int DT>
__device__ __forceinline__ void st_t(void* p, size_t i, float v) {
    if (DT == ILLM_BF16) ((bf16_t*)p)[i] = f32_to_bf16(v);
    else ((float*)p)[i] = v;
}

template <int DT>                                       // the storage type of P, A and the tail
__global__ void __launch_bounds__(256)
delta_prepare_kernel(const void* __restrict__ P, int p_dt, int p_stride, int b_off,
                     const void* __restrict__ A, int a_dt, int a_stride, int a_off,
                     const float* __restrict__ conv_w, int taps, void* __restrict__ tail,
                     int tail_dt, const int32_t* __restrict__ row_slot,
                     const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                     float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ vv,
                     float* __restrict__ beta, float* __restrict__ dec, int G, int H, int dk, int dv,
                     int DW, int update_tail) {
    const int r = blockIdx.x, tid = threadIdx.x, NB = gridDim.y;
    const int C = 2 * G * dk + H * dv, K = taps - 1;
    const int slot = row_slot[r];
    int before = 0;                                     // rows of this sequence ahead of r in the step, up to K
    while (before < K && r - before - 1 >= 0 && row_slot[r - before - 1] == slot) ++before;
    const int w = wave_index(), lane = tid & 63;
    const float qscale = 1.0f / sqrtf((float)dk);
    for (int vct = blockIdx.y * 4 + w; vct < 2 * G + H; vct += 4 * NB) {
        const bool is_v = vct >= 2 * G;
        const int L = is_v ? dv : dk;
        const int c0 = is_v ? 2 * G * dk + (vct - 2 * G) * dv : vct * dk;
        float y[DELTA_VEC_MAX];
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < DELTA_VEC_MAX; ++e) {
            const int i = lane + 64 * e;
            y[e] = 0.f;
            if (i < L) {
                const int c = c0 + i;
                // every tap's input and weight is asked for before the first is used
                float x[DELTA_MAX_TAPS], cw[DELTA_MAX_TAPS];
#pragma unroll
                for (int j = 0; j < DELTA_MAX_TAPS; ++j) {
                    x[j] = cw[j] = 0.f;
                    if (j < taps) {
                        const int d = K - j;            // tap j looks d tokens back
                        x[j] = d <= before ? ld_t<DT>(P, (size_t)(r - d) * p_stride + c)
                                           : ld_t<DT>(tail, ((size_t)slot * K + (K - (d - before))) * C + c);
                        cw[j] = conv_w[(size_t)c * taps + j];
                    }
                }
                float a = 0.f;
#pragma unroll
                for (int j = 0; j < DELTA_MAX_TAPS; ++j) {
                    if (j < taps) {
                        a = fmaf(cw[j], x[j], a);
                        if (update_tail && j > 0) st_t<DT>(tail, ((size_t)slot * K + (j - 1)) * C + c, x[j]);
                    }
                }
                y[e] = a * sigmoid_f(a);
                ss += y[e] * y[e];
            }
        }
        float inv = 1.0f;
        if (!is_v) inv = (vct < G ? qscale : 1.0f) / sqrtf(wave_sum(ss) + 1e-6f);
        float* dst = is_v ? vv + ((size_t)r * H + (vct - 2 * G)) * dv
                          : (vct < G ? qn + ((size_t)r * G + vct) * dk : kn + ((size_t)r * G + (vct - G)) * dk);
#pragma unroll
        for (int e = 0; e < DELTA_VEC_MAX; ++e)
            if (lane + 64 * e < L) dst[lane + 64 * e] = y[e] * inv;
    }
    for (int i = blockIdx.y * 256 + tid; i < H; i += 256 * NB)
        beta[(size_t)r * H + i] = sigmoid_f(ld_t<DT>(P, (size_t)r * p_stride + b_off + i));
    for (int i = blockIdx.y * 256 + tid; i < H * DW; i += 256 * NB) {
        const int hh = i / DW;
        const float a = ld_t<DT>(A, (size_t)r * a_stride + a_off + i) + dt_bias[i];
        dec[(size_t)r * H * DW + i] = expf(-expf(a_log[hh]) * softplus_f(a));
    }
}

extern "C" int illm_delta_prepare(const void* P, int p_dt, int p_stride, int b_off, const void* A,
                                  int a_dt, int a_stride, int a_off, const float* conv_w, int taps,
                                  void* tail, int tail_dt, const int32_t* row_slot,
                                  const float* a_log, const float* dt_bias, float* qn, float* kn,
                                  float* vv, float* beta, float* dec, int T, int G, int H, int dk,
                                  int dv, int DW, int update_tail, void* stream) {
    if (T < 0 || G <= 0 || H <= 0 || H % G || dk <= 0 || dv <= 0 || (DW != 1 && DW != dk) ||
        dk > 64 * DELTA_VEC_MAX || dv > 64 * DELTA_VEC_MAX ||
        taps < 1 || taps > DELTA_MAX_TAPS || !illm_dtype_ok(p_dt) || a_dt != p_dt || tail_dt != p_dt)
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    // blocks a row: enough to fill the chip when the rows are few
    const int most = (2 * G + H + 3) / 4;
    int nb = T >= 2048 ? 1 : (2048 + T - 1) / T;
    nb = nb > most ? most : nb;
#define GO(DT_)                                                                                    \
    hipLaunchKernelGGL(delta_prepare_kernel<DT_>, dim3(T, nb), dim3(256), 0, (hipStream_t)stream, P, p_dt, \
                       p_stride, b_off, A, a_dt, a_stride, a_off, conv_w, taps, tail, tail_dt, row_slot, \
                       a_log, dt_bias, qn, kn, vv, beta, dec, G, H, dk, dv, DW, update_tail)
    if (p_dt == ILLM_BF16) GO(ILLM_BF16);
    else GO(ILLM_F32);
#undef GO
    return illm_launch_status();
}

// grid (sequences, ceil(C / 256)): tail[slot][j] <- the input at position end - K + j, from the
// step's rows or, for the positions before them, from the old tail.
__global__ void __launch_bounds__(256)
delta_conv_tail_kernel(const void* __restrict__ P, int p_dt, int p_stride, void* __restrict__ tail,
                       int tail_dt, const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_slot,
                       int C, int K) {
    const int b = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int r0 = cu[b], n = cu[b + 1] - r0;
    if (n <= 0) return;
    const int slot = seq_slot[b];
    float keep[DELTA_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < DELTA_MAX_TAPS; ++j) {
        if (j >= K) continue;
        const int at = n - K + j;                       // row of the step, or before it
        keep[j] = at >= 0 ? ld_f(P, p_dt, (size_t)(r0 + at) * p_stride + c)
                          : ld_f(tail, tail_dt, ((size_t)slot * K + (j + n)) * C + c);
    }
#pragma unroll
    for (int j = 0; j < DELTA_MAX_TAPS; ++j)
        if (j < K) st_f(tail, tail_dt, ((size_t)slot * K + j) * C + c, keep[j]);
}

extern "C" int illm_delta_conv_tail(const void* P, int p_dt, int p_stride, void* tail, int tail_dt,
                                    const int32_t* cu, const int32_t* seq_slot, int n_seqs, int C,
                                    int taps, void* stream) {
    if (n_seqs < 0 || C <= 0 || taps < 1 || taps > DELTA_MAX_TAPS || !illm_dtype_ok(p_dt) ||
        !illm_dtype_ok(tail_dt) || (C + 255) / 256 > 65535)
        return ILLM_ERR_ARG;
    if (n_seqs == 0 || taps == 1) return ILLM_OK;
    hipLaunchKernelGGL(delta_conv_tail_kernel, dim3(n_seqs, (C + 255) / 256), dim3(256), 0,
                       (hipStream_t)stream, P, p_dt, p_stride, tail, tail_dt, cu, seq_slot, C, taps - 1);
    return illm_launch_status();
}

// The recurrence.  grid (ceil(dv / COLS), H, sequences), COLS = 64 / PARTS; one wave: lane = part +
// PARTS * column; a lane holds rows [part NS, part NS + NS) of its column of S, so S^T k and S^T q
// are NS multiply-adds a lane and a sum over the PARTS neighbouring lanes, which stays inside a
// row of 16 lanes (data-parallel moves, no trip through LDS).  Long sequences take 16 parts (the
// chain of dependent operations a token is what bounds them), steps of few tokens take 4 (the
// state's rows are then read and written 64 bytes a piece).  The next token's k, q and decays are
// asked for before this token's arithmetic.  state [slots][H][dk][dv] float32.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// The sum over the PARTS lanes of a group; every lane of the group gets the same bits.
template <int PARTS>
__device__ __forceinline__ float group_sum(float v) {
    v += dpp_move<0xB1>(v);                 // lanes 1 0 3 2 of every four
    v += dpp_move<0x4E>(v);                 // lanes 2 3 0 1
    if (PARTS == 16) {
        v += dpp_move<0x141>(v);            // the other four of every eight (mirrored)
        v += dpp_move<0x140>(v);            // the other eight of the sixteen (mirrored)
    }
    return v;
}

// Steps of few tokens a sequence (single tokens above all): what counts is the state's bytes.
// grid (ceil(dv / 64), H, sequences); 4 waves: a lane is a column, wave w holds rows [w NS, w NS + NS)
// of it, so a row of S is read and written 256 bytes a wave; k, q and the decays of a row are the
// same for a whole wave.  The waves' partial sums meet in LDS, in wave order.
template <int NS, bool CORRECT>
__global__ void __launch_bounds__(256)
delta_step_kernel(const float* __restrict__ qn, const float* __restrict__ kn,
                  const float* __restrict__ vv, const float* __restrict__ beta,
                  const float* __restrict__ dec, int DW, float* __restrict__ state,
                  const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_slot,
                  float* __restrict__ o, int G, int H, int dk, int dv) {
    __shared__ float red[2][4][64];
    const int b = blockIdx.z, h = blockIdx.y, lane = threadIdx.x & 63, w = wave_index();
    const int col = blockIdx.x * 64 + lane;
    const int r0 = cu[b], n = cu[b + 1] - r0;
    if (n <= 0) return;                                 // the whole block
    const int slot = seq_slot[b], gh = h / (H / G), i0 = w * NS;
    const bool live = col < dv;
    float* sp = state + (((size_t)slot * H + h) * dk) * dv + col;
    float s[NS];
#pragma unroll
    for (int ii = 0; ii < NS; ++ii) s[ii] = (live && i0 + ii < dk) ? sp[(size_t)(i0 + ii) * dv] : 0.f;
    for (int t = 0; t < n; ++t) {
        const int row = r0 + t;
        const float* kp = kn + ((size_t)row * G + gh) * dk;
        const float* qp = qn + ((size_t)row * G + gh) * dk;
        const float* dp = dec + ((size_t)row * H + h) * DW;
        float kc[NS], pa[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ii = 0; ii < NS; ++ii) {
            const int i = i0 + ii;
            kc[ii] = i < dk ? kp[i] : 0.f;
            s[ii] *= i < dk ? (DW == 1 ? dp[0] : dp[i]) : 1.f;
            pa[ii & 3] = fmaf(s[ii], kc[ii], pa[ii & 3]);
        }
        float kv = 0.f;
        if (CORRECT) {
            red[0][w][lane] = (pa[0] + pa[1]) + (pa[2] + pa[3]);
            __syncthreads();
            kv = (red[0][0][lane] + red[0][1][lane]) + (red[0][2][lane] + red[0][3][lane]);
        }
        const float v = live ? vv[((size_t)row * H + h) * dv + col] : 0.f;
        const float u = beta[(size_t)row * H + h] * (v - kv);
        pa[0] = pa[1] = pa[2] = pa[3] = 0.f;
#pragma unroll
        for (int ii = 0; ii < NS; ++ii) {
            const int i = i0 + ii;
            s[ii] = fmaf(kc[ii], u, s[ii]);
            pa[ii & 3] = fmaf(s[ii], i < dk ? qp[i] : 0.f, pa[ii & 3]);
        }
        // (the two buffers take turns by token where the first is not used for S^T k, so that a
        // wave may write the next token's sums while another still reads this token's)
        float (*rd)[64] = red[CORRECT ? 1 : (t & 1)];
        rd[w][lane] = (pa[0] + pa[1]) + (pa[2] + pa[3]);
        __syncthreads();
        if (w == 0 && live)
            o[((size_t)row * H + h) * dv + col] = (rd[0][lane] + rd[1][lane]) + (rd[2][lane] + rd[3][lane]);
    }
#pragma unroll
    for (int ii = 0; ii < NS; ++ii)
        if (live && i0 + ii < dk) sp[(size_t)(i0 + ii) * dv] = s[ii];
}

// The same recurrence for long runs of tokens (16 parts a column, part p holding rows p, p + 16, ...).  What bounds it is the chain of
// dependent operations a token, so nothing may wait for memory inside it: the k, q and decay rows of
// DELTA_CHUNK tokens go through LDS in two buffers, the next chunk's loads (and its v and beta, in
// registers) are issued before this chunk's arithmetic and stored after it.  One wave a block;
// dynamic LDS: 2 * DELTA_CHUNK * 3 * 16 NS floats.
#define DELTA_CHUNK 8
template <int NS, bool CORRECT>
__global__ void __launch_bounds__(64)
delta_scan_long_kernel(const float* __restrict__ qn, const float* __restrict__ kn,
                       const float* __restrict__ vv, const float* __restrict__ beta,
                       const float* __restrict__ dec, int DW, float* __restrict__ state,
                       const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_slot,
                       float* __restrict__ o, int G, int H, int dk, int dv) {
    constexpr int PARTS = 16, COLS = 4, TC = DELTA_CHUNK;
    constexpr int DKP = PARTS * NS;                     // a row of k, q or decays in LDS, filled up
    constexpr int JJ = (DKP + 63) / 64;                 // pieces of 64 floats in it
    constexpr int NA = NS >= 4 ? 4 : NS;
    extern __shared__ float stage[];                    // [2][TC][k | q | decay][DKP]
    const int b = blockIdx.z, h = blockIdx.y, lane = threadIdx.x;
    const int part = lane % PARTS, col = blockIdx.x * COLS + lane / PARTS;
    const int r0 = cu[b], n = cu[b + 1] - r0;
    if (n <= 0) return;
    const int slot = seq_slot[b], gh = h / (H / G);
    const bool live = col < dv;
    float* sp = state + (((size_t)slot * H + h) * dk) * dv + col;
    float s[NS];
#pragma unroll
    for (int ii = 0; ii < NS; ++ii)      // row part + 16 ii: the 16 parts read neighbouring words of LDS
        s[ii] = (live && part + PARTS * ii < dk) ? sp[(size_t)(part + PARTS * ii) * dv] : 0.f;
    const float* kbase = kn + ((size_t)r0 * G + gh) * dk;
    const float* qbase = qn + ((size_t)r0 * G + gh) * dk;
    const float* dbase = dec + ((size_t)r0 * H + h) * DW;
    const float* vbase = vv + ((size_t)r0 * H + h) * dv + (live ? col : 0);
    const float* bbase = beta + (size_t)r0 * H + h;
    float* op = o + ((size_t)r0 * H + h) * dv + col;
    const int kstep = G * dk, dstep = H * DW, vstep = H * dv;
    float sk[TC][JJ], sq[TC][JJ], sg[TC][JJ], sv[TC], sb[TC];
    // Rows beyond dk are filled with k = q = 0 and decay 1, and the tokens of the last chunk beyond
    // the sequence with k = q = v = beta = 0 and decay 1, which leave the state as it is: the
    // arithmetic needs no bounds and no branches.  A whole chunk is loaded through pointers that
    // step from token to token; the last, partial one with every row's place computed and clamped.
    bool in_k[JJ];
#pragma unroll
    for (int jj = 0; jj < JJ; ++jj) in_k[jj] = lane + 64 * jj < dk;
    const int jlast = dk - 1;
#define DELTA_LOAD(T0)                                                                            \
    if ((T0) + TC <= n) {                                                                         \
        const float* kp = kbase + (size_t)(T0) * kstep;                                           \
        const float* qp = qbase + (size_t)(T0) * kstep;                                           \
        const float* dp = dbase + (size_t)(T0) * dstep;                                           \
        const float* vp = vbase + (size_t)(T0) * vstep;                                           \
        const float* bp = bbase + (size_t)(T0) * H;                                               \
        _Pragma("unroll") for (int tt = 0; tt < TC; ++tt) {                                       \
            _Pragma("unroll") for (int jj = 0; jj < JJ; ++jj) {                                   \
                const int j = in_k[jj] ? lane + 64 * jj : jlast;      /* read in bounds, then choose */ \
                const float kx = kp[j], qx = qp[j], gx = dp[DW == 1 ? 0 : j];                     \
                sk[tt][jj] = in_k[jj] ? kx : 0.f;                                                 \
                sq[tt][jj] = in_k[jj] ? qx : 0.f;                                                 \
                sg[tt][jj] = in_k[jj] ? gx : 1.f;                                                 \
            }                                                                                     \
            sv[tt] = *vp;                                                                         \
            sb[tt] = *bp;                                                                         \
            kp += kstep; qp += kstep; dp += dstep; vp += vstep; bp += H;                          \
        }                                                                                         \
    } else {                                                                                      \
        _Pragma("unroll") for (int tt = 0; tt < TC; ++tt) {                                       \
            const bool ok = (T0) + tt < n;                                                        \
            const int at = ok ? (T0) + tt : n - 1;                                                \
            _Pragma("unroll") for (int jj = 0; jj < JJ; ++jj) {                                   \
                const int j = in_k[jj] ? lane + 64 * jj : jlast;                                  \
                const bool use = ok && in_k[jj];                                                  \
                sk[tt][jj] = use ? kbase[(size_t)at * kstep + j] : 0.f;                           \
                sq[tt][jj] = use ? qbase[(size_t)at * kstep + j] : 0.f;                           \
                sg[tt][jj] = use ? dbase[(size_t)at * dstep + (DW == 1 ? 0 : j)] : 1.f;           \
            }                                                                                     \
            sv[tt] = ok ? vbase[(size_t)at * vstep] : 0.f;                                        \
            sb[tt] = ok ? bbase[(size_t)at * H] : 0.f;                                            \
        }                                                                                         \
    }
#define DELTA_STORE(BUF)                                                                          \
    _Pragma("unroll") for (int tt = 0; tt < TC; ++tt) {                                           \
        float* dst = stage + ((size_t)(BUF) * TC + tt) * 3 * DKP;                                 \
        _Pragma("unroll") for (int jj = 0; jj < JJ; ++jj) {                                       \
            const int j = lane + 64 * jj;                                                         \
            if (j < DKP) { dst[j] = sk[tt][jj]; dst[DKP + j] = sq[tt][jj]; dst[2 * DKP + j] = sg[tt][jj]; } \
        }                                                                                         \
    }
    DELTA_LOAD(0)
    DELTA_STORE(0)
    __syncthreads();
    const bool writes = part == 0 && live;
    for (int t0 = 0, buf = 0; t0 < n; t0 += TC, buf ^= 1) {
        float cv[TC], cb[TC];
#pragma unroll
        for (int tt = 0; tt < TC; ++tt) { cv[tt] = sv[tt]; cb[tt] = sb[tt]; }
        const bool more = t0 + TC < n;
        if (more) { DELTA_LOAD(t0 + TC) }
        const float* src0 = stage + (size_t)buf * TC * 3 * DKP + part;
        float ovs[TC];
#pragma unroll
        for (int tt = 0; tt < TC; ++tt) {
            const float* src = src0 + tt * 3 * DKP;
            float kc[NS], pa[NA];
#pragma unroll
            for (int a = 0; a < NA; ++a) pa[a] = 0.f;
#pragma unroll
            for (int ii = 0; ii < NS; ++ii) {
                kc[ii] = src[PARTS * ii];
                s[ii] *= src[2 * DKP + PARTS * ii];
                pa[ii % NA] = fmaf(s[ii], kc[ii], pa[ii % NA]);
            }
            float kv = 0.f;
            if (CORRECT) {
                kv = pa[0];
#pragma unroll
                for (int a = 1; a < NA; ++a) kv += pa[a];
                kv = group_sum<PARTS>(kv);
            }
            const float u = cb[tt] * (cv[tt] - kv);
#pragma unroll
            for (int a = 0; a < NA; ++a) pa[a] = 0.f;
#pragma unroll
            for (int ii = 0; ii < NS; ++ii) {
                s[ii] = fmaf(kc[ii], u, s[ii]);
                pa[ii % NA] = fmaf(s[ii], src[DKP + PARTS * ii], pa[ii % NA]);
            }
            float ov = pa[0];
#pragma unroll
            for (int a = 1; a < NA; ++a) ov += pa[a];
            ovs[tt] = group_sum<PARTS>(ov);
        }
        if (writes) {
#pragma unroll
            for (int tt = 0; tt < TC; ++tt)
                if (t0 + tt < n) op[(size_t)tt * vstep] = ovs[tt];
        }
        op += (size_t)TC * vstep;
        if (more) { DELTA_STORE(buf ^ 1) }
        __syncthreads();
    }
#undef DELTA_LOAD
#undef DELTA_STORE
#pragma unroll
    for (int ii = 0; ii < NS; ++ii)
        if (live && part + PARTS * ii < dk) sp[(size_t)(part + PARTS * ii) * dv] = s[ii];
}

// `max_rows`: the most rows a sequence of the step has.  It chooses the layout (16 parts from 16
// rows on), and the layout the order of a row's sums: a row of a long step and the same row as a
// single token differ in rounding, in nothing else.
extern "C" int illm_gated_scan(const float* qn, const float* kn, const float* vv, const float* beta,
                               const float* dec, int DW, float* state, const int32_t* cu,
                               const int32_t* seq_slot, float* o, int n_seqs, int max_rows, int G,
                               int H, int dk, int dv, int correct, void* stream) {
    if (n_seqs < 0 || G <= 0 || H <= 0 || H % G || dk <= 0 || dk > 256 || dv <= 0 ||
        (DW != 1 && DW != dk) || H > 65535 || n_seqs > 65535)
        return ILLM_ERR_ARG;
    if (n_seqs == 0) return ILLM_OK;
    hipStream_t st = (hipStream_t)stream;
    if (max_rows >= 16) {
        const int ns = (dk + 15) / 16;
        const size_t lds = (size_t)2 * DELTA_CHUNK * 3 * 16 * (ns <= 1 ? 1 : ns <= 2 ? 2 : ns <= 4 ? 4 : ns <= 8 ? 8 : 16) * sizeof(float);
        const dim3 grid((dv + 3) / 4, H, n_seqs);
#define GOL(NS_)                                                                                  \
    if (correct)                                                                                  \
        hipLaunchKernelGGL((delta_scan_long_kernel<NS_, true>), grid, dim3(64), lds, st, qn, kn, vv, beta, \
                           dec, DW, state, cu, seq_slot, o, G, H, dk, dv);                        \
    else                                                                                          \
        hipLaunchKernelGGL((delta_scan_long_kernel<NS_, false>), grid, dim3(64), lds, st, qn, kn, vv, beta, \
                           dec, DW, state, cu, seq_slot, o, G, H, dk, dv)
        if (ns <= 1) { GOL(1); }
        else if (ns <= 2) { GOL(2); }
        else if (ns <= 4) { GOL(4); }
        else if (ns <= 8) { GOL(8); }
        else { GOL(16); }
#undef GOL
    } else {
        const int ns = (dk + 3) / 4;
        const dim3 grid((dv + 63) / 64, H, n_seqs);
#define GOS(NS_)                                                                                  \
    if (correct)                                                                                  \
        hipLaunchKernelGGL((delta_step_kernel<NS_, true>), grid, dim3(256), 0, st, qn, kn, vv, beta, dec, \
                           DW, state, cu, seq_slot, o, G, H, dk, dv);                             \
    else                                                                                          \
        hipLaunchKernelGGL((delta_step_kernel<NS_, false>), grid, dim3(256), 0, st, qn, kn, vv, beta, dec, \
                           DW, state, cu, seq_slot, o, G, H, dk, dv)
        if (ns <= 4) { GOS(4); }
        else if (ns <= 8) { GOS(8); }
        else if (ns <= 16) { GOS(16); }
        else if (ns <= 32) { GOS(32); }
        else { GOS(64); }
#undef GOS
    }
    return illm_launch_status();
}

extern "C" int illm_delta_scan(const float* qn, const float* kn, const float* vv, const float* beta,
                               const float* dec, int DW, float* state, const int32_t* cu,
                               const int32_t* seq_slot, float* o, int n_seqs, int max_rows, int G,
                               int H, int dk, int dv, void* stream) {
    return illm_gated_scan(qn, kn, vv, beta, dec, DW, state, cu, seq_slot, o, n_seqs, max_rows, G, H, dk,
                           dv, 1, stream);
}

// grid (rows, H); one wave: out[r, h dv + j] = o / sqrt(mean_j o^2 + eps) * w[j] * act(z[r, h dv + j]),
// act = silu (gate_kind 0) or sigmoid (1); Z [T, z_stride] + z_off.
__global__ void __launch_bounds__(64)
delta_finish_kernel(const float* __restrict__ o, const void* __restrict__ w, int w_dt,
                    const void* __restrict__ Z, int z_dt, int z_stride, int z_off, int gate_kind,
                    void* __restrict__ out, int out_dt, int H, int dv, float eps) {
    const size_t r = blockIdx.x;
    const int h = blockIdx.y, lane = threadIdx.x;
    const float* op = o + (r * H + h) * dv;
    float ss = 0.f;
    for (int j = lane; j < dv; j += 64) ss += op[j] * op[j];
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
    for (int j = lane; j < dv; j += 64) {
        const float z = ld_f(Z, z_dt, r * z_stride + z_off + (size_t)h * dv + j);
        const float g = gate_kind ? sigmoid_f(z) : z * sigmoid_f(z);
        st_f(out, out_dt, (r * H + h) * dv + j, op[j] * inv * ld_f(w, w_dt, j) * g);
    }
}

extern "C" int illm_delta_finish(const float* o, const void* w, int w_dt, const void* Z, int z_dt,
                                 int z_stride, int z_off, int gate_kind, void* out, int out_dt, int T,
                                 int H, int dv, float eps, void* stream) {
    if (T < 0 || H <= 0 || H > 65535 || dv <= 0 || !illm_dtype_ok(w_dt) || !illm_dtype_ok(z_dt) ||
        !illm_dtype_ok(out_dt) || (gate_kind != 0 && gate_kind != 1))
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(delta_finish_kernel, dim3(T, H), dim3(64), 0, (hipStream_t)stream, o, w, w_dt, Z,
                       z_dt, z_stride, z_off, gate_kind, out, out_dt, H, dv, eps);
    return illm_launch_status();
}
