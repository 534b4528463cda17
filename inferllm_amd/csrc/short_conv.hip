// A short causal convolution over time on every channel of packed rows, with the inputs before
// a step's first row kept per sequence:
//     in(t)  = X[t, x_off + c] (+ in_bias[c])
//     y(t)   = (add_input ? in(t) : 0) + bias[c] + sum_{j < taps} w[c, j] in(t - (taps - 1 - j))
// in(t) is zero before a sequence's first token.  A sequence's rows in a step are consecutive; what
// lies before the step's first row comes from `tail` [slots][taps - 1][C] (the newest input last),
// which a fresh slot holds as zeros.  A step of single tokens moves the tail on in the same launch
// (`update_tail`: the thread that has read a channel's taps writes them back); after a step of
// several tokens a sequence `short_conv_tail` does.  With `in_bias` the inputs are rounded to the
// tail's storage type wherever they are read, so a row sees the same numbers whether its
// neighbours came in this step or an earlier one.  Sums are float32 in the order of the taps.
#include <math.h>

#include "api.h"
#include "common.h"

#define CONV_MAX_TAPS 8

__device__ __forceinline__ float conv_round(float v, int dt) {
    return dt == ILLM_BF16 ? bf16_to_f32(f32_to_bf16(v)) : v;
}

__device__ __forceinline__ float4 sc_ld4(const void* p, int dt, size_t i4) {
    if (dt == ILLM_BF16) {
        const uint2 u = ((const uint2*)p)[i4];
        return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                           __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
    }
    return ((const float4*)p)[i4];
}

__device__ __forceinline__ void sc_st4(void* p, int dt, size_t i4, float4 v) {
    if (dt == ILLM_BF16) {
        uint2 u;
        u.x = pack_bf16x2(v.x, v.y);
        u.y = pack_bf16x2(v.z, v.w);
        ((uint2*)p)[i4] = u;
    } else {
        ((float4*)p)[i4] = v;
    }
}

// Four channels a thread where the rows allow (C, the offset and the strides multiples of 4): grid
// (rows, ceil(C / 1024)).
__global__ void __launch_bounds__(256)
short_conv_vec4_kernel(const void* __restrict__ X, int x_dt, int x_stride, int x_off,
                       const float* __restrict__ in_bias, const float* __restrict__ w,
                       const float* __restrict__ bias, int taps, void* __restrict__ tail, int tail_dt,
                       const int32_t* __restrict__ row_slot, int add_input, void* __restrict__ out,
                       int out_dt, int out_stride, int C, int update_tail) {
    const int r = blockIdx.x, c4 = blockIdx.y * 256 + threadIdx.x;
    if (4 * c4 >= C) return;
    const int K = taps - 1, slot = row_slot[r];
    int above[CONV_MAX_TAPS];
#pragma unroll
    for (int j = 1; j < CONV_MAX_TAPS; ++j) above[j] = (j <= K && r - j >= 0) ? row_slot[r - j] : -1;
    float4 ib = make_float4(0.f, 0.f, 0.f, 0.f);
    if (in_bias) ib = ((const float4*)in_bias)[c4];
    // the rows above are asked for together with their slots, before it is known how many of them
    // belong to this sequence (a row of another sequence is then read and dropped): one trip to
    // memory instead of two in a row
    float4 in[CONV_MAX_TAPS];                   // (indexed by constants only: the array stays in registers)
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
        if (j >= taps) continue;
        const int rr = max(r - (K - j), 0);
        in[j] = sc_ld4(X, x_dt, ((size_t)rr * x_stride + x_off) / 4 + c4);
    }
    int n = 0;
#pragma unroll
    for (int j = 1; j < CONV_MAX_TAPS; ++j)
        if (n == j - 1 && above[j] == slot) n = j;
    float4 cur = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
        if (j >= taps) continue;
        const int back = K - j;
        if (back <= n) {
            float4 v = in[j];
            v.x += ib.x; v.y += ib.y; v.z += ib.z; v.w += ib.w;
            if (in_bias) {
                v.x = conv_round(v.x, tail_dt); v.y = conv_round(v.y, tail_dt);
                v.z = conv_round(v.z, tail_dt); v.w = conv_round(v.w, tail_dt);
            }
            in[j] = v;
        } else {
            in[j] = sc_ld4(tail, tail_dt, ((size_t)slot * K + (K - (back - n))) * (C / 4) + c4);
        }
        if (back == 0) cur = in[j];
    }
    float y[4];
    if (bias) { const float4 b4 = ((const float4*)bias)[c4]; y[0] = b4.x; y[1] = b4.y; y[2] = b4.z; y[3] = b4.w; }
    else y[0] = y[1] = y[2] = y[3] = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float* cw = w + (size_t)(4 * c4 + e) * taps;
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS; ++j)
            if (j < taps) y[e] = fmaf(cw[j], ((const float*)&in[j])[e], y[e]);
        if (add_input) y[e] += ((const float*)&cur)[e];
    }
    sc_st4(out, out_dt, ((size_t)r * out_stride) / 4 + c4, make_float4(y[0], y[1], y[2], y[3]));
    if (update_tail) {
#pragma unroll
        for (int j = 1; j < CONV_MAX_TAPS; ++j)
            if (j < taps) sc_st4(tail, tail_dt, ((size_t)slot * K + (j - 1)) * (C / 4) + c4, in[j]);
    }
}

// grid (rows, ceil(C / 256)); 256 threads, one a channel.
__global__ void __launch_bounds__(256)
short_conv_kernel(const void* __restrict__ X, int x_dt, int x_stride, int x_off,
                  const float* __restrict__ in_bias, const float* __restrict__ w,
                  const float* __restrict__ bias, int taps, void* __restrict__ tail, int tail_dt,
                  const int32_t* __restrict__ row_slot, int add_input, void* __restrict__ out,
                  int out_dt, int out_stride, int C, int update_tail) {
    const int r = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int K = taps - 1, slot = row_slot[r];
    int above[CONV_MAX_TAPS];                   // the slots of the rows above, all asked for at once
#pragma unroll
    for (int j = 1; j < CONV_MAX_TAPS; ++j) above[j] = (j <= K && r - j >= 0) ? row_slot[r - j] : -1;
    int n = 0;                                  // rows of the same sequence right above this one
#pragma unroll
    for (int j = 1; j < CONV_MAX_TAPS; ++j)
        if (n == j - 1 && above[j] == slot) n = j;
    const float ib = in_bias ? in_bias[c] : 0.f;
    float in[CONV_MAX_TAPS];                    // in[j]: the input taps - 1 - j rows back (indexed by
    float cur = 0.f;                            // constants only: the array stays in registers)
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
        if (j >= taps) continue;
        const int back = K - j;
        if (back <= n) {
            const float v = ld_f(X, x_dt, (size_t)(r - back) * x_stride + x_off + c) + ib;
            in[j] = in_bias ? conv_round(v, tail_dt) : v;
        } else {
            in[j] = ld_f(tail, tail_dt, ((size_t)slot * K + (K - (back - n))) * C + c);
        }
        if (back == 0) cur = in[j];
    }
    float y = bias ? bias[c] : 0.f;
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j)
        if (j < taps) y = fmaf(w[(size_t)c * taps + j], in[j], y);
    if (add_input) y += cur;
    st_f(out, out_dt, (size_t)r * out_stride + c, y);
    if (update_tail) {
#pragma unroll
        for (int j = 1; j < CONV_MAX_TAPS; ++j)
            if (j < taps) st_f(tail, tail_dt, ((size_t)slot * K + (j - 1)) * C + c, in[j]);
    }
}

extern "C" int illm_short_conv(const void* X, int x_dt, int x_stride, int x_off, const float* in_bias,
                               const float* w, const float* bias, int taps, void* tail, int tail_dt,
                               const int32_t* row_slot, int add_input, void* out, int out_dt,
                               int out_stride, int T, int C, int update_tail, void* stream) {
    if (T < 0 || C <= 0 || taps < 1 || taps > CONV_MAX_TAPS || !illm_dtype_ok(x_dt) ||
        !illm_dtype_ok(tail_dt) || !illm_dtype_ok(out_dt) || x_off < 0 || x_off + C > x_stride ||
        out_stride < C || (C + 255) / 256 > 65535)
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    if (C % 4 == 0 && x_off % 4 == 0 && x_stride % 4 == 0 && out_stride % 4 == 0) {
        hipLaunchKernelGGL(short_conv_vec4_kernel, dim3(T, (C / 4 + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                           X, x_dt, x_stride, x_off, in_bias, w, bias, taps, tail, tail_dt, row_slot,
                           add_input, out, out_dt, out_stride, C, taps > 1 ? update_tail : 0);
        return illm_launch_status();
    }
    hipLaunchKernelGGL(short_conv_kernel, dim3(T, (C + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                       X, x_dt, x_stride, x_off, in_bias, w, bias, taps, tail, tail_dt, row_slot,
                       add_input, out, out_dt, out_stride, C, taps > 1 ? update_tail : 0);
    return illm_launch_status();
}

// The last taps - 1 inputs of every sequence of a step into `tail`.  grid (sequences, ceil(C / 256)).
__global__ void __launch_bounds__(256)
short_conv_tail_kernel(const void* __restrict__ X, int x_dt, int x_stride, int x_off,
                       const float* __restrict__ in_bias, void* __restrict__ tail, int tail_dt,
                       const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_slot, int C, int K) {
    const int b = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int r0 = cu[b], n = cu[b + 1] - r0;
    if (n <= 0) return;
    const int slot = seq_slot[b];
    const float ib = in_bias ? in_bias[c] : 0.f;
    float keep[CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
        if (j >= K) continue;
        const int at = n - K + j;                       // row of the step, or before it
        keep[j] = at >= 0 ? ld_f(X, x_dt, (size_t)(r0 + at) * x_stride + x_off + c) + ib
                          : ld_f(tail, tail_dt, ((size_t)slot * K + (j + n)) * C + c);
    }
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j)
        if (j < K) st_f(tail, tail_dt, ((size_t)slot * K + j) * C + c, keep[j]);
}

extern "C" int illm_short_conv_tail(const void* X, int x_dt, int x_stride, int x_off,
                                    const float* in_bias, void* tail, int tail_dt, const int32_t* cu,
                                    const int32_t* seq_slot, int n_seqs, int C, int taps, void* stream) {
    if (n_seqs < 0 || C <= 0 || taps < 1 || taps > CONV_MAX_TAPS || !illm_dtype_ok(x_dt) ||
        !illm_dtype_ok(tail_dt) || x_off < 0 || x_off + C > x_stride || (C + 255) / 256 > 65535)
        return ILLM_ERR_ARG;
    if (n_seqs == 0 || taps == 1) return ILLM_OK;
    hipLaunchKernelGGL(short_conv_tail_kernel, dim3(n_seqs, (C + 255) / 256), dim3(256), 0,
                       (hipStream_t)stream, X, x_dt, x_stride, x_off, in_bias, tail, tail_dt, cu,
                       seq_slot, C, taps - 1);
    return illm_launch_status();
}

// ---------------------------------------------------------------- norm of a sublayer's output
// out[r, :] = gain * a[r, :] / sqrt(mean(a[r]^2) + eps) * w, float32: what a sublayer whose output
// passes a norm of its own leaves to be added to the residual stream.  grid (rows); 256 threads.
__global__ void __launch_bounds__(256)
rms_rows_gain_kernel(const void* __restrict__ a, int a_dt, const void* __restrict__ w, int w_dt,
                     float* __restrict__ out, int E, float eps, float gain) {
    __shared__ float red[16];
    const size_t base = (size_t)blockIdx.x * E;
    float ss = 0.f;
    for (int i = threadIdx.x; i < E; i += 256) {
        const float v = ld_f(a, a_dt, base + i);
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)E + eps);
    for (int i = threadIdx.x; i < E; i += 256)
        out[base + i] = gain * (ld_f(a, a_dt, base + i) * inv * ld_f(w, w_dt, i));
}

extern "C" int illm_rms_rows_gain(const void* a, int a_dt, const void* w, int w_dt, float* out,
                                  int rows, int E, float eps, float gain, void* stream) {
    if (rows < 0 || E <= 0 || !illm_dtype_ok(a_dt) || !illm_dtype_ok(w_dt)) return ILLM_ERR_ARG;
    if (rows == 0) return ILLM_OK;
    hipLaunchKernelGGL(rms_rows_gain_kernel, dim3(rows), dim3(256), 0, (hipStream_t)stream, a, a_dt, w,
                       w_dt, out, E, eps, gain);
    return illm_launch_status();
}

// ---------------------------------------------------------------- clamped gate * (up + 1)
// gate_up [T, 2F] = [gate | up]: g = min(gate, limit), u = clamp(up, -limit, limit),
// out = g sigmoid(alpha g) (u + 1).  grid (ceil(F / 256), rows).
__global__ void __launch_bounds__(256)
clamped_swish_mul_kernel(const void* __restrict__ gu, void* __restrict__ out, int dt, int F,
                         float limit, float alpha) {
    const size_t t = blockIdx.y;
    const int f = blockIdx.x * 256 + threadIdx.x;
    if (f >= F) return;
    const float g = fminf(ld_f(gu, dt, t * 2 * F + f), limit);
    const float u = fminf(fmaxf(ld_f(gu, dt, t * 2 * F + F + f), -limit), limit);
    st_f(out, dt, t * F + f, g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
}

// bfloat16 rows with F % 8 == 0: 8 values (16 bytes) of gate and of up a thread
__global__ void __launch_bounds__(256)
clamped_swish_mul_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int F, float limit,
                                float alpha) {
    const size_t t = blockIdx.y;
    const int f = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (f >= F) return;
    const uint4 g = *(const uint4*)(gu + t * 2 * F + f);
    const uint4 u = *(const uint4*)(gu + t * 2 * F + F + f);
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t ow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float g0 = fminf(__uint_as_float(gw[i] << 16), limit), g1 = fminf(__uint_as_float(gw[i] & 0xffff0000u), limit);
        const float u0 = fminf(fmaxf(__uint_as_float(uw[i] << 16), -limit), limit);
        const float u1 = fminf(fmaxf(__uint_as_float(uw[i] & 0xffff0000u), -limit), limit);
        ow[i] = pack_bf16x2(g0 / (1.0f + expf(-alpha * g0)) * (u0 + 1.0f), g1 / (1.0f + expf(-alpha * g1)) * (u1 + 1.0f));
    }
    *(uint4*)(out + t * F + f) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

extern "C" int illm_clamped_swish_mul(const void* gate_up, void* out, int dt, int T, int F,
                                      float limit, float alpha, void* stream) {
    if (T < 0 || F <= 0 || !illm_dtype_ok(dt) || !(limit > 0.f)) return ILLM_ERR_ARG;
    if (dt == ILLM_BF16 && F % 8 == 0) {
        for (int t0 = 0; t0 < T; t0 += 65535) {
            const int rows = T - t0 < 65535 ? T - t0 : 65535;
            hipLaunchKernelGGL(clamped_swish_mul_bf16x8_kernel, dim3((F / 8 + 255) / 256, rows), dim3(256), 0,
                               (hipStream_t)stream, (const bf16_t*)gate_up + (size_t)t0 * 2 * F,
                               (bf16_t*)out + (size_t)t0 * F, F, limit, alpha);
        }
        return illm_launch_status();
    }
    const size_t esz = dt == ILLM_BF16 ? 2 : 4;
    for (int t0 = 0; t0 < T; t0 += 65535) {
        const int rows = T - t0 < 65535 ? T - t0 : 65535;
        hipLaunchKernelGGL(clamped_swish_mul_kernel, dim3((F + 255) / 256, rows), dim3(256), 0,
                           (hipStream_t)stream, (const void*)((const char*)gate_up + (size_t)t0 * 2 * F * esz),
                           (void*)((char*)out + (size_t)t0 * F * esz), dt, F, limit, alpha);
    }
    return illm_launch_status();
}

// ---------------------------------------------------------------- one pass between two sublayers
// What stands between a sublayer that has its own norm behind it and the next sublayer's input:
//     x <- x + gain * a / sqrt(mean(a^2) + post_eps) * post_w          (a null: nothing is added)
//     h  = x / sqrt(mean(x^2) + eps) * w                                (rounded to the output's type)
//     out = h + sum_j conv_w[:, j] h(t - (taps - 1 - j))                (conv_w null: out = h)
// With `row_idx` only those rows are formed and x is left as it is.  The convolution is for steps of
// one row a sequence: the earlier inputs come from tail [slots][taps - 1][E], which is moved on.
// grid (rows); 256 threads.  A thread owns NV groups of 4 consecutive columns (E % 4 == 0, E <= 1024
// NV) and asks for everything it reads of a pass before it uses any of it; other widths take the
// plain loop (NV 0), which keeps the row's sum in LDS (E floats) between the passes.
template <int NV>
__global__ void __launch_bounds__(256)
post_add_rmsnorm_kernel(float* __restrict__ x, const void* __restrict__ a, int a_dt,
                        const void* __restrict__ post_w, int post_w_dt, float post_eps, float gain,
                        const void* __restrict__ w, int w_dt, void* __restrict__ out, int out_dt,
                        const int32_t* __restrict__ row_idx, int E, float eps,
                        const float* __restrict__ conv_w, int taps, void* __restrict__ tail, int tail_dt,
                        const int32_t* __restrict__ row_slot) {
    extern __shared__ float row[];
    __shared__ float red[16];
    const int r = blockIdx.x;
    const int in_row = row_idx ? row_idx[r] : r;
    const size_t ib = (size_t)in_row * E, ob = (size_t)r * E;
    const int K = taps - 1;
    const int slot = conv_w ? row_slot[r] : 0;
    if (NV > 0) {
        const int n4 = E / 4;
        float4 xv[NV > 0 ? NV : 1], av[NV > 0 ? NV : 1], pwv[NV > 0 ? NV : 1], wv4[NV > 0 ? NV : 1];
        const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int i4 = threadIdx.x + 256 * k;
            xv[k] = i4 < n4 ? ((const float4*)(x + ib))[i4] : zero4;
            av[k] = (a && i4 < n4) ? sc_ld4(a, a_dt, ib / 4 + i4) : zero4;
            pwv[k] = (a && i4 < n4) ? sc_ld4(post_w, post_w_dt, i4) : zero4;
            wv4[k] = i4 < n4 ? sc_ld4(w, w_dt, i4) : zero4;
        }
        if (a) {
            float sa = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k) sa += av[k].x * av[k].x + av[k].y * av[k].y + av[k].z * av[k].z + av[k].w * av[k].w;
            sa = block_sum(sa, red);
            const float inv_a = 1.0f / sqrtf(sa / (float)E + post_eps);
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const int i4 = threadIdx.x + 256 * k;
                if (i4 >= n4) continue;
                const float4 pw = pwv[k];
                xv[k].x += gain * (av[k].x * inv_a * pw.x);
                xv[k].y += gain * (av[k].y * inv_a * pw.y);
                xv[k].z += gain * (av[k].z * inv_a * pw.z);
                xv[k].w += gain * (av[k].w * inv_a * pw.w);
                if (!row_idx) ((float4*)(x + ib))[i4] = xv[k];
            }
        }
        float ss = 0.f;
#pragma unroll
        for (int k = 0; k < NV; ++k) ss += xv[k].x * xv[k].x + xv[k].y * xv[k].y + xv[k].z * xv[k].z + xv[k].w * xv[k].w;
        ss = block_sum(ss, red);
        const float scale = 1.0f / sqrtf(ss / (float)E + eps);
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int i4 = threadIdx.x + 256 * k;
            if (i4 >= n4) continue;
            const float4 wv = wv4[k];
            float h[4] = {(xv[k].x * scale) * wv.x, (xv[k].y * scale) * wv.y, (xv[k].z * scale) * wv.z,
                          (xv[k].w * scale) * wv.w};
            if (conv_w) {
                float4 old[CONV_MAX_TAPS - 1];
#pragma unroll
                for (int j = 0; j < CONV_MAX_TAPS - 1; ++j)
                    if (j < K) old[j] = sc_ld4(tail, tail_dt, ((size_t)slot * K + j) * n4 + i4);
                float hq[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    hq[e] = conv_round(h[e], out_dt);
                    const float* cw = conv_w + (size_t)(4 * i4 + e) * taps;
                    float c = 0.f;
#pragma unroll
                    for (int j = 0; j < CONV_MAX_TAPS - 1; ++j)
                        if (j < K) c = fmaf(cw[j], ((const float*)&old[j])[e], c);
                    c = fmaf(cw[K], hq[e], c);
                    h[e] = hq[e] + c;
                }
                // the tail moves on by the new input
#pragma unroll
                for (int j = 1; j < CONV_MAX_TAPS - 1; ++j)
                    if (j < K) sc_st4(tail, tail_dt, ((size_t)slot * K + (j - 1)) * n4 + i4, old[j]);
                sc_st4(tail, tail_dt, ((size_t)slot * K + (K - 1)) * n4 + i4, make_float4(hq[0], hq[1], hq[2], hq[3]));
            }
            sc_st4(out, out_dt, ob / 4 + i4, make_float4(h[0], h[1], h[2], h[3]));
        }
        return;
    }
    float inv_a = 0.f;
    if (a) {
        float sa = 0.f;
        for (int i = threadIdx.x; i < E; i += 256) {
            const float v = ld_f(a, a_dt, ib + i);
            sa = fmaf(v, v, sa);
        }
        sa = block_sum(sa, red);
        inv_a = 1.0f / sqrtf(sa / (float)E + post_eps);
    }
    float ss = 0.f;
    for (int i = threadIdx.x; i < E; i += 256) {
        float v = x[ib + i];
        if (a) {
            v += gain * (ld_f(a, a_dt, ib + i) * inv_a * ld_f(post_w, post_w_dt, i));
            if (!row_idx) x[ib + i] = v;
        }
        row[i] = v;
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)E + eps);
    for (int i = threadIdx.x; i < E; i += 256) {
        float h = (row[i] * scale) * ld_f(w, w_dt, i);
        if (conv_w) {
            h = conv_round(h, out_dt);
            float in[CONV_MAX_TAPS];
#pragma unroll
            for (int j = 0; j < CONV_MAX_TAPS; ++j) {
                if (j >= taps) continue;
                in[j] = j == K ? h : ld_f(tail, tail_dt, ((size_t)slot * K + j) * E + i);
            }
            float c = 0.f;
#pragma unroll
            for (int j = 0; j < CONV_MAX_TAPS; ++j)
                if (j < taps) c = fmaf(conv_w[(size_t)i * taps + j], in[j], c);
#pragma unroll
            for (int j = 1; j < CONV_MAX_TAPS; ++j)
                if (j < taps) st_f(tail, tail_dt, ((size_t)slot * K + (j - 1)) * E + i, in[j]);
            h += c;
        }
        st_f(out, out_dt, ob + i, h);
    }
}

extern "C" int illm_post_add_rmsnorm(float* x, const void* a, int a_dt, const void* post_w, int post_w_dt,
                                     float post_eps, float gain, const void* w, int w_dt, void* out,
                                     int out_dt, const int32_t* row_idx, int rows, int E, float eps,
                                     const float* conv_w, int taps, void* tail, int tail_dt,
                                     const int32_t* row_slot, void* stream) {
    if (rows < 0 || E <= 0 || !illm_dtype_ok(w_dt) || !illm_dtype_ok(out_dt) ||
        (a && (!illm_dtype_ok(a_dt) || !illm_dtype_ok(post_w_dt) || !post_w)) ||
        (conv_w && (taps < 2 || taps > CONV_MAX_TAPS || !tail || !row_slot || row_idx || !illm_dtype_ok(tail_dt))))
        return ILLM_ERR_ARG;
    if (rows == 0) return ILLM_OK;
    hipStream_t st = (hipStream_t)stream;
#define GO(NV_, LDS_)                                                                                   \
    hipLaunchKernelGGL(post_add_rmsnorm_kernel<NV_>, dim3(rows), dim3(256), LDS_, st, x, a, a_dt, post_w,   \
                       post_w_dt, post_eps, gain, w, w_dt, out, out_dt, row_idx, E, eps, conv_w, taps, tail, \
                       tail_dt, row_slot)
    if (E % 4 == 0 && E <= 8192) {
        if (E <= 1024) GO(1, 0);
        else if (E <= 2048) GO(2, 0);
        else if (E <= 4096) GO(4, 0);
        else GO(8, 0);
        return illm_launch_status();
    }
    const size_t lds = (size_t)E * sizeof(float);
    if (lds > 64 * 1024) return ILLM_ERR_ARG;
    if (lds > 48 * 1024 &&
        hipFuncSetAttribute((const void*)post_add_rmsnorm_kernel<0>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
        return ILLM_ERR_LAUNCH;
    GO(0, lds);
#undef GO
    return illm_launch_status();
}
