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
// Everything but the stored projections is float32.  A sequence's rows in a step are consecutive;
// a step may go on from any state (single tokens, portions of a prompt) or start from the zeros a
// fresh slot holds.  Sums run in an order fixed by the sizes alone.
#include <math.h>

#include "api.h"
#include "common.h"

#define DELTA_MAX_TAPS 8

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// grid (rows); 256 threads; dynamic LDS: C floats.
// P [T, p_stride]: columns [0, C) = q (G dk) | k (G dk) | v (H dv) before the convolution, b_off: H
// columns of b.  A [T, a_stride] + a_off: the decays' pre-activations, DW a head (1 or dk).
__global__ void __launch_bounds__(256)
delta_prepare_kernel(const void* __restrict__ P, int p_dt, int p_stride, int b_off,
                     const void* __restrict__ A, int a_dt, int a_stride, int a_off,
                     const float* __restrict__ conv_w, int taps, const void* __restrict__ tail,
                     int tail_dt, const int32_t* __restrict__ row_slot,
                     const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                     float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ vv,
                     float* __restrict__ beta, float* __restrict__ dec, int G, int H, int dk, int dv,
                     int DW) {
    extern __shared__ float cs[];
    const int r = blockIdx.x, tid = threadIdx.x;
    const int C = 2 * G * dk + H * dv, K = taps - 1;
    const int slot = row_slot[r];
    int before = 0;                                     // rows of this sequence ahead of r in the step, up to K
    while (before < K && r - before - 1 >= 0 && row_slot[r - before - 1] == slot) ++before;
    for (int c = tid; c < C; c += 256) {
        float a = 0.f;
        for (int j = 0; j < taps; ++j) {
            const int d = K - j;                        // tap j looks d tokens back
            float x;
            if (d <= before) x = ld_f(P, p_dt, (size_t)(r - d) * p_stride + c);
            else x = ld_f(tail, tail_dt, ((size_t)slot * K + (K - (d - before))) * C + c);
            a = fmaf(conv_w[(size_t)c * taps + j], x, a);
        }
        cs[c] = a * sigmoid_f(a);
    }
    __syncthreads();
    const int w = tid >> 6, lane = tid & 63;
    const float qscale = 1.0f / sqrtf((float)dk);
    for (int vct = w; vct < 2 * G; vct += 4) {          // q heads, then k heads
        const float* src = cs + (size_t)vct * dk;
        float ss = 0.f;
        for (int i = lane; i < dk; i += 64) ss += src[i] * src[i];
        ss = wave_sum(ss);
        const float inv = (vct < G ? qscale : 1.0f) / sqrtf(ss + 1e-6f);
        float* dst = vct < G ? qn + ((size_t)r * G + vct) * dk : kn + ((size_t)r * G + (vct - G)) * dk;
        for (int i = lane; i < dk; i += 64) dst[i] = src[i] * inv;
    }
    for (int i = tid; i < H * dv; i += 256) vv[(size_t)r * H * dv + i] = cs[2 * G * dk + i];
    for (int i = tid; i < H; i += 256)
        beta[(size_t)r * H + i] = sigmoid_f(ld_f(P, p_dt, (size_t)r * p_stride + b_off + i));
    for (int i = tid; i < H * DW; i += 256) {
        const int hh = i / DW;
        const float a = ld_f(A, a_dt, (size_t)r * a_stride + a_off + i) + dt_bias[i];
        dec[(size_t)r * H * DW + i] = expf(-expf(a_log[hh]) * softplus_f(a));
    }
}

extern "C" int illm_delta_prepare(const void* P, int p_dt, int p_stride, int b_off, const void* A,
                                  int a_dt, int a_stride, int a_off, const float* conv_w, int taps,
                                  const void* tail, int tail_dt, const int32_t* row_slot,
                                  const float* a_log, const float* dt_bias, float* qn, float* kn,
                                  float* vv, float* beta, float* dec, int T, int G, int H, int dk,
                                  int dv, int DW, void* stream) {
    if (T < 0 || G <= 0 || H <= 0 || H % G || dk <= 0 || dv <= 0 || (DW != 1 && DW != dk) ||
        taps < 1 || taps > DELTA_MAX_TAPS || !illm_dtype_ok(p_dt) || !illm_dtype_ok(a_dt) ||
        !illm_dtype_ok(tail_dt))
        return ILLM_ERR_ARG;
    const size_t C = 2 * (size_t)G * dk + (size_t)H * dv;
    if (C * sizeof(float) > 150 * 1024) return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    if (C * sizeof(float) > 48 * 1024 &&
        hipFuncSetAttribute((const void*)delta_prepare_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)(C * sizeof(float))) != hipSuccess)
        return ILLM_ERR_LAUNCH;
    hipLaunchKernelGGL(delta_prepare_kernel, dim3(T), dim3(256), C * sizeof(float), (hipStream_t)stream,
                       P, p_dt, p_stride, b_off, A, a_dt, a_stride, a_off, conv_w, taps, tail, tail_dt,
                       row_slot, a_log, dt_bias, qn, kn, vv, beta, dec, G, H, dk, dv, DW);
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

// The recurrence.  grid (ceil(dv / 16), H, sequences); one wave: lane = column + 16 part; a lane
// holds rows [part NS, part NS + NS) of its column of S, so S^T k and S^T q are NS multiply-adds
// and two exchanges a lane.  The next token's k, q and decays are asked for before this token's
// arithmetic.  state [slots][H][dk][dv] float32.
template <int NS>
__global__ void __launch_bounds__(64)
delta_scan_kernel(const float* __restrict__ qn, const float* __restrict__ kn,
                  const float* __restrict__ vv, const float* __restrict__ beta,
                  const float* __restrict__ dec, int DW, float* __restrict__ state,
                  const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_slot,
                  float* __restrict__ o, int G, int H, int dk, int dv) {
    const int b = blockIdx.z, h = blockIdx.y, lane = threadIdx.x;
    const int col = blockIdx.x * 16 + (lane & 15), part = lane >> 4;
    const int r0 = cu[b], n = cu[b + 1] - r0;
    if (n <= 0) return;
    const int slot = seq_slot[b], gh = h / (H / G), i0 = part * NS;
    const bool live = col < dv;
    float* sp = state + (((size_t)slot * H + h) * dk) * dv + col;
    float s[NS], kc[NS], qc[NS], gc[NS];
#pragma unroll
    for (int ii = 0; ii < NS; ++ii) s[ii] = (live && i0 + ii < dk) ? sp[(size_t)(i0 + ii) * dv] : 0.f;
    auto fetch = [&](int row, float* k_, float* q_, float* g_, float& v_, float& b_) {
        const float* kp = kn + ((size_t)row * G + gh) * dk;
        const float* qp = qn + ((size_t)row * G + gh) * dk;
        const float* dp = dec + ((size_t)row * H + h) * DW;
#pragma unroll
        for (int ii = 0; ii < NS; ++ii) {
            const int i = i0 + ii;
            const bool in = i < dk;
            k_[ii] = in ? kp[i] : 0.f;
            q_[ii] = in ? qp[i] : 0.f;
            g_[ii] = in ? (DW == 1 ? dp[0] : dp[i]) : 1.f;
        }
        v_ = live ? vv[((size_t)row * H + h) * dv + col] : 0.f;
        b_ = beta[(size_t)row * H + h];
    };
    float vc, bc;
    fetch(r0, kc, qc, gc, vc, bc);
    for (int t = 0; t < n; ++t) {
        const int row = r0 + t;
        float kx[NS], qx[NS], gx[NS], vx, bx;
        fetch(t + 1 < n ? row + 1 : row, kx, qx, gx, vx, bx);
        float kv = 0.f;
#pragma unroll
        for (int ii = 0; ii < NS; ++ii) {
            s[ii] *= gc[ii];
            kv = fmaf(s[ii], kc[ii], kv);
        }
        kv += __shfl_xor(kv, 16, 64);
        kv += __shfl_xor(kv, 32, 64);
        const float u = bc * (vc - kv);
        float ov = 0.f;
#pragma unroll
        for (int ii = 0; ii < NS; ++ii) {
            s[ii] = fmaf(kc[ii], u, s[ii]);
            ov = fmaf(s[ii], qc[ii], ov);
        }
        ov += __shfl_xor(ov, 16, 64);
        ov += __shfl_xor(ov, 32, 64);
        if (part == 0 && live) o[((size_t)row * H + h) * dv + col] = ov;
#pragma unroll
        for (int ii = 0; ii < NS; ++ii) { kc[ii] = kx[ii]; qc[ii] = qx[ii]; gc[ii] = gx[ii]; }
        vc = vx; bc = bx;
    }
#pragma unroll
    for (int ii = 0; ii < NS; ++ii)
        if (live && i0 + ii < dk) sp[(size_t)(i0 + ii) * dv] = s[ii];
}

extern "C" int illm_delta_scan(const float* qn, const float* kn, const float* vv, const float* beta,
                               const float* dec, int DW, float* state, const int32_t* cu,
                               const int32_t* seq_slot, float* o, int n_seqs, int G, int H, int dk,
                               int dv, void* stream) {
    if (n_seqs < 0 || G <= 0 || H <= 0 || H % G || dk <= 0 || dk > 256 || dv <= 0 ||
        (DW != 1 && DW != dk) || H > 65535 || n_seqs > 65535)
        return ILLM_ERR_ARG;
    if (n_seqs == 0) return ILLM_OK;
    const dim3 grid((dv + 15) / 16, H, n_seqs);
    hipStream_t st = (hipStream_t)stream;
#define GO(NS_)                                                                                  \
    hipLaunchKernelGGL(delta_scan_kernel<NS_>, grid, dim3(64), 0, st, qn, kn, vv, beta, dec, DW, \
                       state, cu, seq_slot, o, G, H, dk, dv)
    const int ns = (dk + 3) / 4;
    if (ns <= 4) GO(4);
    else if (ns <= 8) GO(8);
    else if (ns <= 16) GO(16);
    else if (ns <= 24) GO(24);
    else if (ns <= 32) GO(32);
    else if (ns <= 48) GO(48);
    else GO(64);
#undef GO
    return illm_launch_status();
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
