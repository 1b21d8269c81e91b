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

// The recurrence.  grid (ceil(dv / COLS), H, sequences), COLS = 64 / PARTS; one wave: lane = part +
// PARTS * column; a lane holds rows [part NS, part NS + NS) of its column of S, so S^T k and S^T q
// are NS multiply-adds a lane and a sum over the PARTS neighbouring lanes, which stays inside a
// row of 16 lanes (data-parallel moves, no trip through LDS).  Long sequences take 16 parts (the
// chain of dependent operations a token is what bounds them), steps of few tokens take 4 (the
// state's rows are then read and written 64 bytes a piece).  The next token's k, q and decays are
// asked for before this token's arithmetic.  state [slots][H][dk][dv] float32.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
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

template <int NS, int PARTS>
__global__ void __launch_bounds__(64)
delta_scan_kernel(const float* __restrict__ qn, const float* __restrict__ kn,
                  const float* __restrict__ vv, const float* __restrict__ beta,
                  const float* __restrict__ dec, int DW, float* __restrict__ state,
                  const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_slot,
                  float* __restrict__ o, int G, int H, int dk, int dv) {
    constexpr int COLS = 64 / PARTS;
    constexpr int NA = NS >= 4 ? 4 : NS;                // partial sums, to keep the chains short
    const int b = blockIdx.z, h = blockIdx.y, lane = threadIdx.x;
    const int part = lane % PARTS, col = blockIdx.x * COLS + lane / PARTS;
    const int r0 = cu[b], n = cu[b + 1] - r0;
    if (n <= 0) return;
    const int slot = seq_slot[b], gh = h / (H / G), i0 = part * NS;
    const bool live = col < dv;
    float* sp = state + (((size_t)slot * H + h) * dk) * dv + col;
    float s[NS], kc[NS], qc[NS], gc[NS];
#pragma unroll
    for (int ii = 0; ii < NS; ++ii) s[ii] = (live && i0 + ii < dk) ? sp[(size_t)(i0 + ii) * dv] : 0.f;
    float vc, bc;
#define DELTA_FETCH(ROW, K_, Q_, G_, V_, B_)                                                      \
    {                                                                                             \
        const float* kp = kn + ((size_t)(ROW) * G + gh) * dk;                                     \
        const float* qp = qn + ((size_t)(ROW) * G + gh) * dk;                                     \
        const float* dp = dec + ((size_t)(ROW) * H + h) * DW;                                     \
        _Pragma("unroll") for (int ii = 0; ii < NS; ++ii) {                                       \
            const int i = i0 + ii;                                                                \
            const bool in = i < dk;                                                               \
            K_[ii] = in ? kp[i] : 0.f;                                                            \
            Q_[ii] = in ? qp[i] : 0.f;                                                            \
            G_[ii] = in ? (DW == 1 ? dp[0] : dp[i]) : 1.f;                                        \
        }                                                                                         \
        V_ = live ? vv[((size_t)(ROW) * H + h) * dv + col] : 0.f;                                 \
        B_ = beta[(size_t)(ROW) * H + h];                                                         \
    }
    DELTA_FETCH(r0, kc, qc, gc, vc, bc)
    for (int t = 0; t < n; ++t) {
        const int row = r0 + t;
        float kx[NS], qx[NS], gx[NS], vx, bx;
        const int nxt = t + 1 < n ? row + 1 : row;
        DELTA_FETCH(nxt, kx, qx, gx, vx, bx)
        float pa[NA];
#pragma unroll
        for (int a = 0; a < NA; ++a) pa[a] = 0.f;
#pragma unroll
        for (int ii = 0; ii < NS; ++ii) {
            s[ii] *= gc[ii];
            pa[ii % NA] = fmaf(s[ii], kc[ii], pa[ii % NA]);
        }
        float kv = pa[0];
#pragma unroll
        for (int a = 1; a < NA; ++a) kv += pa[a];
        kv = group_sum<PARTS>(kv);
        const float u = bc * (vc - kv);
#pragma unroll
        for (int a = 0; a < NA; ++a) pa[a] = 0.f;
#pragma unroll
        for (int ii = 0; ii < NS; ++ii) {
            s[ii] = fmaf(kc[ii], u, s[ii]);
            pa[ii % NA] = fmaf(s[ii], qc[ii], pa[ii % NA]);
        }
        float ov = pa[0];
#pragma unroll
        for (int a = 1; a < NA; ++a) ov += pa[a];
        ov = group_sum<PARTS>(ov);
        if (part == 0 && live) o[((size_t)row * H + h) * dv + col] = ov;
#pragma unroll
        for (int ii = 0; ii < NS; ++ii) { kc[ii] = kx[ii]; qc[ii] = qx[ii]; gc[ii] = gx[ii]; }
        vc = vx; bc = bx;
    }
#undef DELTA_FETCH
#pragma unroll
    for (int ii = 0; ii < NS; ++ii)
        if (live && i0 + ii < dk) sp[(size_t)(i0 + ii) * dv] = s[ii];
}

// The same recurrence for long runs of tokens (16 parts a column, part p holding rows p, p + 16, ...).  What bounds it is the chain of
// dependent operations a token, so nothing may wait for memory inside it: the k, q and decay rows of
// DELTA_CHUNK tokens go through LDS in two buffers, the next chunk's loads (and its v and beta, in
// registers) are issued before this chunk's arithmetic and stored after it.  One wave a block;
// dynamic LDS: 2 * DELTA_CHUNK * (2 dk + DW) floats.
#define DELTA_CHUNK 8
template <int NS>
__global__ void __launch_bounds__(64)
delta_scan_long_kernel(const float* __restrict__ qn, const float* __restrict__ kn,
                       const float* __restrict__ vv, const float* __restrict__ beta,
                       const float* __restrict__ dec, int DW, float* __restrict__ state,
                       const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_slot,
                       float* __restrict__ o, int G, int H, int dk, int dv) {
    constexpr int PARTS = 16, COLS = 4, TC = DELTA_CHUNK;
    constexpr int JJ = NS >= 4 ? NS / 4 : 1;            // pieces of 64 floats in a row of 16 NS
    constexpr int NA = NS >= 4 ? 4 : NS;
    extern __shared__ float stage[];
    const int b = blockIdx.z, h = blockIdx.y, lane = threadIdx.x;
    const int part = lane % PARTS, col = blockIdx.x * COLS + lane / PARTS;
    const int r0 = cu[b], n = cu[b + 1] - r0;
    if (n <= 0) return;
    const int slot = seq_slot[b], gh = h / (H / G);
    const bool live = col < dv;
    const int RW = 2 * dk + DW;
    float* sp = state + (((size_t)slot * H + h) * dk) * dv + col;
    float s[NS];
#pragma unroll
    for (int ii = 0; ii < NS; ++ii)      // row part + 16 ii: the 16 parts read neighbouring words of LDS
        s[ii] = (live && part + PARTS * ii < dk) ? sp[(size_t)(part + PARTS * ii) * dv] : 0.f;
    float sk[TC][JJ], sq[TC][JJ], sg[TC][JJ], sv[TC], sb[TC];
#define DELTA_LOAD(T0)                                                                            \
    _Pragma("unroll") for (int tt = 0; tt < TC; ++tt) {                                           \
        const int row = r0 + ((T0) + tt < n ? (T0) + tt : n - 1);                                 \
        const float* kp = kn + ((size_t)row * G + gh) * dk;                                       \
        const float* qp = qn + ((size_t)row * G + gh) * dk;                                       \
        const float* dp = dec + ((size_t)row * H + h) * DW;                                       \
        _Pragma("unroll") for (int jj = 0; jj < JJ; ++jj) {                                       \
            const int j = lane + 64 * jj;                                                         \
            sk[tt][jj] = j < dk ? kp[j] : 0.f;                                                    \
            sq[tt][jj] = j < dk ? qp[j] : 0.f;                                                    \
            sg[tt][jj] = j < DW ? dp[j] : 1.f;                                                    \
        }                                                                                         \
        sv[tt] = live ? vv[((size_t)row * H + h) * dv + col] : 0.f;                               \
        sb[tt] = beta[(size_t)row * H + h];                                                       \
    }
#define DELTA_STORE(BUF)                                                                          \
    _Pragma("unroll") for (int tt = 0; tt < TC; ++tt) {                                           \
        float* dst = stage + ((size_t)(BUF) * TC + tt) * RW;                                      \
        _Pragma("unroll") for (int jj = 0; jj < JJ; ++jj) {                                       \
            const int j = lane + 64 * jj;                                                         \
            if (j < dk) { dst[j] = sk[tt][jj]; dst[dk + j] = sq[tt][jj]; }                        \
            if (j < DW) dst[2 * dk + j] = sg[tt][jj];                                             \
        }                                                                                         \
    }
    DELTA_LOAD(0)
    DELTA_STORE(0)
    __syncthreads();
    for (int t0 = 0, buf = 0; t0 < n; t0 += TC, buf ^= 1) {
        float cv[TC], cb[TC];
#pragma unroll
        for (int tt = 0; tt < TC; ++tt) { cv[tt] = sv[tt]; cb[tt] = sb[tt]; }
        const bool more = t0 + TC < n;
        if (more) DELTA_LOAD(t0 + TC)
#pragma unroll
        for (int tt = 0; tt < TC; ++tt) {
            if (t0 + tt < n) {
                const float* src = stage + ((size_t)buf * TC + tt) * RW;
                float kc[NS], qc[NS], gc[NS];
#pragma unroll
                for (int ii = 0; ii < NS; ++ii) {
                    const int i = part + PARTS * ii;
                    const bool in = i < dk;
                    kc[ii] = in ? src[i] : 0.f;
                    qc[ii] = in ? src[dk + i] : 0.f;
                    gc[ii] = in ? src[2 * dk + (DW == 1 ? 0 : i)] : 1.f;
                }
                float pa[NA];
#pragma unroll
                for (int a = 0; a < NA; ++a) pa[a] = 0.f;
#pragma unroll
                for (int ii = 0; ii < NS; ++ii) {
                    s[ii] *= gc[ii];
                    pa[ii % NA] = fmaf(s[ii], kc[ii], pa[ii % NA]);
                }
                float kv = pa[0];
#pragma unroll
                for (int a = 1; a < NA; ++a) kv += pa[a];
                kv = group_sum<PARTS>(kv);
                const float u = cb[tt] * (cv[tt] - kv);
#pragma unroll
                for (int a = 0; a < NA; ++a) pa[a] = 0.f;
#pragma unroll
                for (int ii = 0; ii < NS; ++ii) {
                    s[ii] = fmaf(kc[ii], u, s[ii]);
                    pa[ii % NA] = fmaf(s[ii], qc[ii], pa[ii % NA]);
                }
                float ov = pa[0];
#pragma unroll
                for (int a = 1; a < NA; ++a) ov += pa[a];
                ov = group_sum<PARTS>(ov);
                if (part == 0 && live) o[((size_t)(r0 + t0 + tt) * H + h) * dv + col] = ov;
            }
        }
        if (more) DELTA_STORE(buf ^ 1)
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
extern "C" int illm_delta_scan(const float* qn, const float* kn, const float* vv, const float* beta,
                               const float* dec, int DW, float* state, const int32_t* cu,
                               const int32_t* seq_slot, float* o, int n_seqs, int max_rows, int G,
                               int H, int dk, int dv, void* stream) {
    if (n_seqs < 0 || G <= 0 || H <= 0 || H % G || dk <= 0 || dk > 256 || dv <= 0 ||
        (DW != 1 && DW != dk) || H > 65535 || n_seqs > 65535)
        return ILLM_ERR_ARG;
    if (n_seqs == 0) return ILLM_OK;
    hipStream_t st = (hipStream_t)stream;
#define GO(NS_, PARTS_)                                                                          \
    hipLaunchKernelGGL((delta_scan_kernel<NS_, PARTS_>), dim3((dv + 64 / PARTS_ - 1) / (64 / PARTS_), H, n_seqs), \
                       dim3(64), 0, st, qn, kn, vv, beta, dec, DW, state, cu, seq_slot, o, G, H, dk, dv)
    if (max_rows >= 16) {
        const int ns = (dk + 15) / 16;
        const size_t lds = (size_t)2 * DELTA_CHUNK * (2 * dk + DW) * sizeof(float);
        const dim3 grid((dv + 3) / 4, H, n_seqs);
#define GOL(NS_)                                                                                  \
    hipLaunchKernelGGL(delta_scan_long_kernel<NS_>, grid, dim3(64), lds, st, qn, kn, vv, beta, dec, DW, \
                       state, cu, seq_slot, o, G, H, dk, dv)
        if (ns <= 1) GOL(1);
        else if (ns <= 2) GOL(2);
        else if (ns <= 4) GOL(4);
        else if (ns <= 8) GOL(8);
        else GOL(16);
#undef GOL
    } else {
        const int ns = (dk + 3) / 4;
        if (ns <= 4) GO(4, 4);
        else if (ns <= 8) GO(8, 4);
        else if (ns <= 16) GO(16, 4);
        else if (ns <= 32) GO(32, 4);
        else GO(64, 4);
    }
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
