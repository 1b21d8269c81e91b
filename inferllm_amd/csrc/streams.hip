// Several residual streams (hyper-connections).  Every row keeps S copies x_0 .. x_{S-1} of width
// E, float32 [T, S, E].  A sublayer reads one weighted sum of them and writes its output back
// into all of them at once:
//     read:   u = sum_s read[s] x_s            (read null: every weight 1)
//     write:  x_t <- sum_s mix[s, t] x_s + out[t] y     for every t, from the old streams
// One kernel does the write of the sublayer before and the read and RMS norm of the sublayer that
// follows, as the single-stream norm does with the residual add: the streams go through memory
// once a sublayer.  y = ya * y1 (+ yb * y2): a block whose two parts read the same rows hands both.
// All arithmetic float32; sums over the streams in rising s, over the width in a fixed order.
#include "api.h"
#include "common.h"

#define STREAMS_MAX 8

__device__ __forceinline__ void ld4(const void* p, int dt, size_t i, float* o) {
    if (dt == ILLM_BF16) {
        const uint2 u = *(const uint2*)((const bf16_t*)p + i);
        o[0] = __uint_as_float(u.x << 16); o[1] = __uint_as_float(u.x & 0xffff0000u);
        o[2] = __uint_as_float(u.y << 16); o[3] = __uint_as_float(u.y & 0xffff0000u);
    } else {
        const float4 f = *(const float4*)((const float*)p + i);
        o[0] = f.x; o[1] = f.y; o[2] = f.z; o[3] = f.w;
    }
}

// grid (rows); dynamic LDS: E floats (u) + 16.  VEC: E is a multiple of 4.
template <int S, bool VEC>
__global__ void __launch_bounds__(256)
stream_mix_norm_kernel(float* __restrict__ x, const void* __restrict__ y1, int y1_dt, float ya,
                       const void* __restrict__ y2, int y2_dt, float yb,
                       const float* __restrict__ mix, const float* __restrict__ outw,
                       const float* __restrict__ read, const void* __restrict__ w, int w_dt,
                       void* __restrict__ h, int h_dt, const int32_t* __restrict__ row_idx, int E,
                       float eps) {
    extern __shared__ float smem[];
    float* us = smem;
    float* red = smem + E;
    const size_t r = blockIdx.x;
    const size_t row = row_idx ? (size_t)row_idx[r] : r;
    float* xr = x + row * (size_t)S * E;
    float m[S][S], ow[S], rd[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
        ow[s] = y1 ? outw[s] : 0.f;
        rd[s] = read ? read[s] : 1.f;
#pragma unroll
        for (int t = 0; t < S; ++t) m[s][t] = y1 ? mix[s * S + t] : (s == t ? 1.f : 0.f);
    }
    float ss = 0.f;
    if (VEC) {
        // four neighbouring columns a thread: 16-byte loads and stores of every stream
        for (int i = threadIdx.x * 4; i < E; i += 1024) {
            float4 xs[S];
            float xn[S][4];
#pragma unroll
            for (int s = 0; s < S; ++s) xs[s] = *(const float4*)(xr + (size_t)s * E + i);
            if (y1) {
                float y[4];
                ld4(y1, y1_dt, row * E + i, y);
#pragma unroll
                for (int c = 0; c < 4; ++c) y[c] *= ya;
                if (y2) {
                    float z[4];
                    ld4(y2, y2_dt, row * E + i, z);
#pragma unroll
                    for (int c = 0; c < 4; ++c) y[c] += yb * z[c];
                }
#pragma unroll
                for (int t = 0; t < S; ++t) {
                    float a[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < S; ++s) {
                        a[0] += m[s][t] * xs[s].x; a[1] += m[s][t] * xs[s].y;
                        a[2] += m[s][t] * xs[s].z; a[3] += m[s][t] * xs[s].w;
                    }
#pragma unroll
                    for (int c = 0; c < 4; ++c) xn[t][c] = a[c] + ow[t] * y[c];
                    if (!row_idx)
                        *(float4*)(xr + (size_t)t * E + i) = make_float4(xn[t][0], xn[t][1], xn[t][2], xn[t][3]);
                }
            } else {
#pragma unroll
                for (int t = 0; t < S; ++t) {
                    xn[t][0] = xs[t].x; xn[t][1] = xs[t].y; xn[t][2] = xs[t].z; xn[t][3] = xs[t].w;
                }
            }
            float u[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < S; ++s)
#pragma unroll
                for (int c = 0; c < 4; ++c) u[c] += rd[s] * xn[s][c];
            *(float4*)(us + i) = make_float4(u[0], u[1], u[2], u[3]);
            ss += u[0] * u[0]; ss += u[1] * u[1]; ss += u[2] * u[2]; ss += u[3] * u[3];
        }
    } else
    for (int i = threadIdx.x; i < E; i += 256) {
        float xs[S], xn[S];
#pragma unroll
        for (int s = 0; s < S; ++s) xs[s] = xr[(size_t)s * E + i];
        if (y1) {
            float y = ya * ld_f(y1, y1_dt, row * E + i);
            if (y2) y += yb * ld_f(y2, y2_dt, row * E + i);
#pragma unroll
            for (int t = 0; t < S; ++t) {
                float a = 0.f;
#pragma unroll
                for (int s = 0; s < S; ++s) a += m[s][t] * xs[s];
                xn[t] = a + ow[t] * y;
            }
            if (!row_idx) {
#pragma unroll
                for (int t = 0; t < S; ++t) xr[(size_t)t * E + i] = xn[t];
            }
        } else {
#pragma unroll
            for (int t = 0; t < S; ++t) xn[t] = xs[t];
        }
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < S; ++s) u += rd[s] * xn[s];
        us[i] = u;
        ss += u * u;
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)E + eps);
    for (int i = threadIdx.x; i < E; i += 256)
        st_f(h, h_dt, r * E + i, us[i] * inv * ld_f(w, w_dt, i));
}

extern "C" int illm_stream_mix_norm(float* x, int S, const void* y1, int y1_dt, float ya,
                                    const void* y2, int y2_dt, float yb, const float* mix,
                                    const float* outw, const float* read, const void* w, int w_dt,
                                    void* h, int h_dt, const int32_t* row_idx, int rows, int E,
                                    float eps, void* stream) {
    if (S < 1 || S > STREAMS_MAX || rows < 0 || E <= 0 || E > 32768 || !illm_dtype_ok(w_dt) ||
        !illm_dtype_ok(h_dt) || (y1 && (!illm_dtype_ok(y1_dt) || !mix || !outw)) ||
        (y2 && (!y1 || !illm_dtype_ok(y2_dt))))
        return ILLM_ERR_ARG;
    if (rows == 0) return ILLM_OK;
    const size_t lds = ((size_t)E + 16) * sizeof(float);
    hipStream_t st = (hipStream_t)stream;
#define GO1(S_, V_)                                                                               \
    {                                                                                             \
        if (lds > 48 * 1024 &&                                                                    \
            hipFuncSetAttribute((const void*)stream_mix_norm_kernel<S_, V_>,                      \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
            return ILLM_ERR_LAUNCH;                                                               \
        hipLaunchKernelGGL((stream_mix_norm_kernel<S_, V_>), dim3(rows), dim3(256), lds, st, x, y1, y1_dt, \
                           ya, y2, y2_dt, yb, mix, outw, read, w, w_dt, h, h_dt, row_idx, E, eps); \
    }
#define GO(S_)                                                                                    \
    case S_:                                                                                      \
        if (E % 4 == 0) GO1(S_, true) else GO1(S_, false)                                         \
        break;
    switch (S) {
        GO(1) GO(2) GO(3) GO(4) GO(5) GO(6) GO(7) GO(8)
    }
#undef GO
#undef GO1
    return illm_launch_status();
}

// out[t, s, :] = table[tokens[t], :] * scale for s < S: every stream starts as the embedded row.
__global__ void embed_streams_kernel(const int32_t* __restrict__ tokens, const void* __restrict__ table,
                                     int table_dt, float* __restrict__ out, int E, int V, int S,
                                     float scale) {
    const int t = blockIdx.x;
    int id = tokens[t];
    id = id < 0 ? 0 : (id >= V ? V - 1 : id);
    const size_t src = (size_t)id * E, dst = (size_t)t * S * E;
    for (int i = threadIdx.x; i < E; i += blockDim.x) {
        const float v = ld_f(table, table_dt, src + i) * scale;
        for (int s = 0; s < S; ++s) out[dst + (size_t)s * E + i] = v;
    }
}

extern "C" int illm_embed_streams(const int32_t* tokens, const void* table, int table_dt, float* out,
                                  int T, int E, int V, int S, float scale, void* stream) {
    if (T < 0 || E <= 0 || V <= 0 || S < 1 || !illm_dtype_ok(table_dt)) return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(embed_streams_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, tokens, table,
                       table_dt, out, E, V, S, scale);
    return illm_launch_status();
}
