// Routed feed-forward (mixture of experts): the router's choice, the grouping of (token, choice)
// pairs by expert, the experts' products over their own rows, and the weighted sum.
//
// A pair p = t * top + k is token t's k-th choice.  Pairs are grouped by expert into tiles of at
// most MOE_TILE rows; a block of the product kernels takes one tile and some output columns, a wave
// one column at a time with the lanes cutting K among them, so a matrix is read once per tile and
// a row's sum depends on nothing but the row (its order over K is fixed by the lane pattern).  The
// order of the pairs inside an expert's group is whatever the grouping's counters gave: it moves
// rows between tiles and changes no value.
#include "api.h"
#include "common.h"

#define MOE_TILE 8

// ---------------------------------------------------------------- router
// One wave per token: s = softmax(z) over all NE outputs (float32), choice score = s + correction,
// the `top` largest choice scores (lowest index on ties) in falling order; weights are s.
#define MOE_EPL 8                                   // outputs a lane holds: up to 512 experts
__global__ void __launch_bounds__(64)
moe_route_kernel(const float* __restrict__ z, const void* __restrict__ corr, int corr_dt, int NE,
                 int top, int32_t* __restrict__ idx, float* __restrict__ wt) {
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* zr = z + (size_t)t * NE;
    float s[MOE_EPL], c[MOE_EPL];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < MOE_EPL; ++i) {
        const int e = lane + 64 * i;
        s[i] = e < NE ? zr[e] : -INFINITY;
        mx = fmaxf(mx, s[i]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < MOE_EPL; ++i) {
        s[i] = lane + 64 * i < NE ? expf(s[i] - mx) : 0.f;
        sum += s[i];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int i = 0; i < MOE_EPL; ++i) {
        const int e = lane + 64 * i;
        s[i] = s[i] / sum;
        c[i] = e < NE ? s[i] + (corr ? ld_f(corr, corr_dt, e) : 0.f) : -INFINITY;
    }
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int be = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < MOE_EPL; ++i) {
            const int e = lane + 64 * i;
            if (e < NE && (c[i] > best || (c[i] == best && e < be))) { best = c[i]; be = e; }
        }
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oe = __shfl_xor(be, o, 64);
            if (ob > best || (ob == best && oe < be)) { best = ob; be = oe; }
        }
        float w = 0.f;
#pragma unroll
        for (int i = 0; i < MOE_EPL; ++i)
            if (lane + 64 * i == be) { w = s[i]; c[i] = -INFINITY; }
        w = wave_sum(w);                               // only the owner's lane holds a value
        if (lane == 0) { idx[(size_t)t * top + k] = be; wt[(size_t)t * top + k] = w; }
    }
}

extern "C" int illm_moe_route(const float* z, const void* corr, int corr_dt, int T, int NE, int top,
                              int32_t* idx, float* wt, void* stream) {
    if (T < 0 || NE <= 0 || NE > 64 * MOE_EPL || top <= 0 || top > NE || (corr && !illm_dtype_ok(corr_dt)))
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(moe_route_kernel, dim3(T), dim3(64), 0, (hipStream_t)stream, z, corr, corr_dt,
                       NE, top, idx, wt);
    return illm_launch_status();
}

// ---------------------------------------------------------------- grouping
// One block.  order[NP]: the pairs whose expert is a real one (< NEr), grouped by expert.
// tiles[3 i ..]: (expert, first place in `order`, rows) of tile i; tiles[3 max_tiles] = number of
// tiles.  Counters live in LDS and are cleared here, so nothing needs clearing between calls.
#define MOE_MAX_EXPERTS 512
__global__ void __launch_bounds__(1024)
moe_group_kernel(const int32_t* __restrict__ idx, int NP, int NEr, int32_t* __restrict__ order,
                 int32_t* __restrict__ tiles, int max_tiles) {
    __shared__ int cnt[MOE_MAX_EXPERTS], offs[MOE_MAX_EXPERTS], tile0[MOE_MAX_EXPERTS + 1];
    for (int e = threadIdx.x; e < NEr; e += blockDim.x) cnt[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < NP; p += blockDim.x) {
        const int e = idx[p];
        if (e >= 0 && e < NEr) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int o = 0, tl = 0;
        for (int e = 0; e < NEr; ++e) {
            offs[e] = o; tile0[e] = tl;
            o += cnt[e];
            tl += (cnt[e] + MOE_TILE - 1) / MOE_TILE;
        }
        tile0[NEr] = tl;
        tiles[3 * (size_t)max_tiles] = tl < max_tiles ? tl : max_tiles;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < NEr; e += blockDim.x) {
        const int n = cnt[e];
        for (int s = 0, i = tile0[e]; s < n && i < max_tiles; s += MOE_TILE, ++i) {
            tiles[3 * (size_t)i] = e;
            tiles[3 * (size_t)i + 1] = offs[e] + s;
            tiles[3 * (size_t)i + 2] = n - s < MOE_TILE ? n - s : MOE_TILE;
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < NEr; e += blockDim.x) cnt[e] = offs[e];     // now the write cursors
    __syncthreads();
    for (int p = threadIdx.x; p < NP; p += blockDim.x) {
        const int e = idx[p];
        if (e >= 0 && e < NEr) order[atomicAdd(&cnt[e], 1)] = p;
    }
}

extern "C" int illm_moe_tile_rows(void) { return MOE_TILE; }

extern "C" int illm_moe_group(const int32_t* idx, int NP, int NEr, int32_t* order, int32_t* tiles,
                              int max_tiles, void* stream) {
    if (NP < 0 || NEr < 0 || NEr > MOE_MAX_EXPERTS || max_tiles < 0) return ILLM_ERR_ARG;
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, idx, NP, NEr,
                       order, tiles, max_tiles);
    return illm_launch_status();
}

// ---------------------------------------------------------------- the experts' products
// Four elements of a row as float32; V = 4: one 8- or 16-byte load, V = 1: element by element.
template <int DT>
__device__ __forceinline__ float4 ld4(const void* p, size_t i) {
    if (DT == ILLM_BF16) {
        const uint2 u = *(const uint2*)((const bf16_t*)p + i);
        return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                           __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
    }
    return *(const float4*)((const float*)p + i);
}

template <int DT>
__device__ __forceinline__ float ld1(const void* p, size_t i) {
    return DT == ILLM_BF16 ? bf16_to_f32(((const bf16_t*)p)[i]) : ((const float*)p)[i];
}

// Sum over the wave of n <= MOE_TILE values per lane.
__device__ __forceinline__ void wave_sums(float* v, int n) {
#pragma unroll
    for (int r = 0; r < MOE_TILE; ++r)
        if (r < n) v[r] = wave_sum(v[r]);
}

// grid (tiles, column groups).  X rows: pair p reads row p / x_div of X (x_div = top for the
// tokens' rows, 1 for rows that are per pair already).  GATED: W holds [gate (N) | up (N)] rows per
// expert and Y = silu(X Wg^T) * (X Wu^T); else Y = X W^T.  Y rows are per pair.
template <int DT, int V, bool GATED>
__global__ void __launch_bounds__(256)
moe_rows_kernel(const void* __restrict__ X, int x_div, const void* __restrict__ W,
                const int32_t* __restrict__ order, const int32_t* __restrict__ tiles, int max_tiles,
                void* __restrict__ Y, int N, int K, int cols_per_block) {
    const int tile = blockIdx.x;
    if (tile >= tiles[3 * (size_t)max_tiles]) return;
    const int e = tiles[3 * (size_t)tile], first = tiles[3 * (size_t)tile + 1];
    const int n = tiles[3 * (size_t)tile + 2];
    const int w = wave_index(), lane = threadIdx.x & 63;
    int pair[MOE_TILE];
#pragma unroll
    for (int r = 0; r < MOE_TILE; ++r) pair[r] = r < n ? order[first + r] : 0;
    const size_t wrows = GATED ? 2 * (size_t)N : (size_t)N;
    const int c_end = min(N, (int)(blockIdx.y + 1) * cols_per_block);
    for (int col = blockIdx.y * cols_per_block + w; col < c_end; col += 4) {
        const size_t wa = ((size_t)e * wrows + col) * K, wb = wa + (size_t)N * K;
        float a[MOE_TILE], g[MOE_TILE];
#pragma unroll
        for (int r = 0; r < MOE_TILE; ++r) { a[r] = 0.f; g[r] = 0.f; }
        for (int k = lane * V; k < K; k += 64 * V) {
            if (V == 4) {
                const float4 w0 = ld4<DT>(W, wa + k);
                float4 w1 = w0;
                if (GATED) w1 = ld4<DT>(W, wb + k);
#pragma unroll
                for (int r = 0; r < MOE_TILE; ++r) {
                    if (r < n) {
                        const float4 x = ld4<DT>(X, (size_t)(pair[r] / x_div) * K + k);
                        a[r] += x.x * w0.x; a[r] += x.y * w0.y; a[r] += x.z * w0.z; a[r] += x.w * w0.w;
                        if (GATED) {
                            g[r] += x.x * w1.x; g[r] += x.y * w1.y; g[r] += x.z * w1.z; g[r] += x.w * w1.w;
                        }
                    }
                }
            } else {
                const float w0 = ld1<DT>(W, wa + k);
                const float w1 = GATED ? ld1<DT>(W, wb + k) : 0.f;
#pragma unroll
                for (int r = 0; r < MOE_TILE; ++r) {
                    if (r < n) {
                        const float x = ld1<DT>(X, (size_t)(pair[r] / x_div) * K + k);
                        a[r] += x * w0;
                        if (GATED) g[r] += x * w1;
                    }
                }
            }
        }
        wave_sums(a, n);
        if (GATED) wave_sums(g, n);
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < MOE_TILE; ++r) {
                if (r < n) {
                    float v = a[r];
                    if (GATED) {
                        // the products take the activations' type before the activation, as a
                        // product of its own would leave them
                        float gate = a[r], up = g[r];
                        if (DT == ILLM_BF16) { gate = bf16_to_f32(f32_to_bf16(gate)); up = bf16_to_f32(f32_to_bf16(up)); }
                        v = (gate / (1.0f + expf(-gate))) * up;
                    }
                    if (DT == ILLM_BF16) ((bf16_t*)Y)[(size_t)pair[r] * N + col] = f32_to_bf16(v);
                    else ((float*)Y)[(size_t)pair[r] * N + col] = v;
                }
            }
        }
    }
}

extern "C" int illm_moe_rows(const void* X, int x_div, const void* W, int dt, int gated,
                             const int32_t* order, const int32_t* tiles, int max_tiles, void* Y,
                             int N, int K, void* stream) {
    if (x_div <= 0 || N <= 0 || K <= 0 || max_tiles < 0 || max_tiles > 2147483647 / 3 ||
        !illm_dtype_ok(dt))
        return ILLM_ERR_ARG;
    if (max_tiles == 0) return ILLM_OK;
    const int cols = 32;
    const dim3 grid(max_tiles, (N + cols - 1) / cols);
    if (grid.y > 65535) return ILLM_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = K % 4 == 0;
#define GO(DT_, V_, G_)                                                                          \
    hipLaunchKernelGGL((moe_rows_kernel<DT_, V_, G_>), grid, dim3(256), 0, st, X, x_div, W, order, \
                       tiles, max_tiles, Y, N, K, cols)
    if (dt == ILLM_BF16) {
        if (vec) { if (gated) GO(ILLM_BF16, 4, true); else GO(ILLM_BF16, 4, false); }
        else { if (gated) GO(ILLM_BF16, 1, true); else GO(ILLM_BF16, 1, false); }
    } else {
        if (vec) { if (gated) GO(ILLM_F32, 4, true); else GO(ILLM_F32, 4, false); }
        else { if (gated) GO(ILLM_F32, 1, true); else GO(ILLM_F32, 1, false); }
    }
#undef GO
    return illm_launch_status();
}

// ---------------------------------------------------------------- weighted sum
// One block per token: out[t] = sum_k wt[t, k] * (idx[t, k] < NEr ? Y[t top + k] : h[t])
//                               (+ sigmoid(h[t] . sg) * shared[t]), float32.
__global__ void __launch_bounds__(256)
moe_combine_kernel(const void* __restrict__ h, int dt, const int32_t* __restrict__ idx,
                   const float* __restrict__ wt, const void* __restrict__ Y,
                   const void* __restrict__ shared, const void* __restrict__ sg, int sg_dt,
                   float* __restrict__ out, int E, int top, int NEr) {
    __shared__ float red[16];
    const size_t t = blockIdx.x;
    float gate = 0.f;
    if (shared) {
        gate = 1.f;
        if (sg) {
            float d = 0.f;
            for (int i = threadIdx.x; i < E; i += blockDim.x) d += ld_f(h, dt, t * E + i) * ld_f(sg, sg_dt, i);
            d = block_sum(d, red);
            gate = 1.0f / (1.0f + expf(-d));
        }
    }
    for (int i = threadIdx.x; i < E; i += blockDim.x) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            const int e = idx[t * top + k];
            const float v = e < NEr ? ld_f(Y, dt, (t * top + k) * E + i) : ld_f(h, dt, t * E + i);
            acc += wt[t * top + k] * v;
        }
        if (shared) acc += gate * ld_f(shared, dt, t * E + i);
        out[t * E + i] = acc;
    }
}

extern "C" int illm_moe_combine(const void* h, int dt, const int32_t* idx, const float* wt,
                                const void* Y, const void* shared, const void* sg, int sg_dt,
                                float* out, int T, int E, int top, int NEr, void* stream) {
    if (T < 0 || E <= 0 || top <= 0 || !illm_dtype_ok(dt) || (sg && !illm_dtype_ok(sg_dt)))
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, h, dt, idx,
                       wt, Y, shared, sg, sg_dt, out, E, top, NEr);
    return illm_launch_status();
}
