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
// z[t, e] = sum_k x[t, k] w[e, k] with a float32 matrix of few rows (a router): float32 products
// and sums.  A wave takes 4 outputs and 8 tokens at a time (a chunk of a row of w serves 8 tokens,
// a chunk of a token's row 4 outputs), lanes over K; every sum runs over K in the same order
// whatever its companions.  grid (ceil(T / 8), ceil(NE / 16)).
__device__ __forceinline__ float4 ld4_f32(const void* p, int dt, size_t i) {
    if (dt == ILLM_BF16) {
        const uint2 u = *(const uint2*)((const bf16_t*)p + i);
        return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                           __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
    }
    return *(const float4*)((const float*)p + i);
}

template <int EW>
__global__ void __launch_bounds__(256)
few_outputs_f32_kernel(const void* __restrict__ x, int x_dt, const float* __restrict__ w,
                       float* __restrict__ z, int T, int NE, int K) {
    const int t0 = blockIdx.x * 8;
    const int e0 = (blockIdx.y * 4 + wave_index()) * EW, lane = threadIdx.x & 63;
    if (e0 >= NE) return;
    const int nt = T - t0 < 8 ? T - t0 : 8;
    const float* wr[EW];
    size_t xr[8];
#pragma unroll
    for (int j = 0; j < EW; ++j) wr[j] = w + (size_t)(e0 + j < NE ? e0 + j : NE - 1) * K;
#pragma unroll
    for (int i = 0; i < 8; ++i) xr[i] = (size_t)(i < nt ? t0 + i : t0) * K;
    float acc[8][EW];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < EW; ++j) acc[i][j] = 0.f;
    if (K % 4 == 0) {
        // four neighbouring k a lane: one 16-byte load of w and one of 8 or 16 bytes of x
#pragma unroll 2
        for (int k = lane * 4; k < K; k += 256) {
            float4 wv[EW], xv[8];
#pragma unroll
            for (int j = 0; j < EW; ++j) wv[j] = *(const float4*)(wr[j] + k);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                xv[i] = i < nt ? ld4_f32(x, x_dt, xr[i] + k) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < EW; ++j) {
                    acc[i][j] += xv[i].x * wv[j].x; acc[i][j] += xv[i].y * wv[j].y;
                    acc[i][j] += xv[i].z * wv[j].z; acc[i][j] += xv[i].w * wv[j].w;
                }
        }
    } else {
#pragma unroll 4
        for (int k = lane; k < K; k += 64) {
            float wv[EW], xv[8];
#pragma unroll
            for (int j = 0; j < EW; ++j) wv[j] = wr[j][k];
#pragma unroll
            for (int i = 0; i < 8; ++i) xv[i] = i < nt ? ld_f(x, x_dt, xr[i] + k) : 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < EW; ++j) acc[i][j] += xv[i] * wv[j];
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if (i >= nt) continue;
#pragma unroll
        for (int j = 0; j < EW; ++j) {
            const float v = wave_sum(acc[i][j]);
            if (lane == 0 && e0 + j < NE) z[(size_t)(t0 + i) * NE + e0 + j] = v;
        }
    }
}

extern "C" int illm_few_outputs_f32(const void* x, int x_dt, const float* w, float* z, int T, int NE,
                                    int K, void* stream) {
    if (T < 0 || NE <= 0 || NE > 65535 * 4 || K <= 0 || !illm_dtype_ok(x_dt)) return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    if (T <= 16)        // few tokens: an output a wave, so that more waves share the reading
        hipLaunchKernelGGL(few_outputs_f32_kernel<1>, dim3((T + 7) / 8, (NE + 3) / 4), dim3(256), 0,
                           (hipStream_t)stream, x, x_dt, w, z, T, NE, K);
    else
        hipLaunchKernelGGL(few_outputs_f32_kernel<4>, dim3((T + 7) / 8, (NE + 15) / 16), dim3(256), 0,
                           (hipStream_t)stream, x, x_dt, w, z, T, NE, K);
    return illm_launch_status();
}

// Scores of a router's outputs: their softmax, or every output's sigmoid.
#define MOE_SCORE_SOFTMAX 0
#define MOE_SCORE_SIGMOID 1
// What an expert does with its gate and up products: silu(gate) * up, or with both clamped
// (gate from above, up on both sides, at `limit`) gate * sigmoid(1.702 gate) * (up + 1).
#define MOE_ACT_SILU 0
#define MOE_ACT_CLAMPED 1
__device__ __forceinline__ float moe_act(float gate, float up, int act_kind, float limit) {
    if (act_kind == MOE_ACT_SILU) return (gate / (1.0f + expf(-gate))) * up;
    gate = fminf(gate, limit);
    up = fminf(fmaxf(up, -limit), limit);
    return (gate / (1.0f + expf(-1.702f * gate))) * (up + 1.0f);
}

// One wave per token: s = the scores of all NE outputs (float32), choice score = s + correction,
// the `top` largest choice scores (lowest index on ties) in falling order; weights are s.
#define MOE_EPL 8                                   // outputs a lane holds: up to 512 experts
__device__ __forceinline__ void
moe_route_row(const float* zr, const void* __restrict__ corr, int corr_dt, int NE, int top,
              int32_t* __restrict__ idx_row, float* __restrict__ wt_row, int32_t* idx_copy,
              int score_kind) {
    const int lane = threadIdx.x & 63;
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
        // softmax over all outputs, or every output's own sigmoid
        s[i] = score_kind == MOE_SCORE_SIGMOID ? (e < NE ? 1.0f / (1.0f + expf(-zr[e])) : 0.f) : s[i] / sum;
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
        if (lane == 0) {
            idx_row[k] = be;
            wt_row[k] = w;
            if (idx_copy) idx_copy[k] = be;
        }
    }
}

__global__ void __launch_bounds__(64)
moe_route_kernel(const float* __restrict__ z, const void* __restrict__ corr, int corr_dt, int NE,
                 int top, int32_t* __restrict__ idx, float* __restrict__ wt, int score_kind) {
    const size_t t = blockIdx.x;
    moe_route_row(z + t * NE, corr, corr_dt, NE, top, idx + t * top, wt + t * top, nullptr, score_kind);
}

extern "C" int illm_moe_route(const float* z, const void* corr, int corr_dt, int T, int NE, int top,
                              int32_t* idx, float* wt, int score_kind, void* stream) {
    if ((score_kind != MOE_SCORE_SOFTMAX && score_kind != MOE_SCORE_SIGMOID) || T < 0 || NE <= 0 || NE > 64 * MOE_EPL || top <= 0 || top > NE || (corr && !illm_dtype_ok(corr_dt)))
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(moe_route_kernel, dim3(T), dim3(64), 0, (hipStream_t)stream, z, corr, corr_dt,
                       NE, top, idx, wt, score_kind);
    return illm_launch_status();
}

// ---------------------------------------------------------------- grouping
// One block.  order[NP]: the pairs whose expert is a real one (< NEr), grouped by expert.
// tiles[3 i ..]: (expert, first place in `order`, rows) of tile i; tiles[3 max_tiles] = number of
// tiles.  Counters live in LDS and are cleared here, so nothing needs clearing between calls.
#define MOE_MAX_EXPERTS 512
__device__ __forceinline__ void
moe_group_pairs(const int32_t* idx, int NP, int NEr, int32_t* __restrict__ order,
                int32_t* __restrict__ tiles, int max_tiles, int tile_rows) {
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
            tl += (cnt[e] + tile_rows - 1) / tile_rows;
        }
        tile0[NEr] = tl;
        tiles[3 * (size_t)max_tiles] = tl < max_tiles ? tl : max_tiles;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < NEr; e += blockDim.x) {
        const int n = cnt[e];
        for (int s = 0, i = tile0[e]; s < n && i < max_tiles; s += tile_rows, ++i) {
            tiles[3 * (size_t)i] = e;
            tiles[3 * (size_t)i + 1] = offs[e] + s;
            tiles[3 * (size_t)i + 2] = n - s < tile_rows ? n - s : tile_rows;
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

__global__ void __launch_bounds__(1024)
moe_group_kernel(const int32_t* __restrict__ idx, int NP, int NEr, int32_t* __restrict__ order,
                 int32_t* __restrict__ tiles, int max_tiles, int tile_rows) {
    moe_group_pairs(idx, NP, NEr, order, tiles, max_tiles, tile_rows);
}

extern "C" int illm_moe_tile_rows(void) { return MOE_TILE; }

extern "C" int illm_moe_group(const int32_t* idx, int NP, int NEr, int32_t* order, int32_t* tiles,
                              int max_tiles, int tile_rows, void* stream) {
    if (NP < 0 || NEr < 0 || NEr > MOE_MAX_EXPERTS || max_tiles < 0 || tile_rows <= 0)
        return ILLM_ERR_ARG;
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, idx, NP, NEr,
                       order, tiles, max_tiles, tile_rows);
    return illm_launch_status();
}

// ---------------------------------------------------------------- the experts' products
// V elements of a row as float32: bfloat16 V = 8 (one 16-byte load), float32 V = 4, or V = 1.
template <int DT, int V>
__device__ __forceinline__ void ldv(const void* p, size_t i, float* o) {
    if (V == 8) {
        const uint4 u = *(const uint4*)((const bf16_t*)p + i);
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            o[2 * j] = __uint_as_float(w[j] << 16);
            o[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        }
    } else if (V == 4) {
        const float4 f = *(const float4*)((const float*)p + i);
        o[0] = f.x; o[1] = f.y; o[2] = f.z; o[3] = f.w;
    } else {
        o[0] = DT == ILLM_BF16 ? bf16_to_f32(((const bf16_t*)p)[i]) : ((const float*)p)[i];
    }
}

// grid (tiles, column groups).  X rows: pair p reads row p / x_div of X (x_div = top for the
// tokens' rows, 1 for rows that are per pair already).  GATED: W holds [gate (N) | up (N)] rows per
// expert and Y = silu(X Wg^T) * (X Wu^T); else Y = X W^T.  Y rows are per pair.  A wave takes two
// columns at a time, so that their rows of W are in flight together.
template <int DT, int V, bool GATED>
__global__ void __launch_bounds__(256)
moe_rows_kernel(const void* __restrict__ X, int x_div, const void* __restrict__ W,
                const int32_t* __restrict__ order, const int32_t* __restrict__ tiles, int max_tiles,
                void* __restrict__ Y, int N, int K, int cols_per_block, int act_kind, float limit,
                const float* __restrict__ row_w) {
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
    for (int col = blockIdx.y * cols_per_block + 2 * w; col < c_end; col += 8) {
        const bool two = col + 1 < c_end;
        const size_t wa0 = ((size_t)e * wrows + col) * K, wa1 = two ? wa0 + K : wa0;
        const size_t up = (size_t)N * K;
        float a[2][MOE_TILE], g[2][MOE_TILE];
#pragma unroll
        for (int r = 0; r < MOE_TILE; ++r) { a[0][r] = a[1][r] = 0.f; g[0][r] = g[1][r] = 0.f; }
#pragma unroll 2
        for (int k = lane * V; k < K; k += 64 * V) {
            float w0[V], w1[V], u0[V], u1[V];
            ldv<DT, V>(W, wa0 + k, w0);
            ldv<DT, V>(W, wa1 + k, w1);
            if (GATED) { ldv<DT, V>(W, wa0 + up + k, u0); ldv<DT, V>(W, wa1 + up + k, u1); }
#pragma unroll
            for (int r = 0; r < MOE_TILE; ++r) {
                if (r < n) {
                    float x[V];
                    ldv<DT, V>(X, (size_t)(pair[r] / x_div) * K + k, x);
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        a[0][r] += x[j] * w0[j];
                        a[1][r] += x[j] * w1[j];
                        if (GATED) { g[0][r] += x[j] * u0[j]; g[1][r] += x[j] * u1[j]; }
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < MOE_TILE; ++r) {
            if (r < n) {
                a[0][r] = wave_sum(a[0][r]); a[1][r] = wave_sum(a[1][r]);
                if (GATED) { g[0][r] = wave_sum(g[0][r]); g[1][r] = wave_sum(g[1][r]); }
            }
        }
        if (lane < 2 && (lane == 0 || two)) {
#pragma unroll
            for (int r = 0; r < MOE_TILE; ++r) {
                if (r < n) {
                    float v = lane ? a[1][r] : a[0][r];
                    if (GATED) {
                        // the products take the activations' type before the activation, as a
                        // product of its own would leave them
                        float gate = v, upv = lane ? g[1][r] : g[0][r];
                        if (row_w) { gate *= row_w[pair[r]]; upv *= row_w[pair[r]]; }   // W (w x) = w (W x)
                        if (DT == ILLM_BF16) { gate = bf16_to_f32(f32_to_bf16(gate)); upv = bf16_to_f32(f32_to_bf16(upv)); }
                        v = moe_act(gate, upv, act_kind, limit);
                    }
                    if (DT == ILLM_BF16) ((bf16_t*)Y)[(size_t)pair[r] * N + col + lane] = f32_to_bf16(v);
                    else ((float*)Y)[(size_t)pair[r] * N + col + lane] = v;
                }
            }
        }
    }
}

extern "C" int illm_moe_rows(const void* X, int x_div, const void* W, int dt, int gated,
                             const int32_t* order, const int32_t* tiles, int max_tiles, void* Y,
                             int N, int K, int act_kind, float limit, const float* row_w,
                             void* stream) {
    if ((act_kind != MOE_ACT_SILU && act_kind != MOE_ACT_CLAMPED) || x_div <= 0 || N <= 0 || K <= 0 || max_tiles < 0 || max_tiles > 2147483647 / 3 ||
        !illm_dtype_ok(dt))
        return ILLM_ERR_ARG;
    if (max_tiles == 0) return ILLM_OK;
    const int cols = 32;
    const dim3 grid(max_tiles, (N + cols - 1) / cols);
    if (grid.y > 65535) return ILLM_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
#define GO(DT_, V_, G_)                                                                          \
    hipLaunchKernelGGL((moe_rows_kernel<DT_, V_, G_>), grid, dim3(256), 0, st, X, x_div, W, order, \
                       tiles, max_tiles, Y, N, K, cols, act_kind, limit, row_w)
    if (dt == ILLM_BF16) {
        if (K % 8 == 0) { if (gated) GO(ILLM_BF16, 8, true); else GO(ILLM_BF16, 8, false); }
        else { if (gated) GO(ILLM_BF16, 1, true); else GO(ILLM_BF16, 1, false); }
    } else {
        if (K % 4 == 0) { if (gated) GO(ILLM_F32, 4, true); else GO(ILLM_F32, 4, false); }
        else { if (gated) GO(ILLM_F32, 1, true); else GO(ILLM_F32, 1, false); }
    }
#undef GO
    return illm_launch_status();
}

// The same products for tiles of up to 16 MT pairs on the matrix cores (bfloat16, K % 32 == 0):
// MFMA 16x16x32 with 16 rows of W as the A operand and 16 of the tile's X rows as the B operand,
// both read in operand order straight from memory (lane (r, q) = (lane % 16, lane / 16) holds 8
// consecutive k of row r at k0 + 8 q; the tile's X rows stay in the caches, W is read once a
// tile).  A wave takes NT groups of 16 output columns at a time and all MT row groups, so an X
// operand serves NT (gated: 2 NT) products; the sum over K runs in one fixed order, so a row's
// result does not depend on its tile.  grid (tiles, column groups of 64 NT).
typedef __bf16 moe_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float moe_f32x4_t __attribute__((ext_vector_type(4)));

template <int MT, int NT, bool GATED, bool AHEAD, int KU>
__global__ void __launch_bounds__(256)
moe_rows_mfma_kernel(const bf16_t* __restrict__ X, int x_div, const bf16_t* __restrict__ W,
                     const int32_t* __restrict__ order, const int32_t* __restrict__ tiles,
                     int max_tiles, bf16_t* __restrict__ Y, int N, int K, int act_kind, float limit,
                     const float* __restrict__ row_w) {
    const int tile = blockIdx.x;
    if (tile >= tiles[3 * (size_t)max_tiles]) return;
    const int e = tiles[3 * (size_t)tile], first = tiles[3 * (size_t)tile + 1];
    const int n = tiles[3 * (size_t)tile + 2];
    const int w = wave_index(), lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    int pair[MT];
    const bf16_t* xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int i = mt * 16 + r;
        pair[mt] = order[first + (i < n ? i : n - 1)];          // rows beyond the tile: read, not written
        xp[mt] = X + (size_t)(pair[mt] / x_div) * K + q * 8;
    }
    const size_t wrows = GATED ? 2 * (size_t)N : (size_t)N;
    const int n0 = (blockIdx.y * 4 + w) * 16 * NT;
    if (n0 >= N) return;
    const bf16_t* wa[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int wr = n0 + nt * 16 + r < N ? n0 + nt * 16 + r : N - 1;
        wa[nt] = W + ((size_t)e * wrows + wr) * K + q * 8;
    }
    const size_t up = (size_t)N * K;
    moe_f32x4_t a[NT][MT], g[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            a[nt][mt] = (moe_f32x4_t){0.f, 0.f, 0.f, 0.f};
            g[nt][mt] = a[nt][mt];
        }
    if (KU > 1) {
        // few accumulators (single tokens): KU steps of 32 k at a time, all their loads first
        for (int k = 0; k < K; k += 32 * KU) {
            moe_bf16x8_t w0[KU][NT], w1[KU][NT], x[KU][MT];
#pragma unroll
            for (int u = 0; u < KU; ++u) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    w0[u][nt] = *(const moe_bf16x8_t*)(wa[nt] + k + 32 * u);
                    if (GATED) w1[u][nt] = *(const moe_bf16x8_t*)(wa[nt] + up + k + 32 * u);
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) x[u][mt] = *(const moe_bf16x8_t*)(xp[mt] + k + 32 * u);
            }
#pragma unroll
            for (int u = 0; u < KU; ++u)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        a[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0[u][nt], x[u][mt], a[nt][mt], 0, 0, 0);
                        if (GATED)
                            g[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[u][nt], x[u][mt], g[nt][mt], 0, 0, 0);
                    }
        }
    } else {
        // the operands of the next 32 k are asked for before this step's products are issued
        moe_bf16x8_t w0[NT], w1[NT], x[MT];
    #pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            w0[nt] = *(const moe_bf16x8_t*)(wa[nt]);
            if (GATED) w1[nt] = *(const moe_bf16x8_t*)(wa[nt] + up);
        }
    #pragma unroll
        for (int mt = 0; mt < MT; ++mt) x[mt] = *(const moe_bf16x8_t*)(xp[mt]);
        for (int k = 0; k < K; k += 32) {
            moe_bf16x8_t w0n[NT], w1n[NT], xn[MT];
            const int kn = k + 32 < K ? k + 32 : k;            // the last step loads its own again
            if (!AHEAD && k > 0) {
                // (many accumulators: no second set of operands; other waves hide the loads)
    #pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    w0[nt] = *(const moe_bf16x8_t*)(wa[nt] + k);
                    if (GATED) w1[nt] = *(const moe_bf16x8_t*)(wa[nt] + up + k);
                }
    #pragma unroll
                for (int mt = 0; mt < MT; ++mt) x[mt] = *(const moe_bf16x8_t*)(xp[mt] + k);
            }
            if (AHEAD) {
    #pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    w0n[nt] = *(const moe_bf16x8_t*)(wa[nt] + kn);
                    if (GATED) w1n[nt] = *(const moe_bf16x8_t*)(wa[nt] + up + kn);
                }
    #pragma unroll
                for (int mt = 0; mt < MT; ++mt) xn[mt] = *(const moe_bf16x8_t*)(xp[mt] + kn);
            }
    #pragma unroll
            for (int nt = 0; nt < NT; ++nt)
    #pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    a[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0[nt], x[mt], a[nt][mt], 0, 0, 0);
                    if (GATED)
                        g[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[nt], x[mt], g[nt][mt], 0, 0, 0);
                }
            if (AHEAD) {
    #pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    w0[nt] = w0n[nt];
                    if (GATED) w1[nt] = w1n[nt];
                }
    #pragma unroll
                for (int mt = 0; mt < MT; ++mt) x[mt] = xn[mt];
            }
        }
    }
    // a[nt][mt][i] belongs to the pair of row mt * 16 + r and column n0 + 16 nt + 4 q + i
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (mt * 16 + r >= n) continue;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int col = n0 + 16 * nt + 4 * q + i;
                if (col >= N) continue;
                float v = a[nt][mt][i];
                if (GATED) {
                    const float rw = row_w ? row_w[pair[mt]] : 1.0f;          // W (w x) = w (W x)
                    const float gate = bf16_to_f32(f32_to_bf16(a[nt][mt][i] * rw));
                    const float upv = bf16_to_f32(f32_to_bf16(g[nt][mt][i] * rw));
                    v = moe_act(gate, upv, act_kind, limit);
                }
                Y[(size_t)pair[mt] * N + col] = f32_to_bf16(v);
            }
    }
}

// Tiles of 64 pairs (prompts), K % 64 == 0: as above with the tile's X rows shared by the block's
// four waves through LDS, 64 k at a time in two buffers (a thread brings 32 bytes of one row; the
// 16-byte pieces of a row are placed at piece ^ (row % 8), so that the 16 rows a product's operand
// reads lie in different banks); one barrier a slab.  W stays a stream of each wave's own rows,
// asked for one slab ahead.
template <int NT, bool GATED>
__global__ void __launch_bounds__(256)
moe_rows_mfma_lds_kernel(const bf16_t* __restrict__ X, int x_div, const bf16_t* __restrict__ W,
                         const int32_t* __restrict__ order, const int32_t* __restrict__ tiles,
                         int max_tiles, bf16_t* __restrict__ Y, int N, int K, int act_kind,
                         float limit, const float* __restrict__ row_w) {
    constexpr int MT = 4;
    __shared__ uint4 xs[2][64 * 8];
    const int tile = blockIdx.x;
    if (tile >= tiles[3 * (size_t)max_tiles]) return;          // the whole block leaves together
    const int e = tiles[3 * (size_t)tile], first = tiles[3 * (size_t)tile + 1];
    const int n = tiles[3 * (size_t)tile + 2];
    const int w = wave_index(), lane = threadIdx.x & 63;
    const int r = lane & 15, q = lane >> 4;
    const int lr = threadIdx.x >> 2, lc = (threadIdx.x & 3) * 2;       // the row and pieces this thread brings
    const bf16_t* lx = X + (size_t)(order[first + (lr < n ? lr : n - 1)] / x_div) * K + lc * 8;
    const int s0 = lr * 8 + (lc ^ (lr & 7)), s1 = lr * 8 + ((lc + 1) ^ (lr & 7));
    int pair[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int i = mt * 16 + r;
        pair[mt] = order[first + (i < n ? i : n - 1)];
    }
    const size_t wrows = GATED ? 2 * (size_t)N : (size_t)N;
    const int n0 = (blockIdx.y * 4 + w) * 16 * NT;             // (a wave beyond N works on row N - 1 and writes nothing)
    const bf16_t* wa[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int wr = n0 + nt * 16 + r < N ? n0 + nt * 16 + r : N - 1;
        wa[nt] = W + ((size_t)e * wrows + wr) * K + q * 8;
    }
    const size_t up = (size_t)N * K;
    moe_f32x4_t a[NT][MT], g[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            a[nt][mt] = (moe_f32x4_t){0.f, 0.f, 0.f, 0.f};
            g[nt][mt] = a[nt][mt];
        }
    moe_bf16x8_t w0[2][NT], w1[2][NT];
    uint4 xa = *(const uint4*)lx, xb = *(const uint4*)(lx + 8);
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            w0[u][nt] = *(const moe_bf16x8_t*)(wa[nt] + 32 * u);
            if (GATED) w1[u][nt] = *(const moe_bf16x8_t*)(wa[nt] + up + 32 * u);
        }
    xs[0][s0] = xa;
    xs[0][s1] = xb;
    __syncthreads();
    for (int k = 0; k < K; k += 64) {
        const int buf = (k >> 6) & 1;
        const int kn = k + 64 < K ? k + 64 : k;                  // the last slab asks for itself again
        moe_bf16x8_t w0n[2][NT], w1n[2][NT];
        xa = *(const uint4*)(lx + kn);
        xb = *(const uint4*)(lx + kn + 8);
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                w0n[u][nt] = *(const moe_bf16x8_t*)(wa[nt] + kn + 32 * u);
                if (GATED) w1n[u][nt] = *(const moe_bf16x8_t*)(wa[nt] + up + kn + 32 * u);
            }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            moe_bf16x8_t x[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const uint4 v = xs[buf][(mt * 16 + r) * 8 + ((u * 4 + q) ^ (r & 7))];
                x[mt] = *(const moe_bf16x8_t*)&v;
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    a[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0[u][nt], x[mt], a[nt][mt], 0, 0, 0);
                    if (GATED)
                        g[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[u][nt], x[mt], g[nt][mt], 0, 0, 0);
                }
        }
        xs[buf ^ 1][s0] = xa;
        xs[buf ^ 1][s1] = xb;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                w0[u][nt] = w0n[u][nt];
                if (GATED) w1[u][nt] = w1n[u][nt];
            }
        __syncthreads();
    }
    if (n0 >= N) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (mt * 16 + r >= n) continue;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int col = n0 + 16 * nt + 4 * q + i;
                if (col >= N) continue;
                float v = a[nt][mt][i];
                if (GATED) {
                    const float rw = row_w ? row_w[pair[mt]] : 1.0f;          // W (w x) = w (W x)
                    const float gate = bf16_to_f32(f32_to_bf16(a[nt][mt][i] * rw));
                    const float upv = bf16_to_f32(f32_to_bf16(g[nt][mt][i] * rw));
                    v = moe_act(gate, upv, act_kind, limit);
                }
                Y[(size_t)pair[mt] * N + col] = f32_to_bf16(v);
            }
    }
}

extern "C" int illm_moe_rows_mfma(const void* X, int x_div, const void* W, int gated, int tile_rows,
                                  const int32_t* order, const int32_t* tiles, int max_tiles,
                                  void* Y, int N, int K, int act_kind, float limit,
                                  const float* row_w, void* stream) {
    if ((act_kind != MOE_ACT_SILU && act_kind != MOE_ACT_CLAMPED) || x_div <= 0 || N <= 0 || K <= 0 || K % 32 || max_tiles < 0 || max_tiles > 2147483647 / 3 ||
        (tile_rows != 16 && tile_rows != 32 && tile_rows != 64))
        return ILLM_ERR_ARG;
    if (max_tiles == 0) return ILLM_OK;
    hipStream_t st = (hipStream_t)stream;
    if (tile_rows == 64 && K % 64 == 0) {
        const int nt = gated ? 2 : 4;
        const dim3 grid(max_tiles, (N + 64 * nt - 1) / (64 * nt));
        if (grid.y > 65535) return ILLM_ERR_ARG;
        if (gated)
            hipLaunchKernelGGL((moe_rows_mfma_lds_kernel<2, true>), grid, dim3(256), 0, st, (const bf16_t*)X,
                               x_div, (const bf16_t*)W, order, tiles, max_tiles, (bf16_t*)Y, N, K, act_kind, limit, row_w);
        else
            hipLaunchKernelGGL((moe_rows_mfma_lds_kernel<4, false>), grid, dim3(256), 0, st, (const bf16_t*)X,
                               x_div, (const bf16_t*)W, order, tiles, max_tiles, (bf16_t*)Y, N, K, act_kind, limit, row_w);
        return illm_launch_status();
    }
#define GO(MT_, NT_, G_, KU_)                                                                      \
    do {                                                                                           \
        const dim3 grid(max_tiles, (N + 64 * NT_ - 1) / (64 * NT_));                               \
        if (grid.y > 65535) return ILLM_ERR_ARG;                                                   \
        hipLaunchKernelGGL((moe_rows_mfma_kernel<MT_, NT_, G_, (MT_ * NT_ <= 16), KU_>), grid, dim3(256), 0, st, \
                           (const bf16_t*)X, x_div, (const bf16_t*)W, order, tiles, max_tiles,     \
                           (bf16_t*)Y, N, K, act_kind, limit, row_w);                              \
    } while (0)
    if (tile_rows == 16 && (long)max_tiles * ((N + 255) / 256) < 512) {
        // few tiles (single tokens): 16 columns a wave, so that more waves share the reading
        if (K % 256 == 0) { if (gated) GO(1, 1, true, 8); else GO(1, 1, false, 8); }
        else if (K % 128 == 0) { if (gated) GO(1, 1, true, 4); else GO(1, 1, false, 4); }
        else if (K % 64 == 0) { if (gated) GO(1, 1, true, 2); else GO(1, 1, false, 2); }
        else { if (gated) GO(1, 1, true, 1); else GO(1, 1, false, 1); }
    } else if (tile_rows == 16) {
        if (K % 64 == 0) { if (gated) GO(1, 4, true, 2); else GO(1, 4, false, 2); }
        else { if (gated) GO(1, 4, true, 1); else GO(1, 4, false, 1); }
    }
    else if (tile_rows == 32) { if (gated) GO(2, 4, true, 1); else GO(2, 4, false, 1); }
    else { if (gated) GO(4, 2, true, 1); else GO(4, 4, false, 1); }    // wider column blocks measured slower
#undef GO
    return illm_launch_status();
}

// ---------------------------------------------------------------- weighted sum
// grid (tokens, chunks of 256 columns): out[t] = sum_k wt[t, k] * (idx[t, k] < NEr ? Y[t top + k] : h[t])
//                                         (+ sigmoid(h[t] . sg) * shared[t]), float32.
#define MOE_COMBINE_TOP 16                          // choices held in registers (more: read again)
__global__ void __launch_bounds__(256)
moe_combine_kernel(const void* __restrict__ h, int dt, const int32_t* __restrict__ idx,
                   const float* __restrict__ wt, const void* __restrict__ Y,
                   const void* __restrict__ shared, const void* __restrict__ sg, int sg_dt,
                   float* __restrict__ out, int E, int top, int NEr) {
    __shared__ float red[16];
    const size_t t = blockIdx.x;
    int ce[MOE_COMBINE_TOP];
    float cw[MOE_COMBINE_TOP];
#pragma unroll
    for (int k = 0; k < MOE_COMBINE_TOP; ++k) {
        ce[k] = k < top ? idx[t * top + k] : 0;
        cw[k] = k < top ? (wt ? wt[t * top + k] : 1.f) : 0.f;
    }
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
    const int i_end = min(E, (int)(blockIdx.y + 1) * 256);
    for (int i = blockIdx.y * 256 + threadIdx.x; i < i_end; i += 256) {
        const float hv = ld_f(h, dt, t * E + i);
        float acc = 0.f;
        if (top <= MOE_COMBINE_TOP) {
            float v[MOE_COMBINE_TOP];
#pragma unroll
            for (int k = 0; k < MOE_COMBINE_TOP; ++k)
                v[k] = k < top && ce[k] < NEr ? ld_f(Y, dt, (t * top + k) * E + i) : hv;
#pragma unroll
            for (int k = 0; k < MOE_COMBINE_TOP; ++k)
                if (k < top) acc += cw[k] * v[k];
        } else {
            for (int k = 0; k < top; ++k) {
                const int e = idx[t * top + k];
                acc += (wt ? wt[t * top + k] : 1.f) * (e < NEr ? ld_f(Y, dt, (t * top + k) * E + i) : hv);
            }
        }
        if (shared) acc += gate * ld_f(shared, dt, t * E + i);
        out[t * E + i] = acc;
    }
}

extern "C" int illm_moe_combine(const void* h, int dt, const int32_t* idx, const float* wt,
                                const void* Y, const void* shared, const void* sg, int sg_dt,
                                float* out, int T, int E, int top, int NEr, void* stream) {
    if (T < 0 || E <= 0 || top <= 0 || !illm_dtype_ok(dt) || (sg && !illm_dtype_ok(sg_dt)) ||
        (E + 255) / 256 > 65535)
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(moe_combine_kernel, dim3(T, (E + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                       h, dt, idx, wt, Y, shared, sg, sg_dt, out, E, top, NEr);
    return illm_launch_status();
}
