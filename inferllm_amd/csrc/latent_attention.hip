// Latent attention: every token keeps one low-rank latent row c [R] (RMS-normed) and one rotated
// key part kr [dr] that all heads share; a head's key is [W_uk c | kr] and its value W_uv c.
//
// Rows of several tokens (whole prompts) build every head's keys and values from the step's own
// latent rows (`illm_latent_pack`) and go through the library's prompt attention.  Single tokens
// never build them: with qa_h = [W_uk,h^T q_h | q_h,rot] the score of key j is qa_h . [c_j | kr_j],
// and the weighted sum of values is W_uv,h (sum_j p_j c_j), so one token's attention is a walk over
// the cached latent rows that all heads of a block share (`illm_latent_attn_decode`), followed by
// the small product with W_uv and the output gate (`illm_latent_merge_up`).
//
// Scores, softmax statistics, the norm of the latent, rotation and the running sums are float32.
#include "api.h"
#include "common.h"

// ---------------------------------------------------------------- norm, rotation, cache store
// One block per row of y = [q: H (dn + dr) | down: R + dr | gate: H] (row stride ncols).
// The latent is normed (float32 statistics), the shared key part and every head's rotated query
// part are rotated in pairs (2i, 2i+1), i < rot/2, by the float32 table [max_pos][rot/2][2];
// latent and key part go to the paged cache [page][row][R + dr] and to c_out / kr_out.
__device__ __forceinline__ void
latent_store_row(const int t, void* __restrict__ y, int dt, int ncols, int H, int dn, int dr, int R,
                 int rot, const float* __restrict__ cos_sin, int max_pos,
                 const void* __restrict__ nw, int nw_dt, float eps,
                 const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
                 const int32_t* __restrict__ slot_len, void* __restrict__ cache,
                 const int32_t* __restrict__ page_table, int table_stride, int page_size,
                 int ring, void* __restrict__ c_out, void* __restrict__ kr_out,
                 void* __restrict__ cache_t, const bool rotate_q) {
    __shared__ float red[16];
    int pos = row_pos[t];
    const size_t row = (size_t)t * ncols;
    const size_t down = row + (size_t)H * (dn + dr);
    float ss = 0.f;
    for (int i = threadIdx.x; i < R; i += blockDim.x) {
        const float v = ld_f(y, dt, down + i);
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)R + eps);
    bool store = cache != nullptr;
    size_t dst = 0, dst_t = 0;
    if (store) {
        const int slot = row_slot[t];
        if (ring > 0 && slot_len) {
            // a later row of this step lands on the same ring page: this one is already outside
            const int last_page = (slot_len[slot] - 1) / page_size;
            if (pos / page_size + ring <= last_page) store = false;
        }
        if (store) {
            int lp = pos / page_size;
            if (ring > 0) lp %= ring;
            const int phys = page_table[(size_t)slot * table_stride + lp];
            dst = ((size_t)phys * page_size + (pos % page_size)) * (size_t)(R + dr);
            dst_t = (size_t)phys * R * page_size + (pos % page_size);
        }
    }
    for (int i = threadIdx.x; i < R; i += blockDim.x) {
        const float v = (ld_f(y, dt, down + i) * scale) * ld_f(nw, nw_dt, i);
        if (c_out) st_f(c_out, dt, (size_t)t * R + i, v);
        if (store) st_f(cache, dt, dst + i, v);
        if (store && cache_t) st_f(cache_t, dt, dst_t + (size_t)i * page_size, v);   // [page][dim][row]
    }
    if (pos >= max_pos) pos = max_pos - 1;
    const float* cs = cos_sin ? cos_sin + (size_t)pos * rot : nullptr;   // [rot/2][2]
    const int half = cs ? rot / 2 : 0;
    const size_t ksrc = down + R;
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        const float c = cs[2 * i], s = cs[2 * i + 1];
        const float u = ld_f(y, dt, ksrc + 2 * i), v = ld_f(y, dt, ksrc + 2 * i + 1);
        const float a = u * c - v * s, b = v * c + u * s;
        if (kr_out) { st_f(kr_out, dt, (size_t)t * dr + 2 * i, a); st_f(kr_out, dt, (size_t)t * dr + 2 * i + 1, b); }
        if (store) { st_f(cache, dt, dst + R + 2 * i, a); st_f(cache, dt, dst + R + 2 * i + 1, b); }
    }
    for (int e = 2 * half + threadIdx.x; e < dr; e += blockDim.x) {       // dims beyond the rotated ones
        const float v = ld_f(y, dt, ksrc + e);
        if (kr_out) st_f(kr_out, dt, (size_t)t * dr + e, v);
        if (store) st_f(cache, dt, dst + R + e, v);
    }
    for (int u = threadIdx.x; rotate_q && u < H * half; u += blockDim.x) {
        const int h = u / half, i = u - h * half;
        const size_t base = row + (size_t)h * (dn + dr) + dn;
        const float c = cs[2 * i], s = cs[2 * i + 1];
        const float a = ld_f(y, dt, base + 2 * i), b = ld_f(y, dt, base + 2 * i + 1);
        st_f(y, dt, base + 2 * i, a * c - b * s);
        st_f(y, dt, base + 2 * i + 1, b * c + a * s);
    }
}

__global__ void __launch_bounds__(256)
latent_rope_store_kernel(void* __restrict__ y, int dt, int ncols, int H, int dn, int dr, int R,
                         int rot, const float* __restrict__ cos_sin, int max_pos,
                         const void* __restrict__ nw, int nw_dt, float eps,
                         const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
                         const int32_t* __restrict__ slot_len, void* __restrict__ cache,
                         const int32_t* __restrict__ page_table, int table_stride, int page_size,
                         int ring, void* __restrict__ c_out, void* __restrict__ kr_out,
                         void* __restrict__ cache_t) {
    latent_store_row(blockIdx.x, y, dt, ncols, H, dn, dr, R, rot, cos_sin, max_pos, nw, nw_dt, eps,
                     row_pos, row_slot, slot_len, cache, page_table, table_stride, page_size, ring,
                     c_out, kr_out, cache_t, true);
}

extern "C" int illm_latent_rope_store(void* y, int dt, int ncols, int T, int H, int dn, int dr,
                                      int R, int rot, const float* cos_sin, int max_pos,
                                      const void* norm_w, int norm_dt, float eps,
                                      const int32_t* row_pos, const int32_t* row_slot,
                                      const int32_t* slot_len, void* cache,
                                      const int32_t* page_table, int table_stride, int page_size,
                                      int ring, void* c_out, void* kr_out, void* cache_t,
                                      void* stream) {
    if (T < 0 || H <= 0 || dn < 0 || dr < 0 || R <= 0 || !illm_dtype_ok(dt) || !illm_dtype_ok(norm_dt) ||
        ncols < H * (dn + dr) + R + dr)
        return ILLM_ERR_ARG;
    if (cos_sin && (rot <= 0 || rot > dr || (rot & 1) || max_pos <= 0)) return ILLM_ERR_ARG;
    if (cache && (!page_table || !row_slot || page_size <= 0 || table_stride <= 0)) return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(latent_rope_store_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, y, dt,
                       ncols, H, dn, dr, R, rot, cos_sin, max_pos, norm_w, norm_dt, eps, row_pos,
                       row_slot, slot_len, cache, page_table, table_stride, page_size, ring, c_out,
                       kr_out, cache_t);
    return illm_launch_status();
}

// ---------------------------------------------------------------- packed rows for prompt attention
// out[t] = [q heads | k heads | v heads], every head P wide: q_h = [y's q_h (dn + dr) | 0],
// k_h = [kvu's key part h (dn) | kr (dr) | 0], v_h = [kvu's value part h (dv) | 0].
// kvu [T, H dn + H dv] is the product of the latent rows with [W_uk ; W_uv].
__global__ void __launch_bounds__(256)
latent_pack_kernel(const void* __restrict__ y, int dt, int ncols, const void* __restrict__ kvu,
                   const void* __restrict__ kr, void* __restrict__ out, int H, int dn, int dr,
                   int dv, int P) {
    const size_t t = blockIdx.x;
    const int HP = H * P, dq = dn + dr;
    const size_t kvrow = t * (size_t)(H * (dn + dv));
    for (int e = threadIdx.x; e < 3 * HP; e += blockDim.x) {
        const int which = e / HP, rem = e - which * HP;
        const int h = rem / P, d = rem - h * P;
        float v = 0.f;
        if (which == 0) {
            if (d < dq) v = ld_f(y, dt, t * ncols + (size_t)h * dq + d);
        } else if (which == 1) {
            if (d < dn) v = ld_f(kvu, dt, kvrow + (size_t)h * dn + d);
            else if (d < dq) v = ld_f(kr, dt, t * dr + (d - dn));
        } else if (d < dv) {
            v = ld_f(kvu, dt, kvrow + (size_t)H * dn + (size_t)h * dv + d);
        }
        st_f(out, dt, t * (size_t)(3 * HP) + e, v);
    }
}

extern "C" int illm_latent_pack(const void* y, int dt, int ncols, const void* kvu, const void* kr,
                                void* out, int T, int H, int dn, int dr, int dv, int P,
                                void* stream) {
    if (T < 0 || H <= 0 || dn < 0 || dr < 0 || dv <= 0 || P < dn + dr || P < dv || !illm_dtype_ok(dt))
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(latent_pack_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, y, dt, ncols,
                       kvu, kr, out, H, dn, dr, dv, P);
    return illm_launch_status();
}

// out[t, h dv + v] = attn[t, h P + v] * sigmoid(y[t, gate_off + h]): the output gate per head.
__global__ void __launch_bounds__(256)
latent_gate_kernel(const void* __restrict__ attn, const void* __restrict__ y, int dt, int ncols,
                   int gate_off, void* __restrict__ out, int H, int dv, int P) {
    const size_t t = blockIdx.x;
    for (int e = threadIdx.x; e < H * dv; e += blockDim.x) {
        const int h = e / dv, v = e - h * dv;
        const float g = ld_f(y, dt, t * ncols + gate_off + h);
        const float a = ld_f(attn, dt, t * (size_t)(H * P) + (size_t)h * P + v);
        st_f(out, dt, t * (size_t)(H * dv) + e, a * (1.0f / (1.0f + expf(-g))));
    }
}

extern "C" int illm_latent_gate(const void* attn, const void* y, int dt, int ncols, int gate_off,
                                void* out, int T, int H, int dv, int P, void* stream) {
    if (T < 0 || H <= 0 || dv <= 0 || P < dv || gate_off < 0 || gate_off + H > ncols || !illm_dtype_ok(dt))
        return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(latent_gate_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, attn, y, dt,
                       ncols, gate_off, out, H, dv, P);
    return illm_launch_status();
}

// ---------------------------------------------------------------- queries against latent rows
struct LatentStore {              // what the store of a row needs (see illm_latent_rope_store)
    int rot, max_pos, nw_dt, table_stride, page_size, ring;
    float eps;
    const float* cos_sin;
    const void* nw;
    const int32_t* row_pos;
    const int32_t* row_slot;
    void* cache;
    void* cache_t;
    const int32_t* page_table;
};

// The rot part of a head's query in LDS (qs[dn ..]) rotated at the row's position.
__device__ __forceinline__ void rotate_in_lds(float* qs, int dn, const LatentStore& st, int b) {
    if (!st.cos_sin) return;
    int pos = st.row_pos[b];
    if (pos >= st.max_pos) pos = st.max_pos - 1;
    const float* cs = st.cos_sin + (size_t)pos * st.rot;
    for (int i = threadIdx.x; i < st.rot / 2; i += blockDim.x) {
        const float c = cs[2 * i], s = cs[2 * i + 1];
        const float a = qs[dn + 2 * i], v = qs[dn + 2 * i + 1];
        qs[dn + 2 * i] = a * c - v * s;
        qs[dn + 2 * i + 1] = v * c + a * s;
    }
    __syncthreads();
}

// qa[b, h] = [sum_d q[b, h, d] W_uk[h dn + d, :] (R) | q[b, h, dn:] (dr)], float32.  grid (B, H).
// FUSED (grid (B, H + 1)): the query's rot part is rotated here, on its way (y keeps the
// unrotated one), and block (b, H) norms, rotates and stores row b's latent and key part.
template <bool FUSED>
__global__ void __launch_bounds__(256)
latent_absorb_q_kernel(void* __restrict__ y, int dt, int ncols, const void* __restrict__ wuk,
                       int w_dt, void* __restrict__ qa, int qa_dt, int H, int dn, int dr, int R,
                       LatentStore st) {
    extern __shared__ float qs[];
    const int b = blockIdx.x, h = blockIdx.y;
    if (FUSED && h == H) {
        latent_store_row(b, y, dt, ncols, H, dn, dr, R, st.rot, st.cos_sin, st.max_pos, st.nw, st.nw_dt,
                         st.eps, st.row_pos, st.row_slot, nullptr, st.cache, st.page_table,
                         st.table_stride, st.page_size, st.ring, nullptr, nullptr, st.cache_t, false);
        return;
    }
    const size_t src = (size_t)b * ncols + (size_t)h * (dn + dr);
    for (int d = threadIdx.x; d < dn + dr; d += blockDim.x) qs[d] = ld_f(y, dt, src + d);
    __syncthreads();
    if (FUSED) rotate_in_lds(qs, dn, st, b);
    const size_t dst = ((size_t)b * H + h) * (size_t)(R + dr);
    for (int r = threadIdx.x; r < R; r += blockDim.x) {
        float acc = 0.f;
#pragma unroll 8
        for (int d = 0; d < dn; ++d) acc += qs[d] * ld_f(wuk, w_dt, ((size_t)h * dn + d) * R + r);
        st_f(qa, qa_dt, dst + r, acc);
    }
    for (int e = threadIdx.x; e < dr; e += blockDim.x) st_f(qa, qa_dt, dst + R + e, qs[dn + e]);
}

// The same for bfloat16 W_uk with R % 8 == 0 and R <= 512: a thread holds 8 neighbouring latent
// dims (one 16-byte load a row of W_uk) and takes every (256 / (R / 8))-th plain dim; the groups'
// sums are added through LDS in group order.
template <bool FUSED>
__global__ void __launch_bounds__(256)
latent_absorb_q_bf16_kernel(void* __restrict__ y, int dt, int ncols,
                            const bf16_t* __restrict__ wuk, void* __restrict__ qa, int qa_dt, int H,
                            int dn, int dr, int R, LatentStore st) {
    extern __shared__ float sm[];
    float* qs = sm;                       // [dn + dr]
    float* part = sm + dn + dr;           // [groups][R]
    const int b = blockIdx.x, h = blockIdx.y;
    if (FUSED && h == H) {
        latent_store_row(b, y, dt, ncols, H, dn, dr, R, st.rot, st.cos_sin, st.max_pos, st.nw, st.nw_dt,
                         st.eps, st.row_pos, st.row_slot, nullptr, st.cache, st.page_table,
                         st.table_stride, st.page_size, st.ring, nullptr, nullptr, st.cache_t, false);
        return;
    }
    const size_t src = (size_t)b * ncols + (size_t)h * (dn + dr);
    for (int d = threadIdx.x; d < dn + dr; d += 256) qs[d] = ld_f(y, dt, src + d);
    __syncthreads();
    if (FUSED) rotate_in_lds(qs, dn, st, b);
    const int per_row = R / 8, groups = 256 / per_row;
    const int c = threadIdx.x % per_row, g = threadIdx.x / per_row;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    if (g < groups) {
        const bf16_t* wp = wuk + (size_t)h * dn * R + c * 8;
#pragma unroll 4
        for (int d = g; d < dn; d += groups) {
            const uint4 u = *(const uint4*)(wp + (size_t)d * R);
            const float q = qs[d];
            const uint32_t uw[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[2 * i] += q * __uint_as_float(uw[i] << 16);
                acc[2 * i + 1] += q * __uint_as_float(uw[i] & 0xffff0000u);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) part[(size_t)g * R + c * 8 + i] = acc[i];
    }
    __syncthreads();
    const size_t dst = ((size_t)b * H + h) * (size_t)(R + dr);
    for (int r = threadIdx.x; r < R; r += 256) {
        float a = 0.f;
        for (int gg = 0; gg < groups; ++gg) a += part[(size_t)gg * R + r];
        st_f(qa, qa_dt, dst + r, a);
    }
    for (int e = threadIdx.x; e < dr; e += 256) st_f(qa, qa_dt, dst + R + e, qs[dn + e]);
}

template <bool FUSED>
static int launch_absorb_q(void* y, int dt, int ncols, const void* wuk, int w_dt, void* qa, int qa_dt,
                           int B, int H, int dn, int dr, int R, const LatentStore& st,
                           hipStream_t stream) {
    const dim3 grid(B, FUSED ? H + 1 : H);
    if (w_dt == ILLM_BF16 && R % 8 == 0 && R <= 512 && R >= 8) {
        const int groups = 256 / (R / 8);
        const size_t smem = ((size_t)(dn + dr) + (size_t)groups * R) * sizeof(float);
        if (smem <= 48 * 1024) {
            hipLaunchKernelGGL(latent_absorb_q_bf16_kernel<FUSED>, grid, dim3(256), smem, stream, y, dt,
                               ncols, (const bf16_t*)wuk, qa, qa_dt, H, dn, dr, R, st);
            return illm_launch_status();
        }
    }
    hipLaunchKernelGGL(latent_absorb_q_kernel<FUSED>, grid, dim3(256), (size_t)(dn + dr) * sizeof(float),
                       stream, y, dt, ncols, wuk, w_dt, qa, qa_dt, H, dn, dr, R, st);
    return illm_launch_status();
}

extern "C" int illm_latent_absorb_q(const void* y, int dt, int ncols, const void* wuk, int w_dt,
                                    void* qa, int qa_dt, int B, int H, int dn, int dr, int R,
                                    void* stream) {
    if (B < 0 || H <= 0 || H > 65534 || dn < 0 || dr < 0 || R <= 0 || !illm_dtype_ok(dt) ||
        !illm_dtype_ok(w_dt) || !illm_dtype_ok(qa_dt) || ncols < H * (dn + dr))
        return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
    LatentStore st = {};
    return launch_absorb_q<false>((void*)y, dt, ncols, wuk, w_dt, qa, qa_dt, B, H, dn, dr, R, st,
                                  (hipStream_t)stream);
}

extern "C" int illm_latent_store_absorb(void* y, int dt, int ncols, int B, int H, int dn, int dr,
                                        int R, int rot, const float* cos_sin, int max_pos,
                                        const void* norm_w, int norm_dt, float eps,
                                        const int32_t* row_pos, const int32_t* row_slot, void* cache,
                                        const int32_t* page_table, int table_stride, int page_size,
                                        int ring, void* cache_t, const void* wuk, int w_dt, void* qa,
                                        int qa_dt, void* stream) {
    if (B < 0 || H <= 0 || H > 65534 || dn < 0 || dr < 0 || R <= 0 || !illm_dtype_ok(dt) ||
        !illm_dtype_ok(w_dt) || !illm_dtype_ok(qa_dt) || !illm_dtype_ok(norm_dt) ||
        ncols < H * (dn + dr) + R + dr || !row_pos)
        return ILLM_ERR_ARG;
    if (cos_sin && (rot <= 0 || rot > dr || (rot & 1) || max_pos <= 0)) return ILLM_ERR_ARG;
    if (cache && (!page_table || !row_slot || page_size <= 0 || table_stride <= 0)) return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
    LatentStore st;
    st.rot = rot; st.max_pos = max_pos; st.nw_dt = norm_dt; st.table_stride = table_stride;
    st.page_size = page_size; st.ring = ring; st.eps = eps; st.cos_sin = cos_sin; st.nw = norm_w;
    st.row_pos = row_pos; st.row_slot = row_slot; st.cache = cache; st.cache_t = cache_t;
    st.page_table = page_table;
    return launch_absorb_q<true>(y, dt, ncols, wuk, w_dt, qa, qa_dt, B, H, dn, dr, R, st,
                                 (hipStream_t)stream);
}

// ---------------------------------------------------------------- one token over the latent cache
// grid (sequences, splits, groups of HG = 4 HGW heads); 256 threads.  A split takes whole tiles of
// TK keys aligned at absolute positions; a tile of latent rows goes through LDS once for all heads
// of the block.  Wave w owns heads 4-wise: HGW heads, whose scores, softmax statistics and sums it
// keeps to itself; lane = (key of the tile, part of the row), lanes of one key share the row's
// dims in turn and add their partial scores.  For the sums a lane holds latent dims lane + 64 c.
// Each block leaves (sums [R], max, weight) per head in `partial`.
template <int DT>
__device__ __forceinline__ float lds_elem(const char* ks, size_t i) {
    return DT == ILLM_BF16 ? bf16_to_f32(((const bf16_t*)ks)[i]) : ((const float*)ks)[i];
}

template <int DT, int HGW, int RC>
__global__ void __launch_bounds__(256)
latent_decode_kernel(const float* __restrict__ qa, const void* __restrict__ cache,
                     const int32_t* __restrict__ page_table, int table_stride, int page_size,
                     int ring, const int32_t* __restrict__ seq_slot,
                     const int32_t* __restrict__ seq_len, int len_more,
                     float* __restrict__ partial, int nsplit, int H, int R, int dr, float scale,
                     int window, int TK, int kstride) {
    extern __shared__ size_t smem_raw[];
    const int D = R + dr, HG = 4 * HGW;
    size_t* rowoff = smem_raw;                         // [TK]
    float* qs = (float*)(rowoff + TK);                 // [HG][D]
    float* ps = qs + (size_t)HG * D;                   // [HG][TK]
    char* ks = (char*)(ps + (size_t)HG * TK);          // [TK][kstride] in storage type
    const int b = blockIdx.x, split = blockIdx.y, h0 = blockIdx.z * HG;
    const int len = seq_len[b] + len_more, slot = seq_slot[b];
    const int lo = window > 0 ? (len - window > 0 ? len - window : 0) : 0;
    const int tile0 = lo / TK, tile1 = (len - 1) / TK + 1;
    const int per = (tile1 - tile0 + nsplit - 1) / nsplit;
    const int ta = tile0 + split * per;
    const int tb = ta + per < tile1 ? ta + per : tile1;
    for (int e = threadIdx.x; e < HG * D; e += 256) {
        const int hh = e / D, d = e - hh * D;
        qs[e] = h0 + hh < H ? qa[((size_t)b * H + h0 + hh) * D + d] : 0.f;
    }
    const int w = wave_index(), lane = threadIdx.x & 63;
    const int NP = 64 / TK, j = lane % TK, part = lane / TK;
    float m[HGW], l[HGW], acc[HGW][RC];
#pragma unroll
    for (int i = 0; i < HGW; ++i) {
        m[i] = -INFINITY; l[i] = 0.f;
#pragma unroll
        for (int c = 0; c < RC; ++c) acc[i][c] = 0.f;
    }
    for (int tile = ta; tile < tb; ++tile) {
        const int k0 = tile * TK;
        __syncthreads();                               // the tile before has been used up
        if (threadIdx.x < TK) {
            const int p = k0 + threadIdx.x;
            int lp = p / page_size;
            if (ring > 0) lp %= ring;
            const int phys = page_table[(size_t)slot * table_stride + lp];
            rowoff[threadIdx.x] = ((size_t)phys * page_size + (p % page_size)) * (size_t)D;
        }
        __syncthreads();
        for (int e = threadIdx.x; e < TK * D; e += 256) {
            const int jj = e / D, d = e - jj * D;
            const int p = k0 + jj;
            const bool ok = p >= lo && p < len;
            if (DT == ILLM_BF16)
                ((bf16_t*)ks)[(size_t)jj * kstride + d] = ok ? ((const bf16_t*)cache)[rowoff[jj] + d] : (bf16_t)0;
            else
                ((float*)ks)[(size_t)jj * kstride + d] = ok ? ((const float*)cache)[rowoff[jj] + d] : 0.f;
        }
        __syncthreads();
        float s[HGW];
#pragma unroll
        for (int i = 0; i < HGW; ++i) s[i] = 0.f;
        for (int d = part; d < D; d += NP) {
            const float kv = lds_elem<DT>(ks, (size_t)j * kstride + d);
#pragma unroll
            for (int i = 0; i < HGW; ++i) s[i] += qs[(size_t)(w * HGW + i) * D + d] * kv;
        }
        for (int off = TK; off < 64; off <<= 1) {
#pragma unroll
            for (int i = 0; i < HGW; ++i) s[i] += __shfl_xor(s[i], off, 64);
        }
        const int p = k0 + j;
        const bool ok = p >= lo && p < len;
#pragma unroll
        for (int i = 0; i < HGW; ++i) {
            const float sc = ok ? s[i] * scale : -INFINITY;
            const float mn = fmaxf(m[i], wave_max(sc));
            const float alpha = m[i] == -INFINITY ? 0.f : expf(m[i] - mn);
            const float pj = ok ? expf(sc - mn) : 0.f;
            l[i] = l[i] * alpha + wave_sum(part == 0 ? pj : 0.f);
            m[i] = mn;
            if (part == 0) ps[(size_t)(w * HGW + i) * TK + j] = pj;
#pragma unroll
            for (int c = 0; c < RC; ++c) acc[i][c] *= alpha;
        }
        __syncthreads();
        const int j_lo = lo - k0 > 0 ? lo - k0 : 0;
        const int j_hi = len - k0 < TK ? len - k0 : TK;
        for (int jj = j_lo; jj < j_hi; ++jj) {
            float pw[HGW];
#pragma unroll
            for (int i = 0; i < HGW; ++i) pw[i] = ps[(size_t)(w * HGW + i) * TK + jj];
#pragma unroll
            for (int c = 0; c < RC; ++c) {
                const int r = lane + 64 * c;
                const float kv = r < R ? lds_elem<DT>(ks, (size_t)jj * kstride + r) : 0.f;
#pragma unroll
                for (int i = 0; i < HGW; ++i) acc[i][c] += pw[i] * kv;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < HGW; ++i) {
        const int h = h0 + w * HGW + i;
        if (h >= H) continue;
        float* dst = partial + (((size_t)b * H + h) * nsplit + split) * (size_t)(R + 4);
#pragma unroll
        for (int c = 0; c < RC; ++c) {
            const int r = lane + 64 * c;
            if (r < R) dst[r] = acc[i][c];
        }
        if (lane == 0) { dst[R] = m[i]; dst[R + 1] = l[i]; }
    }
}

template <int DT, int HGW>
static int launch_latent_decode(int RC, dim3 grid, size_t smem, hipStream_t st, const float* qa,
                                const void* cache, const int32_t* page_table, int table_stride,
                                int page_size, int ring, const int32_t* seq_slot,
                                const int32_t* seq_len, int len_more, float* partial, int nsplit,
                                int H, int R, int dr, float scale, int window, int TK, int kstride) {
#define GO(RC_)                                                                                   \
    do {                                                                                          \
        if (smem > 48 * 1024 &&                                                                   \
            hipFuncSetAttribute((const void*)latent_decode_kernel<DT, HGW, RC_>,                  \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) { \
            (void)hipGetLastError();                                                              \
            return ILLM_ERR_ARG;                                                                  \
        }                                                                                         \
        hipLaunchKernelGGL((latent_decode_kernel<DT, HGW, RC_>), grid, dim3(256), smem, st, qa,   \
                           cache, page_table, table_stride, page_size, ring, seq_slot, seq_len,   \
                           len_more, partial, nsplit, H, R, dr, scale, window, TK, kstride);      \
        return illm_launch_status();                                                              \
    } while (0)
    switch (RC) {
        case 1: GO(1);
        case 2: GO(2);
        case 4: GO(4);
        case 8: GO(8);
        default: GO(16);
    }
#undef GO
}

extern "C" int illm_latent_attn_decode(const float* qa, const void* cache, int dt,
                                       const int32_t* page_table, int table_stride, int page_size,
                                       int ring, const int32_t* seq_slot, const int32_t* seq_len,
                                       int len_more, float* partial, int nsplit, int B, int H,
                                       int R, int dr, float scale, int window, void* stream) {
    if (B < 0 || H <= 0 || R <= 0 || R > 1024 || dr < 0 || nsplit < 1 || nsplit > 65535 ||
        page_size <= 0 || page_size % 8 || table_stride <= 0 || !illm_dtype_ok(dt) || !partial)
        return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
    const int D = R + dr;
    const int HGW = H >= 16 ? 4 : (H >= 8 ? 2 : 1), HG = 4 * HGW;
    const int groups = (H + HG - 1) / HG;
    if (groups > 65535) return ILLM_ERR_ARG;
    const int rc = (R + 63) / 64;
    const int RC = rc <= 1 ? 1 : (rc <= 2 ? 2 : (rc <= 4 ? 4 : (rc <= 8 ? 8 : 16)));
    // row stride of a tile in LDS: lanes that read the same dim of different keys hit different banks
    int kstride;
    if (dt == ILLM_BF16) {
        kstride = (D + 1) & ~1;
        if ((kstride / 2) % 2 == 0) kstride += 2;
    } else {
        kstride = D | 1;
    }
    const size_t esz = dt == ILLM_BF16 ? 2 : 4;
    int TK = 64;
    size_t smem = 0;
    for (; TK >= 8; TK >>= 1) {
        smem = (size_t)TK * 8 + (size_t)HG * D * 4 + (size_t)HG * TK * 4 + (size_t)TK * kstride * esz;
        if (page_size % TK == 0 && smem <= 128 * 1024) break;
    }
    if (TK < 8) return ILLM_ERR_ARG;
    const dim3 grid(B, nsplit, groups);
    hipStream_t st = (hipStream_t)stream;
#define CALL(DT_, HGW_)                                                                            \
    return launch_latent_decode<DT_, HGW_>(RC, grid, smem, st, qa, cache, page_table, table_stride, \
                                           page_size, ring, seq_slot, seq_len, len_more, partial,   \
                                           nsplit, H, R, dr, scale, window, TK, kstride)
    if (dt == ILLM_BF16) {
        if (HGW == 4) CALL(ILLM_BF16, 4);
        if (HGW == 2) CALL(ILLM_BF16, 2);
        CALL(ILLM_BF16, 1);
    }
    if (HGW == 4) CALL(ILLM_F32, 4);
    if (HGW == 2) CALL(ILLM_F32, 2);
    CALL(ILLM_F32, 1);
#undef CALL
}

// The same walk on the matrix cores for a bfloat16 cache (R % 16 == 0, (R + dr) % 8 == 0, pages of
// a multiple of 32 rows), with a second copy of the latent rows laid out [page][dim][row]
// (`cache_t`).  A block is one wave: a group of 16 heads, one range of keys, 32 keys at a time.
// Scores: MFMA 16x16x32 with 16 keys as the A operand (8 neighbouring dims of a cache row, read in
// operand order straight from memory) and the 16 heads' queries as the B operand (bfloat16, read
// the same way; they stay in the cache): lane (r, q) = (lane % 16, lane / 16) is left with head r's scores of keys 4 q .. 4 q + 3 of
// either half of the 32.  Those 8 weights are the B operand of the second product as they stand:
// its contraction takes the keys in that order, and the A operand, 16 latent dims by these 8 keys,
// is two 8-byte loads from the transposed copy.  Keys that are not seen get weight 0 and their
// loaded values are masked (a freed page may hold anything).  The sums stay in registers
// (R / 16 accumulators of 4); statistics in float32.
typedef __bf16 la_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float la_f32x4_t __attribute__((ext_vector_type(4)));

template <int RT>
__global__ void __launch_bounds__(64)
latent_decode_mfma_kernel(const bf16_t* __restrict__ qa, const bf16_t* __restrict__ cache,
                          const bf16_t* __restrict__ cache_t,
                          const int32_t* __restrict__ page_table, int table_stride, int page_size,
                          int ring, const int32_t* __restrict__ seq_slot,
                          const int32_t* __restrict__ seq_len, int len_more,
                          float* __restrict__ partial, int nsplit, int H, int R, int dr, float scale,
                          int window) {
    const int D = R + dr;
    const int b = blockIdx.x, split = blockIdx.y, h0 = blockIdx.z * 16;
    const int lane = threadIdx.x, r = lane & 15, q = lane >> 4;
    const int len = seq_len[b] + len_more, slot = seq_slot[b];
    const int lo = window > 0 ? (len - window > 0 ? len - window : 0) : 0;
    const int tile0 = lo / 32, tile1 = (len - 1) / 32 + 1;
    const int per = (tile1 - tile0 + nsplit - 1) / nsplit;
    const int ta = tile0 + split * per;
    const int tb = ta + per < tile1 ? ta + per : tile1;
    // the lane's query row (heads beyond the last read the last one's; their results are dropped)
    const bf16_t* qp = qa + ((size_t)b * H + (h0 + r < H ? h0 + r : H - 1)) * D + 8 * q;
    la_f32x4_t o[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) o[rt] = (la_f32x4_t){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    const la_bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int tile = ta; tile < tb; ++tile) {
        const int k0 = tile * 32;
        int lp = k0 / page_size;
        if (ring > 0) lp %= ring;
        const int phys = page_table[(size_t)slot * table_stride + lp];
        const int rowb = k0 % page_size;
        const bf16_t* kp0 = cache + ((size_t)phys * page_size + rowb + r) * D + 8 * q;
        const bf16_t* kp1 = kp0 + (size_t)16 * D;
        la_f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = s0;
        // six steps of 32 dims at a time: all their loads are asked for before the first product
        int d0 = 0;
        for (; d0 + 192 <= D; d0 += 192) {
            la_bf16x8_t qv[6], ka[6], kb[6];
#pragma unroll
            for (int u = 0; u < 6; ++u) {
                qv[u] = *(const la_bf16x8_t*)(qp + d0 + 32 * u);
                ka[u] = *(const la_bf16x8_t*)(kp0 + d0 + 32 * u);
                kb[u] = *(const la_bf16x8_t*)(kp1 + d0 + 32 * u);
            }
#pragma unroll
            for (int u = 0; u < 6; ++u) {
                s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[u], qv[u], s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb[u], qv[u], s1, 0, 0, 0);
            }
        }
        for (; d0 < D; d0 += 32) {                   // what is left, the last step maybe in part
            la_bf16x8_t qv = zero8, ka = zero8, kb = zero8;
            if (d0 + 8 * q < D) {
                qv = *(const la_bf16x8_t*)(qp + d0);
                ka = *(const la_bf16x8_t*)(kp0 + d0);
                kb = *(const la_bf16x8_t*)(kp1 + d0);
            }
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qv, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb, qv, s1, 0, 0, 0);
        }
        float sc[8];
        bool ok[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int p0 = k0 + 4 * q + i, p1 = p0 + 16;
            ok[i] = p0 >= lo && p0 < len;
            ok[4 + i] = p1 >= lo && p1 < len;
            sc[i] = ok[i] ? s0[i] * scale : -INFINITY;
            sc[4 + i] = ok[4 + i] ? s1[i] * scale : -INFINITY;
        }
        float mt = sc[0];
#pragma unroll
        for (int i = 1; i < 8; ++i) mt = fmaxf(mt, sc[i]);
        mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
        mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
        const float mn = fmaxf(m, mt);
        const float alpha = m == -INFINITY ? 0.f : expf(m - mn);
        float pw[8], ls = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            pw[i] = ok[i] ? expf(sc[i] - mn) : 0.f;
            ls += pw[i];
        }
        ls += __shfl_xor(ls, 16, 64);
        ls += __shfl_xor(ls, 32, 64);
        l = l * alpha + ls;
        m = mn;
        uint4 pu;
        pu.x = pack_bf16x2(pw[0], pw[1]); pu.y = pack_bf16x2(pw[2], pw[3]);
        pu.z = pack_bf16x2(pw[4], pw[5]); pu.w = pack_bf16x2(pw[6], pw[7]);
        const la_bf16x8_t pv = *(const la_bf16x8_t*)&pu;
        const uint32_t k01 = (ok[0] ? 0xffffu : 0u) | (ok[1] ? 0xffff0000u : 0u);
        const uint32_t k23 = (ok[2] ? 0xffffu : 0u) | (ok[3] ? 0xffff0000u : 0u);
        const uint32_t k45 = (ok[4] ? 0xffffu : 0u) | (ok[5] ? 0xffff0000u : 0u);
        const uint32_t k67 = (ok[6] ? 0xffffu : 0u) | (ok[7] ? 0xffff0000u : 0u);
        const bf16_t* tp = cache_t + ((size_t)phys * R + r) * page_size + rowb + 4 * q;
        constexpr int CH = RT < 8 ? RT : 8;          // row groups whose loads are in flight together
#pragma unroll
        for (int r0 = 0; r0 < RT; r0 += CH) {
            uint2 c0[CH], c1[CH];
#pragma unroll
            for (int u = 0; u < CH; ++u) {
                const int rt = (r0 + u) * 16 < R ? r0 + u : 0;      // beyond R: loaded, not used
                c0[u] = *(const uint2*)(tp + (size_t)rt * 16 * page_size);
                c1[u] = *(const uint2*)(tp + (size_t)rt * 16 * page_size + 16);
            }
#pragma unroll
            for (int u = 0; u < CH; ++u) {
                const int rt = r0 + u;
                if (rt * 16 < R) {
                    uint4 cu;
                    cu.x = c0[u].x & k01; cu.y = c0[u].y & k23; cu.z = c1[u].x & k45; cu.w = c1[u].y & k67;
                    o[rt][0] *= alpha; o[rt][1] *= alpha; o[rt][2] *= alpha; o[rt][3] *= alpha;
                    o[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const la_bf16x8_t*)&cu, pv, o[rt], 0, 0, 0);
                }
            }
        }
    }
    // o[rt][i] = sum of head h0 + r over latent dim 16 rt + 4 q + i
    const int h = h0 + r;
    if (h < H) {
        float* dst = partial + (((size_t)b * H + h) * nsplit + split) * (size_t)(R + 4);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            if (rt * 16 < R) {
                *(la_f32x4_t*)(dst + rt * 16 + 4 * q) = o[rt];       // rows of R + 4 floats: 16-byte aligned
            }
        }
        if (q == 0) { dst[R] = m; dst[R + 1] = l; }
    }
}

extern "C" int illm_latent_attn_decode_mfma(const void* qa, const void* cache, const void* cache_t,
                                            const int32_t* page_table, int table_stride,
                                            int page_size, int ring, const int32_t* seq_slot,
                                            const int32_t* seq_len, int len_more, float* partial,
                                            int nsplit, int B, int H, int R, int dr, float scale,
                                            int window, void* stream) {
    if (B < 0 || H <= 0 || R <= 0 || R > 512 || R % 16 || dr < 0 || (R + dr) % 8 || nsplit < 1 ||
        nsplit > 65535 || page_size <= 0 || page_size % 32 || table_stride <= 0 || !partial ||
        !cache || !cache_t)
        return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
    const int groups = (H + 15) / 16;
    if (groups > 65535) return ILLM_ERR_ARG;
    const dim3 grid(B, nsplit, groups);
    hipStream_t st = (hipStream_t)stream;
#define GO(RT_)                                                                                   \
    hipLaunchKernelGGL((latent_decode_mfma_kernel<RT_>), grid, dim3(64), 0, st,                    \
                       (const bf16_t*)qa, (const bf16_t*)cache, (const bf16_t*)cache_t, page_table, table_stride,     \
                       page_size, ring, seq_slot, seq_len, len_more, partial, nsplit, H, R, dr,    \
                       scale, window)
    if (R <= 64) GO(4);
    else if (R <= 128) GO(8);
    else if (R <= 256) GO(16);
    else GO(32);
#undef GO
    return illm_launch_status();
}

// grid (B, H, chunks of 32 value dims): combine the splits, multiply the combined latent sum by
// W_uv's rows of the head (a wave a value dim, lanes over the latent dims) and by the head's
// output gate.  Every chunk's block combines the splits for itself.
__global__ void __launch_bounds__(256)
latent_merge_up_kernel(const float* __restrict__ partial, int nsplit, const void* __restrict__ wuv,
                       int w_dt, const void* __restrict__ y, int dt, int ncols, int gate_off,
                       void* __restrict__ out, int H, int R, int dv) {
    extern __shared__ float ol[];                      // [R] combined sums, then [nsplit] weights
    float* ws = ol + R;
    const int b = blockIdx.x, h = blockIdx.y;
    const float* base = partial + ((size_t)b * H + h) * nsplit * (size_t)(R + 4);
    const int w = wave_index(), lane = threadIdx.x & 63;
    if (w == 0) {
        // the ranges' (max, weight): lane s holds range s, s + 64, ...; weights exp(m_s - M) / total
        float M = -INFINITY;
        for (int s = lane; s < nsplit; s += 64) M = fmaxf(M, base[(size_t)s * (R + 4) + R]);
        M = wave_max(M);
        float tot = 0.f;
        for (int s = lane; s < nsplit; s += 64) {
            const float ms = base[(size_t)s * (R + 4) + R];
            const float e = ms == -INFINITY ? 0.f : expf(ms - M);
            ws[s] = e;
            tot += base[(size_t)s * (R + 4) + R + 1] * e;
        }
        tot = wave_sum(tot);
        for (int s = lane; s < nsplit; s += 64) ws[s] = ws[s] / tot;
    }
    __syncthreads();
    for (int r = threadIdx.x; r < R; r += 256) {
        float a = 0.f;
        for (int s = 0; s < nsplit; ++s) a += base[(size_t)s * (R + 4) + r] * ws[s];
        ol[r] = a;
    }
    __syncthreads();
    const float g = ld_f(y, dt, (size_t)b * ncols + gate_off + h);
    const float gate = 1.0f / (1.0f + expf(-g));
    if (w_dt == ILLM_BF16 && R % 8 == 0) {
        // 16-byte loads: a lane takes 8 neighbouring latent dims of a row of W_uv
        const bf16_t* wp = (const bf16_t*)wuv;
        const int v_end = min(dv, (int)(blockIdx.z + 1) * 32);
        for (int v0 = blockIdx.z * 32 + 4 * w; v0 < v_end; v0 += 16) {   // four rows of W_uv in flight a wave
            float dot[4] = {0.f, 0.f, 0.f, 0.f};
            for (int r = lane * 8; r < R; r += 512) {
                uint4 u[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int v = v0 + j < v_end ? v0 + j : v_end - 1;
                    u[j] = *(const uint4*)(wp + ((size_t)h * dv + v) * R + r);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t uw[4] = {u[j].x, u[j].y, u[j].z, u[j].w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        dot[j] += __uint_as_float(uw[i] << 16) * ol[r + 2 * i];
                        dot[j] += __uint_as_float(uw[i] & 0xffff0000u) * ol[r + 2 * i + 1];
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float d = wave_sum(dot[j]);
                if (lane == 0 && v0 + j < v_end)
                    st_f(out, dt, (size_t)b * H * dv + (size_t)h * dv + v0 + j, d * gate);
            }
        }
        return;
    }
    const int v_hi = min(dv, (int)(blockIdx.z + 1) * 32);
    for (int v = blockIdx.z * 32 + w; v < v_hi; v += 4) {
        const size_t wr = ((size_t)h * dv + v) * R;
        float dot = 0.f;
        for (int r = lane; r < R; r += 64) dot += ld_f(wuv, w_dt, wr + r) * ol[r];
        dot = wave_sum(dot);
        if (lane == 0) st_f(out, dt, (size_t)b * H * dv + (size_t)h * dv + v, dot * gate);
    }
}

extern "C" int illm_latent_merge_up(const float* partial, int nsplit, const void* wuv, int w_dt,
                                    const void* y, int dt, int ncols, int gate_off, void* out,
                                    int B, int H, int R, int dv, void* stream) {
    if (B < 0 || H <= 0 || H > 65535 || R <= 0 || dv <= 0 || nsplit < 1 || !illm_dtype_ok(dt) ||
        !illm_dtype_ok(w_dt) || gate_off < 0 || gate_off + H > ncols)
        return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
    if ((dv + 31) / 32 > 65535) return ILLM_ERR_ARG;
    hipLaunchKernelGGL(latent_merge_up_kernel, dim3(B, H, (dv + 31) / 32), dim3(256), (size_t)(R + nsplit) * sizeof(float),
                       (hipStream_t)stream, partial, nsplit, wuv, w_dt, y, dt, ncols, gate_off, out,
                       H, R, dv);
    return illm_launch_status();
}
