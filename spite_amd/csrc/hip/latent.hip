// Latent attention: every head's keys and values are projections of one small latent vector
// per position, and only that latent (R elements, normed) and one rotated key part (r elements,
// shared by all heads) are cached: a cache row is [latent | rotated part], Dk = R + r wide.
//
// The per-head projections are folded into the query and the output instead of being applied
// to every cached row: with q_h = [a_h | b_h] (unrotated, rotated) and per-head matrices U_h
// (keys) and V_h (values) of the latent c_j,
//     score_h(i, j) = a_h . (U_h c_j) + b_h . k_j = (U_h^T a_h) . c_j + b_h . k_j
//     out_h(i)      = sum_j p_ij (V_h c_j)        = V_h (sum_j p_ij c_j)
// so the attention itself is one shared "kv head" of key width Dk whose value is the first R
// elements of the key row; the query rows [U_h^T a_h | rot(b_h)] and the up-projection of the
// result are grouped products over the heads (row lists, see gemm_generic.hip).
//
// latent_prepare: the elementwise part between the fused projection and those products.
// attn_latent_generic: the plain kernel of the 32-bit path and of sizes that the MFMA kernel
// (attn_latent_mfma.hip) refuses.
#include "common.h"

// One workgroup per token.  `q` row: H heads of [n | r] query elements; `dkv` row (own): R + r
// elements of the down-projection.  Writes
//   qa[(t*H + h) * Dk + R + e] = the rotated part of head h's query (the first `rot_dims` elements
//       turn, adjacent pairs (2i, 2i+1) by pos * inv_freq[i]; the rest pass);
//   (own) the cache row slot_map[t]: the latent, RMS-normed with weight `w_norm`, then the
//       rotated shared key part;
//   rows_th[h*T + t] = t*H + h and offsets_h[h] = h*T: the row list by which a grouped product
//       with one group per head walks rows that lie token by token.
// Angles, rotation and norm are fp32; sine and cosine are the accurate routines.
template <typename T>
__global__ __launch_bounds__(256)
void latent_prepare_kernel(const T* __restrict__ qd, int ldq, const T* __restrict__ dkv_all, int ld_dkv, T* __restrict__ qa, T* __restrict__ kv_pages,
                           const int* __restrict__ positions, const int* __restrict__ slot_map,
                           const float* __restrict__ inv_freq, const float* __restrict__ w_norm, float eps,
                           int H, int n, int r, int R, int rot_dims, int own,
                           int* __restrict__ rows_th, int* __restrict__ offsets_h, int T_all) {
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int Dk = R + r, hw = n + r;
    const float pos = (float)positions[t];
    const T* row = qd + (size_t)t * ldq;
    auto turned = [&](const T* part, int e) -> float {
        if (e >= rot_dims) return to_f32<T>(part[e]);
        const int i = e >> 1;
        float sn, cs;
        sincosf(pos * inv_freq[i], &sn, &cs);
        const float u = to_f32<T>(part[2 * i]), v = to_f32<T>(part[2 * i + 1]);
        return (e & 1) ? v * cs + u * sn : u * cs - v * sn;
    };
    for (int i = tid; i < H * r; i += 256) {
        const int h = i / r, e = i - h * r;
        qa[((size_t)t * H + h) * Dk + R + e] = from_f32<T>(turned(row + (size_t)h * hw + n, e));
    }
    if (own) {
        const T* dkv = dkv_all + (size_t)t * ld_dkv;
        float sq = 0.f;
        for (int e = tid; e < R; e += 256) { const float x = to_f32<T>(dkv[e]); sq += x * x; }
        const float scale = 1.0f / sqrtf(block_sum<256>(sq, red) / (float)R + eps);
        const int slot = slot_map[t];
        if (slot >= 0) {
            T* out = kv_pages + (size_t)slot * Dk;
            for (int e = tid; e < R; e += 256) out[e] = from_f32<T>(to_f32<T>(dkv[e]) * scale * w_norm[e]);
            for (int e = tid; e < r; e += 256) out[R + e] = from_f32<T>(turned(dkv + R, e));
        }
    }
    for (int h = tid; h < H; h += 256) rows_th[(size_t)h * T_all + t] = t * H + h;
    if (t == 0) for (int h = tid; h <= H; h += 256) offsets_h[h] = h * T_all;
}

extern "C" int spite_latent_prepare(const void* qd, int ldq, const void* dkv, int ld_dkv, void* qa, void* kv_pages, int dtype, const int* positions,
                                    const int* slot_map, const float* inv_freq, const float* w_norm, float eps,
                                    int T, int H, int n, int r, int R, int rot_dims, int own,
                                    int* rows_th, int* offsets_h, hipStream_t st) {
    SP_REQUIRE(T >= 0 && H > 0 && n > 0 && r >= 0 && R > 0, "latent_prepare: bad sizes T=%d H=%d n=%d r=%d R=%d", T, H, n, r, R);
    SP_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= r, "latent_prepare: %d turning elements of %d", rot_dims, r);
    SP_REQUIRE(ldq >= H * (n + r) && (!own || ld_dkv >= R + r), "latent_prepare: rows of %d or %d are too short", ldq, ld_dkv);
    SP_REQUIRE(!own || (dkv && kv_pages && slot_map && w_norm && eps > 0.f), "latent_prepare: the cache row needs pages, slots and the norm");
    SP_REQUIRE((long)T * H < (1L << 31), "latent_prepare: too many rows");
    if (T == 0) return 0;
    if (dtype == SP_F32)
        latent_prepare_kernel<float><<<T, 256, 0, st>>>((const float*)qd, ldq, (const float*)dkv, ld_dkv, (float*)qa, (float*)kv_pages, positions, slot_map,
            inv_freq, w_norm, eps, H, n, r, R, rot_dims, own, rows_th, offsets_h, T);
    else if (dtype == SP_BF16)
        latent_prepare_kernel<bf16><<<T, 256, 0, st>>>((const bf16*)qd, ldq, (const bf16*)dkv, ld_dkv, (bf16*)qa, (bf16*)kv_pages, positions, slot_map,
            inv_freq, w_norm, eps, H, n, r, R, rot_dims, own, rows_th, offsets_h, T);
    else return sp_fail("latent_prepare: unknown dtype %d", dtype);
    SP_LAUNCH_CHECK("latent_prepare");
    return 0;
}

// ------------------------------------------------------------------ the plain attention kernel
// One wave per query row (token t, head h): q row (t*H + h) of width Dk against the cache rows
// [first_visible(p), p] of the token's request; the value of a key is the first R elements of
// its row.  Keys are walked in tiles of 64 that start at first_visible(p), so the order of every
// sum depends on p alone.  Scores, maximum, sum and output are fp32, exp is the accurate one.
#define LAT_MAX_V 16  // latents up to 1,024

template <typename T>
__global__ __launch_bounds__(64)
void attn_latent_generic_kernel(const T* __restrict__ q, const T* __restrict__ kv_pages, T* __restrict__ out,
                                const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                                const int* __restrict__ block_table, int max_blocks, int H, int Dk, int R, int ps,
                                int vis, int span, float scale) {
    extern __shared__ float smem[];
    float* q_sh = smem;                            // [Dk]
    float* p_sh = smem + Dk;                       // [64]
    long long* row_sh = (long long*)(p_sh + 64 + (Dk & 1));   // [64] first element of each key's row, -1 = none
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int p = positions[t];
    const int* bt = block_table + (size_t)seq_of_token[t] * max_blocks;
    const int lo = sp_first_visible(p, vis, span);
    const T* qr = q + ((size_t)t * H + h) * Dk;
    for (int c = lane; c < Dk; c += 64) q_sh[c] = to_f32<T>(qr[c]);
    __syncthreads();
    float m = -INFINITY, l = 0.f;
    float o[LAT_MAX_V];
#pragma unroll
    for (int u = 0; u < LAT_MAX_V; ++u) o[u] = 0.f;
    for (int j0 = lo; j0 <= p; j0 += 64) {
        const int j = j0 + lane;
        float s = -INFINITY;
        long long row = -1;
        if (j <= p) {
            const int page = bt[j / ps];
            if (page < 0) {
                s = NAN;   // a page that was given back is asked for: poison the result
            } else {
                row = ((long long)page * ps + j % ps) * Dk;
                const T* kr = kv_pages + row;
                float acc = 0.f;
                for (int c = 0; c < Dk; ++c) acc = fmaf(q_sh[c], to_f32<T>(kr[c]), acc);
                s = acc * scale;
            }
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float alpha = expf(m - m_new);
        const float pj = (j <= p) ? expf(s - m_new) : 0.f;
        l = l * alpha + wave_sum(pj);
        m = m_new;
        __syncthreads();
        p_sh[lane] = pj;
        row_sh[lane] = row;
        __syncthreads();
        const int n_valid = (p - j0 + 1) < 64 ? (p - j0 + 1) : 64;
#pragma unroll
        for (int u = 0; u < LAT_MAX_V; ++u) {
            const int c = lane + u * 64;
            if (c < R) {
                float acc = o[u] * alpha;
                for (int jj = 0; jj < n_valid; ++jj) {
                    const long long rr = row_sh[jj];
                    acc = fmaf(p_sh[jj], rr >= 0 ? to_f32<T>(kv_pages[rr + c]) : 0.f, acc);
                }
                o[u] = acc;
            }
        }
    }
    const float inv = 1.0f / fmaxf(l, 1e-30f);
    T* orow = out + ((size_t)t * H + h) * R;
#pragma unroll
    for (int u = 0; u < LAT_MAX_V; ++u) {
        const int c = lane + u * 64;
        if (c < R) orow[c] = from_f32<T>(o[u] * inv);
    }
}

extern "C" int spite_attn_latent_generic(const void* q, const void* kv_pages, void* out, int dtype, const int* positions,
                                         const int* seq_of_token, const int* block_table, int max_blocks, int T, int H,
                                         int Dk, int R, int page_size, int vis, int span, float scale, hipStream_t st) {
    SP_REQUIRE(T >= 0 && H > 0 && H <= 65535, "latent attention: %d heads", H);
    SP_REQUIRE(R > 0 && R <= Dk && R <= 64 * LAT_MAX_V, "latent attention: latent of %d in rows of %d (at most %d)", R, Dk, 64 * LAT_MAX_V);
    SP_REQUIRE(page_size > 0 && max_blocks > 0, "latent attention: bad page size %d or table width %d", page_size, max_blocks);
    SP_REQUIRE(vis >= 0 && vis < SP_VIS_COUNT && (!sp_vis_has_span(vis) || span > 0), "latent attention: chunk or window of %d", span);
    if (T == 0) return 0;
    dim3 grid(T, H);
    const size_t sh = (size_t)(Dk + 64 + (Dk & 1)) * sizeof(float) + 64 * sizeof(long long);
    if (dtype == SP_F32)
        attn_latent_generic_kernel<float><<<grid, 64, sh, st>>>((const float*)q, (const float*)kv_pages, (float*)out, positions,
            seq_of_token, block_table, max_blocks, H, Dk, R, page_size, vis, span, scale);
    else if (dtype == SP_BF16)
        attn_latent_generic_kernel<bf16><<<grid, 64, sh, st>>>((const bf16*)q, (const bf16*)kv_pages, (bf16*)out, positions,
            seq_of_token, block_table, max_blocks, H, Dk, R, page_size, vis, span, scale);
    else return sp_fail("latent attention: unknown dtype %d", dtype);
    SP_LAUNCH_CHECK("attn_latent_generic");
    return 0;
}
