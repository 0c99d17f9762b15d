// Latent attention on the matrix units (bfloat16): query rows [Dk] against cache rows [Dk] of one
// shared kv head, the value of a key being the first R elements of its row (see latent.hip).
//
// Because all heads read the same rows, the heads are the kernel's batch: query row t*H + h is
// one column of a 16-column MFMA tile, so a decoded token alone fills tiles with its heads, and a
// prompt's portion fills them with (token, head) pairs.  A workgroup takes up to 128 consecutive
// query rows of one request (the list `wg`, built on the host from the step's entries: first row
// and number of rows), one wave per 16 rows.  All waves walk the same blocks of 32 keys, from the
// first key that the first row may read to the last row's own position; a block is staged once
// in LDS for all of them: the rows (the S^T = K Q^T operand, in the order of the tiles' rows), and their first R
// elements transposed (the O^T = V^T P^T operand).  Every row masks by its own position.
//
// Tiles: S^T tile tt (of 2) holds the keys (r/4)*8 + tt*4 + r%4 of the block in its rows r, so the
// eight scores a lane holds are eight consecutive keys: P^T is the next product's operand without a
// shuffle.  Scores, maximum, sum and the output are fp32.
//
// Few workgroups with many keys (decoded tokens of a few requests over long contexts): the blocks
// of keys are dealt to `n_splits` workgroups a work item (grid.y), each leaves a record (output not
// yet divided, maximum, sum) per query row, and a second kernel joins the records.
#include "common.h"

#define LM_ROWS 128        // query rows per workgroup at most (8 waves of 16)
#define LM_PRE 12          // 16-byte pieces of a key's row that a staging thread keeps in registers, per block in flight
#define LM_KROW_BLOCKS 128 // blocks of keys whose cache rows the staging waves look up ahead of their loop
#define LM_VT_LD 40        // row stride of the transposed values in LDS (32 keys + 8: no bank conflicts, 16-byte rows)

template <int KQ, int NV>   // Dk <= 32*KQ, R <= 16*NV
__global__ __launch_bounds__(512)
void attn_latent_mfma_kernel(const bf16* __restrict__ q, const bf16* __restrict__ kv_pages, bf16* __restrict__ out,
                             const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                             const int* __restrict__ block_table, int max_blocks, const int* __restrict__ wg,
                             int H, int Dk, int R, int ps, int vis, int span, float scale,
                             float* __restrict__ part, int n_splits) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int kq = (Dk + 31) >> 5, nv = (R + 15) >> 4;
    const int ks_ld = kq * 32 + 8;                                  // row stride of the staged rows
    bf16* Ks = (bf16*)lds_raw;                                      // [32][ks_ld]
    bf16* Vt = Ks + 32 * ks_ld;                                     // [nv*16][LM_VT_LD]
    int* kflag = (int*)(Vt + nv * 16 * LM_VT_LD);                   // [32] 1: the key's page was given back
    int* krow = kflag + 32;                                         // [LM_KROW_BLOCKS * 32] cache rows of the share's keys (staging waves)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthreads = blockDim.x;
    const int row0 = wg[2 * blockIdx.x], nrows = wg[2 * blockIdx.x + 1];
    const int t_first = row0 / H, t_last = (row0 + nrows - 1) / H;
    const int* bt = block_table + (size_t)seq_of_token[t_first] * max_blocks;
    const int key_lo = sp_first_visible(positions[t_first], vis, span), key_hi = positions[t_last];

    // the staged rows' elements past Dk are zero for good
    for (int i = tid; i < 32 * (ks_ld - Dk); i += nthreads) {
        const int key = i / (ks_ld - Dk), f = Dk + i % (ks_ld - Dk);
        Ks[key * ks_ld + f] = (bf16)0.f;
    }
    for (int i = tid; i < (nv * 16 - R) * LM_VT_LD; i += nthreads) Vt[R * LM_VT_LD + i] = (bf16)0.f;

    const int chunks = Dk >> 3;                                     // 16-byte pieces of a row

    // this workgroup's share of the blocks of keys
    int blk_first = key_lo >> 5, blk_end = (key_hi >> 5) + 1;
    if (n_splits > 1) {
        const int per = (blk_end - blk_first + n_splits - 1) / n_splits;
        blk_first += (int)blockIdx.y * per;
        blk_end = blk_first + per < blk_end ? blk_first + per : blk_end;
    }
    // Waves beyond the ones that hold query rows do all the staging when they can keep a block's
    // pieces in registers (2 threads a key and wave, PRE pieces a thread) and the share's cache rows
    // fit their table: they fetch the next two blocks while the others compute on this one.  Their loop
    // holds no load but the rows' own, so nothing makes them wait for the youngest load; the table
    // entries of the whole share are looked up before it.
    constexpr int PRE = KQ <= 6 ? 4 : (KQ <= 10 ? 8 : LM_PRE);      // smaller rows leave the other instantiations their registers
    const int n_cw = (nrows + 15) >> 4, n_lw = (nthreads >> 6) - n_cw, n_blk = blk_end - blk_first;
    const bool roles = n_lw * 2 * PRE >= chunks && n_blk <= LM_KROW_BLOCKS && n_blk > 0;
    if (roles && wave >= n_cw) {
        const int lt = tid - n_cw * 64, key = lt & 31, piece0 = lt >> 5, piece_step = n_lw * 2;
        bf16* ks_row = Ks + ((((key >> 2) & 1) << 4) + ((key >> 3) << 2) + (key & 3)) * ks_ld;
        for (int i = lt; i < n_blk * 32; i += n_lw * 64) {
            const int j = (blk_first << 5) + i;
            int r = -2;
            if (j >= key_lo && j <= key_hi) { const int page = bt[j / ps]; r = page >= 0 ? page * ps + j % ps : -1; }
            krow[i] = r;
        }
        __syncthreads();                                            // (the rows' waves meet it before their loop)
        bf16x8 preA[PRE], preB[PRE];
        auto fetch = [&](bf16x8* pre, int r) {
#pragma unroll
            for (int u = 0; u < PRE; ++u) {
                const int pc = piece0 + u * piece_step;
#pragma unroll
                for (int e = 0; e < 8; ++e) pre[u][e] = (bf16)0.f;
                if (r >= 0 && pc < chunks) pre[u] = *(const bf16x8*)(kv_pages + (size_t)r * Dk + (pc << 3));
            }
        };
        auto stage = [&](const bf16x8* pre, int r) {
            __syncthreads();                                        // the last block's readers are done
#pragma unroll
            for (int u = 0; u < PRE; ++u) {
                const int pc = piece0 + u * piece_step, f = pc << 3;
                if (pc < chunks) {
                    *(bf16x8*)(ks_row + f) = pre[u];
                    if (f < R) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) Vt[(f + e) * LM_VT_LD + key] = pre[u][e];
                    }
                }
            }
            if (lt < 32) kflag[key] = r == -1;
            __syncthreads();
        };
        int rA = krow[key], rB = n_blk > 1 ? krow[32 + key] : -2;
        fetch(preA, rA);
        if (n_blk > 1) fetch(preB, rB);
        for (int b = 0; b < n_blk; b += 2) {
            stage(preA, rA);
            if (b + 2 < n_blk) { rA = krow[(b + 2) * 32 + key]; fetch(preA, rA); }   // on its way while the others compute
            if (b + 1 < n_blk) {
                stage(preB, rB);
                if (b + 3 < n_blk) { rB = krow[(b + 3) * 32 + key]; fetch(preB, rB); }
            }
        }
        return;
    }

    const int c = lane & 15, g4 = lane >> 4;
    // this lane's query row: a column of every tile
    const int my = wave * 16 + c;
    const bool row_ok = my < nrows;
    const int row = row0 + (row_ok ? my : 0);
    const int my_p = positions[row / H];
    const int my_lo = sp_first_visible(my_p, vis, span);
    // what this wave's rows read at all (its first and last row bound it: positions grow with the rows)
    const int w_first = wave * 16 < nrows ? wave * 16 : 0;
    const int w_last = wave * 16 + 15 < nrows ? wave * 16 + 15 : nrows - 1;
    const int wave_lo = sp_first_visible(positions[(row0 + w_first) / H], vis, span);
    const int wave_hi = wave * 16 < nrows ? positions[(row0 + w_last) / H] : -1;

    bf16x8 qf[KQ];
#pragma unroll
    for (int k = 0; k < KQ; ++k) {
        const int f = k * 32 + g4 * 8;
        bf16x8 z;
#pragma unroll
        for (int e = 0; e < 8; ++e) z[e] = (bf16)0.f;
        qf[k] = (k < kq && f < Dk) ? *(const bf16x8*)(q + (size_t)row * Dk + f) : z;
    }
    float m_run = -INFINITY, l_run = 0.f;
    f32x4 o[NV];
#pragma unroll
    for (int a = 0; a < NV; ++a) o[a] = f32x4{0.f, 0.f, 0.f, 0.f};
    // Staging: a thread keeps one key of the block (consecutive lanes take consecutive keys, so the
    // transposed copy's 2-byte stores fall into consecutive LDS words instead of one bank) and walks
    // that key's 16-byte pieces.  Where the key's row lies is looked up one block ahead, so the table
    // entry's way from memory is hidden behind the block before.
    const int key = tid & 31, piece0 = tid >> 5, piece_step = nthreads >> 5;
    // LDS row of a key: the 16 rows of S^T tile tt lie together, tile row (key/8)*4 + key%4
    bf16* ks_row = Ks + ((((key >> 2) & 1) << 4) + ((key >> 3) << 2) + (key & 3)) * ks_ld;
    auto row_of = [&](int blk0) -> long long {       // first element of the key's cache row; -1: page given back; -2: not read
        const int j = blk0 + key;
        if (j < key_lo || j > key_hi) return -2;
        const int page = bt[j / ps];
        return page >= 0 ? ((long long)page * ps + j % ps) * Dk : -1;
    };
    auto put = [&](int f, const bf16x8& v) {
        *(bf16x8*)(ks_row + f) = v;
        if (f < R) {
#pragma unroll
            for (int e = 0; e < 8; ++e) Vt[(f + e) * LM_VT_LD + key] = v[e];
        }
    };
    if (roles) __syncthreads();                                     // the staging waves have looked up the share's rows
    long long row_cur = (!roles && blk_first < blk_end) ? row_of(blk_first << 5) : -2;
    for (int blk0 = blk_first << 5; blk0 < (blk_end << 5); blk0 += 32) {
      if (roles) {
        __syncthreads();
        __syncthreads();                                            // the staging waves have filled the block
      } else {
        const long long row_next = blk0 + 32 < (blk_end << 5) ? row_of(blk0 + 32) : -2;
        __syncthreads();                                            // the last block's readers are done
        const bf16* src = kv_pages + (row_cur >= 0 ? row_cur : 0);
        for (int pc = piece0; pc < chunks; pc += 2 * piece_step) {  // two loads in flight before their stores
            bf16x8 v0, v1;
#pragma unroll
            for (int e = 0; e < 8; ++e) { v0[e] = (bf16)0.f; v1[e] = (bf16)0.f; }
            const bool two = pc + piece_step < chunks;
            if (row_cur >= 0) {
                v0 = *(const bf16x8*)(src + (pc << 3));
                if (two) v1 = *(const bf16x8*)(src + ((pc + piece_step) << 3));
            }
            put(pc << 3, v0);
            if (two) put((pc + piece_step) << 3, v1);
        }
        if (tid < 32) kflag[key] = row_cur == -1;
        row_cur = row_next;
        __syncthreads();
      }
        if (blk0 + 31 < wave_lo || blk0 > wave_hi) continue;        // nothing here for this wave's rows

        f32x4 s[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
            s[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
            const bf16* kr = Ks + (tt * 16 + c) * ks_ld + g4 * 8;
#pragma unroll
            for (int k = 0; k < KQ; ++k)
                if (k < kq) s[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8*)(kr + k * 32), qf[k], s[tt], 0, 0, 0);
        }
        float mx = -INFINITY;
        bool ok[2][4];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = g4 * 8 + tt * 4 + i, j = blk0 + key;
                ok[tt][i] = row_ok && j >= my_lo && j <= my_p;
                const float v = ok[tt][i] ? (kflag[key] ? NAN : s[tt][i] * scale) : -INFINITY;
                s[tt][i] = v;
                mx = fmaxf(mx, v);
            }
        mx = rows4_max(mx);
        const float m_new = fmaxf(m_run, mx);
        const float alpha = (m_run == -INFINITY) ? 0.f : __expf(m_run - m_new);
        float sum = 0.f;
        bf16x8 pf;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = ok[tt][i] ? __expf(s[tt][i] - m_new) : 0.f;
                sum += e;
                pf[tt * 4 + i] = (bf16)e;
            }
        sum = rows4_sum(sum);
        l_run = l_run * alpha + sum;
        m_run = m_new;
#pragma unroll
        for (int a = 0; a < NV; ++a) {
            if (a < nv) {
                o[a] = o[a] * alpha;
                o[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8*)(Vt + (a * 16 + c) * LM_VT_LD + g4 * 8), pf, o[a], 0, 0, 0);
            }
        }
    }
    if (!row_ok) return;
    // o[a][i] of lane (c, g4) is O[row c][a*16 + g4*4 + i]
    if (n_splits > 1) {
        float* rec = part + ((size_t)row * n_splits + blockIdx.y) * (R + 2);
#pragma unroll
        for (int a = 0; a < NV; ++a) {
            const int col = a * 16 + g4 * 4;
            if (a < nv && col < R) {
#pragma unroll
                for (int i = 0; i < 4; ++i) rec[col + i] = o[a][i];
            }
        }
        if (g4 == 0) { rec[R] = m_run; rec[R + 1] = l_run; }
        return;
    }
    const float inv = 1.0f / fmaxf(l_run, 1e-30f);
    bf16* orow = out + (size_t)row * R;
#pragma unroll
    for (int a = 0; a < NV; ++a) {
        const int col = a * 16 + g4 * 4;
        if (a < nv && col < R) {
            bf16x4 w;
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = (bf16)(o[a][i] * inv);
            *(bf16x4*)(orow + col) = w;
        }
    }
}

// Joins the records [row][split][R + 2] of a split call: one workgroup a query row.
__global__ __launch_bounds__(256)
void attn_latent_join_kernel(const float* __restrict__ part, bf16* __restrict__ out, int R, int n_splits) {
    __shared__ float wsh[1024];          // weight of every split: exp(m_s - M) / L
    __shared__ float red[8];
    const size_t row = blockIdx.x;
    const float* rec = part + row * n_splits * (R + 2);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // the first 1024 splits' maxima and sums, four a thread
    float ms[4], ls[4], M = -INFINITY;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int s = tid + u * 256;
        ms[u] = s < n_splits ? rec[(size_t)s * (R + 2) + R] : -INFINITY;
        ls[u] = s < n_splits ? rec[(size_t)s * (R + 2) + R + 1] : 0.f;
        M = fmaxf(M, ms[u]);
    }
    M = wave_max(M);
    if (lane == 0) red[wave] = M;
    __syncthreads();
    M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float L = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int s = tid + u * 256;
        const float w = ms[u] == -INFINITY ? 0.f : __expf(ms[u] - M);
        if (s < n_splits) wsh[s] = w;
        L += w * ls[u];
    }
    L = wave_sum(L);
    if (lane == 0) red[4 + wave] = L;
    __syncthreads();
    const float inv = 1.0f / fmaxf(red[4] + red[5] + red[6] + red[7], 1e-30f);
    for (int c = tid; c < R; c += 256) {
        float acc = 0.f;
        for (int s = 0; s < n_splits; ++s) {
            const float w = wsh[s];
            if (w != 0.f) acc += w * rec[(size_t)s * (R + 2) + c];
        }
        out[row * R + c] = (bf16)(acc * inv);
    }
}

// `wg`: int32 pairs (first query row, rows <= 128) on the device, `n_wg` of them, each within one
// request's rows of the step; `max_rows`: the most rows of any pair (it sizes the workgroups).
// `n_splits` > 1: the keys of every pair are dealt to that many workgroups; `part` (fp32,
// rows * n_splits * (R + 2) floats, rows = T * H) holds their records.
extern "C" int spite_attn_latent_mfma(const void* q, const void* kv_pages, void* out, const int* positions,
                                      const int* seq_of_token, const int* block_table, int max_blocks, const int* wg,
                                      int n_wg, int max_rows, int H, int Dk, int R, int page_size, int vis, int span,
                                      float scale, float* part, int n_splits, int n_rows, hipStream_t st) {
    SP_REQUIRE(H > 0 && n_wg >= 0 && max_rows >= 0 && max_rows <= LM_ROWS, "latent attention: %d rows a workgroup, at most %d", max_rows, LM_ROWS);
    SP_REQUIRE(Dk > 0 && Dk % 8 == 0 && R > 0 && R % 8 == 0 && R <= Dk && Dk <= 576 && R <= 512,
               "latent attention (MFMA): rows of %d with a latent of %d: multiples of 8, at most 576 and 512", Dk, R);
    SP_REQUIRE(page_size > 0 && max_blocks > 0, "latent attention: bad page size %d or table width %d", page_size, max_blocks);
    SP_REQUIRE(vis >= 0 && vis < SP_VIS_COUNT && (!sp_vis_has_span(vis) || span > 0), "latent attention: chunk or window of %d", span);
    SP_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)kv_pages & 15) == 0 && ((uintptr_t)out & 7) == 0, "latent attention: operands must be 16-byte aligned");
    SP_REQUIRE(n_splits >= 1 && n_splits <= 1024 && (n_splits == 1 || part), "latent attention: %d splits", n_splits);
    if (n_wg == 0 || max_rows == 0) return 0;
    const int kq = (Dk + 31) / 32, nv = (R + 15) / 16;
    // a wave for every 16 query rows, and enough waves that staging a block of 32 keys takes a thread
    // no more than about four 16-byte pieces (waves without rows only stage)
    int nw = (max_rows + 15) / 16;
    const int pre = kq <= 6 ? 4 : (kq <= 10 ? 8 : LM_PRE);
    const int fetch_waves = (Dk / 8 + 2 * pre - 1) / (2 * pre);         // staging waves (see the kernel)
    if (nw + fetch_waves <= 8) nw += fetch_waves;
    else {
        const int stage_waves = (32 * (Dk / 8) + 255) / 256;
        if (nw < stage_waves) nw = stage_waves < 8 ? stage_waves : 8;
    }
    const size_t sh = ((size_t)32 * (kq * 32 + 8) + (size_t)nv * 16 * LM_VT_LD) * sizeof(bf16) + (32 + LM_KROW_BLOCKS * 32) * sizeof(int);
#define SP_LM(KQV, NVV) do { \
        auto kern = attn_latent_mfma_kernel<KQV, NVV>; \
        static bool allowed = false; \
        if (sh > 48 * 1024 && !allowed) { hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh); \
            if (e != hipSuccess) return sp_fail("latent attention: %zu bytes of LDS refused: %s", sh, hipGetErrorString(e)); allowed = true; } \
        kern<<<dim3(n_wg, n_splits), nw * 64, sh, st>>>((const bf16*)q, (const bf16*)kv_pages, (bf16*)out, positions, seq_of_token, \
                                        block_table, max_blocks, wg, H, Dk, R, page_size, vis, span, scale, part, n_splits); } while (0)
    if (kq <= 6 && nv <= 8) SP_LM(6, 8);
    else if (kq <= 10 && nv <= 16) SP_LM(10, 16);
    else SP_LM(18, 32);
#undef SP_LM
    SP_LAUNCH_CHECK("attn_latent_mfma");
    if (n_splits > 1) {
        attn_latent_join_kernel<<<n_rows, 256, 0, st>>>(part, (bf16*)out, R, n_splits);
        SP_LAUNCH_CHECK("attn_latent_join");
    }
    return 0;
}
