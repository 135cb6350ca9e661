// Attention with a temperature and a log-distance penalty a head, over a window or the row's own block
// of positions, values from the key cache: the matrix-core kernel for bfloat16 heads whose size is a
// multiple of 16.  It serves portions of prompts and single decoded rows alike.
//
// A workgroup of four waves takes 16 consecutive rows of one sequence (a "tile", counted from the first
// row that the sequence has in this step) and one head.  The keys from the first one that the tile's first
// row sees to the tile's last row are walked 16 at a time, the four waves taking every fourth 16 each with
// sums of their own, which are merged through LDS at the end (nearest keys first).  Each (row, key) pair is masked on its own,
// so a tile may lie across the edge of a block of positions.  A wave brings its 16 keys into LDS with
// 16-byte loads (a page lookup a lane and pass) and reads both matrix operands from there.
//
#include "common.h"

typedef __attribute__((ext_vector_type(4))) short bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

union Frag4 {
    uint2 u;
    bf16_t e[4];
    bf16x4 v;
};

#ifndef ABM_WAVES
#define ABM_WAVES 4
#endif
#define ABM_PAD 8          // bfloat16 elements between the rows of a key tile in LDS (16 bytes: rows stay 16-byte aligned
                           // and the four lane groups of a gather fall into different banks)

__device__ __forceinline__ int abm_first_visible(int pos, int mask_kind, int mask_size) {
    if (mask_kind == 1) return max(0, pos - mask_size + 1);
    if (mask_kind == 2) return pos - pos % mask_size;
    return 0;
}

static inline size_t abm_lds_bytes(int D, int CT) {
    const size_t tiles = (size_t)ABM_WAVES * 16 * (D + ABM_PAD) * 2;
    const size_t merge = (size_t)(ABM_WAVES - 1) * CT * (16 * D + 32) * 4;
    return tiles > merge ? tiles : merge;
}

// ND = head_dim / 16; CT: a tile is 16 * CT rows, and each wave keeps CT sets of 16 columns that share the key
// tile's operands.  values: null (the values are the keys) or the value cache [page][kv head][d][slot].
template <int ND, int CT>
__global__ __launch_bounds__(64 * ABM_WAVES) void attention_biased_mfma_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ row_start, const int* __restrict__ seq_start,
    int num_seqs, const int* __restrict__ tables, int table_width, int page_size, int num_pages, int heads,
    int kv_heads, float scale, const float* __restrict__ temp, const float* __restrict__ r1,
    const float* __restrict__ r2, int mask_kind, int mask_size, int grouped) {
    constexpr int D = ND * 16, LD = D + ABM_PAD, CHUNKS = 16 * (D / 8), ROWS = 16 * CT;      // CHUNKS: 16-byte pieces of a key tile
    extern __shared__ __align__(16) unsigned char abm_lds[];
    const int lane = threadIdx.x % 64, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int col = lane % 16, grp = lane / 16;
    // grouped > 0 (steps of single rows): a tile is one row, its columns are the `grouped` query heads that share
    // kv head blockIdx.y, so that a key tile is fetched once for all of them; else blockIdx.y is the query head
    const int per_tile = grouped ? 1 : ROWS;
    // which sequence and which of its tiles
    int tile = blockIdx.x, seq = 0, first_row = 0, count = 0;
    for (; seq < num_seqs; ++seq) {
        first_row = row_start[seq];
        count = row_start[seq + 1] - first_row;
        const int nt = (count + per_tile - 1) / per_tile;
        if (tile < nt) break;
        tile -= nt;
    }
    if (seq >= num_seqs) return;                                        // (the whole workgroup)
    const int head = grouped ? blockIdx.y * grouped + min(col, grouped - 1) : blockIdx.y;     // of this lane's column
    const int g = grouped ? blockIdx.y : head / (heads / kv_heads);
    const int* table = tables + (size_t)seq * table_width;
    const int live = min(per_tile, count - tile * per_tile);            // rows of this tile
    const int row0 = first_row + tile * per_tile;
    const int pos0 = seq_start[seq] + tile * per_tile;
    const int lo = abm_first_visible(pos0, mask_kind, mask_size), hi = pos0 + live - 1;
    const float mul = scale * (temp ? temp[head] : 1.0f);
    const float pen1 = r1 ? r1[head] : 0.f, pen2 = r1 ? r2[head] : 0.f;
    const size_t page_stride = (size_t)kv_heads * page_size * D;
    const int page_shift = __builtin_ctz(page_size), page_mask = page_size - 1;      // (a power of two: the launcher checks)
    const int live_cols = grouped ? grouped : live;                     // columns that are stored

    int qpos[CT], qlo[CT];
    Frag4 qf[CT][ND];
    f32x4 acc[CT][ND];
    float m[CT], l[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int my = min(ct * 16 + col, live - 1);                    // (idle columns repeat the last row; never stored)
        qpos[ct] = pos0 + my;
        qlo[ct] = abm_first_visible(qpos[ct], mask_kind, mask_size);
        const bf16_t* q_row = q + ((size_t)(row0 + my) * heads + head) * D;
#pragma unroll
        for (int j = 0; j < ND; ++j) {
            qf[ct][j].u = *reinterpret_cast<const uint2*>(q_row + j * 16 + grp * 4);
            acc[ct][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
        m[ct] = -INFINITY;
        l[ct] = 0.f;
    }
    bf16_t* kt = reinterpret_cast<bf16_t*>(abm_lds) + (size_t)wave * 16 * LD;     // this wave's key tile [16][LD]

    // A key tile's 16-byte pieces, one a lane and pass: keys outside lo..hi, or without a page, as zeros.  The
    // loads of the next tile are asked for before the current one is worked on.
    constexpr int PASSES = (CHUNKS + 63) / 64;
    uint4 next[PASSES];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            const int c = ps * 64 + lane;
            next[ps] = make_uint4(0, 0, 0, 0);
            if (CHUNKS % 64 == 0 || c < CHUNKS) {
                const int key = k0 + c / (D / 8);
                if (key >= lo && key <= hi) {
                    const int page = table[key >> page_shift];
                    if (page >= 0 && page < num_pages)
                        next[ps] = *reinterpret_cast<const uint4*>(k_cache + (size_t)page * page_stride +
                                                                   ((size_t)g * page_size + (key & page_mask)) * D + (c % (D / 8)) * 8);
                }
            }
        }
    };
    // from the nearest keys to the farthest: with a penalty that grows with the distance the maxima settle in the
    // first tiles, and the accumulators are rarely rescaled after them
    const int k_low = lo - lo % 16, k_first = hi - hi % 16 - 16 * wave;
    if (k_first >= k_low) fetch(k_first);
    for (int k0 = k_first; k0 >= k_low; k0 -= 16 * ABM_WAVES) {
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            const int c = ps * 64 + lane;
            if (CHUNKS % 64 == 0 || c < CHUNKS)
                *reinterpret_cast<uint4*>(kt + (c / (D / 8)) * LD + (c % (D / 8)) * 8) = next[ps];
        }
        if (k0 - 16 * ABM_WAVES >= k_low) fetch(k0 - 16 * ABM_WAVES);
        wave_lds_sync();
        // scores: A = the key k0 + col, this lane group's dims, shared by the sets of columns
        f32x4 s[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) s[ct] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < ND; ++j) {
            Frag4 a;
            a.u = *reinterpret_cast<const uint2*>(kt + col * LD + j * 16 + grp * 4);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
                s[ct] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, qf[ct][j].v, s[ct], 0, 0, 0);
        }
        // this lane: keys k0 + 4 grp + i of column col of every set
        Frag4 p[CT];
        float corr[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            float w[4];
            float mx = -INFINITY;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = k0 + grp * 4 + i;
                float v = s[ct][i] * mul;
                if (r1) v -= pen1 * __logf(1.0f + pen2 * (float)(qpos[ct] - key));
                w[i] = (key >= qlo[ct] && key <= qpos[ct]) ? v : -INFINITY;
                mx = fmaxf(mx, w[i]);
            }
            mx = quad_rows_max(mx);
            const float m_new = fmaxf(m[ct], mx);
            // (a column whose keys so far are all hidden keeps m = -inf: its weights and its correction are 0)
            corr[ct] = (m_new == -INFINITY) ? 0.f : __expf(m[ct] - m_new);
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = (w[i] == -INFINITY) ? 0.f : __expf(w[i] - m_new);
                p[ct].e[i] = f32_to_bf16(e);
                sum += bf16_to_f32(p[ct].e[i]);         // the weights as the values meet them
            }
            l[ct] = l[ct] * corr[ct] + quad_rows_sum(sum);
            m[ct] = m_new;
        }
        bool moved = false;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) moved = moved || corr[ct] != 1.0f;
        const bool rescale = __any(moved);              // (the same for the whole wave)
        // A of the output: dim 16 j + col of the keys k0 + 4 grp + i
        const bf16_t* vp[4] = {nullptr, nullptr, nullptr, nullptr};
        if (v_cache) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = k0 + grp * 4 + i;
                if (key >= lo && key <= hi) {
                    const int page = table[key >> page_shift];
                    if (page >= 0 && page < num_pages)
                        vp[i] = v_cache + (size_t)page * page_stride + (size_t)g * page_size * D + (size_t)col * page_size + (key & page_mask);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < ND; ++j) {
            Frag4 a;
            if (v_cache) {
#pragma unroll
                for (int i = 0; i < 4; ++i) a.e[i] = vp[i] ? vp[i][(size_t)j * 16 * page_size] : (bf16_t)0;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) a.e[i] = kt[(grp * 4 + i) * LD + j * 16 + col];
            }
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                if (rescale) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[ct][j][i] *= corr[ct];
                }
                acc[ct][j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, p[ct].v, acc[ct][j], 0, 0, 0);
            }
        }
        wave_lds_sync();                                // the tile is read before the next one is written over it
    }
    // the four waves' sums into wave 0: each of the others leaves (m, l) a column and its accumulators
    __syncthreads();
    float* merge = reinterpret_cast<float*>(abm_lds);
    constexpr int PER_SET = 16 * D + 32, PER_WAVE = CT * PER_SET;
    if (wave > 0) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            float* mine = merge + (size_t)(wave - 1) * PER_WAVE + ct * PER_SET;
            if (grp == 0) {
                mine[col] = m[ct];
                mine[16 + col] = l[ct];
            }
#pragma unroll
            for (int j = 0; j < ND; ++j)
                *reinterpret_cast<f32x4*>(mine + 32 + ((size_t)j * 64 + lane) * 4) = acc[ct][j];
        }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        if (ct * 16 >= live_cols) break;
        float mt = m[ct];
#pragma unroll
        for (int w = 0; w < ABM_WAVES - 1; ++w) mt = fmaxf(mt, merge[(size_t)w * PER_WAVE + ct * PER_SET + col]);
        const float f0 = (m[ct] == -INFINITY) ? 0.f : __expf(m[ct] - mt);
        float lt = l[ct] * f0;
#pragma unroll
        for (int j = 0; j < ND; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[ct][j][i] *= f0;
#pragma unroll
        for (int w = 0; w < ABM_WAVES - 1; ++w) {
            const float* theirs = merge + (size_t)w * PER_WAVE + ct * PER_SET;
            const float mw = theirs[col];
            const float f = (mw == -INFINITY) ? 0.f : __expf(mw - mt);
            lt += theirs[16 + col] * f;
#pragma unroll
            for (int j = 0; j < ND; ++j) {
                const f32x4 a = *reinterpret_cast<const f32x4*>(theirs + 32 + ((size_t)j * 64 + lane) * 4);
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[ct][j][i] += a[i] * f;
            }
        }
        if (ct * 16 + col >= live_cols) continue;
        const float inv = lt > 0.f ? 1.0f / lt : 0.f;
        bf16_t* o_row = out + ((size_t)(row0 + (grouped ? 0 : ct * 16 + col)) * heads + head) * D;
#pragma unroll
        for (int j = 0; j < ND; ++j) {
            uint2 st;
            st.x = pack_bf16x2(acc[ct][j][0] * inv, acc[ct][j][1] * inv);
            st.y = pack_bf16x2(acc[ct][j][2] * inv, acc[ct][j][3] * inv);
            *reinterpret_cast<uint2*>(o_row + j * 16 + grp * 4) = st;
        }
    }
}

// rows_a_tile: 16 or 32 (heads up to 128 only); tiles: an upper bound of the sum over the sequences of
// ceil(rows / rows_a_tile) (workgroups past the last tile leave at once).  grouped = heads / kv_heads (at most 16):
// a tile is one row with the heads of a kv head as its columns, and tiles counts the rows.
extern "C" int tli_attention_biased_mfma_bf16(
    const void* q, void* out, const void* k_cache, const void* v_cache, const int* row_start, const int* seq_start,
    int num_seqs, int tiles, int rows_a_tile, const int* tables, int table_width, int page_size, int num_pages, int heads,
    int kv_heads, int head_dim, float scale, const float* temp, const float* r1, const float* r2, int mask_kind,
    int mask_size, int grouped, void* stream) {
    if (num_seqs <= 0 || tiles <= 0) return 0;
    if (head_dim % 16 || head_dim < 16 || head_dim > 256)
        return tli_fail("attention: the matrix-core kernel takes heads of 16 to 256 in steps of 16, not %d", head_dim);
    if (rows_a_tile != 16 && !(rows_a_tile == 32 && head_dim <= 128))
        return tli_fail("attention: tiles of %d rows with heads of %d", rows_a_tile, head_dim);
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads)
        return tli_fail("attention: heads %d must be a multiple of kv heads %d", heads, kv_heads);
    if (page_size <= 0 || table_width <= 0 || num_pages <= 0) return tli_fail("attention: bad cache geometry");
    if (page_size & (page_size - 1)) return tli_fail("attention: the matrix-core kernel takes pages of a power of two, not %d", page_size);
    if (mask_kind < 0 || mask_kind > 2 || (mask_kind && mask_size <= 0)) return tli_fail("attention: bad mask %d of %d", mask_kind, mask_size);
    if ((r1 == nullptr) != (r2 == nullptr)) return tli_fail("attention: the distance penalty needs both of its numbers");
    if ((((uintptr_t)q | (uintptr_t)out | (uintptr_t)k_cache) & 15)) return tli_fail("attention: operands must be 16-byte aligned");
    if (heads > 65535) return tli_fail("attention: %d heads exceed the grid limit 65535", heads);
    if (grouped && (grouped != heads / kv_heads || grouped > 16 || rows_a_tile != 16))
        return tli_fail("attention: %d heads a kv head cannot be one tile's columns", grouped);
    const dim3 grid(tiles, grouped ? kv_heads : heads);
    hipStream_t s = (hipStream_t)stream;
    const int ct = rows_a_tile / 16;
#define ABM_ARGS (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)k_cache, (const bf16_t*)v_cache, row_start, seq_start, num_seqs, \
        tables, table_width, page_size, num_pages, heads, kv_heads, scale, temp, r1, r2, mask_kind, mask_size, grouped
#define ABM_CASE(N) case N: attention_biased_mfma_kernel<N, 1><<<grid, 64 * ABM_WAVES, abm_lds_bytes(16 * N, 1), s>>>(ABM_ARGS); break;
#define ABM_CASE2(N) case N: if (ct == 2) attention_biased_mfma_kernel<N, 2><<<grid, 64 * ABM_WAVES, abm_lds_bytes(16 * N, 2), s>>>(ABM_ARGS); \
        else attention_biased_mfma_kernel<N, 1><<<grid, 64 * ABM_WAVES, abm_lds_bytes(16 * N, 1), s>>>(ABM_ARGS); break;
    switch (head_dim / 16) {
        ABM_CASE2(1) ABM_CASE2(2) ABM_CASE2(3) ABM_CASE2(4) ABM_CASE2(5) ABM_CASE2(6) ABM_CASE2(7) ABM_CASE2(8)
        ABM_CASE(9) ABM_CASE(10) ABM_CASE(11) ABM_CASE(12) ABM_CASE(13) ABM_CASE(14) ABM_CASE(15) ABM_CASE(16)
    }
#undef ABM_CASE
#undef ABM_CASE2
#undef ABM_ARGS
    return tli_check_launch("attention_biased_mfma");
}
