// Attention with a temperature and a log-distance penalty a head, over a window or the row's own block
// of positions, values from the key cache: the matrix-core kernel for bfloat16 heads whose size is a
// multiple of 16.  It serves portions of prompts and single decoded rows alike.
//
// One wave takes 16 consecutive rows of one sequence (a "tile", counted from the first row that the
// sequence has in this step) and one head; the four waves of a workgroup take four heads next to each
// other, which read the same keys where they share a kv head.  Keys are walked 16 at a time from the
// first one that the tile's first row sees to the tile's last row, each (row, key) pair masked on its own,
// so a tile may lie across the edge of a block of positions.
//
// Transposed throughout, so that a row's numbers stay in the lanes of one column (lane % 16):
//   S^T [16 keys x 16 rows]  = K [16 keys x d] . Q^T            A: a key's 4 dims of a lane group, 8 bytes from the cache
//                                                               B: a row's 4 dims, 8 bytes of q
//   s = S^T * scale * temp - r1 * ln(1 + r2 * (row position - key position)), float32
//   weights with a running maximum a row; maxima and sums go over the four lane groups of a column
//   O^T [d x 16 rows]       += V^T [16 d x 16 keys] . P^T       A: 4 keys of one dim (2-byte loads: the cache keeps
//                                                               a key's dims together); B: the weights as they lie
// Lane l of a 16x16x16 tile holds, of A, row l % 16 and k = 4 * (l / 16) .. + 3, of B, column l % 16 and the
// same k, of the result, column l % 16 and rows 4 * (l / 16) .. + 3.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) short bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

union Frag4 {
    uint2 u;
    bf16_t e[4];
    bf16x4 v;
};

#define ABM_WAVES 4

__device__ __forceinline__ int abm_first_visible(int pos, int mask_kind, int mask_size) {
    if (mask_kind == 1) return max(0, pos - mask_size + 1);
    if (mask_kind == 2) return pos - pos % mask_size;
    return 0;
}

// ND = head_dim / 16.  values: null (the values are the keys) or the value cache [page][kv head][d][slot].
template <int ND>
__global__ __launch_bounds__(64 * ABM_WAVES) void attention_biased_mfma_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ row_start, const int* __restrict__ seq_start,
    int num_seqs, const int* __restrict__ tables, int table_width, int page_size, int num_pages, int heads,
    int kv_heads, float scale, const float* __restrict__ temp, const float* __restrict__ r1,
    const float* __restrict__ r2, int mask_kind, int mask_size) {
    constexpr int D = ND * 16;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int col = lane % 16, grp = lane / 16;
    const int head = blockIdx.y * ABM_WAVES + wave;
    if (head >= heads) return;
    // which sequence and which of its tiles
    int tile = blockIdx.x, seq = 0, first_row = 0, count = 0;
    for (; seq < num_seqs; ++seq) {
        first_row = row_start[seq];
        count = row_start[seq + 1] - first_row;
        const int nt = (count + 15) / 16;
        if (tile < nt) break;
        tile -= nt;
    }
    if (seq >= num_seqs) return;
    const int g = head / (heads / kv_heads);
    const int* table = tables + (size_t)seq * table_width;
    const int live = min(16, count - tile * 16);                        // rows of this tile
    const int row0 = first_row + tile * 16;
    const int pos0 = seq_start[seq] + tile * 16;
    const int my = min(col, live - 1);                                  // (idle columns repeat the last row; never stored)
    const int qpos = pos0 + my;
    const int qlo = abm_first_visible(qpos, mask_kind, mask_size);
    const int lo = abm_first_visible(pos0, mask_kind, mask_size), hi = pos0 + live - 1;
    const float mul = scale * (temp ? temp[head] : 1.0f);
    const float pen1 = r1 ? r1[head] : 0.f, pen2 = r1 ? r2[head] : 0.f;
    const size_t page_stride = (size_t)kv_heads * page_size * D;

    Frag4 qf[ND];
    const bf16_t* q_row = q + ((size_t)(row0 + my) * heads + head) * D;
#pragma unroll
    for (int j = 0; j < ND; ++j) qf[j].u = *reinterpret_cast<const uint2*>(q_row + j * 16 + grp * 4);

    f32x4 acc[ND];
#pragma unroll
    for (int j = 0; j < ND; ++j) acc[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    for (int k0 = lo - lo % 16; k0 <= hi; k0 += 16) {
        // A of the scores: key k0 + col, this lane group's dims
        const int ka = k0 + col;
        const bf16_t* kp = nullptr;
        if (ka >= lo && ka <= hi) {
            const int page = table[ka / page_size];
            if (page >= 0 && page < num_pages)
                kp = k_cache + (size_t)page * page_stride + ((size_t)g * page_size + ka % page_size) * D + grp * 4;
        }
        f32x4 s = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < ND; ++j) {
            Frag4 a;
            a.u = kp ? *reinterpret_cast<const uint2*>(kp + j * 16) : make_uint2(0, 0);
            s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, qf[j].v, s, 0, 0, 0);
        }
        // this lane: keys k0 + 4 grp + i of column col
        float w[4];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = k0 + grp * 4 + i;
            float v = s[i] * mul;
            if (r1) v -= pen1 * log1pf(pen2 * (float)(qpos - key));
            w[i] = (key >= qlo && key <= qpos) ? v : -INFINITY;
            mx = fmaxf(mx, w[i]);
        }
        mx = quad_rows_max(mx);
        const float m_new = fmaxf(m, mx);
        // (a column whose keys so far are all hidden keeps m = -inf: its weights and its correction are 0)
        const float corr = (m_new == -INFINITY) ? 0.f : __expf(m - m_new);
        float sum = 0.f;
        Frag4 p;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float e = (w[i] == -INFINITY) ? 0.f : __expf(w[i] - m_new);
            p.e[i] = f32_to_bf16(e);
            sum += bf16_to_f32(p.e[i]);                 // the weights as the values meet them
        }
        l = l * corr + quad_rows_sum(sum);
        m = m_new;
        // A of the output: dim 16 j + col of the keys k0 + 4 grp + i
        const bf16_t* vp[4];
        size_t vstep;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = k0 + grp * 4 + i;
            vp[i] = nullptr;
            if (key >= lo && key <= hi) {
                const int page = table[key / page_size];
                if (page >= 0 && page < num_pages) {
                    if (v_cache) vp[i] = v_cache + (size_t)page * page_stride + (size_t)g * page_size * D + (size_t)col * page_size + key % page_size;
                    else vp[i] = k_cache + (size_t)page * page_stride + ((size_t)g * page_size + key % page_size) * D + col;
                }
            }
        }
        vstep = v_cache ? (size_t)16 * page_size : 16;
#pragma unroll
        for (int j = 0; j < ND; ++j) {
            Frag4 a;
#pragma unroll
            for (int i = 0; i < 4; ++i) a.e[i] = vp[i] ? vp[i][j * vstep] : (bf16_t)0;
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[j][i] *= corr;
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, p.v, acc[j], 0, 0, 0);
        }
    }
    if (col >= live) return;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    bf16_t* o_row = out + ((size_t)(row0 + col) * heads + head) * D;
#pragma unroll
    for (int j = 0; j < ND; ++j) {
        uint2 st;
        st.x = pack_bf16x2(acc[j][0] * inv, acc[j][1] * inv);
        st.y = pack_bf16x2(acc[j][2] * inv, acc[j][3] * inv);
        *reinterpret_cast<uint2*>(o_row + j * 16 + grp * 4) = st;
    }
}

// tiles: an upper bound of sum over the sequences of ceil(rows / 16) (workgroups past the last tile leave at once)
extern "C" int tli_attention_biased_mfma_bf16(
    const void* q, void* out, const void* k_cache, const void* v_cache, const int* row_start, const int* seq_start,
    int num_seqs, int tiles, const int* tables, int table_width, int page_size, int num_pages, int heads, int kv_heads,
    int head_dim, float scale, const float* temp, const float* r1, const float* r2, int mask_kind, int mask_size,
    void* stream) {
    if (num_seqs <= 0 || tiles <= 0) return 0;
    if (head_dim % 16 || head_dim < 16 || head_dim > 256)
        return tli_fail("attention: the matrix-core kernel takes heads of 16 to 256 in steps of 16, not %d", head_dim);
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads)
        return tli_fail("attention: heads %d must be a multiple of kv heads %d", heads, kv_heads);
    if (page_size <= 0 || table_width <= 0 || num_pages <= 0) return tli_fail("attention: bad cache geometry");
    if (mask_kind < 0 || mask_kind > 2 || (mask_kind && mask_size <= 0)) return tli_fail("attention: bad mask %d of %d", mask_kind, mask_size);
    if ((r1 == nullptr) != (r2 == nullptr)) return tli_fail("attention: the distance penalty needs both of its numbers");
    if ((((uintptr_t)q | (uintptr_t)out | (uintptr_t)k_cache) & 7)) return tli_fail("attention: operands must be 8-byte aligned");
    const dim3 grid(tiles, (heads + ABM_WAVES - 1) / ABM_WAVES);
    hipStream_t s = (hipStream_t)stream;
#define ABM_CASE(N) case N: attention_biased_mfma_kernel<N><<<grid, 64 * ABM_WAVES, 0, s>>>( \
        (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)k_cache, (const bf16_t*)v_cache, row_start, seq_start, num_seqs, \
        tables, table_width, page_size, num_pages, heads, kv_heads, scale, temp, r1, r2, mask_kind, mask_size); break;
    switch (head_dim / 16) {
        ABM_CASE(1) ABM_CASE(2) ABM_CASE(3) ABM_CASE(4) ABM_CASE(5) ABM_CASE(6) ABM_CASE(7) ABM_CASE(8)
        ABM_CASE(9) ABM_CASE(10) ABM_CASE(11) ABM_CASE(12) ABM_CASE(13) ABM_CASE(14) ABM_CASE(15) ABM_CASE(16)
    }
#undef ABM_CASE
    return tli_check_launch("attention_biased_mfma");
}
