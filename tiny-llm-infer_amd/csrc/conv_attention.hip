// Attention whose queries and keys pass a short causal convolution over time and whose values are its
// keys: the plain kernels (any sizes, float32 or bfloat16 storage, float32 arithmetic).
//
// conv_heads:   the raw projections qk [rows][C] (C = q_dim + kv_dim, q first) get their bias and are
//               mixed over time, channel by channel:
//                   y[p][c] = sum_j w[j][c] * (qk[p - taps + 1 + j][c] + b[c]),   nothing before position 0
//               (w is kept tap by tap, [taps][C], so that neighbouring channels' weights lie together).
//               Rows before the step's first row of the sequence come from the sequence's kept rows
//               (state [slots][taps - 1][C], raw projections, oldest first).  The q channels go to
//               q_out [rows][q_dim], the k channels into the paged cache [page][kv head][slot][d].
// conv_keep:    afterwards, the last taps - 1 raw rows of every sequence replace its kept rows (one
//               thread a channel moves them oldest first, so that it reads nothing it has written).
// attention_biased_plain: one workgroup per (row, head).  Row at position p, head a, kv head g:
//                   s_t = (q_a . K_t,g) * scale * temp_a - r1_a * ln(1 + r2_a * (p - t))      t = lo..p
//                   out_a = sum_t softmax(s)_t V_t,g
//               lo = 0, p - size + 1 (window) or p - p % size (chunk).  The values are read from the
//               value cache [page][kv head][d][slot] or, without one, are the keys themselves.
#include "common.h"

#define CA_THREADS 256
#define CA_MAX_HEAD_DIM 512
#define CA_MAX_TAPS 64

// KEEP: every sequence has one row in this step, and the thread that mixed a channel also moves the
// sequence's kept rows of that channel up by one and puts the new row last (conv_keep's work).
template <typename T, bool KEEP>
__global__ void conv_heads_kernel(const T* __restrict__ qk, const float* __restrict__ bias,
                                  const float* __restrict__ conv_w, T* __restrict__ state,
                                  T* __restrict__ q_out, T* __restrict__ k_cache,
                                  const int* __restrict__ positions, const int* __restrict__ seq_of_row,
                                  const int* __restrict__ row_start, const int* __restrict__ slots,
                                  const int* __restrict__ tables, int table_width, int page_size, int num_pages,
                                  int C, int q_dim, int kv_heads, int head_dim, int taps) {
    const int r = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int pos = positions[r];
    const int seq = seq_of_row[r];
    const int first = row_start[seq];
    T* kept = state ? state + (size_t)slots[seq] * (taps - 1) * C : nullptr;
    const float b = bias ? bias[c] : 0.f;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j;
        if (pos - back < 0) continue;
        const int src = r - back;
        float u;
        if (src >= first) u = to_f32(qk[(size_t)src * C + c]);
        else u = to_f32(kept[(size_t)(taps - 1 + src - first) * C + c]);
        acc += conv_w[(size_t)j * C + c] * (u + b);
    }
    if (KEEP && kept) {
        for (int i = 0; i + 2 < taps; ++i) kept[(size_t)i * C + c] = kept[(size_t)(i + 1) * C + c];
        kept[(size_t)(taps - 2) * C + c] = qk[(size_t)r * C + c];
    }
    if (c < q_dim) {
        from_f32(q_out + (size_t)r * q_dim + c, acc);
        return;
    }
    const int kc = c - q_dim, g = kc / head_dim, d = kc % head_dim;
    const int page = tables[(size_t)seq * table_width + pos / page_size];
    if (page < 0 || page >= num_pages) return;
    T v;
    from_f32(&v, acc);
    k_cache[(size_t)page * kv_heads * page_size * head_dim + ((size_t)g * page_size + pos % page_size) * head_dim + d] =
        cache_value(v);
}


// The same for bfloat16 with eight channels a thread (16-byte loads and stores): head_dim % 8 == 0.
template <bool KEEP>
__global__ void conv_heads_vec_kernel(const bf16_t* __restrict__ qk, const float* __restrict__ bias,
                                      const float* __restrict__ conv_w, bf16_t* __restrict__ state,
                                      bf16_t* __restrict__ q_out, bf16_t* __restrict__ k_cache,
                                      const int* __restrict__ positions, const int* __restrict__ seq_of_row,
                                      const int* __restrict__ row_start, const int* __restrict__ slots,
                                      const int* __restrict__ tables, int table_width, int page_size, int num_pages,
                                      int C, int q_dim, int kv_heads, int head_dim, int taps) {
    const int r = blockIdx.x;
    const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
    if (c >= C) return;
    const int pos = positions[r];
    const int seq = seq_of_row[r];
    const int first = row_start[seq];
    bf16_t* kept = state ? state + (size_t)slots[seq] * (taps - 1) * C : nullptr;
    float b[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (bias) {
        const float4 b0 = *reinterpret_cast<const float4*>(bias + c), b1 = *reinterpret_cast<const float4*>(bias + c + 4);
        b[0] = b0.x; b[1] = b0.y; b[2] = b0.z; b[3] = b0.w; b[4] = b1.x; b[5] = b1.y; b[6] = b1.z; b[7] = b1.w;
    }
    uint4 newest = make_uint4(0, 0, 0, 0);
    for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j;
        if (pos - back < 0) continue;
        const int src = r - back;
        const uint4 v = src >= first ? *reinterpret_cast<const uint4*>(qk + (size_t)src * C + c)
                                     : *reinterpret_cast<const uint4*>(kept + (size_t)(taps - 1 + src - first) * C + c);
        if (back == 0) newest = v;
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        const float4 t0 = *reinterpret_cast<const float4*>(conv_w + (size_t)j * C + c);
        const float4 t1 = *reinterpret_cast<const float4*>(conv_w + (size_t)j * C + c + 4);
        const float t[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            acc[2 * e] += t[2 * e] * (__uint_as_float(w[e] << 16) + b[2 * e]);
            acc[2 * e + 1] += t[2 * e + 1] * (__uint_as_float(w[e] & 0xFFFF0000u) + b[2 * e + 1]);
        }
    }
    if (KEEP && kept) {
        for (int i = 0; i + 2 < taps; ++i)
            *reinterpret_cast<uint4*>(kept + (size_t)i * C + c) = *reinterpret_cast<const uint4*>(kept + (size_t)(i + 1) * C + c);
        *reinterpret_cast<uint4*>(kept + (size_t)(taps - 2) * C + c) = newest;
    }
    uint32_t o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const bf16_t lo = cache_value(f32_to_bf16(acc[2 * e])), hi = cache_value(f32_to_bf16(acc[2 * e + 1]));
        o[e] = (uint32_t)lo | ((uint32_t)hi << 16);
    }
    const uint4 y = make_uint4(o[0], o[1], o[2], o[3]);
    if (c < q_dim) {
        *reinterpret_cast<uint4*>(q_out + (size_t)r * q_dim + c) = y;
        return;
    }
    const int kc = c - q_dim, g = kc / head_dim, d = kc % head_dim;
    const int page = tables[(size_t)seq * table_width + pos / page_size];
    if (page < 0 || page >= num_pages) return;
    *reinterpret_cast<uint4*>(k_cache + (size_t)page * kv_heads * page_size * head_dim +
                              ((size_t)g * page_size + pos % page_size) * head_dim + d) = y;
}

template <typename T>
__global__ void conv_keep_kernel(const T* __restrict__ qk, T* __restrict__ state, const int* __restrict__ row_start,
                                 const int* __restrict__ slots, int C, int taps) {
    const int seq = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int first = row_start[seq], n = row_start[seq + 1] - first;
    T* kept = state + (size_t)slots[seq] * (taps - 1) * C;
    for (int i = 0; i < taps - 1; ++i) {
        const int src = n - (taps - 1) + i;          // row of this step that becomes kept row i
        kept[(size_t)i * C + c] = src >= 0 ? qk[(size_t)(first + src) * C + c] : kept[(size_t)(i + n) * C + c];
    }
}

extern "C" int tli_conv_heads(const void* qk, const float* bias, const float* conv_w, void* state, void* q_out,
                              void* k_cache, const int* positions, const int* seq_of_row, const int* row_start,
                              const int* slots, int rows, int seqs, const int* tables, int table_width,
                              int page_size, int num_pages, int heads, int kv_heads, int head_dim, int taps,
                              int one_row_each, int dtype, void* stream) {
    if (rows <= 0) return 0;
    if (heads <= 0 || kv_heads <= 0 || head_dim <= 0) return tli_fail("conv_heads: bad head sizes");
    if (taps <= 0 || taps > CA_MAX_TAPS) return tli_fail("conv_heads: %d taps are outside 1..%d", taps, CA_MAX_TAPS);
    if (taps > 1 && !state) return tli_fail("conv_heads: a convolution of %d taps needs the sequences' kept rows", taps);
    if (page_size <= 0 || table_width <= 0 || num_pages <= 0) return tli_fail("conv_heads: bad cache geometry");
    const int q_dim = heads * head_dim, C = q_dim + kv_heads * head_dim;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(rows, (C + CA_THREADS - 1) / CA_THREADS), keep(seqs, (C + CA_THREADS - 1) / CA_THREADS);
    if (one_row_each && rows != seqs) return tli_fail("conv_heads: %d rows of %d sequences are not one row each", rows, seqs);
#define CA_ARGS(T) (const T*)qk, bias, conv_w, (T*)state, (T*)q_out, (T*)k_cache, positions, seq_of_row, row_start, slots, \
        tables, table_width, page_size, num_pages, C, q_dim, kv_heads, head_dim, taps
    if (dtype == TLI_F32) {
        if (one_row_each) conv_heads_kernel<float, true><<<grid, CA_THREADS, 0, s>>>(CA_ARGS(float));
        else {
            conv_heads_kernel<float, false><<<grid, CA_THREADS, 0, s>>>(CA_ARGS(float));
            if (taps > 1) conv_keep_kernel<float><<<keep, CA_THREADS, 0, s>>>((const float*)qk, (float*)state, row_start, slots, C, taps);
        }
    } else if (dtype == TLI_BF16 && head_dim % 8 == 0 &&
               !(((uintptr_t)qk | (uintptr_t)state | (uintptr_t)q_out | (uintptr_t)k_cache | (uintptr_t)bias | (uintptr_t)conv_w) & 15)) {
        const int groups = C / 8, threads = groups >= 256 ? 256 : (groups + 63) / 64 * 64;
        const dim3 vgrid(rows, (groups + threads - 1) / threads);
        if (one_row_each) conv_heads_vec_kernel<true><<<vgrid, threads, 0, s>>>(CA_ARGS(bf16_t));
        else {
            conv_heads_vec_kernel<false><<<vgrid, threads, 0, s>>>(CA_ARGS(bf16_t));
            if (taps > 1) conv_keep_kernel<bf16_t><<<keep, CA_THREADS, 0, s>>>((const bf16_t*)qk, (bf16_t*)state, row_start, slots, C, taps);
        }
    } else if (dtype == TLI_BF16) {
        if (one_row_each) conv_heads_kernel<bf16_t, true><<<grid, CA_THREADS, 0, s>>>(CA_ARGS(bf16_t));
        else {
            conv_heads_kernel<bf16_t, false><<<grid, CA_THREADS, 0, s>>>(CA_ARGS(bf16_t));
            if (taps > 1) conv_keep_kernel<bf16_t><<<keep, CA_THREADS, 0, s>>>((const bf16_t*)qk, (bf16_t*)state, row_start, slots, C, taps);
        }
    } else {
        return tli_fail("conv_heads: unknown dtype %d", dtype);
    }
    return tli_check_launch("conv_heads");
}

// mask_kind: 0 every key up to the row's own, 1 a window of mask_size keys, 2 the row's own block of mask_size positions
__device__ __forceinline__ int first_visible(int pos, int mask_kind, int mask_size) {
    if (mask_kind == 1) return max(0, pos - mask_size + 1);
    if (mask_kind == 2) return pos - pos % mask_size;
    return 0;
}

template <typename T>
__global__ void attention_biased_plain_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ seq_of_row, const int* __restrict__ tables,
    int table_width, int page_size, int num_pages, int heads, int kv_heads, int head_dim, float scale,
    const float* __restrict__ temp, const float* __restrict__ r1, const float* __restrict__ r2,
    int mask_kind, int mask_size) {
    __shared__ float q_s[CA_MAX_HEAD_DIM];
    __shared__ float p_s[CA_THREADS];
    __shared__ float red[16];
    const int row = blockIdx.x, head = blockIdx.y;
    const int tid = threadIdx.x;
    const int g = head / (heads / kv_heads);
    const int pos = positions[row];
    const int seq = seq_of_row[row];
    const int* table = tables + (size_t)seq * table_width;
    const int lo = first_visible(pos, mask_kind, mask_size);
    const size_t page_stride = (size_t)kv_heads * page_size * head_dim;
    const float mul = scale * (temp ? temp[head] : 1.0f);
    const float pen1 = r1 ? r1[head] : 0.f, pen2 = r1 ? r2[head] : 0.f;

    const T* q_row = q + ((size_t)row * heads + head) * head_dim;
    for (int d = tid; d < head_dim; d += CA_THREADS) q_s[d] = to_f32(q_row[d]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc0 = 0.f, acc1 = 0.f;      // output elements tid and tid + 256
    for (int base = lo; base <= pos; base += CA_THREADS) {
        const int t = base + tid;
        float s = -INFINITY;
        if (t <= pos) {
            const int page = table[t / page_size];
            if (page >= 0 && page < num_pages) {
                const T* kp = k_cache + (size_t)page * page_stride + ((size_t)g * page_size + (t % page_size)) * head_dim;
                float dot = 0.f;
                for (int d = 0; d < head_dim; ++d) dot += q_s[d] * to_f32(kp[d]);
                s = dot * mul;
                if (r1) s -= pen1 * log1pf(pen2 * (float)(pos - t));
            }
        }
        const float tile_max = block_max(s, red);
        const float m_new = fmaxf(m, tile_max);
        const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
        const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
        const float tile_sum = block_sum(p, red);
        l = l * corr + tile_sum;
        p_s[tid] = p;
        __syncthreads();
        const int count = min(CA_THREADS, pos - base + 1);
        for (int half = 0; half < 2; ++half) {
            const int d = tid + half * CA_THREADS;
            if (d >= head_dim) break;
            float a = (half == 0 ? acc0 : acc1) * corr;
            for (int j = 0; j < count; ++j) {
                const int tt = base + j;
                const int page = table[tt / page_size];
                if (page < 0 || page >= num_pages) continue;
                float v;
                if (v_cache) v = to_f32(v_cache[(size_t)page * page_stride + (size_t)g * page_size * head_dim + (tt % page_size) + (size_t)d * page_size]);
                else v = to_f32(k_cache[(size_t)page * page_stride + ((size_t)g * page_size + (tt % page_size)) * head_dim + d]);
                a += p_s[j] * v;
            }
            if (half == 0) acc0 = a; else acc1 = a;
        }
        m = m_new;
        __syncthreads();
    }
    T* o_row = out + ((size_t)row * heads + head) * head_dim;
    const float inv = (l > 0.f) ? 1.0f / l : 0.f;
    if (tid < head_dim) from_f32(o_row + tid, acc0 * inv);
    if (tid + CA_THREADS < head_dim) from_f32(o_row + tid + CA_THREADS, acc1 * inv);
}

extern "C" int tli_attention_biased_plain(
    const void* q, void* out, const void* k_cache, const void* v_cache, const int* positions, const int* seq_of_row,
    const int* tables, int table_width, int page_size, int num_pages, int rows, int heads, int kv_heads, int head_dim,
    float scale, const float* temp, const float* r1, const float* r2, int mask_kind, int mask_size, int dtype,
    void* stream) {
    if (rows <= 0) return 0;
    if (head_dim <= 0 || head_dim > CA_MAX_HEAD_DIM)
        return tli_fail("attention: head_dim %d is outside 1..%d", head_dim, CA_MAX_HEAD_DIM);
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads)
        return tli_fail("attention: heads %d must be a multiple of kv heads %d", heads, kv_heads);
    if (heads > 65535) return tli_fail("attention: %d heads exceed the grid limit 65535", heads);
    if (page_size <= 0 || table_width <= 0 || num_pages <= 0) return tli_fail("attention: bad cache geometry");
    if (mask_kind < 0 || mask_kind > 2 || (mask_kind && mask_size <= 0)) return tli_fail("attention: bad mask %d of %d", mask_kind, mask_size);
    if ((r1 == nullptr) != (r2 == nullptr)) return tli_fail("attention: the distance penalty needs both of its numbers");
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(rows, heads);
    if (dtype == TLI_F32)
        attention_biased_plain_kernel<float><<<grid, CA_THREADS, 0, s>>>(
            (const float*)q, (float*)out, (const float*)k_cache, (const float*)v_cache, positions, seq_of_row, tables,
            table_width, page_size, num_pages, heads, kv_heads, head_dim, scale, temp, r1, r2, mask_kind, mask_size);
    else if (dtype == TLI_BF16)
        attention_biased_plain_kernel<bf16_t><<<grid, CA_THREADS, 0, s>>>(
            (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)k_cache, (const bf16_t*)v_cache, positions, seq_of_row, tables,
            table_width, page_size, num_pages, heads, kv_heads, head_dim, scale, temp, r1, r2, mask_kind, mask_size);
    else
        return tli_fail("attention: unknown dtype %d", dtype);
    return tli_check_launch("attention_biased_plain");
}
