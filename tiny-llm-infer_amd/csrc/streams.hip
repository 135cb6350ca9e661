// Several copies of the residual stream side by side (hyper-connections), and the token shift.
//
// The residual is float32 [rows][S][n].  A sublayer that read u = sum_s in[s] x_s and gave y is
// written back as x_t <- sum_s mix[s][t] x_s + out[t] y, every stream from the old ones.
//
// streams_open:  x[r][s][:] = e[r][:] for every s.
// streams_norm:  one workgroup a row: (1) if a sublayer's y is still owed, the streams are
//                rewritten as above; (2) u = sum_s in[s] x_s of the new streams; (3)
//                h = w * u / sqrt(mean(u^2) + eps).  With a list of rows only those are computed
//                and the streams are left as they are (the last norm of a step, with in = 1: the
//                streams' sum).  All arithmetic is float32; u is kept in LDS between the passes.
//                With a shift (steps of one row a sequence): h is mixed with the sequence's
//                kept row and replaces it, as token_shift does.
// token_shift:   out[r] = h[r] + (prev - h[r]) * mu, prev the row before of the same sequence:
//                in this step, or the kept row of the sequence's slot (nothing at position 0).
//                The workgroup of a sequence's first row, having read the kept row, replaces it
//                by the sequence's last row of this step: each element is read and written by
//                the same thread.
#include "common.h"

#define ST_MAX_STREAMS 8
#define ST_MAX_WIDTH 15360          // a row of u in LDS: 60 KiB

__global__ void streams_open_kernel(const float* __restrict__ e, float* __restrict__ x, int n, int S) {
    const size_t row = blockIdx.x;
    if (n % 4 == 0 && !(((uintptr_t)e | (uintptr_t)x) & 15)) {
        for (int i = threadIdx.x * 4; i < n; i += blockDim.x * 4) {
            const float4 v = *reinterpret_cast<const float4*>(e + row * n + i);
            for (int s = 0; s < S; ++s) *reinterpret_cast<float4*>(x + (row * S + s) * n + i) = v;
        }
        return;
    }
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = e[row * n + i];
        for (int s = 0; s < S; ++s) x[(row * S + s) * n + i] = v;
    }
}

extern "C" int tli_streams_open(const float* e, float* x, int rows, int n, int streams, void* stream) {
    if (rows <= 0) return 0;
    if (n <= 0 || streams <= 0) return tli_fail("streams_open: bad sizes n=%d streams=%d", n, streams);
    streams_open_kernel<<<rows, 256, 0, (hipStream_t)stream>>>(e, x, n, streams);
    return tli_check_launch("streams_open");
}

struct ShiftArgs {
    const float* mu;          // null: no shift
    float* kept;              // [slots][n]
    const int* slots;         // [seqs]
    const int* seq_start;     // [seqs]
    const int* seq_of_row;    // [rows]
};

template <typename TD, typename TO, int S>
__global__ void streams_norm_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                    const float* __restrict__ mix, const float* __restrict__ out_w,
                                    const float* __restrict__ in_w, const float* __restrict__ weight,
                                    TO* __restrict__ out, const int* __restrict__ rows, int n, float eps,
                                    int total_rows, ShiftArgs sh, const float* __restrict__ sums, int parts) {
    extern __shared__ float u_s[];
    __shared__ float scratch[16];
    const int out_row = blockIdx.x;
    int r = rows ? rows[out_row] : out_row;
    if (r < 0 || r >= total_rows) r = 0;
    float* x = resid + (size_t)r * S * n;
    const bool owed = delta != nullptr || parts > 0;
    const bool update = owed && rows == nullptr;
    const size_t plane = (size_t)total_rows * n;             // of the partial sums [parts][total_rows][n]
    const float* sum_row = parts > 0 ? sums + (size_t)r * n : nullptr;
    float m[S][S], o[S], a[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
        a[s] = in_w[s];
        o[s] = owed ? out_w[s] : 0.f;
#pragma unroll
        for (int t = 0; t < S; ++t) m[s][t] = owed ? mix[s * S + t] : 0.f;
    }
    const TD* y_row = delta ? delta + (size_t)r * n : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float xs[S];
#pragma unroll
        for (int s = 0; s < S; ++s) xs[s] = x[(size_t)s * n + i];
        if (owed) {
            float y;
            if (parts > 0) {
                float a = 0.f;
                for (int k = 0; k < parts; ++k) a += sum_row[(size_t)k * plane + i];
                y = bf16_to_f32(f32_to_bf16(a));              // as the product's own reduction would have stored it
            } else {
                y = to_f32(y_row[i]);
            }
            float xn[S];
#pragma unroll
            for (int t = 0; t < S; ++t) {
                float acc = 0.f;
#pragma unroll
                for (int s = 0; s < S; ++s) acc += m[s][t] * xs[s];
                xn[t] = acc + o[t] * y;
            }
#pragma unroll
            for (int t = 0; t < S; ++t) {
                xs[t] = xn[t];
                if (update) x[(size_t)t * n + i] = xn[t];
            }
        }
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < S; ++s) u += a[s] * xs[s];
        u_s[i] = u;
        ss += u * u;
    }
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)n + eps);
    TO* dst = out + (size_t)out_row * n;
    if (sh.mu == nullptr) {
        for (int i = threadIdx.x; i < n; i += blockDim.x) from_f32(dst + i, weight[i] * u_s[i] * scale);
        return;
    }
    const int seq = sh.seq_of_row[r];
    float* kept = sh.kept + (size_t)sh.slots[seq] * n;
    const bool fresh = sh.seq_start[seq] <= 0;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float h = weight[i] * u_s[i] * scale;
        const float prev = fresh ? 0.f : kept[i];
        kept[i] = h;
        from_f32(dst + i, h + (prev - h) * sh.mu[i]);
    }
}


// four consecutive elements at once (16-byte aligned float rows, 8-byte aligned bfloat16 rows)
__device__ __forceinline__ void st_load4(const float* p, float v[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void st_load4(const bf16_t* p, float v[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xFFFF0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xFFFF0000u);
}
__device__ __forceinline__ void st_store4(float* p, const float v[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void st_store4(bf16_t* p, const float v[4]) {
    *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
}

// The same, four elements a thread and turn (n % 4 == 0, every row 16-byte aligned).
template <typename TD, typename TO, int S>
__global__ void streams_norm_vec_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                        const float* __restrict__ mix, const float* __restrict__ out_w,
                                        const float* __restrict__ in_w, const float* __restrict__ weight,
                                        TO* __restrict__ out, const int* __restrict__ rows, int n, float eps,
                                        int total_rows, ShiftArgs sh, const float* __restrict__ sums, int parts) {
    extern __shared__ __align__(16) float u_s[];
    __shared__ float scratch[16];
    const int out_row = blockIdx.x;
    int r = rows ? rows[out_row] : out_row;
    if (r < 0 || r >= total_rows) r = 0;
    float* x = resid + (size_t)r * S * n;
    const bool owed = delta != nullptr || parts > 0;
    const bool update = owed && rows == nullptr;
    const size_t plane = (size_t)total_rows * n;             // of the partial sums [parts][total_rows][n]
    const float* sum_row = parts > 0 ? sums + (size_t)r * n : nullptr;
    float m[S][S], o[S], a[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
        a[s] = in_w[s];
        o[s] = owed ? out_w[s] : 0.f;
#pragma unroll
        for (int t = 0; t < S; ++t) m[s][t] = owed ? mix[s * S + t] : 0.f;
    }
    const TD* y_row = delta ? delta + (size_t)r * n : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x * 4; i < n; i += blockDim.x * 4) {
        float xs[S][4];
#pragma unroll
        for (int s = 0; s < S; ++s) st_load4(x + (size_t)s * n + i, xs[s]);
        if (owed) {
            float y[4], xn[S][4];
            if (parts > 0) {
                float a[4] = {0.f, 0.f, 0.f, 0.f};
                for (int k = 0; k < parts; ++k) {
                    float pv[4];
                    st_load4(sum_row + (size_t)k * plane + i, pv);
#pragma unroll
                    for (int e = 0; e < 4; ++e) a[e] += pv[e];
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) y[e] = bf16_to_f32(f32_to_bf16(a[e]));      // as the product's own reduction would have stored it
            } else {
                st_load4(y_row + i, y);
            }
#pragma unroll
            for (int t = 0; t < S; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float acc = 0.f;
#pragma unroll
                    for (int s = 0; s < S; ++s) acc += m[s][t] * xs[s][e];
                    xn[t][e] = acc + o[t] * y[e];
                }
#pragma unroll
            for (int t = 0; t < S; ++t) {
#pragma unroll
                for (int e = 0; e < 4; ++e) xs[t][e] = xn[t][e];
                if (update) st_store4(x + (size_t)t * n + i, xn[t]);
            }
        }
        float u[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            u[e] = 0.f;
#pragma unroll
            for (int s = 0; s < S; ++s) u[e] += a[s] * xs[s][e];
            ss += u[e] * u[e];
        }
        st_store4(u_s + i, u);
    }
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)n + eps);
    TO* dst = out + (size_t)out_row * n;
    const bool shift = sh.mu != nullptr;
    float* kept = nullptr;
    bool fresh = true;
    if (shift) {
        const int seq = sh.seq_of_row[r];
        kept = sh.kept + (size_t)sh.slots[seq] * n;
        fresh = sh.seq_start[seq] <= 0;
    }
    for (int i = threadIdx.x * 4; i < n; i += blockDim.x * 4) {
        float u[4], w[4], h[4];
        st_load4(u_s + i, u);
        st_load4(weight + i, w);
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = w[e] * u[e] * scale;
        if (shift) {
            float prev[4] = {0.f, 0.f, 0.f, 0.f}, mu[4];
            if (!fresh) st_load4(kept + i, prev);
            st_load4(sh.mu + i, mu);
            st_store4(kept + i, h);
#pragma unroll
            for (int e = 0; e < 4; ++e) h[e] = h[e] + (prev[e] - h[e]) * mu[e];
        }
        st_store4(dst + i, h);
    }
}

template <typename TD, typename TO, int S>
static void launch_streams_norm_s(float* resid, const void* delta, const float* mix, const float* out_w, const float* in_w,
                                  const float* weight, void* out, const int* rows, int out_rows, int total_rows, int n,
                                  float eps, ShiftArgs sh, const float* sums, int parts, hipStream_t s) {
    const bool aligned = !(((uintptr_t)resid | (uintptr_t)delta | (uintptr_t)weight | (uintptr_t)out | (uintptr_t)sh.mu |
                            (uintptr_t)sh.kept | (uintptr_t)sums) & 15);
    if (n % 4 == 0 && aligned) {
        const int groups = n / 4;
        const int threads = groups >= 512 ? 512 : (groups + 63) / 64 * 64;
        streams_norm_vec_kernel<TD, TO, S><<<out_rows, threads, (size_t)n * sizeof(float), s>>>(
            resid, (const TD*)delta, mix, out_w, in_w, weight, (TO*)out, rows, n, eps, total_rows, sh, sums, parts);
        return;
    }
    const int threads = n >= 2048 ? 512 : 256;
    streams_norm_kernel<TD, TO, S><<<out_rows, threads, (size_t)n * sizeof(float), s>>>(
        resid, (const TD*)delta, mix, out_w, in_w, weight, (TO*)out, rows, n, eps, total_rows, sh, sums, parts);
}

template <typename TD, typename TO>
static int launch_streams_norm(int S, float* resid, const void* delta, const float* mix, const float* out_w,
                               const float* in_w, const float* weight, void* out, const int* rows, int out_rows,
                               int total_rows, int n, float eps, ShiftArgs sh, const float* sums, int parts, hipStream_t s) {
#define ST_CASE(N) case N: launch_streams_norm_s<TD, TO, N>(resid, delta, mix, out_w, in_w, weight, out, rows, out_rows, total_rows, n, eps, sh, sums, parts, s); break;
    switch (S) {
        ST_CASE(1) ST_CASE(2) ST_CASE(3) ST_CASE(4) ST_CASE(5) ST_CASE(6) ST_CASE(7) ST_CASE(8)
        default: return tli_fail("streams_norm: %d streams, at most %d", S, ST_MAX_STREAMS);
    }
#undef ST_CASE
    return 0;
}

// delta_dtype: of the owed rows y [total_rows][n] (ignored without them); out_dtype: of the normed rows.
// parts > 0: the owed rows come as float32 partial sums `delta` [parts][total_rows][n] of a product whose k range
// was split (bfloat16 runs): they are added in order and rounded to bfloat16.
// mu != null: the shift for steps of one row a sequence (rows must be null).
extern "C" int tli_streams_norm(float* resid, const void* delta, const float* mix, const float* out_w,
                                const float* in_w, const float* weight, void* out, const int* rows, int out_rows,
                                int total_rows, int n, int streams, float eps, int delta_dtype, int out_dtype,
                                const float* mu, float* kept, const int* slots, const int* seq_start,
                                const int* seq_of_row, int parts, void* stream) {
    if (out_rows <= 0) return 0;
    if (n <= 0 || n > ST_MAX_WIDTH) return tli_fail("streams_norm: row size %d is outside 1..%d", n, ST_MAX_WIDTH);
    if ((delta || parts > 0) && (!mix || !out_w)) return tli_fail("streams_norm: owed rows need their mix and out weights");
    if (mu && (rows || !kept || !slots || !seq_start || !seq_of_row))
        return tli_fail("streams_norm: the shift takes every row of a step and the sequences' slots");
    if (parts < 0 || (parts > 0 && (!delta || delta_dtype != TLI_BF16)))
        return tli_fail("streams_norm: partial sums (%d) go with bfloat16 rows only", parts);
    const float* sums = parts > 0 ? (const float*)delta : nullptr;
    if (parts > 0) delta = nullptr;
    if (!delta) delta_dtype = out_dtype == TLI_F32 ? TLI_F32 : TLI_BF16;
    const ShiftArgs sh{mu, kept, slots, seq_start, seq_of_row};
    hipStream_t s = (hipStream_t)stream;
    int rc;
    if (delta_dtype == TLI_F32 && out_dtype == TLI_F32)
        rc = launch_streams_norm<float, float>(streams, resid, delta, mix, out_w, in_w, weight, out, rows, out_rows, total_rows, n, eps, sh, sums, parts, s);
    else if (delta_dtype == TLI_BF16 && out_dtype == TLI_BF16)
        rc = launch_streams_norm<bf16_t, bf16_t>(streams, resid, delta, mix, out_w, in_w, weight, out, rows, out_rows, total_rows, n, eps, sh, sums, parts, s);
    else if (delta_dtype == TLI_BF16 && out_dtype == TLI_F32)
        rc = launch_streams_norm<bf16_t, float>(streams, resid, delta, mix, out_w, in_w, weight, out, rows, out_rows, total_rows, n, eps, sh, sums, parts, s);
    else
        return tli_fail("streams_norm: owed rows of dtype %d with normed rows of dtype %d", delta_dtype, out_dtype);
    if (rc) return rc;
    return tli_check_launch("streams_norm");
}

template <typename TO>
__global__ void token_shift_kernel(const float* __restrict__ h, const float* __restrict__ mu, float* __restrict__ kept,
                                   TO* __restrict__ out, const int* __restrict__ seq_of_row,
                                   const int* __restrict__ row_start, const int* __restrict__ seq_start,
                                   const int* __restrict__ slots, int n) {
    const int r = blockIdx.x;
    const int seq = seq_of_row[r];
    const int first = row_start[seq], last = row_start[seq + 1] - 1;
    const float* cur = h + (size_t)r * n;
    TO* dst = out + (size_t)r * n;
    if (r > first) {
        const float* before = h + (size_t)(r - 1) * n;
        if (n % 4 == 0 && !(((uintptr_t)h | (uintptr_t)mu | (uintptr_t)out) & 15)) {
            for (int i = threadIdx.x * 4; i < n; i += blockDim.x * 4) {
                float c[4], b[4], w[4];
                st_load4(cur + i, c);
                st_load4(before + i, b);
                st_load4(mu + i, w);
#pragma unroll
                for (int e = 0; e < 4; ++e) c[e] = c[e] + (b[e] - c[e]) * w[e];
                st_store4(dst + i, c);
            }
            return;
        }
        for (int i = threadIdx.x; i < n; i += blockDim.x) from_f32(dst + i, cur[i] + (before[i] - cur[i]) * mu[i]);
        return;
    }
    float* k = kept + (size_t)slots[seq] * n;
    const float* end = h + (size_t)last * n;
    const bool fresh = seq_start[seq] <= 0;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float prev = fresh ? 0.f : k[i];
        k[i] = end[i];
        from_f32(dst + i, cur[i] + (prev - cur[i]) * mu[i]);
    }
}

extern "C" int tli_token_shift(const float* h, const float* mu, float* kept, void* out, const int* seq_of_row,
                               const int* row_start, const int* seq_start, const int* slots, int rows, int n,
                               int out_dtype, void* stream) {
    if (rows <= 0) return 0;
    if (n <= 0) return tli_fail("token_shift: bad row size %d", n);
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == TLI_F32)
        token_shift_kernel<float><<<rows, 256, 0, s>>>(h, mu, kept, (float*)out, seq_of_row, row_start, seq_start, slots, n);
    else if (out_dtype == TLI_BF16)
        token_shift_kernel<bf16_t><<<rows, 256, 0, s>>>(h, mu, kept, (bf16_t*)out, seq_of_row, row_start, seq_start, slots, n);
    else
        return tli_fail("token_shift: unknown dtype %d", out_dtype);
    return tli_check_launch("token_shift");
}
