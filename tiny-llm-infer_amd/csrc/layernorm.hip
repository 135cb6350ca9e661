// Residual add + layer norm without bias, for one or two weight vectors at once.
//
//   v = resid[r] + (d1[r] + d2[r])          (what the parts before still owe the residual; float32)
//   m = mean(v),  s = mean((v - m)^2)       (two passes: the variance is of the deviations)
//   out_a = (v - m) / sqrt(s + eps) * w_a   for a = 1 (and 2: two norms of the same row share m and s)
//
// With a row list only those rows are computed and the residual is left as it is.
#include "common.h"

template <typename T>
struct Owed {
    const T* d1;
    const T* d2;
    __device__ __forceinline__ bool any() const { return d1 != nullptr || d2 != nullptr; }
    __device__ __forceinline__ float at(int i) const {
        float d = d1 ? to_f32(d1[i]) : 0.f;
        if (d2) d = d1 ? d + to_f32(d2[i]) : to_f32(d2[i]);
        return d;
    }
};

template <typename T>
__global__ void add_layernorm_kernel(float* __restrict__ resid, const T* __restrict__ d1, const T* __restrict__ d2,
                                     const float* __restrict__ w1, const float* __restrict__ w2,
                                     T* __restrict__ out1, T* __restrict__ out2, const int* __restrict__ rows,
                                     int n, float eps, int total_rows) {
    __shared__ float scratch[16];
    const int out_row = blockIdx.x;
    int r = rows ? rows[out_row] : out_row;
    if (r < 0 || r >= total_rows) r = 0;
    float* x = resid + (size_t)r * n;
    const Owed<T> d{d1 ? d1 + (size_t)r * n : nullptr, d2 ? d2 + (size_t)r * n : nullptr};
    const bool update = rows == nullptr && d.any();
    const bool again = d.any() && !update;           // the sum is not stored: every pass makes it anew
    float sum = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = x[i];
        if (d.any()) v += d.at(i);
        if (update) x[i] = v;
        sum += v;
    }
    const float mean = block_sum(sum, scratch) / (float)n;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = x[i];
        if (again) v += d.at(i);
        ss += (v - mean) * (v - mean);
    }
    const float scale = 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
    T* o1 = out1 + (size_t)out_row * n;
    T* o2 = out2 ? out2 + (size_t)out_row * n : nullptr;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = x[i];
        if (again) v += d.at(i);
        const float z = (v - mean) * scale;
        from_f32(o1 + i, z * w1[i]);
        if (o2) from_f32(o2 + i, z * w2[i]);
    }
}

// The row in registers: n % 4 == 0 and n <= 4 * IT * blockDim.x, everything 16-byte aligned.
__device__ __forceinline__ void ln_load4(const float* p, float v[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void ln_load4(const bf16_t* p, float v[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = bf16_to_f32((bf16_t)(t.x & 0xffffu)); v[1] = bf16_to_f32((bf16_t)(t.x >> 16));
    v[2] = bf16_to_f32((bf16_t)(t.y & 0xffffu)); v[3] = bf16_to_f32((bf16_t)(t.y >> 16));
}
__device__ __forceinline__ void ln_store4(float* p, const float v[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void ln_store4(bf16_t* p, const float v[4]) {
    *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
}

template <typename T, int IT>
__global__ void add_layernorm_vec_kernel(float* __restrict__ resid, const T* __restrict__ d1, const T* __restrict__ d2,
                                         const float* __restrict__ w1, const float* __restrict__ w2,
                                         T* __restrict__ out1, T* __restrict__ out2, const int* __restrict__ rows,
                                         int n, float eps, int total_rows) {
    __shared__ float scratch[16];
    const int out_row = blockIdx.x;
    int r = rows ? rows[out_row] : out_row;
    if (r < 0 || r >= total_rows) r = 0;
    float* x = resid + (size_t)r * n;
    const bool update = rows == nullptr && (d1 || d2);
    float v[IT][4];
    float sum = 0.f;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int i = (threadIdx.x + it * blockDim.x) * 4;
        if (i < n) {
            ln_load4(x + i, v[it]);
            float a[4], b[4];
            if (d1) ln_load4(d1 + (size_t)r * n + i, a);
            if (d2) ln_load4(d2 + (size_t)r * n + i, b);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (d1 && d2) v[it][e] += a[e] + b[e];
                else if (d1) v[it][e] += a[e];
                else if (d2) v[it][e] += b[e];
                sum += v[it][e];
            }
            if (update) ln_store4(x + i, v[it]);
        }
    }
    const float mean = block_sum(sum, scratch) / (float)n;
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int i = (threadIdx.x + it * blockDim.x) * 4;
        if (i < n) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[it][e] -= mean;
                ss += v[it][e] * v[it][e];
            }
        }
    }
    const float scale = 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int i = (threadIdx.x + it * blockDim.x) * 4;
        if (i < n) {
            float w[4], o[4];
            ln_load4(w1 + i, w);
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = v[it][e] * scale * w[e];
            ln_store4(out1 + (size_t)out_row * n + i, o);
            if (out2) {
                ln_load4(w2 + i, w);
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = v[it][e] * scale * w[e];
                ln_store4(out2 + (size_t)out_row * n + i, o);
            }
        }
    }
}

template <typename T>
static void launch_add_layernorm(float* resid, const void* d1, const void* d2, const float* w1, const float* w2,
                                 void* out1, void* out2, const int* rows, int out_rows, int total_rows, int n,
                                 float eps, hipStream_t s) {
    const uintptr_t all = (uintptr_t)resid | (uintptr_t)d1 | (uintptr_t)d2 | (uintptr_t)w1 | (uintptr_t)w2 |
                          (uintptr_t)out1 | (uintptr_t)out2;
    if (n % 4 == 0 && !(all & 15) && n <= 4 * 4 * 1024) {
        const int quads = n / 4;
        int threads = 64;
        while (threads < 1024 && threads * 2 <= quads) threads *= 2;      // at least one quad a thread
        const int it = (quads + threads - 1) / threads;
#define TLI_LN(IT) hipLaunchKernelGGL((add_layernorm_vec_kernel<T, IT>), dim3(out_rows), dim3(threads), 0, s, resid, \
                                      (const T*)d1, (const T*)d2, w1, w2, (T*)out1, (T*)out2, rows, n, eps, total_rows)
        if (it <= 1) TLI_LN(1);
        else if (it == 2) TLI_LN(2);
        else if (it == 3) TLI_LN(3);
        else TLI_LN(4);
#undef TLI_LN
        return;
    }
    hipLaunchKernelGGL((add_layernorm_kernel<T>), dim3(out_rows), dim3(256), 0, s, resid, (const T*)d1, (const T*)d2,
                       w1, w2, (T*)out1, (T*)out2, rows, n, eps, total_rows);
}

extern "C" int tli_add_layernorm(float* resid, const void* d1, const void* d2, const float* w1, const float* w2,
                                 void* out1, void* out2, const int* rows, int out_rows, int total_rows, int n,
                                 float eps, int dtype, void* stream) {
    if (out_rows <= 0) return 0;
    if (n <= 0) return tli_fail("add_layernorm: bad row size %d", n);
    if (!w1 || !out1 || (out2 && !w2)) return tli_fail("add_layernorm: an output without its weight");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TLI_F32)
        launch_add_layernorm<float>(resid, d1, d2, w1, w2, out1, out2, rows, out_rows, total_rows, n, eps, s);
    else if (dtype == TLI_BF16)
        launch_add_layernorm<bf16_t>(resid, d1, d2, w1, w2, out1, out2, rows, out_rows, total_rows, n, eps, s);
    else
        return tli_fail("add_layernorm: unknown dtype %d", dtype);
    return tli_check_launch("add_layernorm");
}
