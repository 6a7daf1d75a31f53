// Small utility kernels: zero fill, f32 -> bf16, synthetic normal tensors for benchmarks.
#include "internal.hpp"

namespace {

__global__ __launch_bounds__(256) void k_zero_bytes(uint8_t *dst, size_t bytes) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < bytes) dst[i] = 0;
}

__device__ __forceinline__ uint16_t bf16_rne(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

__global__ __launch_bounds__(256) void k_f32_to_bf16(const float *__restrict__ src, uint16_t *__restrict__ dst,
                                                      size_t n) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = bf16_rne(src[i]);
}

__device__ __forceinline__ uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

// Two normals per counter (Box-Muller); element i depends only on (seed, i).
__global__ __launch_bounds__(256) void k_fill_normal(float *__restrict__ dst, size_t n, uint64_t seed, float std,
                                                      float outlier_rate, float outlier_mag) {
    const size_t stride = (size_t)gridDim.x * 256;
    const size_t n_pairs = (n + 1) / 2;
    for (size_t p = (size_t)blockIdx.x * 256 + threadIdx.x; p < n_pairs; p += stride) {
        const uint64_t r = splitmix64(seed * 0xD1342543DE82EF95ull + p);
        const float u1 = ((float)(uint32_t)(r >> 40) + 1.0f) * (1.0f / 16777216.0f);  // (0, 1]
        const float u2 = (float)(uint32_t)((r >> 8) & 0xFFFFFFu) * (1.0f / 16777216.0f);
        const float rad = std * __builtin_sqrtf(-2.0f * __logf(u1));
        float s, c;
        __sincosf(6.28318530718f * u2, &s, &c);
        float v0 = rad * c, v1 = rad * s;
        if (outlier_rate > 0.0f) {
            const uint64_t o = splitmix64(r);
            const float o0 = (float)(uint32_t)(o & 0xFFFFFFu) * (1.0f / 16777216.0f);
            const float o1 = (float)(uint32_t)((o >> 24) & 0xFFFFFFu) * (1.0f / 16777216.0f);
            if (o0 < outlier_rate) v0 = (o >> 62 & 1) ? outlier_mag : -outlier_mag;
            if (o1 < outlier_rate) v1 = (o >> 63) ? outlier_mag : -outlier_mag;
        }
        dst[2 * p] = v0;
        if (2 * p + 1 < n) dst[2 * p + 1] = v1;
    }
}

inline unsigned capped_grid(size_t items) {
    size_t g = (items + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

}  // namespace

namespace pmh {

hipError_t launch_zero_bytes(uint8_t *dst, size_t bytes, hipStream_t s) {
    if (bytes == 0) return hipSuccess;
    hipLaunchKernelGGL(k_zero_bytes, dim3((unsigned)((bytes + 255) / 256)), dim3(256), 0, s, dst, bytes);
    return hipGetLastError();
}

hipError_t launch_f32_to_bf16(const float *src, uint16_t *dst, size_t n, hipStream_t s) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_f32_to_bf16, dim3(capped_grid(n)), dim3(256), 0, s, src, dst, n);
    return hipGetLastError();
}

hipError_t launch_fill_normal(float *dst, size_t n, uint64_t seed, float std, float outlier_rate,
                              float outlier_mag, hipStream_t s) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_fill_normal, dim3(capped_grid((n + 1) / 2)), dim3(256), 0, s, dst, n, seed, std,
                       outlier_rate, outlier_mag);
    return hipGetLastError();
}

}  // namespace pmh
