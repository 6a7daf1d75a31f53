// Small utility kernels: zero fill, f32 -> bf16, synthetic normal tensors for benchmarks, and a probe of the
// matrix-core rate the machine sustains.
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

// Register-only loop of v_mfma_f32_32x32x16_f16: 8 waves per workgroup (two per SIMD), four independent
// accumulators per wave, no memory traffic.  With `vary` the operands differ per lane and one register of an operand changes
// sign after every four matrix instructions (one v_xor with a compile-time register index: the loop body is eight such
// groups written out, so nothing is selected at run time); without it they are all 1.0.  `iters` counts groups of four
// matrix instructions and is rounded down to a multiple of eight.
typedef _Float16 probe_half8 __attribute__((ext_vector_type(8)));
typedef float probe_float16 __attribute__((ext_vector_type(16)));
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(512) void k_mfma_probe(int iters, int vary, float *__restrict__ sink) {
    probe_half8 a, b;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = (_Float16)(vary ? (float)((threadIdx.x * 37 + i * 11) % 97) * 0.37f - 17.0f : 1.0f);
        b[i] = (_Float16)(vary ? (float)((threadIdx.x * 13 + i * 7) % 89) * 0.21f - 9.0f : 1.0f);
    }
    const uint32_t flip = vary ? 0x80008000u : 0u;  // the sign bits of the two halves of a register
    probe_float16 c0, c1, c2, c3;
#pragma unroll
    for (int i = 0; i < 16; i++) c0[i] = 0.0f, c1[i] = 0.0f, c2[i] = 0.0f, c3[i] = 0.0f;
    for (int i = 0; i < iters / 8; i++) {
#pragma unroll
        for (int g = 0; g < 8; g++) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c3, 0, 0, 0);
            probe_u32x4 &bits = reinterpret_cast<probe_u32x4 &>((g & 1) ? b : a);
            bits[g >> 1] ^= flip;
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) s += c0[i] + c1[i] + c2[i] + c3[i];
    if (s == 1.2345f) sink[0] = s;  // keeps the loop alive; practically never true
}

// Plain streaming read: every thread loads 16 bytes per step of a grid-wide sweep and folds them into a value that is
// (practically) never stored.  The time of this kernel over n bytes is what the memory system of the machine allows a
// single launch that does nothing but read them.
__global__ __launch_bounds__(256) void k_read_probe(const uint4 *__restrict__ p, size_t n16, uint32_t *__restrict__ sink) {
    const size_t stride = (size_t)gridDim.x * 256;
    uint32_t acc = 0;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) {
        const uint4 v = p[i];
        acc += v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x12345678u) sink[0] = acc;
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

hipError_t launch_read_probe(const void *src, size_t bytes, uint32_t *sink, hipStream_t s) {
    const size_t n16 = bytes / 16;
    if (n16 == 0) return hipSuccess;
    size_t grid = (n16 + 255) / 256;
    if (grid > 2048) grid = 2048;  // eight workgroups per compute unit: the fastest sweep for tensors of tens of MB
    hipLaunchKernelGGL(k_read_probe, dim3((unsigned)grid), dim3(256), 0, s, reinterpret_cast<const uint4 *>(src), n16, sink);
    return hipGetLastError();
}

hipError_t launch_mfma_probe(int iters, int vary, int workgroups, float *sink, hipStream_t s) {
    hipLaunchKernelGGL(k_mfma_probe, dim3((unsigned)workgroups), dim3(512), 0, s, iters, vary, sink);
    return hipGetLastError();
}

}  // namespace pmh
