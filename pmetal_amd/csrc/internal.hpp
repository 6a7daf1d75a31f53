// Internal declarations shared by the translation units of libpmetal_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace pmh {

constexpr uint32_t kTypeQ8_0 = 8, kTypeQ2K = 10, kTypeQ3K = 11, kTypeQ4K = 12, kTypeQ5K = 13, kTypeQ6K = 14, kTypeQ8K = 15;
constexpr uint32_t kOrderRef = 0, kOrderGgml = 1;
constexpr uint32_t kDtypeF32 = 0, kDtypeBf16 = 1;

// ---- codec.hip: bit-exact quantize / dequantize (compiled without fp contraction) ----
hipError_t launch_quantize_q8_0(const float *x, size_t n, uint8_t *dst, hipStream_t s);
hipError_t launch_quantize_legacy32(uint32_t type, const float *x, size_t n, uint8_t *dst, hipStream_t s);
hipError_t launch_dequantize_legacy32(uint32_t type, const uint8_t *src, size_t n, float *dst, hipStream_t s);
hipError_t launch_quantize_q4k(const float *x, size_t n, uint8_t *dst, hipStream_t s);
hipError_t launch_quantize_q5k(const float *x, size_t n, uint8_t *dst, hipStream_t s);
hipError_t launch_quantize_q2k(const float *x, size_t n, uint8_t *dst, hipStream_t s);
hipError_t launch_quantize_q3k(const float *x, size_t n, uint8_t *dst, hipStream_t s);
hipError_t launch_quantize_q6k(const float *x, size_t n, uint8_t *dst, hipStream_t s);
hipError_t launch_dequantize_q8_0(const uint8_t *src, size_t n, float *dst, hipStream_t s);
hipError_t launch_dequantize_q4k(const uint8_t *src, size_t n, float *dst, uint32_t order, hipStream_t s);
hipError_t launch_dequantize_q5k(const uint8_t *src, size_t n, float *dst, uint32_t order, hipStream_t s);
hipError_t launch_dequantize_q2k(const uint8_t *src, size_t n, float *dst, hipStream_t s);
hipError_t launch_dequantize_q3k(const uint8_t *src, size_t n, float *dst, hipStream_t s);
hipError_t launch_dequantize_q6k(const uint8_t *src, size_t n, float *dst, hipStream_t s);

// ---- gemv.hip: dequant-fused y = W x ----
hipError_t launch_qgemv(uint32_t type, const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype,
                        float *y, uint32_t order, hipStream_t s);

// ---- gemv_q4k.hip ----
constexpr int kMaxGemvGroup = 4;

// gemv_q5k.hip: the Q5_K GEMV (every shape with k a multiple of 256 that fits; hipErrorInvalidValue otherwise)
hipError_t launch_qgemv_q5k(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y, uint32_t order,
                            hipStream_t s);
// gemv_q23k.hip: the Q2_K and Q3_K GEMVs (every shape with k a multiple of 256 that fits; hipErrorInvalidValue otherwise)
hipError_t launch_qgemv_q2k(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y, hipStream_t s);
hipError_t launch_qgemv_q3k(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y, hipStream_t s);
// gemv_q6k.hip: the row-staging integer-dot kernel for large Q6_K matrices; false when the shape does not suit it
bool try_launch_qgemv_q6k_chunk(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y,
                                hipStream_t s, hipError_t *err);
// gemv_q8_0.hip: the row-staging integer-dot kernel for large Q8_0 matrices; false when the shape does not suit it
bool try_launch_qgemv_q8_0_chunk(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y,
                                 hipStream_t s, hipError_t *err);
hipError_t launch_qgemv_q4k(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y,
                            uint32_t order, hipStream_t s);
// Several small Q4_K matrices with the same k, x, x_dtype and order in one launch (count <= kMaxGemvGroup);
// launch_qgemv_q4k_pair: two large matrices (not groupable) that share k, x and the element order in one launch of the
// large-matrix kernel; hipErrorNotSupported when the pair does not suit it.
hipError_t launch_qgemv_q4k_pair(const uint8_t *w0, int64_t n0, float *y0, const uint8_t *w1, int64_t n1, float *y1, int64_t k,
                                 const void *x, uint32_t x_dtype, uint32_t order, hipStream_t s);
// qgemv_q4k_groupable tells whether a matrix is small enough to go into a group.
bool qgemv_q4k_groupable(int64_t n, int64_t k);
hipError_t launch_qgemv_q4k_q6k_group(const uint8_t *const *w, const int64_t *n, float *const *y, int count, const uint8_t *w6, int64_t n6,
                                      float *y6, int64_t k, const void *x, uint32_t x_dtype, uint32_t order, hipStream_t s);
hipError_t launch_qgemv_q4k_group(const uint8_t *const *w, const int64_t *n, float *const *y, int count, int64_t k,
                                  const void *x, uint32_t x_dtype, uint32_t order, hipStream_t s);

// ---- gemm.hip: dequant-fused Y = X W^T for Q4_K and Q6_K (every wave owns 32 weight rows) ----
struct GemmPlan {
    int mb;      // 32-row activation blocks per workgroup (1, 2 or 4)
    int mp;      // activation rows padded to a multiple of 32 mb
    int nw;      // waves per workgroup
    int splits;  // workgroups along K (more than one: partial tiles plus a reduction kernel)
    int chunk;   // super-blocks per split
};
bool qgemm_fits(uint32_t type, int64_t m, int64_t n, int64_t k);
// (the padded row count mp does not depend on the type; the K split does)
GemmPlan qgemm_plan(int64_t m, int64_t n, int64_t k, uint32_t type = kTypeQ4K);
// Bytes of device workspace qgemm needs for a weight of `type` at (m, n, k); the caller provides it.
size_t qgemm_workspace_bytes(uint32_t type, int64_t m, int64_t n, int64_t k);
// reuse_prepass: the workspace still holds the converted activations of the previous launch_qgemm on this stream with the same
// x, m, k and weight type (two weights that share their activations: the pre-pass runs once)
hipError_t launch_qgemm(uint32_t type, const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype,
                        int64_t m, void *y, uint32_t y_dtype, uint32_t order, void *workspace, hipStream_t s,
                        bool reuse_prepass = false);

// ---- q8k.hip: Q8_K activation blocks and the integer dot products over them ----
hipError_t launch_quantize_q8k(const float *x, size_t n, uint8_t *dst, hipStream_t s);
hipError_t launch_dequantize_q8k(const uint8_t *src, size_t n, float *dst, hipStream_t s);
// four f64 sums per workgroup (sum (a-b)^2, sum a^2, sum a b, sum b^2) into partial[4 * kl_sums_workgroups(n)]
int kl_sums_workgroups(size_t n);
hipError_t launch_kl_sums(const float *a, const float *b, size_t n, double *partial, hipStream_t s);
// the same sums between `original` and the first n elements decoded from k-quant blocks (never stored), into
// Exact re-blocking of Q5_K / Q3_K / Q2_K super-blocks into Q6_K ones (210 bytes each): W = A (+ B for the formats with
// mins).  reblock_q6k_parts: 2, 1, 2; 0 for any other type.  dst_b is not touched when there is one part.
int reblock_q6k_parts(uint32_t type);
hipError_t launch_reblock_q6k(uint32_t type, const uint8_t *src, size_t n_blocks, uint32_t order, uint8_t *dst_a, uint8_t *dst_b,
                              hipStream_t s);
// y[i] = a[i] + b[i], stored as f32 or bf16
hipError_t launch_add_store(const float *a, const float *b, size_t n, void *y, bool y_bf16, hipStream_t s);
// partial[4 * kl_sums_quantized_workgroups(n)]; hipErrorInvalidValue for a type that is not a k-quant
int kl_sums_quantized_workgroups(size_t n);
hipError_t launch_kl_sums_quantized(uint32_t type, const uint8_t *src, const float *original, size_t n, uint32_t order, double *partial,
                                    hipStream_t s);
// k a multiple of 256 and at most 32768 (the activation blocks live in LDS); type Q4_K or Q6_K
hipError_t launch_qgemv_q8k(uint32_t type, const uint8_t *w, int64_t n, int64_t k, const uint8_t *xq, float *y, hipStream_t s);

// ---- util.hip ----
hipError_t launch_fill_normal(float *dst, size_t n, uint64_t seed, float std, float outlier_rate,
                              float outlier_mag, hipStream_t s);
hipError_t launch_f32_to_bf16(const float *src, uint16_t *dst, size_t n, hipStream_t s);
hipError_t launch_zero_bytes(uint8_t *dst, size_t bytes, hipStream_t s);
hipError_t launch_mfma_probe(int iters, int vary, int workgroups, float *sink, hipStream_t s);
hipError_t launch_read_probe(const void *src, size_t bytes, uint32_t *sink, hipStream_t s);

}  // namespace pmh
