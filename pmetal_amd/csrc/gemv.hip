// Dequant-fused GEMV  y[n] = sum_k W[n,k] * x[k]  for Q6_K and Q8_0 weights on gfx950, and the
// dispatch over weight types (Q4_K lives in gemv_q4k.hip).
//
// W is the packed GGUF block stream, row-major [n, k]; the value of a weight is what the
// reference's dequantize yields (k_quants.rs:474-496 for Q6_K, dequant.rs:466-495 for Q8_0).  The
// reference has no fused kernel: it dequantizes on the CPU at load
// (crates/pmetal-models/src/weight_format.rs:299) and multiplies dense; these kernels are checked
// against exactly that (dequantize, then matmul), to 1e-3.
//
//  * A "team" of T lanes walks one weight row at a time; for Q6_K 8 lanes share a 210-byte
//    super-block, for Q8_0 one lane owns a 34-byte block.  Blocks are only 2-byte aligned, so the
//    loads are unaligned dword loads, which the hardware supports.
//  * Q6_K quants are assembled in registers into bf16 pairs: OR-ing the integer q' = q + 32 (shifted
//    by one) into the mantissa of bf16(64.0) gives exactly 64 + q', and one v_dot2c_f32_bf16
//    multiplies two of them with two activations, accumulating in fp32.  The offsets are removed
//    with per-group sums of x computed once.
//  * x is staged once per workgroup in LDS, already permuted into the pair order the unpacking
//    produces, laid out so that consecutive lanes read consecutive 16-byte words.  f32 activations
//    are split exactly into three bf16 planes (hi + mid + lo) and run through the same path thrice.
//  * The team's partial sums are reduced with DPP (quad_perm, row_half_mirror, row_mirror) and, for
//    teams wider than a 16-lane row, ds_bpermute; lane 0 of the team stores y[row].
#include "gemv_q6k_small.hpp"

namespace {

template <int T, bool XF32>
__global__ __launch_bounds__(256) void k_qgemv_q6k(const uint8_t *__restrict__ W, const void *__restrict__ xg,
                                                    float *__restrict__ y, int n_rows, int spr) {
    extern __shared__ uint4 smem[];
    q6k_small_body<T, XF32>(W, xg, y, n_rows, spr, (int)blockIdx.x, (int)gridDim.x, 256 / T, smem);
}

// ------------------------------------------------------------------------------------------------
// Q8_0 (34-byte blocks of 32, 2-byte aligned).  One lane per block; 8-bit quants do not fit the
// bf16 mantissa trick, so each is sign-extended, converted and multiplied in fp32 with x held as f32
// in LDS (at 8.5 bits per weight the VALU budget per byte is twice that of Q4_K).
// LDS: xf[8][blocks] float4 (elements 32b + 4q .. +3).
// ------------------------------------------------------------------------------------------------
template <bool XF32>
__device__ __forceinline__ void stage_x_q8_0(const void *xg, int bpr, float4 *xf) {
    for (int b = threadIdx.x; b < bpr; b += blockDim.x) {
#pragma unroll
        for (int q = 0; q < 8; q++) {
            float4 v;
            if (XF32) {
                v = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(xg) + (size_t)b * 32)[q];
            } else {
                const uint2 u =
                    reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(xg) + (size_t)b * 32)[q];
                v = make_float4(bf16_to_f32(u.x & 0xFFFFu), bf16_to_f32(u.x >> 16), bf16_to_f32(u.y & 0xFFFFu),
                                bf16_to_f32(u.y >> 16));
            }
            xf[q * bpr + b] = v;
        }
    }
}

__device__ __forceinline__ float q8_0_lane(const uint8_t *blk, const float4 *xf, const int bpr, const int b) {
    const float d = f16_bits_to_f32(*reinterpret_cast<const u16_a2 *>(blk));
    const u32x4_a2 qa = *reinterpret_cast<const u32x4_a2 *>(blk + 2);
    const u32x4_a2 qb = *reinterpret_cast<const u32x4_a2 *>(blk + 18);
    const uint32_t w[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
    float acc = 0.0f;
#pragma unroll
    for (int q = 0; q < 8; q++) {
        const float4 xv = xf[q * bpr + b];
        acc += (float)(int8_t)(w[q]) * xv.x;
        acc += (float)(int8_t)(w[q] >> 8) * xv.y;
        acc += (float)(int8_t)(w[q] >> 16) * xv.z;
        acc += (float)(int8_t)(w[q] >> 24) * xv.w;
    }
    return d * acc;
}

template <int T, bool XF32>
__global__ __launch_bounds__(256) void k_qgemv_q8_0(const uint8_t *__restrict__ W, const void *__restrict__ xg,
                                                     float *__restrict__ y, int n_rows, int bpr) {
    extern __shared__ uint4 smem[];
    float4 *xf = reinterpret_cast<float4 *>(smem);
    stage_x_q8_0<XF32>(xg, bpr, xf);
    __syncthreads();

    const int lt = threadIdx.x & (T - 1);
    const int team = blockIdx.x * (256 / T) + threadIdx.x / T;
    const int n_teams = gridDim.x * (256 / T);
    const int iters = bpr / T;
    const size_t row_bytes = (size_t)bpr * 34;

    for (int row = team; row < n_rows; row += 2 * n_teams) {
        const int row1 = row + n_teams;
        const bool has1 = row1 < n_rows;
        const uint8_t *p0 = W + (size_t)row * row_bytes;
        const uint8_t *p1 = W + (size_t)(has1 ? row1 : row) * row_bytes;
        float acc0 = 0.0f, acc1 = 0.0f;
        for (int it = 0; it < iters; it++) {
            const int b = it * T + lt;
            acc0 += q8_0_lane(p0 + (size_t)b * 34, xf, bpr, b);
            acc1 += q8_0_lane(p1 + (size_t)b * 34, xf, bpr, b);
        }
        acc0 = team_sum<T>(acc0);
        acc1 = team_sum<T>(acc1);
        if (lt == 0) {
            y[row] = acc0;
            if (has1) y[row1] = acc1;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
constexpr int rows_per_team() { return 4; }

// Rows per team: rows_per_team() when that still leaves a workgroup for every compute unit, fewer otherwise
// (a small matrix is spread over the whole chip rather than streamed by a few workgroups).
unsigned grid_for_rows(int64_t n, int teams_per_wg, int64_t r = rows_per_team()) {
    const int64_t cus = compute_units();
    while (r > 1 && (n + teams_per_wg * r - 1) / (teams_per_wg * r) < cus) r /= 2;
    const int64_t per_wg = (int64_t)teams_per_wg * r;
    int64_t g = (n + per_wg - 1) / per_wg;
    if (g < 1) g = 1;
    if (g > (1 << 20)) g = 1 << 20;
    return (unsigned)g;
}

template <typename Kern>
hipError_t launch(Kern kern, unsigned grid, size_t lds, hipStream_t s, const uint8_t *w, const void *x, float *y,
                  int n, int units) {
    if (lds > kMaxLds) return hipErrorInvalidValue;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, s, w, x, y, n, units);
    return hipGetLastError();
}

template <bool XF32>
hipError_t launch_q6k(int team, unsigned grid, size_t lds, hipStream_t s, const uint8_t *w, const void *x, float *y,
                      int n, int spr) {
    switch (team) {
    case 8: return launch(k_qgemv_q6k<8, XF32>, grid, lds, s, w, x, y, n, spr);
    case 16: return launch(k_qgemv_q6k<16, XF32>, grid, lds, s, w, x, y, n, spr);
    case 32: return launch(k_qgemv_q6k<32, XF32>, grid, lds, s, w, x, y, n, spr);
    default: return launch(k_qgemv_q6k<64, XF32>, grid, lds, s, w, x, y, n, spr);
    }
}

template <bool XF32>
hipError_t launch_q8_0(int team, unsigned grid, size_t lds, hipStream_t s, const uint8_t *w, const void *x,
                       float *y, int n, int bpr) {
    switch (team) {
    case 1: return launch(k_qgemv_q8_0<1, XF32>, grid, lds, s, w, x, y, n, bpr);
    case 2: return launch(k_qgemv_q8_0<2, XF32>, grid, lds, s, w, x, y, n, bpr);
    case 4: return launch(k_qgemv_q8_0<4, XF32>, grid, lds, s, w, x, y, n, bpr);
    case 8: return launch(k_qgemv_q8_0<8, XF32>, grid, lds, s, w, x, y, n, bpr);
    case 16: return launch(k_qgemv_q8_0<16, XF32>, grid, lds, s, w, x, y, n, bpr);
    case 32: return launch(k_qgemv_q8_0<32, XF32>, grid, lds, s, w, x, y, n, bpr);
    default: return launch(k_qgemv_q8_0<64, XF32>, grid, lds, s, w, x, y, n, bpr);
    }
}

}  // namespace

namespace pmh {

// Preconditions (checked by the C ABI layer): n > 0, k > 0 a multiple of the block size, n and
// k / block below 2^31, pointers 16-byte aligned, type/order/x_dtype valid.  Returns
// hipErrorInvalidValue when the staged activations do not fit the 160 KiB of LDS.
hipError_t launch_qgemv(uint32_t type, const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype,
                        float *y, uint32_t order, hipStream_t s) {
    const bool xf32 = x_dtype == kDtypeF32;
    const int planes = xf32 ? 3 : 1;
    if (type == kTypeQ4K) return launch_qgemv_q4k(w, n, k, x, x_dtype, y, order, s);
    if (type == kTypeQ5K) return launch_qgemv_q5k(w, n, k, x, x_dtype, y, order, s);
    if (type == kTypeQ2K) return launch_qgemv_q2k(w, n, k, x, x_dtype, y, s);
    if (type == kTypeQ3K) return launch_qgemv_q3k(w, n, k, x, x_dtype, y, s);
    if (type == kTypeQ6K) {
        hipError_t chunk_err = hipSuccess;
        if (try_launch_qgemv_q6k_chunk(w, n, k, x, x_dtype, y, s, &chunk_err)) return chunk_err;
        const int spr = (int)(k / 256);
        const int team = 8 * pow2_divisor(spr, 8);
        const size_t slots = (size_t)spr * 8;
        const size_t lds = slots * 64 * planes + slots * 16;
        // A very tall matrix (an output projection) takes more rows per team, so fewer workgroups
        // each convert x: 151936 x 1024 runs 39.1 us with 4 rows per team, 37.5 with 8, 36.6 with
        // 16 and 40.3 with 32.  The Q8_0 kernel below is fastest at 4.
        const unsigned grid = grid_for_rows(n, 256 / team, n >= 65536 ? 16 : rows_per_team());
        return xf32 ? launch_q6k<true>(team, grid, lds, s, w, x, y, (int)n, spr)
                    : launch_q6k<false>(team, grid, lds, s, w, x, y, (int)n, spr);
    }
    if (type == kTypeQ8_0) {
        hipError_t chunk_err = hipSuccess;
        if (try_launch_qgemv_q8_0_chunk(w, n, k, x, x_dtype, y, s, &chunk_err)) return chunk_err;
        const int bpr = (int)(k / 32);
        const int team = pow2_divisor(bpr, 64);
        const size_t lds = (size_t)bpr * 128;
        const unsigned grid = grid_for_rows(n, 256 / team);
        return xf32 ? launch_q8_0<true>(team, grid, lds, s, w, x, y, (int)n, bpr)
                    : launch_q8_0<false>(team, grid, lds, s, w, x, y, (int)n, bpr);
    }
    return hipErrorInvalidValue;
}

}  // namespace pmh
