// Helpers shared by the GEMV translation units.
#pragma once

#include <cstdlib>

#include "internal.hpp"

namespace pmh {
namespace gemv {

constexpr size_t kMaxLds = 160 * 1024;  // LDS per workgroup on gfx950

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

__device__ __forceinline__ uint32_t bf16_rne(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return __builtin_bit_cast(float, h << 16); }

// v from another lane of the same 16-lane row, selected by a DPP control word:
// 0xB1 quad_perm [1,0,3,2], 0x4E quad_perm [2,3,0,1], 0x141 row_half_mirror, 0x140 row_mirror.
template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
    return __builtin_bit_cast(float,
                              __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Sum over the T lanes of a team (aligned groups of T = 8..64 lanes); every lane gets the total.
template <int T>
__device__ __forceinline__ float team_sum(float v) {
    if (T >= 2) v += dpp<0xB1>(v);
    if (T >= 4) v += dpp<0x4E>(v);
    if (T >= 8) v += dpp<0x141>(v);
    if (T >= 16) v += dpp<0x140>(v);
    if (T >= 32) v += __shfl_xor(v, 16);
    if (T >= 64) v += __shfl_xor(v, 32);
    return v;
}

// Sum over the T lanes of a team using DPP only; the LAST lane of the team gets the total (other lanes
// hold partial sums).  row_bcast:15 adds lane 15 of each row into the next row (rows 1 and 3 enabled),
// row_bcast:31 adds lane 31 into rows 2 and 3.
template <int T>
__device__ __forceinline__ float team_sum_last(float v) {
    v += dpp<0xB1>(v);
    v += dpp<0x4E>(v);
    v += dpp<0x141>(v);
    if (T >= 16) v += dpp<0x140>(v);
    if (T >= 32)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, false));
    if (T >= 64)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xC, 0xF, false));
    return v;
}

// Same as team_sum with a wave-uniform run-time T >= 8.
__device__ __forceinline__ float team_sum_rt(float v, int T) {
    v += dpp<0xB1>(v);
    v += dpp<0x4E>(v);
    v += dpp<0x141>(v);
    if (T >= 16) v += dpp<0x140>(v);
    if (T >= 32) v += __shfl_xor(v, 16);
    if (T >= 64) v += __shfl_xor(v, 32);
    return v;
}

// largest power of two dividing v, capped
inline int pow2_divisor(int64_t v, int cap) {
    int t = 1;
    while (t < cap && v % (2 * t) == 0) t *= 2;
    return t;
}

// compute units of the current device (256 on MI355X); falls back to 256 if the query fails
inline int compute_units() {
    static const int n = [] {
        int dev = 0, cu = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 256;
        if (hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cu <= 0) return 256;
        return cu;
    }();
    return n;
}

}  // namespace gemv

}  // namespace pmh
