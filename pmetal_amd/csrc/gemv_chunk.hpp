// Shared pieces of the row-staging GEMV kernels (gemv_q5k.hip, gemv_q6k.hip, gemv_q8_0.hip, gemv_q23k.hip): one
// workgroup per compute unit, wave (g, h) = chunk h of the rows of row group g, one chunk sum per row through LDS.
#pragma once
#include "gemv_common.hpp"

namespace pmh {
namespace gemv {

__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// Fixed point for a group of activations that shares one power-of-two scale.  `mb` is the largest magnitude of the group
// as float bits; every |x| of the group is then below 2^(eb - 126) with eb the biased exponent.  mult = 2^(148 - eb) puts
// them below 2^22; scale = 2^(eb - 148) undoes it (0 for groups below 2^-126, NaN when the group holds an infinity or a
// NaN, so that every output of the GEMV becomes NaN).
struct GroupScale {
    float mult, scale;
    bool bad;
};
__device__ __forceinline__ GroupScale group_scale(uint32_t mb) {
    int eb = (int)(mb >> 23);
    GroupScale g;
    g.bad = eb == 255;
    eb = eb < 21 ? 21 : eb;
    g.mult = __builtin_bit_cast(float, (uint32_t)(275 - eb) << 23);
    g.scale = g.bad ? __builtin_nanf("") : __builtin_bit_cast(float, (uint32_t)(eb - 21) << 23);
    return g;
}

// Four activations -> one dword per digit plane (three balanced base-256 digits in [-128, 127] per value, value c in
// byte c); returns the sum of the four fixed-point integers.
//  * |v * mult| < 2^22, so adding 1.5 * 2^23 rounds to the integer grid (nearest even, as rintf does) and leaves the
//    integer xi in the low bits of the float.
//  * xi + 0x808080 = sum (d_k + 128) 256^k with every d_k + 128 in [0, 255]: the bytes of the biased value, each with its
//    top bit flipped, are the balanced digits.  The three bytes of the four values are transposed into the three planes
//    with byte permutes.
__device__ __forceinline__ int to_digits(const float (&v)[4], const GroupScale &g, uint32_t (&dig)[3]) {
    constexpr float kMagic = 12582912.0f;                       // 0x4B400000
    constexpr uint32_t kUnbias = 0x4B400000u - 0x00808080u;     // float bits -> xi + 0x808080
    uint32_t u[4];
    int sum = 0;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        u[c] = __builtin_bit_cast(uint32_t, __builtin_fmaf(v[c], g.mult, kMagic)) - kUnbias;
        sum += (int)u[c];
    }
    sum -= 4 * 0x00808080;
    const uint32_t t01 = __builtin_amdgcn_perm(u[1], u[0], 0x05010400u);  // u0.b0 u1.b0 u0.b1 u1.b1
    const uint32_t t23 = __builtin_amdgcn_perm(u[3], u[2], 0x05010400u);
    const uint32_t h01 = __builtin_amdgcn_perm(u[1], u[0], 0x0C0C0602u);  // u0.b2 u1.b2 0 0
    const uint32_t h23 = __builtin_amdgcn_perm(u[3], u[2], 0x0C0C0602u);
    dig[0] = __builtin_amdgcn_perm(t23, t01, 0x05040100u) ^ 0x80808080u;
    dig[1] = __builtin_amdgcn_perm(t23, t01, 0x07060302u) ^ 0x80808080u;
    dig[2] = (h01 | (h23 << 16)) ^ 0x80808080u;
    if (g.bad) dig[0] = dig[1] = dig[2] = 0, sum = 0;  // the group's scale is NaN: its digits only have to be finite work
    return sum;
}

// largest magnitude of four floats, as bits (the order of non-negative floats is that of their bits)
__device__ __forceinline__ uint32_t max_magnitude_bits(const float (&v)[4]) {
    uint32_t mb = 0;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const uint32_t a = __builtin_bit_cast(uint32_t, v[c]) & 0x7FFFFFFFu;
        mb = a > mb ? a : mb;
    }
    return mb;
}

// A task's lane values are added up inside the wave (DPP); lane 63 drops the total into part[group][row][chunk].
__device__ __forceinline__ void store_chunk_sum(float *slot_of_task, float lane_value, int lane) {
    const float total = team_sum_last<64>(lane_value);
    if (lane == 63) *slot_of_task = total;
}

// Row totals after the barrier: one thread per row adds the row's ks chunk sums in chunk order; the workgroup's rows leave
// with one coalesced store.  part is [group][n_nominal][ks].
__device__ __forceinline__ void reduce_rows(const float *part, int ks, int wg_r0, int wg_rows, int rows_per_wave, int n_nominal,
                                            int nthreads, float *__restrict__ y) {
    for (int rl = (int)threadIdx.x; rl < wg_rows; rl += nthreads) {
        const int grp = rl / rows_per_wave, loc = rl - grp * rows_per_wave;
        const float *src = part + (size_t)(grp * n_nominal + loc) * ks;
        float sum = src[0];
        for (int i = 1; i < ks; i++) sum += src[i];
        y[wg_r0 + rl] = sum;
    }
}

// Launch geometry: rows split evenly over one workgroup per compute unit, the workgroup's rows over 16 / ks row groups.
struct ChunkPlan {
    int64_t n_wg, rows_per_wg, rows_per_wave, n_nominal, threads;
    size_t lds;
};
// stage_bytes: LDS of one wave's row chunk; lds_x: LDS of the staged activations (slots = 64 ks lane slots)
inline ChunkPlan plan_chunks(int64_t n, int ks, size_t stage_bytes, size_t lds_x) {
    ChunkPlan p;
    const int64_t want = compute_units();
    p.n_wg = n < want ? n : want;
    p.rows_per_wg = (n + p.n_wg - 1) / p.n_wg;
    p.n_wg = (n + p.rows_per_wg - 1) / p.rows_per_wg;
    int64_t groups = 16 / ks;
    if (groups > p.rows_per_wg) groups = p.rows_per_wg;
    p.rows_per_wave = (p.rows_per_wg + groups - 1) / groups;
    groups = (p.rows_per_wg + p.rows_per_wave - 1) / p.rows_per_wave;
    p.n_nominal = p.rows_per_wave;
    p.threads = ks * groups * 64;
    p.lds = (size_t)(p.threads / 64) * stage_bytes + lds_x + (size_t)groups * (size_t)p.n_nominal * ks * 4;
    return p;
}

}  // namespace gemv
}  // namespace pmh
