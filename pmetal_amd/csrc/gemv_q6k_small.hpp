// The small-matrix Q6_K GEMV as device code: what gemv.hip's kernel runs, and what a launch of mixed types (gemv_q4k.hip)
// runs in the workgroups that belong to a Q6_K matrix.
#pragma once
#include "gemv_common.hpp"

namespace {

using namespace pmh::gemv;

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef uint32_t u32_a2 __attribute__((aligned(2)));
typedef uint16_t u16_a2 __attribute__((aligned(2)));
struct __attribute__((packed, aligned(2))) u32x2_a2 {
    uint32_t x, y;
};
struct __attribute__((packed, aligned(2))) u32x4_a2 {
    uint32_t x, y, z, w;
};

// Integer -> bf16 without a conversion: OR the integer into the mantissa of a power of two whose ulp is
// <= 1.  bf16(16.0) has ulp 1/8, so 0x4180 | (q << 3) is exactly 16 + q for q < 16; bf16(64.0) has ulp
// 1/2, so 0x4280 | (q << 1) is exactly 64 + q for q < 64.  The smallest usable offset keeps the
// cancellation error of "dot - offset * sum(x)" small.
constexpr uint32_t kBf16_64 = 0x42804280u;

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c,
                                           false);
}

// Split an f32 into three bf16 terms hi + mid + lo; 3 x 8 significant bits hold all 24 bits of the
// f32, so the sum is exact (barring underflow of the low terms).
__device__ __forceinline__ void split3(float f, uint32_t &h, uint32_t &m, uint32_t &l) {
    h = bf16_rne(f);
    const float r1 = f - bf16_to_f32(h);
    m = bf16_rne(r1);
    l = bf16_rne(r1 - bf16_to_f32(m));
}

// Load NE (8 or 16) consecutive activations starting at element `e` as PLANES planes of NE/2 packed
// bf16 pairs p[i] = elem 2i | elem 2i+1 << 16 (bf16 input: one plane; f32 input: three planes whose
// sum is the input), and return their f32 sum.
template <bool XF32, int NE>
__device__ __forceinline__ float load_x(const void *xg, size_t e, uint32_t (&pl)[3][NE / 2]) {
    float sum = 0.0f;
    if (XF32) {
        const float4 *p = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(xg) + e);
#pragma unroll
        for (int q = 0; q < NE / 4; q++) {
            const float4 v = p[q];
            const float f[4] = {v.x, v.y, v.z, v.w};
            uint32_t h[4], m[4], l[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                split3(f[c], h[c], m[c], l[c]);
                sum += f[c];
            }
            pl[0][2 * q] = h[0] | (h[1] << 16), pl[0][2 * q + 1] = h[2] | (h[3] << 16);
            pl[1][2 * q] = m[0] | (m[1] << 16), pl[1][2 * q + 1] = m[2] | (m[3] << 16);
            pl[2][2 * q] = l[0] | (l[1] << 16), pl[2][2 * q + 1] = l[2] | (l[3] << 16);
        }
    } else {
        const uint4 *p = reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(xg) + e);
#pragma unroll
        for (int q = 0; q < NE / 8; q++) {
            const uint4 a = p[q];
            pl[0][4 * q] = a.x, pl[0][4 * q + 1] = a.y, pl[0][4 * q + 2] = a.z, pl[0][4 * q + 3] = a.w;
        }
#pragma unroll
        for (int i = 0; i < NE / 2; i++) {
            pl[1][i] = pl[2][i] = 0;
            sum += bf16_to_f32(pl[0][i] & 0xFFFFu) + bf16_to_f32(pl[0][i] >> 16);
        }
    }
    return sum;
}

// From packed (e0|e1), (e2|e3) make the pairs the unpacking produces: (e0|e2) and (e1|e3).
__device__ __forceinline__ void even_odd_pairs(uint32_t p0, uint32_t p1, uint32_t &ev, uint32_t &od) {
    ev = (p0 & 0xFFFFu) | (p1 << 16);
    od = (p0 >> 16) | (p1 & 0xFFFF0000u);
}

// ------------------------------------------------------------------------------------------------
// Q6_K (210-byte super-blocks, only 2-byte aligned).  Lane t of a super-block: half h = t / 4,
// l in [8(t%4), 8(t%4)+8); for each of the 4 groups g it owns elements 128h + 32g + l.
// LDS: xl[PLANES][4][slots] uint4 (index g: pairs (l0,l2) (l1,l3) (l4,l6) (l5,l7)) then xs[slots]
// float4 (per-group sums of x).
// ------------------------------------------------------------------------------------------------
template <int PLANES, bool XF32>
__device__ __forceinline__ void stage_x_q6k(const void *xg, int spr, uint4 *xl, float4 *xs) {
    const int slots = spr * 8;
    for (int slot = threadIdx.x; slot < slots; slot += blockDim.x) {
        const int s = slot >> 3, t = slot & 7;
        const int base = 128 * (t >> 2) + 8 * (t & 3);
        float sums[4];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            uint32_t pl[3][4];
            sums[g] = load_x<XF32, 8>(xg, (size_t)s * 256 + base + 32 * g, pl);
#pragma unroll
            for (int p = 0; p < PLANES; p++) {
                uint4 v;
                even_odd_pairs(pl[p][0], pl[p][1], v.x, v.y);
                even_odd_pairs(pl[p][2], pl[p][3], v.z, v.w);
                xl[(p * 4 + g) * slots + slot] = v;
            }
        }
        xs[slot] = make_float4(sums[0], sums[1], sums[2], sums[3]);
    }
}

// One lane's share of a Q6_K super-block as it lies in memory (loaded ahead of its use).
struct Q6Raw {
    u32x2_a2 qla, qlb, qh, sc8;
    uint32_t d;
};

__device__ __forceinline__ Q6Raw q6k_load(const uint8_t *blk, const int t) {
    const int h = t >> 2, lq = (t & 3) * 8;
    Q6Raw r;
    r.qla = *reinterpret_cast<const u32x2_a2 *>(blk + 64 * h + lq);
    r.qlb = *reinterpret_cast<const u32x2_a2 *>(blk + 64 * h + 32 + lq);
    r.qh = *reinterpret_cast<const u32x2_a2 *>(blk + 128 + 32 * h + lq);
    r.sc8 = *reinterpret_cast<const u32x2_a2 *>(blk + 192 + 8 * h);
    r.d = *reinterpret_cast<const u16_a2 *>(blk + 208);
    return r;
}

template <int PLANES>
__device__ __forceinline__ float q6k_lane(const Q6Raw &raw, const int t, const uint4 *xl, const int slots,
                                          const int slot, const float4 xsum) {
    const int lq = (t & 3) * 8;
    const float d = f16_bits_to_f32(raw.d);
    const uint32_t la[2] = {raw.qla.x, raw.qla.y}, lb[2] = {raw.qlb.x, raw.qlb.y}, hh[2] = {raw.qh.x, raw.qh.y};
    const float xs4[4] = {xsum.x, xsum.y, xsum.z, xsum.w};
    const int shalf = lq >> 4;  // which of the two 16-element scale slots of a group
    float total = 0.0f;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        uint32_t v[2];
#pragma unroll
        for (int r = 0; r < 2; r++) {
            const uint32_t nib = ((g & 1) ? lb[r] : la[r]) >> (g >= 2 ? 4 : 0);
            const uint32_t hi2 = g == 0 ? (hh[r] << 4) : g == 1 ? (hh[r] << 2) : g == 2 ? hh[r] : (hh[r] >> 2);
            v[r] = (nib & 0x0F0F0F0Fu) | (hi2 & 0x30303030u);  // four 6-bit values q + 32
        }
        const uint32_t a0 = ((v[0] << 1) & 0x007E007Eu) | kBf16_64, b0 = ((v[0] >> 7) & 0x007E007Eu) | kBf16_64;
        const uint32_t a1 = ((v[1] << 1) & 0x007E007Eu) | kBf16_64, b1 = ((v[1] >> 7) & 0x007E007Eu) | kBf16_64;
        float dot = 0.0f;
#pragma unroll
        for (int p = 0; p < PLANES; p++) {
            const uint4 xv = xl[(p * 4 + g) * slots + slot];
            dot = dot2(a0, xv.x, dot);
            dot = dot2(b0, xv.y, dot);
            dot = dot2(a1, xv.z, dot);
            dot = dot2(b1, xv.w, dot);
        }
        const int si = 2 * g + shalf;  // scale byte inside this half's 8
        const uint32_t sw = si < 4 ? raw.sc8.x : raw.sc8.y;
        const float sc = (float)(int8_t)(sw >> (8 * (si & 3)));
        total += sc * (dot - 96.0f * xs4[g]);  // stored value is q + 32 and the bf16 trick adds 64
    }
    return d * total;
}

// A team of T lanes walks two rows at a time; the two lanes' shares of the next task (the next chunk of the
// row pair, or the first chunk of the next pair) are requested before the current one is multiplied, and the
// first request goes out before x is converted.
// The body of the kernel, callable from a launch that also holds workgroups of another kind: workgroup `block` of `n_blocks`
// workgroups of this kind, of which the first teams_per_wg teams of every workgroup take rows (the other threads only help
// staging x).
template <int T, bool XF32>
__device__ __forceinline__ void q6k_small_body(const uint8_t *__restrict__ W, const void *__restrict__ xg, float *__restrict__ y,
                                               int n_rows, int spr, int block, int n_blocks, int teams_per_wg, uint4 *smem) {
    constexpr int PLANES = XF32 ? 3 : 1;
    constexpr int SEG = T / 8;
    const int slots = spr * 8;
    uint4 *xl = smem;
    float4 *xs = reinterpret_cast<float4 *>(xl + PLANES * 4 * slots);

    const int lt = threadIdx.x & (T - 1);
    const int t = lt & 7;
    const int team_in_wg = (int)threadIdx.x / T;
    const bool has_rows = team_in_wg < teams_per_wg;  // uniform over a team
    const int team = block * teams_per_wg + (has_rows ? team_in_wg : 0);
    const int n_teams = n_blocks * teams_per_wg;
    const int iters = spr / SEG;
    const size_t row_bytes = (size_t)spr * 210;
    const size_t lane_off = (size_t)(lt >> 3) * 210;

    // task (row, it): rows row and row + n_teams, chunk it; a row past the end is replaced by the last row
    auto block_ptr = [&](int row, int it) -> const uint8_t * {
        const int r = row < n_rows ? row : n_rows - 1;
        return W + (size_t)r * row_bytes + lane_off + (size_t)it * SEG * 210;
    };
    int row = has_rows ? team : n_rows, it = 0;  // a team without rows starts past the end
    Q6Raw c0 = q6k_load(block_ptr(row, 0), t), c1 = q6k_load(block_ptr(row + n_teams, 0), t);

    stage_x_q6k<PLANES, XF32>(xg, spr, xl, xs);
    __syncthreads();

    float acc0 = 0.0f, acc1 = 0.0f;
    while (row < n_rows) {
        int nrow = row, nit = it + 1;
        if (nit == iters) nit = 0, nrow = row + 2 * n_teams;
        const Q6Raw n0 = q6k_load(block_ptr(nrow, nit), t), n1 = q6k_load(block_ptr(nrow + n_teams, nit), t);
        const int slot = it * T + lt;
        const float4 xsum = xs[slot];
        acc0 += q6k_lane<PLANES>(c0, t, xl, slots, slot, xsum);
        acc1 += q6k_lane<PLANES>(c1, t, xl, slots, slot, xsum);
        if (nit == 0) {
            acc0 = team_sum<T>(acc0);
            acc1 = team_sum<T>(acc1);
            if (lt == 0) {
                y[row] = acc0;
                if (row + n_teams < n_rows) y[row + n_teams] = acc1;
            }
            acc0 = acc1 = 0.0f;
        }
        c0 = n0, c1 = n1;
        row = nrow, it = nit;
    }
}


}  // namespace
