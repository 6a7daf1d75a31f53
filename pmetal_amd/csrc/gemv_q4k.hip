// Dequant-fused Q4_K GEMV  y[n] = sum_k W[n,k] * x[k]  for gfx950 -- the batch-1 decode kernel.
//
// W is the packed GGUF stream, row-major [n, k] in 144-byte super-blocks; a weight's value is what the
// reference's dequantize_q4k yields (crates/pmetal-gguf/src/k_quants.rs:358-404) in the element order
// asked for: REF = the order that function emits, GGML = the inverse of quantize_q4k's packing
// (k_quants.rs:946-951).  The reference multiplies the dequantized tensor densely
// (crates/pmetal-models/src/weight_format.rs:299-303); this kernel is checked against that.
//
// HBM-bound by design: each weight byte is read once with 128-bit loads and never unpacked.
//  * 8 lanes share a super-block: lane j loads the 16 quant bytes 16j..16j+15 plus the 16-byte header,
//    so a wave streams 8 consecutive super-blocks (1152 contiguous bytes) per task.
//  * The 4-bit quants are multiplied as they lie in the dword by v_dot8_u32_u4 (8 products per
//    instruction, exact integer accumulation).  For that, x is converted once per workgroup to a
//    per-32-element block fixed point: X = round(x / 2^e) + 2^(4N-1) as N unsigned base-16 digits,
//    digit planes stored in LDS in the nibble order of the weight dwords.  sum(q*X) is N dot8 chains
//    (plus one against 0x11111111 for sum(q)), recombined in fp32; bf16 activations use N = 5
//    (20 bits: exact for every element within 2^-11 of its block maximum), f32 activations N = 6.
//  * Scales: the 6-bit (scale, min) pair of lane j's sub-block is extracted without branches using
//    per-lane shift/mask constants; d*sc*2^e*sum(qX) - dmin*m*sum(x) is accumulated in fp32.
//  * A team of T lanes (T/8 super-blocks per task) walks a contiguous chunk of rows as one linear
//    stream of tasks, T/8 * 144 bytes apart.  Four or eight tasks are in flight per team: they are
//    requested before x is converted, so HBM streams during the staging, and each register buffer is
//    refilled with the task that many ahead as soon as it has been consumed.
//  * When a row is only one or two tasks long (k <= 4096) the digits a lane needs never change, and
//    they are kept in registers instead of being re-read from LDS for every task.
//  * At the end of a row the team's partial sums are reduced with DPP only (quad_perm, row_half_mirror,
//    row_mirror inside a 16-lane row, row_bcast:15 / row_bcast:31 across rows); the last lane of the
//    team stores y[row].
#include "gemv_common.hpp"

namespace {

using namespace pmh::gemv;

// ---- x staging --------------------------------------------------------------------------------
// LDS: xd[NDIG][slots] uint4 (one dword per weight dword d = 0..3), then xm[slots] float4
// (2^e, sum of x over the low-nibble elements, over the high-nibble elements, over both).
// slot = 8 * super_block + j.  Weight dword d of lane j holds bytes 4d..4d+3 of its 16; nibble 2c is
// the low nibble of byte 4d+c -> element lowbase + 4d + c, nibble 2c+1 the high nibble -> element
// highbase + 4d + c, with
//   REF  order: lowbase = 32j,               highbase = lowbase + 16   (both in sub-block j)
//   GGML order: lowbase = 64(j/2) + 16(j%2), highbase = lowbase + 32   (sub-blocks 2(j/2), 2(j/2)+1)

template <bool XF32>
__device__ __forceinline__ void load_x4(const void *xg, size_t e, float (&v)[4]) {
    if (XF32) {
        const float4 f = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(xg) + e);
        v[0] = f.x, v[1] = f.y, v[2] = f.z, v[3] = f.w;
    } else {
        const uint2 u = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(xg) + e);
        v[0] = bf16_to_f32(u.x & 0xFFFFu), v[1] = bf16_to_f32(u.x >> 16);
        v[2] = bf16_to_f32(u.y & 0xFFFFu), v[3] = bf16_to_f32(u.y >> 16);
    }
}

// Four fixed-point values (offset binary, < 2^(4 NDIG)) -> NDIG dwords, digit k of value c in the low
// nibble of byte c of dword k.
template <int NDIG>
__device__ __forceinline__ void digits4(const uint32_t (&xu)[4], uint32_t (&dg)[NDIG]) {
    // byte transposes: B[b] = byte b of each of the four values
    const uint32_t t01 = __builtin_amdgcn_perm(xu[1], xu[0], 0x05010400u);  // x0.b0 x1.b0 x0.b1 x1.b1
    const uint32_t t23 = __builtin_amdgcn_perm(xu[3], xu[2], 0x05010400u);
    const uint32_t b0 = __builtin_amdgcn_perm(t23, t01, 0x05040100u);
    const uint32_t b1 = __builtin_amdgcn_perm(t23, t01, 0x07060302u);
    dg[0] = b0 & 0x0F0F0F0Fu;
    dg[1] = (b0 >> 4) & 0x0F0F0F0Fu;
    dg[2] = b1 & 0x0F0F0F0Fu;
    dg[3] = (b1 >> 4) & 0x0F0F0F0Fu;
    if (NDIG > 4) {
        const uint32_t u01 = __builtin_amdgcn_perm(xu[1], xu[0], 0x0C0C0602u);  // x0.b2 x1.b2 0 0
        const uint32_t u23 = __builtin_amdgcn_perm(xu[3], xu[2], 0x0C0C0602u);
        const uint32_t b2 = u01 | (u23 << 16);
        dg[4] = b2 & 0x0F0F0F0Fu;
        if (NDIG > 5) dg[5] = (b2 >> 4) & 0x0F0F0F0Fu;
    }
}

// Four threads cooperate on a slot, thread d converting the 4 + 4 elements behind weight dword d.
// Element offsets of the 4 + 4 activations thread `idx` of the staging converts:
template <int ORDER>
__device__ __forceinline__ void stage_offsets(int idx, size_t &e_lo, size_t &e_hi) {
    const int slot = idx >> 2, d = idx & 3;
    const int s = slot >> 3, j = slot & 7;
    const int lowbase = ORDER == 0 ? 32 * j : 64 * (j >> 1) + 16 * (j & 1);
    const int highbase = ORDER == 0 ? lowbase + 16 : lowbase + 32;
    e_lo = (size_t)s * 256 + lowbase + 4 * d;
    e_hi = (size_t)s * 256 + highbase + 4 * d;
}

// Convert the 4 + 4 activations of thread `idx` and store their digits.  The four threads of a slot
// are an aligned quad of one wave and are all active together, so the DPP exchanges are safe.
template <int NDIG, bool XF32>
__device__ __forceinline__ void stage_convert(int idx, const float (&lo)[4], const float (&hi)[4], int slots,
                                              uint4 *xd, float4 *xm) {
    constexpr int P = 4 * NDIG - 1;  // magnitude bits of the fixed point
    uint32_t *xd32 = reinterpret_cast<uint32_t *>(xd);
    const int slot = idx >> 2, d = idx & 3;
    float amax = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; c++)
        amax = __builtin_fmaxf(amax, __builtin_fmaxf(__builtin_fabsf(lo[c]), __builtin_fabsf(hi[c])));
    amax = __builtin_fmaxf(amax, dpp<0xB1>(amax));
    amax = __builtin_fmaxf(amax, dpp<0x4E>(amax));  // over the 4 threads of the slot
    // 2^e with |x| / 2^e < 2^P for every x of the slot: e = exponent(amax) + 1 - P
    const int eb = (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xFFu);
    int se = eb + 1 - P;
    se = se < 1 ? 1 : se;  // keep 2^e a normal number
    float scale = __builtin_bit_cast(float, (uint32_t)se << 23);
    const float inv = __builtin_bit_cast(float, (uint32_t)(254 - se) << 23);
    if (eb == 255) scale = amax;  // inf / NaN activations poison the row, as they should
    uint32_t xl[4], xh[4];
#pragma unroll
    for (int c = 0; c < 4; c++) {
        // v * inv is exact (power of two); one rounding to the integer grid, then offset binary
        if (XF32) {
            // an f32 block maximum can round up to 2^P: clamp
            const float rl = __builtin_fminf(__builtin_rintf(lo[c] * inv), (float)((1 << P) - 1));
            const float rh = __builtin_fminf(__builtin_rintf(hi[c] * inv), (float)((1 << P) - 1));
            xl[c] = (uint32_t)((int)rl + (1 << P));
            xh[c] = (uint32_t)((int)rh + (1 << P));
        } else {
            // |v * inv| < 2^22: adding 1.5 * 2^23 rounds to the integer grid (nearest even) and leaves
            // the integer in the low bits of the float; a bf16 maximum never rounds up to 2^P
            constexpr float kMagic = 12582912.0f;  // 0x4B400000
            const float fl = lo[c] * inv + kMagic, fh = hi[c] * inv + kMagic;
            xl[c] = __builtin_bit_cast(uint32_t, fl) - 0x4B400000u + (1u << P);
            xh[c] = __builtin_bit_cast(uint32_t, fh) - 0x4B400000u + (1u << P);
        }
    }
    uint32_t dl[NDIG], dh[NDIG];
    digits4<NDIG>(xl, dl);
    digits4<NDIG>(xh, dh);
#pragma unroll
    for (int k = 0; k < NDIG; k++) xd32[(k * slots + slot) * 4 + d] = dl[k] | (dh[k] << 4);
    float sl = (lo[0] + lo[1]) + (lo[2] + lo[3]), sh = (hi[0] + hi[1]) + (hi[2] + hi[3]);
    sl += dpp<0xB1>(sl), sh += dpp<0xB1>(sh);
    sl += dpp<0x4E>(sl), sh += dpp<0x4E>(sh);
    if (d == 0) xm[slot] = make_float4(scale, sl, sh, sl + sh);
}

// Per-lane constants for the branch-free get_scale_min_k4 (crates/pmetal-gguf/src/quantize.rs:844-855).
// With a, b, c the bytes (j & 3) of the three scale dwords:
//   j <  4: sc = a & 63,                   m = b & 63
//   j >= 4: sc = (c & 15) | (a >> 6) << 4, m = (c >> 4) | (b >> 6) << 4
// both are (c' & cm) | ((a >> sa) & am) with c' = c resp. c >> 4.
struct ScaleSel {
    uint32_t sh;     // 8 * (j & 3)
    uint32_t sh_ab;  // sh + (j < 4 ? 0 : 2)
    uint32_t am;     // j < 4 ? 63 : 0x30
    uint32_t cm;     // j < 4 ? 0 : 15
};

__device__ __forceinline__ ScaleSel scale_sel(int j) {
    ScaleSel s;
    s.sh = 8u * (j & 3);
    s.sh_ab = s.sh + (j < 4 ? 0u : 2u);
    s.am = j < 4 ? 63u : 0x30u;
    s.cm = j < 4 ? 0u : 15u;
    return s;
}

__device__ __forceinline__ void scale_min(const uint4 hdr, const ScaleSel &s, float &sc, float &m) {
    const uint32_t c = hdr.w >> s.sh;
    sc = (float)((c & s.cm) | ((hdr.y >> s.sh_ab) & s.am));
    m = (float)(((c >> 4) & s.cm) | ((hdr.z >> s.sh_ab) & s.am));
}

// sum over the 32 nibbles of (q * X) with X = sum_k 16^k digit_k - 2^P, as fp32
template <int NDIG>
__device__ __forceinline__ float combine(const uint32_t (&acc)[NDIG], uint32_t accq) {
    constexpr int P = 4 * NDIG - 1;
    // the low four digit sums fit an integer exactly; the rest is folded in fp32
    uint32_t t = acc[3];
#pragma unroll
    for (int k = 2; k >= 0; k--) t = (t << 4) + acc[k];
    float f = (float)t;
    if (NDIG > 4) f += 65536.0f * (float)(NDIG > 5 ? acc[4] + (acc[5] << 4) : acc[4]);
    return f - (float)(1 << P) * (float)accq;
}

// One lane's share of one super-block: its 16 quant bytes against the staged digits of its slot.
template <int ORDER, int NDIG>
__device__ __forceinline__ float lane_dot(const uint4 hdr, const uint4 qv, const ScaleSel &s0, const ScaleSel &s1,
                                          const uint4 (&xdig)[NDIG], const float4 xm) {
    const uint32_t w[4] = {qv.x, qv.y, qv.z, qv.w};
    const float d = f16_bits_to_f32(hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(hdr.x >> 16);
    if (ORDER == 0) {
        uint32_t acc[NDIG], accq = 0;
#pragma unroll
        for (int k = 0; k < NDIG; k++) {
            const uint4 xk = xdig[k];
            uint32_t a = __builtin_amdgcn_udot8(w[0], xk.x, 0u, false);
            a = __builtin_amdgcn_udot8(w[1], xk.y, a, false);
            a = __builtin_amdgcn_udot8(w[2], xk.z, a, false);
            acc[k] = __builtin_amdgcn_udot8(w[3], xk.w, a, false);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) accq = __builtin_amdgcn_udot8(w[i], 0x11111111u, accq, false);
        float sc, m;
        scale_min(hdr, s0, sc, m);
        return (d * sc) * (xm.x * combine<NDIG>(acc, accq)) - (dmin * m) * xm.w;
    } else {
        // low nibbles belong to sub-block 2(j/2), high nibbles to 2(j/2)+1: separate sums
        uint32_t wl[4], wh[4];
#pragma unroll
        for (int i = 0; i < 4; i++) wl[i] = w[i] & 0x0F0F0F0Fu, wh[i] = w[i] & 0xF0F0F0F0u;
        uint32_t al[NDIG], ah[NDIG], ql = 0, qh = 0;
#pragma unroll
        for (int k = 0; k < NDIG; k++) {
            const uint4 xk = xdig[k];
            const uint32_t xs[4] = {xk.x, xk.y, xk.z, xk.w};
            al[k] = ah[k] = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                al[k] = __builtin_amdgcn_udot8(wl[i], xs[i], al[k], false);
                ah[k] = __builtin_amdgcn_udot8(wh[i], xs[i], ah[k], false);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            ql = __builtin_amdgcn_udot8(wl[i], 0x11111111u, ql, false);
            qh = __builtin_amdgcn_udot8(wh[i], 0x11111111u, qh, false);
        }
        float sc0, m0, sc1, m1;
        scale_min(hdr, s0, sc0, m0);
        scale_min(hdr, s1, sc1, m1);
        return d * xm.x * (sc0 * combine<NDIG>(al, ql) + sc1 * combine<NDIG>(ah, qh)) -
               dmin * (m0 * xm.y + m1 * xm.z);
    }
}

// Tasks in flight per team.  When a row is one or two tasks long (ITERS = 1, 2) every task of a team uses
// the same one or two x slots, which are then held in registers for the whole kernel; the registers that
// takes are paid for with a shallower prefetch.
template <int ITERS>
struct Depth {
    static constexpr int value = ITERS == 0 ? 8 : 4;
};

#ifdef PMH_TRACE
__device__ unsigned long long *g_trace;  // [workgroup][wave][8] timestamps, set by the harness
#define PMH_STAMP(slot)                                                                              \
    do {                                                                                             \
        if ((threadIdx.x & 63) == 0)                                                                 \
            g_trace[((size_t)blockIdx.x * 16 + (threadIdx.x >> 6)) * 8 + (slot)] = __builtin_readcyclecounter(); \
    } while (0)
#else
#define PMH_STAMP(slot)
#endif

template <int ORDER, bool XF32, int T, int ITERS>
__global__ __launch_bounds__(1024) void k_qgemv_q4k(const uint8_t *__restrict__ W, const void *__restrict__ xg,
                                                     float *__restrict__ y, int n_rows, int spr, int rows_per_wg,
                                                     int per_team) {
    constexpr int NDIG = XF32 ? 6 : 5;
    constexpr int SEG = T / 8;        // super-blocks a team covers per task
    constexpr int STRIDE = SEG * 144; // bytes between a lane's consecutive tasks
    constexpr int kDepth = Depth<ITERS>::value;
    extern __shared__ uint4 smem[];
    const int slots = spr * 8;
    uint4 *xd = smem;
    float4 *xm = reinterpret_cast<float4 *>(xd + NDIG * slots);

    PMH_STAMP(0);
    const int lane = threadIdx.x & 63;
    const int lt = lane & (T - 1);
    const int j = lane & 7;
    const int iters = ITERS ? ITERS : spr / SEG;  // tasks per row
    constexpr int kTeamsPerWave = 64 / T;
    // with full-wave teams everything about a team is wave-uniform: keep it in scalar registers
    auto uni = [](int v) { return T == 64 ? __builtin_amdgcn_readfirstlane(v) : v; };
    const int team = uni((int)(threadIdx.x >> 6) * kTeamsPerWave + lane / T);

    // contiguous chunk of rows for this workgroup, then `per_team` of them for this team
    const int wg_r0 = blockIdx.x * rows_per_wg;
    const int wg_r1 = wg_r0 + rows_per_wg < n_rows ? wg_r0 + rows_per_wg : n_rows;
    const int r0 = wg_r0 + team * per_team;
    const int r1 = r0 + per_team < wg_r1 ? r0 + per_team : wg_r1;
    const int n_tasks = (r1 > r0 ? r1 - r0 : 0) * iters;  // this team's tasks
    const int n_nominal = per_team * iters;               // workgroup-uniform upper bound

    // The first pass of activation loads goes out before the weight loads queue up behind it.
    const int stage_total = slots * 4;
    float x_lo[4], x_hi[4];
    if ((int)threadIdx.x < stage_total) {
        size_t e_lo, e_hi;
        stage_offsets<ORDER>(threadIdx.x, e_lo, e_hi);
        load_x4<XF32>(xg, e_lo, x_lo);
        load_x4<XF32>(xg, e_hi, x_hi);
    }

    // A team's tasks are one linear stream: task t of the team starts STRIDE * t bytes after its first.
    const uint8_t *ph = W + (size_t)(n_tasks > 0 ? r0 : 0) * spr * 144 + (size_t)(lt >> 3) * 144;
    const uint8_t *pq = ph + 16 + 16 * j;

    // kDepth tasks are in flight per team.  They are requested before x is converted, so the memory system
    // streams while the staging runs, and each buffer is refilled as soon as it has been consumed.  (The
    // load unit takes one 1 KiB wave-load per ~32 cycles and a wave stuck issuing loads cannot start
    // converting x, so a deeper initial burst does not pay.)
    uint4 bh[kDepth], bq[kDepth];
#pragma unroll
    for (int i = 0; i < kDepth; i++) {
        if (i < n_tasks) {
            bh[i] = *reinterpret_cast<const uint4 *>(ph + i * STRIDE);
            bq[i] = *reinterpret_cast<const uint4 *>(pq + i * STRIDE);
        }
    }
    PMH_STAMP(1);

    if ((int)threadIdx.x < stage_total) stage_convert<NDIG, XF32>(threadIdx.x, x_lo, x_hi, slots, xd, xm);
    for (int idx = threadIdx.x + blockDim.x; idx < stage_total; idx += blockDim.x) {  // long rows: more passes
        size_t e_lo, e_hi;
        stage_offsets<ORDER>(idx, e_lo, e_hi);
        load_x4<XF32>(xg, e_lo, x_lo);
        load_x4<XF32>(xg, e_hi, x_hi);
        stage_convert<NDIG, XF32>(idx, x_lo, x_hi, slots, xd, xm);
    }
    PMH_STAMP(2);
    __syncthreads();
    PMH_STAMP(3);

    const ScaleSel s0 = scale_sel(ORDER == 0 ? j : 2 * (j >> 1));
    const ScaleSel s1 = scale_sel(ORDER == 0 ? j : 2 * (j >> 1) + 1);
    // register-resident x: slot (it * T + lt) for it < ITERS
    uint4 xr[ITERS ? ITERS : 1][NDIG];
    float4 xmr[ITERS ? ITERS : 1];
    if (ITERS) {
#pragma unroll
        for (int t = 0; t < ITERS; t++) {
#pragma unroll
            for (int k = 0; k < NDIG; k++) xr[t][k] = xd[k * slots + t * T + lt];
            xmr[t] = xm[t * T + lt];
        }
    }
    float acc = 0.0f;
    int it = 0;  // position inside the row: the same for every team of the workgroup
    int row = r0;
    for (int first = 0; first < n_nominal; first += kDepth) {
#pragma unroll
        for (int i = 0; i < kDepth; i++) {
            if (first + i < n_nominal) {
                const bool valid = first + i < n_tasks;
                if (valid) {
                    if (ITERS) {  // kDepth is a multiple of ITERS, so the position in the row is static
                        acc += lane_dot<ORDER, NDIG>(bh[i], bq[i], s0, s1, xr[i % (ITERS ? ITERS : 1)],
                                                     xmr[i % (ITERS ? ITERS : 1)]);
                    } else {
                        const int slot = it * T + lt;
                        uint4 xdig[NDIG];
#pragma unroll
                        for (int k = 0; k < NDIG; k++) xdig[k] = xd[k * slots + slot];
                        acc += lane_dot<ORDER, NDIG>(bh[i], bq[i], s0, s1, xdig, xm[slot]);
                    }
                }
                if (first + i + kDepth < n_tasks) {  // refill this buffer with the task kDepth ahead
                    bh[i] = *reinterpret_cast<const uint4 *>(ph + (size_t)(i + kDepth) * STRIDE);
                    bq[i] = *reinterpret_cast<const uint4 *>(pq + (size_t)(i + kDepth) * STRIDE);
                }
                const bool row_end = ITERS ? (i % (ITERS ? ITERS : 1) == ITERS - 1) : (++it == iters);
                if (row_end) {
                    const float total = team_sum_last<T>(acc);
                    if (lt == T - 1 && valid) y[row] = total;
                    row++;
                    acc = 0.0f;
                    it = 0;
                }
            }
        }
        ph += kDepth * STRIDE;
        pq += kDepth * STRIDE;
        PMH_STAMP(4 + ((first / kDepth) & 3));
    }
}

template <int ORDER, bool XF32>
hipError_t launch_cfg(int T, dim3 grid, dim3 block, size_t lds, hipStream_t s, const uint8_t *w, const void *x,
                      float *y, int n, int spr, int rows_per_wg, int per_team) {
    auto go = [&](auto kern) -> hipError_t {
        if (lds > 64 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kern, grid, block, lds, s, w, x, y, n, spr, rows_per_wg, per_team);
        return hipGetLastError();
    };
    const int iters = spr / (T / 8);
    const bool xreg = iters <= 2 && !XF32 && ORDER == 0;  // the headline path keeps x in registers
    switch (T) {
    case 8: return go(k_qgemv_q4k<ORDER, XF32, 8, 0>);
    case 16: return go(k_qgemv_q4k<ORDER, XF32, 16, 0>);
    case 32:
        if (xreg && iters == 1) return go(k_qgemv_q4k<ORDER, XF32, 32, 1>);
        return go(k_qgemv_q4k<ORDER, XF32, 32, 0>);
    default:
        if (xreg && iters == 1) return go(k_qgemv_q4k<ORDER, XF32, 64, 1>);
        if (xreg && iters == 2) return go(k_qgemv_q4k<ORDER, XF32, 64, 2>);
        return go(k_qgemv_q4k<ORDER, XF32, 64, 0>);
    }
}

}  // namespace

namespace pmh {

// Preconditions as for launch_qgemv.  Returns hipErrorInvalidValue when x does not fit in LDS.
hipError_t launch_qgemv_q4k(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y,
                            uint32_t order, hipStream_t s) {
    const bool xf32 = x_dtype == kDtypeF32;
    const int spr = (int)(k / 256);
    const int T = 8 * gemv::pow2_divisor(spr, 8);
    const size_t slots = (size_t)spr * 8;
    const size_t lds = slots * 16 * (xf32 ? 6 : 5) + slots * 16;
    if (lds > gemv::kMaxLds) return hipErrorInvalidValue;

    // Workgroups own contiguous chunks of rows, about `wgs_per_cu` per compute unit (x is staged once
    // per workgroup), up to 16 waves each; the wave count is the largest that keeps the busiest team's
    // row count minimal.
    const int64_t wgs_per_cu = gemv::tuning("PMETAL_HIP_GEMV_WGS_PER_CU", 1);
    const int64_t want = (int64_t)gemv::compute_units() * (wgs_per_cu > 0 ? wgs_per_cu : 1);
    int64_t n_wg = n < want ? n : want;
    const int64_t rows_per_wg = (n + n_wg - 1) / n_wg;
    n_wg = (n + rows_per_wg - 1) / rows_per_wg;
    const int teams_per_wave = 64 / T;
    int best_waves = 16;
    int64_t best_cost = INT64_MAX;
    for (int waves = 16; waves >= 1; waves--) {  // ties go to more waves: more bytes in flight
        const int64_t teams = (int64_t)waves * teams_per_wave;
        const int64_t per_team = (rows_per_wg + teams - 1) / teams;
        if (per_team < best_cost) best_cost = per_team, best_waves = waves;
    }
    const int forced = (int)gemv::tuning("PMETAL_HIP_GEMV_WAVES", 0);
    if (forced >= 1 && forced <= 16) best_waves = forced;
    const int per_team = (int)((rows_per_wg + (int64_t)best_waves * teams_per_wave - 1) / ((int64_t)best_waves * teams_per_wave));
    const dim3 grid((unsigned)n_wg), block((unsigned)best_waves * 64);
    if (order == kOrderRef)
        return xf32 ? launch_cfg<0, true>(T, grid, block, lds, s, w, x, y, (int)n, spr, (int)rows_per_wg, per_team)
                    : launch_cfg<0, false>(T, grid, block, lds, s, w, x, y, (int)n, spr, (int)rows_per_wg, per_team);
    return xf32 ? launch_cfg<1, true>(T, grid, block, lds, s, w, x, y, (int)n, spr, (int)rows_per_wg, per_team)
                : launch_cfg<1, false>(T, grid, block, lds, s, w, x, y, (int)n, spr, (int)rows_per_wg, per_team);
}

}  // namespace pmh
