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
#include "gemv_q6k_small.hpp"

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

// Four consecutive activations as they lie in memory (f32: 16 bytes, bf16: 8 bytes in .x/.y); unpacking is
// kept apart from the load so that a wave can go on issuing loads while these are in flight.
template <bool XF32>
__device__ __forceinline__ uint4 load_x4_raw(const void *xg, size_t e) {
    if (XF32) return *reinterpret_cast<const uint4 *>(reinterpret_cast<const float *>(xg) + e);
    const uint2 u = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(xg) + e);
    return make_uint4(u.x, u.y, 0u, 0u);
}

template <bool XF32>
__device__ __forceinline__ void unpack_x4(const uint4 r, float (&v)[4]) {
    if (XF32) {
        v[0] = __builtin_bit_cast(float, r.x), v[1] = __builtin_bit_cast(float, r.y);
        v[2] = __builtin_bit_cast(float, r.z), v[3] = __builtin_bit_cast(float, r.w);
    } else {
        v[0] = bf16_to_f32(r.x & 0xFFFFu), v[1] = bf16_to_f32(r.x >> 16);
        v[2] = bf16_to_f32(r.y & 0xFFFFu), v[3] = bf16_to_f32(r.y >> 16);
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
// With a, b, c the bytes (j & 3) of the three scale dwords y, z, w of the header:
//   j <  4: sc = a & 63,                   m = b & 63
//   j >= 4: sc = (c & 15) | (a >> 6) << 4, m = (c >> 4) | (b >> 6) << 4
// Both are  bfe(c-word, off_c, wid_c) | bfe(a-word, off_a, wid_a) << shl  with per-lane field positions
// (a zero-width field reads as 0).
struct ScaleSel {
    uint32_t off_a;  // 8 (j & 3) + (j < 4 ? 0 : 6)
    uint32_t wid_a;  // j < 4 ? 6 : 2
    uint32_t off_c;  // 8 (j & 3)
    uint32_t wid_c;  // j < 4 ? 0 : 4
    uint32_t shl;    // j < 4 ? 0 : 4
};

__device__ __forceinline__ ScaleSel scale_sel(int j) {
    ScaleSel s;
    s.off_c = 8u * (j & 3);
    s.off_a = s.off_c + (j < 4 ? 0u : 6u);
    s.wid_a = j < 4 ? 6u : 2u;
    s.wid_c = j < 4 ? 0u : 4u;
    s.shl = j < 4 ? 0u : 4u;
    return s;
}

__device__ __forceinline__ void scale_min(const uint4 hdr, const ScaleSel &s, float &sc, float &m) {
    const uint32_t a = __builtin_amdgcn_ubfe(hdr.y, s.off_a, s.wid_a);
    const uint32_t b = __builtin_amdgcn_ubfe(hdr.z, s.off_a, s.wid_a);
    const uint32_t c0 = __builtin_amdgcn_ubfe(hdr.w, s.off_c, s.wid_c);
    const uint32_t c1 = __builtin_amdgcn_ubfe(hdr.w, s.off_c + 4u, s.wid_c);
    sc = (float)((a << s.shl) | c0);
    m = (float)((b << s.shl) | c1);
}

// sum over the 32 nibbles of (q * X) with X = sum_k 16^k digit_k - 2^P, as fp32
template <int NDIG>
__device__ __forceinline__ float combine(const uint32_t (&acc)[NDIG], uint32_t accq) {
    if (NDIG == 5) {
        // 2^P = 8 * 16^4: the offset comes off the top digit sum, and the whole signed sum fits 32 bits
        // (|sum| <= 32 * 15 * 2^19 < 2^28): one integer chain, one rounding.
        int t = (int)acc[4] - 8 * (int)accq;
#pragma unroll
        for (int k = 3; k >= 0; k--) t = (t << 4) + (int)acc[k];
        return (float)t;
    }
    constexpr int P = 4 * NDIG - 1;
    // the low four digit sums fit an integer exactly; the rest is folded in fp32
    uint32_t t = acc[3];
#pragma unroll
    for (int k = 2; k >= 0; k--) t = (t << 4) + acc[k];
    float f = (float)t;
    f += 65536.0f * (float)(NDIG > 5 ? acc[4] + (acc[5] << 4) : acc[4]);
    return f - (float)(1 << P) * (float)accq;
}

// One lane's share of one super-block: its 16 quant bytes against the staged digits of its slot.
template <int ORDER, int NDIG>
__device__ __forceinline__ float lane_dot(const uint4 hdr, const uint4 qv, const ScaleSel &s0, const ScaleSel &s1,
                                          const uint4 (&xdig)[NDIG], const float4 xm) {
    const uint32_t w[4] = {qv.x, qv.y, qv.z, qv.w};
    // fma with an f16 operand converted in place
    const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)(hdr.x & 0xFFFFu));
    const float dmin = (float)__builtin_bit_cast(_Float16, (uint16_t)(hdr.x >> 16));
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
        const float u = sc * (xm.x * combine<NDIG>(acc, accq));
        const float v = m * xm.w;
        return __builtin_fmaf(d, u, -(dmin * v));
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

// Conversion of x into LDS in two steps, so that the first pass of activation loads can be requested before
// the weight loads queue up behind it: stage_x_begin loads, stage_x_finish converts (and runs the further
// passes a long row needs).  All threads of the workgroup take part; the caller places the barrier.
constexpr int kStagePre = 2;  // passes of activation loads requested up front

// `live` slots hold activations (8 per super-block of a row); the slots from there to `slots` (the padding of a short last
// chunk) are converted from zeros and read nothing.
template <int ORDER, bool XF32>
__device__ __forceinline__ void stage_x_begin(const void *xg, int slots, int nthreads, uint4 (&r_lo)[kStagePre],
                                              uint4 (&r_hi)[kStagePre], int live) {
#pragma unroll
    for (int ps = 0; ps < kStagePre; ps++) {
        r_lo[ps] = r_hi[ps] = make_uint4(0u, 0u, 0u, 0u);
        const int idx = threadIdx.x + ps * nthreads;
        if (idx < live * 4) {
            size_t e_lo, e_hi;
            stage_offsets<ORDER>(idx, e_lo, e_hi);
            r_lo[ps] = load_x4_raw<XF32>(xg, e_lo);
            r_hi[ps] = load_x4_raw<XF32>(xg, e_hi);
        }
    }
}

template <int ORDER, int NDIG, bool XF32>
__device__ __forceinline__ void stage_x_finish(const void *xg, int slots, int nthreads, const uint4 (&r_lo)[kStagePre],
                                               const uint4 (&r_hi)[kStagePre], uint4 *xd, float4 *xm, int live) {
    const int stage_total = slots * 4;
    float x_lo[4], x_hi[4];
#pragma unroll
    for (int ps = 0; ps < kStagePre; ps++) {
        const int idx = threadIdx.x + ps * nthreads;
        if (idx < stage_total) {
            unpack_x4<XF32>(r_lo[ps], x_lo);
            unpack_x4<XF32>(r_hi[ps], x_hi);
            stage_convert<NDIG, XF32>(idx, x_lo, x_hi, slots, xd, xm);
        }
    }
    for (int idx = threadIdx.x + kStagePre * nthreads; idx < stage_total; idx += nthreads) {
        uint4 a = make_uint4(0u, 0u, 0u, 0u), b = a;
        if (idx < live * 4) {
            size_t e_lo, e_hi;
            stage_offsets<ORDER>(idx, e_lo, e_hi);
            a = load_x4_raw<XF32>(xg, e_lo), b = load_x4_raw<XF32>(xg, e_hi);
        }
        unpack_x4<XF32>(a, x_lo);
        unpack_x4<XF32>(b, x_hi);
        stage_convert<NDIG, XF32>(idx, x_lo, x_hi, slots, xd, xm);
    }
}

// ---- kernel A: one wave per (row group, k-chunk) ------------------------------------------------
// A team of T lanes covers a chunk of T/8 super-blocks of a row; a row is KS = (k/256) / (T/8) chunks.
// The workgroup has KS * G waves: wave (g, h) takes chunk h of the rows of row group g, 64/T rows per task,
// so every task of a wave needs the same x digits, which stay in registers.  Up to kDepth tasks are in
// flight per wave; every load is issued unconditionally (tasks past the end read the first bytes of W, all
// lanes the same address) so that the number of outstanding loads is known at every wait.  A task's lane sums
// are added up inside the wave (DPP) and the team's last lane drops one float per row and chunk into LDS; after
// a barrier one thread per row adds the KS chunk sums and the workgroup stores its rows of y with one coalesced
// store.  (Keeping every lane's partial in LDS and adding them up after the barrier cost 0.5 us per launch at
// 14336 x 4096; stores inside the streaming loop are worse: on this target they share the loads' counter, and
// the counted waits degenerate.)
constexpr int kDepth = 8;  // tasks in flight per wave
constexpr int kPre = 2;    // of which this many are requested before x is converted (the row-owner kernel)
// Kernel A requests three tasks before x is converted (against two: 4096 x 14336 9.9 -> 9.6 us, other shapes unchanged;
// four: 9.7; the row-owner kernel is fastest at two) and then two more per task consumed until the ring is full.
constexpr int kPreA = 3, kFillA = 2;
static_assert(kPreA + kFillA * kDepth >= 2 * kDepth, "after the first round every task of the second is requested");

template <int ORDER, bool XF32, int T, bool SINGLE, bool PAIR, bool RAGGED = false>
__global__ __launch_bounds__(1024) void k_qgemv_q4k_chunk(const uint8_t *__restrict__ W0, const uint8_t *__restrict__ W1,
                                                           const void *__restrict__ xg, int split_wg, int n_rows0, int n_rows1,
                                                           int spr, int rows_per_wg, int rows_per_wave, int n_nominal,
                                                           int nthreads, float *__restrict__ y0, float *__restrict__ y1) {
    // (the arguments needed before the first weight request come first: the leading 16 dwords of the kernel-argument
    // segment are preloaded into scalar registers at wave launch)
    // Two matrices that share k and the activation vector (the gate / up projections) can go through one launch:
    // workgroups [0, split_wg) belong to the first, the others to the second (PAIR; otherwise W1, y1, n_rows1 and split_wg
    // are not looked at).
    const bool second = PAIR && (int)blockIdx.x >= split_wg;  // workgroup-uniform
    const uint8_t *__restrict__ W = second ? W1 : W0;
    float *__restrict__ y = second ? y1 : y0;
    const int n_rows = second ? n_rows1 : n_rows0;
    const int wg_index = second ? (int)blockIdx.x - split_wg : (int)blockIdx.x;
    constexpr int NDIG = XF32 ? 6 : 5;
    constexpr int SEG = T / 8;   // super-blocks a team covers
    constexpr int RPT = 64 / T;  // rows per task
    // RAGGED (T = 64 only): rows that are not whole chunks of eight super-blocks and have too many of them for a
    // narrower team (k = 11008, 13824, 18944, ...).  The last chunk of a row is short: its missing super-blocks get zero
    // activations, their lanes read the row's first block and contribute nothing.
    static_assert(!RAGGED || T == 64, "short last chunks exist for whole-wave teams only");
    extern __shared__ uint4 smem[];
    const int ks = RAGGED ? (spr + SEG - 1) / SEG : spr / SEG;
    const int slots = RAGGED ? ks * 64 : spr * 8;
    uint4 *xd = smem;
    float4 *xm = reinterpret_cast<float4 *>(xd + NDIG * slots);
    float *part = reinterpret_cast<float *>(xm + slots);  // [group][n_nominal * RPT][ks]
    const int lane = threadIdx.x & 63;
    const int lt = lane & (T - 1), tm = lane / T, j = lane & 7;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int h = wave % ks, g = wave / ks;
    const int wg_r0 = wg_index * rows_per_wg;
    const int wg_r1 = wg_r0 + rows_per_wg < n_rows ? wg_r0 + rows_per_wg : n_rows;
    const int wave_r0 = wg_r0 + g * rows_per_wave;
    const int wave_r1 = wave_r0 + rows_per_wave < wg_r1 ? wave_r0 + rows_per_wave : wg_r1;
    const int rows_here = wave_r1 > wave_r0 ? wave_r1 - wave_r0 : 0;
    const int nt_wave = (rows_here + RPT - 1) / RPT;  // real tasks of this wave (wave-uniform)

    const uint32_t rowbytes = (uint32_t)spr * 144u;
    const bool lane_valid = !RAGGED || h * SEG + (lt >> 3) < spr;
    const uint32_t chunk_off = lane_valid ? (uint32_t)(h * SEG + (lt >> 3)) * 144u : 0u;
    const uint32_t chunk_qoff = chunk_off + 16u + 16u * (uint32_t)j;
    auto issue = [&](int t, uint4 &h4, uint4 &q4) {
        const bool real = t < nt_wave;  // wave-uniform
        int row = wave_r0 + t * RPT + tm;
        if (RPT > 1) row = row < wave_r1 ? row : wave_r1 - 1;  // a ragged last task re-reads the last row
        const uint32_t ro = real ? (uint32_t)row * rowbytes : 0u;
        h4 = *reinterpret_cast<const uint4 *>(W + (ro + (real ? chunk_off : 0u)));
        q4 = *reinterpret_cast<const uint4 *>(W + (ro + (real ? chunk_qoff : 0u)));
    };

    uint4 x_lo[kStagePre], x_hi[kStagePre];
    stage_x_begin<ORDER, XF32>(xg, slots, nthreads, x_lo, x_hi, spr * 8);
    uint4 bh[kDepth], bq[kDepth];
#pragma unroll
    for (int i = 0; i < kPreA; i++) issue(i, bh[i], bq[i]);
    stage_x_finish<ORDER, NDIG, XF32>(xg, slots, nthreads, x_lo, x_hi, xd, xm, spr * 8);
    __syncthreads();

    const ScaleSel s0 = scale_sel(ORDER == 0 ? j : 2 * (j >> 1));
    const ScaleSel s1 = scale_sel(ORDER == 0 ? j : 2 * (j >> 1) + 1);
    uint4 xr[NDIG];
#pragma unroll
    for (int k = 0; k < NDIG; k++) xr[k] = xd[k * slots + h * T + lt];
    const float4 xmr = xm[h * T + lt];

    // chunk sums: row (g, t * RPT + tm) of the padded layout, column h
    const int npad = n_nominal * RPT;
    float *pp = part + (size_t)(g * npad + tm) * ks + h;
    const int pstride = RPT * ks;  // floats between consecutive tasks

    auto consume = [&](int t, const uint4 &h4, const uint4 &q4) {
        if (t < nt_wave) {
            const float mine = lane_dot<ORDER, NDIG>(h4, q4, s0, s1, xr, xmr);
            const float v = team_sum_last<T>(RAGGED && !lane_valid ? 0.0f : mine);
            if (lt == T - 1) pp[(size_t)t * pstride] = v;
        }
    };

    // First round: the ring fills up while the first tasks are consumed (kFillA more requests per task consumed),
    // so no wave sits in front of the load unit with nothing to compute.
    int issued = kPreA;
#pragma unroll
    for (int i = 0; i < kDepth; i++) {
        consume(i, bh[i], bq[i]);
        const int upto = SINGLE ? (kPreA + kFillA * (i + 1) < kDepth ? kPreA + kFillA * (i + 1) : kDepth)
                                : (kPreA + kFillA * (i + 1) < kDepth + i + 1 ? kPreA + kFillA * (i + 1) : kDepth + i + 1);
#pragma unroll
        for (; issued < upto; issued++) issue(issued, bh[issued % kDepth], bq[issued % kDepth]);
    }
    if (!SINGLE) {
        // steady rounds: consume task t, refill its buffer with task t + kDepth
        int base = kDepth;
        for (; base + kDepth < n_nominal; base += kDepth) {
#pragma unroll
            for (int i = 0; i < kDepth; i++) {
                consume(base + i, bh[i], bq[i]);
                issue(base + kDepth + i, bh[i], bq[i]);
            }
        }
        // last round: nothing left to request
#pragma unroll
        for (int i = 0; i < kDepth; i++) consume(base + i, bh[i], bq[i]);
    }
    __syncthreads();

    // Row totals: one thread per row adds the row's chunk sums in chunk order.
    const int wg_rows = wg_r1 - wg_r0;
    for (int rl = (int)threadIdx.x; rl < wg_rows; rl += nthreads) {
        const int grp = rl / rows_per_wave, loc = rl - grp * rows_per_wave;
        const float *src = part + (size_t)(grp * npad + loc) * ks;
        float sum = src[0];
        for (int i = 1; i < ks; i++) sum += src[i];
        y[wg_r0 + rl] = sum;
    }
}

// ---- kernel R: a wave owns whole rows ---------------------------------------------------------------
// Rows of KS = 1 or 2 chunks (k = 2048 or 4096) with few enough rows per wave that all of a wave's tasks fit the ring
// (rows per wave * KS <= kDepth): a wave takes both chunks of its rows, so the digits of both stay in registers (48
// VGPRs), adds a row's two lane sums before the in-wave reduction (one reduction per row, not per task), and needs no
// other wave for a row total: the last lane drops it into LDS and, after its last task, the wave reads its own totals
// back (LDS keeps a wave's accesses in order) and stores them as one coalesced store.  No second barrier, no common
// end: two workgroups of eight waves per compute unit run out of step, so that one converts x or stores y while the
// other streams.  From HBM 4.7 % faster than kernel A at 14336 x 4096 (7.28 against 7.63 us on the same machine);
// with the tensor resident in the last-level cache 3 % slower (there one workgroup of 16 waves is the better shape).
constexpr int kRowsWaves = 8;         // waves per workgroup
constexpr int kRowsPerWaveMax = 8;    // row totals a wave keeps in LDS (kDepth tasks of one chunk each)

template <int ORDER, bool XF32, int KS, bool MULTI, bool Q6LAST = false>
__global__ __launch_bounds__(64 * kRowsWaves) void k_qgemv_q4k_rows(const void *__restrict__ xg, const uint8_t *__restrict__ w0,
                                                                     const uint8_t *__restrict__ w1, const uint8_t *__restrict__ w2,
                                                                     const uint8_t *__restrict__ w3, int wg_b1, int wg_b2, int wg_b3,
                                                                     int spr, int rows_per_wg, int n0, int n1, int n2, int n3,
                                                                     float *__restrict__ y0, float *__restrict__ y1,
                                                                     float *__restrict__ y2, float *__restrict__ y3) {
    // Up to four matrices that share k and the activation vector go through one launch (MULTI): workgroups
    // [wg_b(g), wg_b(g + 1)) belong to matrix g (workgroup-uniform selects); otherwise only w0, n0, y0 are looked at.
    static_assert(pmh::kMaxGemvGroup == 4, "the argument list spells out four group members");
    static_assert(MULTI || !Q6LAST, "the Q6_K member is the fourth of a group");
    const int bx = (int)blockIdx.x;
    extern __shared__ uint4 smem[];
    if (Q6LAST && bx >= wg_b3) {
        // Q6LAST: the fourth member is a small Q6_K matrix over the same activations (an attention v projection beside
        // q and k); its workgroups run the small-matrix Q6_K kernel's body, one team per wave
        q6k_small_body<64, XF32>(w3, xg, y3, n3, spr, bx - wg_b3, (int)gridDim.x - wg_b3, kRowsWaves, smem);
        return;
    }
    const int g = MULTI ? (bx >= wg_b1 ? 1 : 0) + (bx >= wg_b2 ? 1 : 0) + (bx >= wg_b3 ? 1 : 0) : 0;
    const uint8_t *__restrict__ W = g == 0 ? w0 : g == 1 ? w1 : g == 2 ? w2 : w3;
    float *__restrict__ y = g == 0 ? y0 : g == 1 ? y1 : g == 2 ? y2 : y3;
    const int n_rows = g == 0 ? n0 : g == 1 ? n1 : g == 2 ? n2 : n3;
    const int wg_index = bx - (g == 0 ? 0 : g == 1 ? wg_b1 : g == 2 ? wg_b2 : wg_b3);
    constexpr int NDIG = XF32 ? 6 : 5;
    constexpr int T = 64, nthreads = 64 * kRowsWaves;
    const int slots = spr * 8;
    uint4 *xd = smem;
    float4 *xm = reinterpret_cast<float4 *>(xd + NDIG * slots);
    float *part = reinterpret_cast<float *>(xm + slots);  // [kRowsWaves][kRowsPerWaveMax]
    const int lane = threadIdx.x & 63, j = lane & 7;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int wg_r0 = wg_index * rows_per_wg;
    const int wg_r1 = wg_r0 + rows_per_wg < n_rows ? wg_r0 + rows_per_wg : n_rows;
    const int wg_rows = wg_r1 - wg_r0;
    // the first `rem` waves take one row more: consecutive waves sit on different SIMDs, so the SIMDs stay balanced
    const int base = wg_rows / kRowsWaves, rem = wg_rows - base * kRowsWaves;
    const int cnt = base + (wave < rem ? 1 : 0);
    const int r0 = wg_r0 + wave * base + (wave < rem ? wave : rem);
    const int nt_wave = cnt * KS;
    const uint32_t rowbytes = (uint32_t)spr * 144u;
    const uint32_t lane_off = (uint32_t)(lane >> 3) * 144u;
    float *pp = part + wave * kRowsPerWaveMax;
    // task t = chunk t % KS of row r0 + t / KS; every load is unconditional (see kernel A)
    auto issue = [&](int t, uint4 &h4, uint4 &q4) {
        const bool real = t < nt_wave;
        const int row = r0 + t / KS, h = t % KS;
        const uint32_t ro = real ? (uint32_t)row * rowbytes + (uint32_t)h * (8u * 144u) + lane_off : 0u;
        h4 = *reinterpret_cast<const uint4 *>(W + ro);
        q4 = *reinterpret_cast<const uint4 *>(W + (ro + (real ? 16u + 16u * (uint32_t)j : 0u)));
    };
    uint4 x_lo[kStagePre], x_hi[kStagePre];
    stage_x_begin<ORDER, XF32>(xg, slots, nthreads, x_lo, x_hi, slots);
    uint4 bh[kDepth], bq[kDepth];
#pragma unroll
    for (int i = 0; i < kPre; i++) issue(i, bh[i], bq[i]);
    stage_x_finish<ORDER, NDIG, XF32>(xg, slots, nthreads, x_lo, x_hi, xd, xm, slots);
    __syncthreads();
    const ScaleSel s0 = scale_sel(ORDER == 0 ? j : 2 * (j >> 1));
    const ScaleSel s1 = scale_sel(ORDER == 0 ? j : 2 * (j >> 1) + 1);
    uint4 xr[KS][NDIG];
    float4 xmr[KS];
#pragma unroll
    for (int h = 0; h < KS; h++) {
#pragma unroll
        for (int k = 0; k < NDIG; k++) xr[h][k] = xd[k * slots + h * T + lane];
        xmr[h] = xm[h * T + lane];
    }
    float rowacc = 0.0f;
    auto consume = [&](int t, int h, const uint4 &h4, const uint4 &q4) {  // h = t % KS, a compile-time constant at every call
        if (t < nt_wave) {
            const float v = lane_dot<ORDER, NDIG>(h4, q4, s0, s1, xr[h], xmr[h]);
            rowacc = h == 0 ? v : rowacc + v;
            if (h == KS - 1) {
                const float total = team_sum_last<T>(rowacc);
                if (lane == T - 1) pp[t / KS] = total;
            }
        }
    };
    static_assert(kDepth % 2 == 0 && kRowsPerWaveMax >= kDepth, "a round holds whole rows, and every row total has its slot");
    // one round: the ring fills up while the first tasks are consumed (two requests per task consumed)
    int issued = kPre;
#pragma unroll
    for (int i = 0; i < kDepth; i++) {
        consume(i, i % KS, bh[i], bq[i]);
        const int upto = kPre + 2 * (i + 1) < kDepth ? kPre + 2 * (i + 1) : kDepth;
#pragma unroll
        for (; issued < upto; issued++) issue(issued, bh[issued % kDepth], bq[issued % kDepth]);
    }
    if (lane < cnt) y[r0 + lane] = pp[lane];
}

// ---- kernel B: general shapes -------------------------------------------------------------------
// A team of T lanes walks a contiguous chunk of rows as one linear stream of tasks, T/8 * 144 bytes apart,
// re-reading its x digits from LDS for every task and reducing with DPP at the end of every row.
constexpr int kRing = 8;

// Up to kMaxGroup weight matrices that share k and the activation vector (the q / k / v or the gate / up
// projections of a decoder layer) go through one launch: x is converted once per workgroup instead of once
// per matrix and launch.  Workgroups [wg_begin[g], wg_begin[g + 1]) belong to matrix g.
struct GemvGroup {
    const uint8_t *w[pmh::kMaxGemvGroup];
    float *y[pmh::kMaxGemvGroup];
    int n[pmh::kMaxGemvGroup];
    int wg_begin[pmh::kMaxGemvGroup + 1];
};

// The arguments come as scalars, the ones needed first up front: the leading 16 dwords of the kernel-argument
// segment are preloaded into scalar registers at wave launch (the translation unit is built with
// -amdgpu-kernarg-preload-count=16), so the first weight request does not wait for an argument fetch.
// Q6LAST: the fourth member is a Q6_K matrix (the v projection of a layer whose q and k are Q4_K): the workgroups from
// wg_b3 on run the small-matrix Q6_K GEMV over it, with q6_teams teams of T lanes each taking rows.
template <int ORDER, bool XF32, int T, bool Q6LAST>
__global__ __launch_bounds__(1024) void k_qgemv_q4k(const void *__restrict__ xg, const uint8_t *__restrict__ w0,
                                                     const uint8_t *__restrict__ w1, const uint8_t *__restrict__ w2,
                                                     const uint8_t *__restrict__ w3, int wg_b1, int wg_b2, int wg_b3,
                                                     int spr, int rows_per_wg, int per_team, int n0, int n1, int n2,
                                                     int n3, float *__restrict__ y0, float *__restrict__ y1,
                                                     float *__restrict__ y2, float *__restrict__ y3, int nthreads, int q6_teams) {
    static_assert(pmh::kMaxGemvGroup == 4, "the argument list spells out four group members");
    const int bx = (int)blockIdx.x;
    if (Q6LAST && bx >= wg_b3) {  // workgroup-uniform
        extern __shared__ uint4 smem6[];
        q6k_small_body<T, XF32>(w3, xg, y3, n3, spr, bx - wg_b3, (int)gridDim.x - wg_b3, q6_teams, smem6);
        return;
    }
    const int g = (bx >= wg_b1 ? 1 : 0) + (bx >= wg_b2 ? 1 : 0) + (bx >= wg_b3 ? 1 : 0);
    const uint8_t *__restrict__ W = g == 0 ? w0 : g == 1 ? w1 : g == 2 ? w2 : w3;
    float *__restrict__ y = g == 0 ? y0 : g == 1 ? y1 : g == 2 ? y2 : y3;
    const int n_rows = g == 0 ? n0 : g == 1 ? n1 : g == 2 ? n2 : n3;
    const int wg_index = bx - (g == 0 ? 0 : g == 1 ? wg_b1 : g == 2 ? wg_b2 : wg_b3);
    constexpr int NDIG = XF32 ? 6 : 5;
    constexpr int SEG = T / 8;         // super-blocks a team covers per task
    constexpr int STRIDE = SEG * 144;  // bytes between a lane's consecutive tasks
    extern __shared__ uint4 smem[];
    const int slots = spr * 8;
    uint4 *xd = smem;
    float4 *xm = reinterpret_cast<float4 *>(xd + NDIG * slots);

    const int lane = threadIdx.x & 63;
    const int lt = lane & (T - 1);
    const int j = lane & 7;
    const int iters = spr / SEG;  // tasks per row
    constexpr int kTeamsPerWave = 64 / T;
    // with full-wave teams everything about a team is wave-uniform: keep it in scalar registers
    auto uni = [](int v) { return T == 64 ? __builtin_amdgcn_readfirstlane(v) : v; };
    const int team = uni((int)(threadIdx.x >> 6) * kTeamsPerWave + lane / T);

    // contiguous chunk of rows for this workgroup, then `per_team` of them for this team
    const int wg_r0 = wg_index * rows_per_wg;
    const int wg_r1 = wg_r0 + rows_per_wg < n_rows ? wg_r0 + rows_per_wg : n_rows;
    const int r0 = wg_r0 + team * per_team;
    const int r1 = r0 + per_team < wg_r1 ? r0 + per_team : wg_r1;
    const int n_tasks = (r1 > r0 ? r1 - r0 : 0) * iters;  // this team's tasks
    const int n_nominal = per_team * iters;               // workgroup-uniform upper bound

    // A team's tasks are one linear stream: task t of the team starts STRIDE * t bytes after its first.
    const uint8_t *ph = W + (size_t)(n_tasks > 0 ? r0 : 0) * spr * 144 + (size_t)(lt >> 3) * 144;
    const uint8_t *pq = ph + 16 + 16 * j;

    // kRing tasks are in flight per team.  They are requested before x is converted, so the memory system
    // streams while the staging runs, and each buffer is refilled as soon as it has been consumed.
    uint4 x_lo[kStagePre], x_hi[kStagePre];
    stage_x_begin<ORDER, XF32>(xg, slots, nthreads, x_lo, x_hi, slots);
    uint4 bh[kRing], bq[kRing];
#pragma unroll
    for (int i = 0; i < kRing; i++) {
        if (i < n_tasks) {
            bh[i] = *reinterpret_cast<const uint4 *>(ph + i * STRIDE);
            bq[i] = *reinterpret_cast<const uint4 *>(pq + i * STRIDE);
        }
    }
    stage_x_finish<ORDER, NDIG, XF32>(xg, slots, nthreads, x_lo, x_hi, xd, xm, slots);
    __syncthreads();

    const ScaleSel s0 = scale_sel(ORDER == 0 ? j : 2 * (j >> 1));
    const ScaleSel s1 = scale_sel(ORDER == 0 ? j : 2 * (j >> 1) + 1);
    float acc = 0.0f;
    int it = 0;  // position inside the row: the same for every team of the workgroup
    int row = r0;
    for (int first = 0; first < n_nominal; first += kRing) {
#pragma unroll
        for (int i = 0; i < kRing; i++) {
            if (first + i < n_nominal) {
                const bool valid = first + i < n_tasks;
                if (valid) {
                    const int slot = it * T + lt;
                    uint4 xdig[NDIG];
#pragma unroll
                    for (int k = 0; k < NDIG; k++) xdig[k] = xd[k * slots + slot];
                    acc += lane_dot<ORDER, NDIG>(bh[i], bq[i], s0, s1, xdig, xm[slot]);
                }
                if (first + i + kRing < n_tasks) {  // refill this buffer with the task kRing ahead
                    bh[i] = *reinterpret_cast<const uint4 *>(ph + (size_t)(i + kRing) * STRIDE);
                    bq[i] = *reinterpret_cast<const uint4 *>(pq + (size_t)(i + kRing) * STRIDE);
                }
                if (++it == iters) {
                    const float total = team_sum_last<T>(acc);
                    if (lt == T - 1 && valid) y[row] = total;
                    row++;
                    acc = 0.0f;
                    it = 0;
                }
            }
        }
        ph += kRing * STRIDE;
        pq += kRing * STRIDE;
    }
}

template <typename Kern, typename... Args>
hipError_t launch_with_lds(Kern kern, dim3 grid, dim3 block, size_t lds, hipStream_t s, Args... args) {
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kern, grid, block, lds, s, args...);
    return hipGetLastError();
}

template <int ORDER, bool XF32>
hipError_t launch_chunk(int T, bool single, dim3 grid, dim3 block, size_t lds, hipStream_t s, const uint8_t *w,
                        const void *x, float *y, int n, int spr, int rows_per_wg, int rows_per_wave, int n_nominal,
                        const uint8_t *w1, int split_wg, float *y1, int n1, bool ragged) {
    if (ragged) {
        if (n1 > 0)
            return single ? launch_with_lds(k_qgemv_q4k_chunk<ORDER, XF32, 64, true, true, true>, grid, block, lds, s, w, w1, x, split_wg, n,
                                            n1, spr, rows_per_wg, rows_per_wave, n_nominal, (int)block.x, y, y1)
                          : launch_with_lds(k_qgemv_q4k_chunk<ORDER, XF32, 64, false, true, true>, grid, block, lds, s, w, w1, x, split_wg, n,
                                            n1, spr, rows_per_wg, rows_per_wave, n_nominal, (int)block.x, y, y1);
        return single ? launch_with_lds(k_qgemv_q4k_chunk<ORDER, XF32, 64, true, false, true>, grid, block, lds, s, w, w1, x, split_wg, n, n1,
                                        spr, rows_per_wg, rows_per_wave, n_nominal, (int)block.x, y, y1)
                      : launch_with_lds(k_qgemv_q4k_chunk<ORDER, XF32, 64, false, false, true>, grid, block, lds, s, w, w1, x, split_wg, n, n1,
                                        spr, rows_per_wg, rows_per_wave, n_nominal, (int)block.x, y, y1);
    }
#define PMH_GO(TT)                                                                                                       \
    if (n1 > 0)                                                                                                                    \
        return single ? launch_with_lds(k_qgemv_q4k_chunk<ORDER, XF32, TT, true, true>, grid, block, lds, s, w, w1, x, split_wg, n, n1,  \
                                        spr, rows_per_wg, rows_per_wave, n_nominal, (int)block.x, y, y1)                      \
                      : launch_with_lds(k_qgemv_q4k_chunk<ORDER, XF32, TT, false, true>, grid, block, lds, s, w, w1, x, split_wg, n, n1, \
                                        spr, rows_per_wg, rows_per_wave, n_nominal, (int)block.x, y, y1);                     \
    return single ? launch_with_lds(k_qgemv_q4k_chunk<ORDER, XF32, TT, true, false>, grid, block, lds, s, w, w1, x, split_wg, n, n1,     \
                                    spr, rows_per_wg, rows_per_wave, n_nominal, (int)block.x, y, y1)                          \
                  : launch_with_lds(k_qgemv_q4k_chunk<ORDER, XF32, TT, false, false>, grid, block, lds, s, w, w1, x, split_wg, n, n1,    \
                                    spr, rows_per_wg, rows_per_wave, n_nominal, (int)block.x, y, y1)
    switch (T) {
    case 8: PMH_GO(8);
    case 16: PMH_GO(16);
    case 32: PMH_GO(32);
    default: PMH_GO(64);
    }
#undef PMH_GO
}

template <int ORDER, bool XF32>
hipError_t launch_general(int T, dim3 grid, dim3 block, size_t lds, hipStream_t s, const GemvGroup &grp, const void *x,
                          int spr, int rows_per_wg, int per_team, int q6_teams = 0) {
    auto go = [&](auto kern) {
        return launch_with_lds(kern, grid, block, lds, s, x, grp.w[0], grp.w[1], grp.w[2], grp.w[3], grp.wg_begin[1],
                               grp.wg_begin[2], grp.wg_begin[3], spr, rows_per_wg, per_team, grp.n[0], grp.n[1], grp.n[2],
                               grp.n[3], grp.y[0], grp.y[1], grp.y[2], grp.y[3], (int)block.x, q6_teams);
    };
    if (q6_teams > 0) {
        switch (T) {
        case 8: return go(k_qgemv_q4k<ORDER, XF32, 8, true>);
        case 16: return go(k_qgemv_q4k<ORDER, XF32, 16, true>);
        case 32: return go(k_qgemv_q4k<ORDER, XF32, 32, true>);
        default: return go(k_qgemv_q4k<ORDER, XF32, 64, true>);
        }
    }
    switch (T) {
    case 8: return go(k_qgemv_q4k<ORDER, XF32, 8, false>);
    case 16: return go(k_qgemv_q4k<ORDER, XF32, 16, false>);
    case 32: return go(k_qgemv_q4k<ORDER, XF32, 32, false>);
    default: return go(k_qgemv_q4k<ORDER, XF32, 64, false>);
    }
}

// One to three small Q4_K matrices and one small Q6_K matrix that share k and x in one launch of kernel B: the workgroups
// are divided between the two kinds by their bytes.
hipError_t launch_group_mixed(const uint8_t *const *w, const int64_t *n, float *const *y, int count, const uint8_t *w6, int64_t n6,
                              float *y6, int64_t k, const void *x, bool xf32, uint32_t order, hipStream_t s) {
    const int spr = (int)(k / 256);
    const int T = 8 * pow2_divisor(spr, 8);
    const size_t slots = (size_t)spr * 8;
    const size_t lds4 = slots * 16 * (xf32 ? 6 : 5) + slots * 16, lds6 = slots * 64 * (xf32 ? 3 : 1) + slots * 16;
    const size_t lds = lds4 > lds6 ? lds4 : lds6;
    if (lds > kMaxLds || count < 1 || count > pmh::kMaxGemvGroup - 1) return hipErrorNotSupported;
    int64_t total = 0;
    for (int i = 0; i < count; i++) total += n[i];
    const int64_t cus = compute_units();
    if (total + n6 < 2 * cus) return hipErrorNotSupported;  // too small to divide
    // a Q6_K byte costs more instructions than a Q4_K byte: its share is weighted by 1.3 (measured flat from 1.15 to 1.8)
    const double b4 = (double)total * spr * 144.0, b6 = (double)n6 * spr * 210.0 * 1.3;
    int64_t wgs6 = (int64_t)((double)cus * b6 / (b4 + b6) + 0.5);
    wgs6 = wgs6 < 1 ? 1 : (wgs6 > cus - count ? cus - count : wgs6);
    const int64_t wgs4 = cus - wgs6;
    int64_t rows_per_wg = (total + wgs4 - 1) / wgs4;
    for (;;) {
        int64_t c = 0;
        for (int i = 0; i < count; i++) c += (n[i] + rows_per_wg - 1) / rows_per_wg;
        if (c <= wgs4 || rows_per_wg >= total) break;
        rows_per_wg++;
    }
    GemvGroup grp{};
    int begin = 0;
    for (int i = 0; i < pmh::kMaxGemvGroup - 1; i++) {
        grp.wg_begin[i] = begin;
        if (i < count) {
            grp.w[i] = w[i], grp.y[i] = y[i], grp.n[i] = (int)n[i];
            begin += (int)((n[i] + rows_per_wg - 1) / rows_per_wg);
        } else {
            grp.w[i] = w[0], grp.y[i] = y[0], grp.n[i] = 0;
        }
    }
    grp.wg_begin[3] = begin;  // the Q6_K member starts here
    grp.w[3] = w6, grp.y[3] = y6, grp.n[3] = (int)n6;
    const dim3 grid((unsigned)(begin + wgs6));
    const int teams_per_wave = 64 / T;
    const int64_t rows6 = (n6 + wgs6 - 1) / wgs6;                 // rows of a Q6_K workgroup: two per team at a time
    int64_t q6_teams = (rows6 + 1) / 2;
    int best_waves = 16;
    int64_t best_cost = INT64_MAX;
    for (int waves = 16; waves >= 1; waves--) {  // as in launch_group_general
        const int64_t teams = (int64_t)waves * teams_per_wave;
        const int64_t per_team = (rows_per_wg + teams - 1) / teams;
        if (per_team < best_cost) best_cost = per_team, best_waves = waves;
    }
    const int64_t teams_avail = (int64_t)best_waves * teams_per_wave;
    q6_teams = q6_teams < 1 ? 1 : (q6_teams > teams_avail ? teams_avail : q6_teams);
    const int per_team = (int)((rows_per_wg + teams_avail - 1) / teams_avail);
    const dim3 block((unsigned)best_waves * 64);
    if (order == pmh::kOrderRef)
        return xf32 ? launch_general<0, true>(T, grid, block, lds, s, grp, x, spr, (int)rows_per_wg, per_team, (int)q6_teams)
                    : launch_general<0, false>(T, grid, block, lds, s, grp, x, spr, (int)rows_per_wg, per_team, (int)q6_teams);
    return xf32 ? launch_general<1, true>(T, grid, block, lds, s, grp, x, spr, (int)rows_per_wg, per_team, (int)q6_teams)
                : launch_general<1, false>(T, grid, block, lds, s, grp, x, spr, (int)rows_per_wg, per_team, (int)q6_teams);
}

// Kernel B over a group of matrices: up to 16 waves; the wave count is the largest that keeps the busiest
// team's row count minimal.
hipError_t launch_group_general(const uint8_t *const *w, const int64_t *n, float *const *y, int count, int64_t k,
                                const void *x, bool xf32, uint32_t order, hipStream_t s) {
    const int spr = (int)(k / 256);
    const int T = 8 * pow2_divisor(spr, 8);
    const size_t slots = (size_t)spr * 8;
    const size_t lds_x = slots * 16 * (xf32 ? 6 : 5) + slots * 16;
    if (lds_x > kMaxLds) return hipErrorInvalidValue;
    int64_t total = 0;
    for (int i = 0; i < count; i++) total += n[i];
    const int64_t want = compute_units();
    int64_t n_wg = total < want ? total : want;
    int64_t rows_per_wg = (total + n_wg - 1) / n_wg;
    // every member rounds its workgroup count up: keep the sum within one workgroup per compute unit (a 257th workgroup
    // would run alone behind the others and nearly double the launch)
    for (;;) {
        int64_t c = 0;
        for (int i = 0; i < count; i++) c += (n[i] + rows_per_wg - 1) / rows_per_wg;
        if (c <= want || rows_per_wg >= total) break;
        rows_per_wg++;
    }
    GemvGroup grp{};
    int begin = 0;
    for (int i = 0; i < pmh::kMaxGemvGroup; i++) {
        grp.wg_begin[i] = begin;
        if (i < count) {
            grp.w[i] = w[i], grp.y[i] = y[i], grp.n[i] = (int)n[i];
            begin += (int)((n[i] + rows_per_wg - 1) / rows_per_wg);
        } else {
            grp.w[i] = w[0], grp.y[i] = y[0], grp.n[i] = 0;
        }
    }
    grp.wg_begin[pmh::kMaxGemvGroup] = begin;
    const dim3 grid((unsigned)begin);
    const int teams_per_wave = 64 / T;
    int best_waves = 16;
    int64_t best_cost = INT64_MAX;
    for (int waves = 16; waves >= 1; waves--) {  // ties go to more waves: more bytes in flight
        const int64_t teams = (int64_t)waves * teams_per_wave;
        const int64_t per_team = (rows_per_wg + teams - 1) / teams;
        if (per_team < best_cost) best_cost = per_team, best_waves = waves;
    }
    const int per_team = (int)((rows_per_wg + (int64_t)best_waves * teams_per_wave - 1) / ((int64_t)best_waves * teams_per_wave));
    const dim3 block((unsigned)best_waves * 64);
    if (order == pmh::kOrderRef)
        return xf32 ? launch_general<0, true>(T, grid, block, lds_x, s, grp, x, spr, (int)rows_per_wg, per_team)
                    : launch_general<0, false>(T, grid, block, lds_x, s, grp, x, spr, (int)rows_per_wg, per_team);
    return xf32 ? launch_general<1, true>(T, grid, block, lds_x, s, grp, x, spr, (int)rows_per_wg, per_team)
                : launch_general<1, false>(T, grid, block, lds_x, s, grp, x, spr, (int)rows_per_wg, per_team);
}

}  // namespace

namespace pmh {

// Kernel R over one to four matrices that share k, x and the element order.  hipErrorNotSupported when the shapes do not
// suit it (rows of more than two chunks or not whole chunks, more rows per wave than the ring holds tasks, offsets beyond
// 32 bits): the caller goes on to another kernel.
template <int ORDER, bool XF32>
static hipError_t launch_rows_kernel(int ks, bool multi, bool q6last, dim3 grid, size_t lds, hipStream_t s, const GemvGroup &grp,
                                     const void *x, int spr, int rows_per_wg) {
    const dim3 block(64 * kRowsWaves);
    auto go = [&](auto kern) {
        return launch_with_lds(kern, grid, block, lds, s, x, grp.w[0], grp.w[1], grp.w[2], grp.w[3], grp.wg_begin[1], grp.wg_begin[2],
                               grp.wg_begin[3], spr, rows_per_wg, grp.n[0], grp.n[1], grp.n[2], grp.n[3], grp.y[0], grp.y[1], grp.y[2],
                               grp.y[3]);
    };
    if (q6last) return ks == 2 ? go(k_qgemv_q4k_rows<ORDER, XF32, 2, true, true>) : go(k_qgemv_q4k_rows<ORDER, XF32, 1, true, true>);
    if (ks == 2) return multi ? go(k_qgemv_q4k_rows<ORDER, XF32, 2, true>) : go(k_qgemv_q4k_rows<ORDER, XF32, 2, false>);
    return multi ? go(k_qgemv_q4k_rows<ORDER, XF32, 1, true>) : go(k_qgemv_q4k_rows<ORDER, XF32, 1, false>);
}

// w6 / n6 / y6: a small Q6_K matrix over the same activations that rides along as the fourth member (n6 == 0: none); its
// workgroups come on top of the Q4_K members' share.
static hipError_t launch_kernel_rows(const uint8_t *const *w, const int64_t *n, float *const *y, int count, int64_t k, const void *x,
                                     bool xf32, uint32_t order, hipStream_t s, const uint8_t *w6 = nullptr, int64_t n6 = 0,
                                     float *y6 = nullptr) {
    const int spr = (int)(k / 256);
    if (spr % 8 != 0 || spr / 8 > 2 || count < 1 || count > kMaxGemvGroup - (n6 > 0 ? 1 : 0)) return hipErrorNotSupported;
    const int ks = spr / 8;
    int64_t total = 0, n_max = 0;
    for (int i = 0; i < count; i++) total += n[i], n_max = n[i] > n_max ? n[i] : n_max;
    if ((uint64_t)n_max * (uint64_t)spr * 144u >= (1ull << 32)) return hipErrorNotSupported;
    // Two workgroups per compute unit; a launch of several matrices that would leave a wave more tasks than the ring holds
    // takes four per compute unit instead (two rounds, and the end of one workgroup overlaps the start of the next).
    const int64_t cus = gemv::compute_units();
    const int64_t max_rows_per_wg = (int64_t)kRowsWaves * (kDepth / ks);
    int64_t want = 2 * cus;
    if (count > 1 && (total + want - 1) / want > max_rows_per_wg) want = 4 * cus;
    // the Q6_K member: a team (one wave) walks two rows at a time, so one workgroup per 16 rows, at most half of all
    int64_t wgs6 = 0;
    if (n6 > 0) {
        if ((uint64_t)n6 * (uint64_t)spr * 210u >= (1ull << 31)) return hipErrorNotSupported;
        wgs6 = (n6 + 2 * kRowsWaves - 1) / (2 * kRowsWaves);
        wgs6 = wgs6 > want / 2 ? want / 2 : wgs6;
        want -= wgs6;
    }
    int64_t n_wg = total < want ? total : want;
    int64_t rows_per_wg = (total + n_wg - 1) / n_wg;
    // every member rounds its workgroup count up: keep the sum within the intended number of workgroups
    for (;;) {
        int64_t c = 0;
        for (int i = 0; i < count; i++) c += (n[i] + rows_per_wg - 1) / rows_per_wg;
        if (c <= want || rows_per_wg >= total) break;
        rows_per_wg++;
    }
    if (rows_per_wg > max_rows_per_wg) return hipErrorNotSupported;
    GemvGroup grp{};
    int begin = 0;
    for (int i = 0; i < kMaxGemvGroup; i++) {
        grp.wg_begin[i] = begin;
        if (i < count) {
            grp.w[i] = w[i], grp.y[i] = y[i], grp.n[i] = (int)n[i];
            begin += (int)((n[i] + rows_per_wg - 1) / rows_per_wg);
        } else {
            grp.w[i] = w[0], grp.y[i] = y[0], grp.n[i] = 0;
        }
    }
    grp.wg_begin[kMaxGemvGroup] = begin;
    const size_t slots = (size_t)spr * 8;
    size_t lds = slots * 16 * (xf32 ? 6 : 5) + slots * 16 + (size_t)kRowsWaves * kRowsPerWaveMax * 4;
    const bool q6last = n6 > 0;
    if (q6last) {  // (the unused members before it hold no workgroups: wg_begin[count .. 3] are all `begin`)
        grp.w[kMaxGemvGroup - 1] = w6, grp.y[kMaxGemvGroup - 1] = y6, grp.n[kMaxGemvGroup - 1] = (int)n6;
        const size_t lds6 = slots * 64 * (xf32 ? 3 : 1) + slots * 16;
        lds = lds6 > lds ? lds6 : lds;
    }
    const dim3 grid((unsigned)(begin + wgs6));
    const bool multi = count > 1 || q6last;
    if (order == kOrderRef)
        return xf32 ? launch_rows_kernel<0, true>(ks, multi, q6last, grid, lds, s, grp, x, spr, (int)rows_per_wg)
                    : launch_rows_kernel<0, false>(ks, multi, q6last, grid, lds, s, grp, x, spr, (int)rows_per_wg);
    return xf32 ? launch_rows_kernel<1, true>(ks, multi, q6last, grid, lds, s, grp, x, spr, (int)rows_per_wg)
                : launch_rows_kernel<1, false>(ks, multi, q6last, grid, lds, s, grp, x, spr, (int)rows_per_wg);
}

// Kernel A over one matrix (n1 == 0) or two that share k, x and the element order.  hipErrorNotSupported when the shape
// does not suit it: a row of more than 16 chunks, offsets beyond 32 bits, partial sums that do not fit in LDS.
static hipError_t launch_kernel_a(const uint8_t *w0, int64_t n0, float *y0, const uint8_t *w1, int64_t n1, float *y1, int64_t k,
                                  const void *x, bool xf32, uint32_t order, hipStream_t s) {
    const int spr = (int)(k / 256);
    int T = 8 * gemv::pow2_divisor(spr, 8);
    // rows that a narrower team would cut into more than 16 chunks: whole-wave teams with a short last chunk
    const bool ragged = T < 64 && spr / (T / 8) > 16 && (spr + 7) / 8 <= 16;
    if (ragged) T = 64;
    const size_t slots = ragged ? (size_t)((spr + 7) / 8) * 64 : (size_t)spr * 8;
    const size_t lds_x = slots * 16 * (xf32 ? 6 : 5) + slots * 16;
    if (lds_x > gemv::kMaxLds) return hipErrorNotSupported;
    // Workgroups own contiguous chunks of rows, one per compute unit (x is staged once per workgroup).
    const int64_t n = n0 + n1, want = gemv::compute_units();
    int64_t n_wg = n < want ? n : want;
    const int64_t rows_per_wg = (n + n_wg - 1) / n_wg;
    const int64_t wg0 = (n0 + rows_per_wg - 1) / rows_per_wg, wg1 = (n1 + rows_per_wg - 1) / rows_per_wg;
    const dim3 grid((unsigned)(wg0 + wg1));
    const int ks = ragged ? (spr + 7) / 8 : spr / (T / 8), rpt = 64 / T;
    const uint64_t w_max = (uint64_t)(n0 > n1 ? n0 : n1) * (uint64_t)spr * 144u;
    if (ks > 16 || w_max >= (1ull << 32)) return hipErrorNotSupported;
    int64_t groups = 16 / ks;
    const int64_t max_groups = (rows_per_wg + rpt - 1) / rpt;
    if (groups > max_groups) groups = max_groups;
    const int64_t rows_per_wave = (rows_per_wg + groups - 1) / groups;
    groups = (rows_per_wg + rows_per_wave - 1) / rows_per_wave;
    const int64_t n_nominal = (rows_per_wave + rpt - 1) / rpt;
    const int64_t threads = ks * groups * 64;
    const size_t lds = lds_x + (size_t)groups * (size_t)n_nominal * rpt * ks * 4;
    if (lds > 128 * 1024) return hipErrorNotSupported;
    const dim3 block((unsigned)threads);
    const bool single = n_nominal <= kDepth;
    const int a_n = (int)n0, a_rpw = (int)rows_per_wg, a_rpv = (int)rows_per_wave, a_nn = (int)n_nominal;
    const uint8_t *b_w = n1 ? w1 : w0;
    float *b_y = n1 ? y1 : y0;
    const int b_split = (int)wg0, b_n = (int)n1;
    if (order == kOrderRef)
        return xf32 ? launch_chunk<0, true>(T, single, grid, block, lds, s, w0, x, y0, a_n, spr, a_rpw, a_rpv, a_nn, b_w, b_split, b_y, b_n, ragged)
                    : launch_chunk<0, false>(T, single, grid, block, lds, s, w0, x, y0, a_n, spr, a_rpw, a_rpv, a_nn, b_w, b_split, b_y, b_n, ragged);
    return xf32 ? launch_chunk<1, true>(T, single, grid, block, lds, s, w0, x, y0, a_n, spr, a_rpw, a_rpv, a_nn, b_w, b_split, b_y, b_n, ragged)
                : launch_chunk<1, false>(T, single, grid, block, lds, s, w0, x, y0, a_n, spr, a_rpw, a_rpv, a_nn, b_w, b_split, b_y, b_n, ragged);
}

// Preconditions as for launch_qgemv.  Returns hipErrorInvalidValue when x does not fit in LDS.
hipError_t launch_qgemv_q4k(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y,
                            uint32_t order, hipStream_t s) {
    const bool xf32 = x_dtype == kDtypeF32;
    const int spr = (int)(k / 256);
    const size_t slots = (size_t)spr * 8;
    const size_t lds_x = slots * 16 * (xf32 ? 6 : 5) + slots * 16;
    if (lds_x > gemv::kMaxLds) return hipErrorInvalidValue;
    const uint64_t w_bytes = (uint64_t)n * (uint64_t)spr * 144u;
    // Measured crossovers against kernel B: the row-owner kernel from about 8 MiB (4096 x 4096: 4.21 against 4.28 us,
    // 5120 x 4096: 4.5 against 5.4; 2048 x 4096: 3.7 against 3.5), kernel A from about 12 MiB.
    if (w_bytes >= (8ull << 20)) {
        const hipError_t e = launch_kernel_rows(&w, &n, &y, 1, k, x, xf32, order, s);
        if (e != hipErrorNotSupported) return e;
    }
    if (w_bytes >= (12ull << 20)) {
        const hipError_t e = launch_kernel_a(w, n, y, nullptr, 0, nullptr, k, x, xf32, order, s);
        if (e != hipErrorNotSupported) return e;
    }
    return launch_group_general(&w, &n, &y, 1, k, x, xf32, order, s);
}

// Two matrices of kernel-A size that share k, x, x_dtype and the element order (the gate / up projections of a large
// model) in one launch.  hipErrorNotSupported when the pair does not suit kernel A: the caller launches them one by one.
hipError_t launch_qgemv_q4k_pair(const uint8_t *w0, int64_t n0, float *y0, const uint8_t *w1, int64_t n1, float *y1, int64_t k,
                                 const void *x, uint32_t x_dtype, uint32_t order, hipStream_t s) {
    const bool xf32 = x_dtype == kDtypeF32;
    const size_t slots = (size_t)(k / 256) * 8;
    if (slots * 16 * (xf32 ? 6 : 5) + slots * 16 > gemv::kMaxLds) return hipErrorNotSupported;
    const uint8_t *ws[2] = {w0, w1};
    const int64_t ns[2] = {n0, n1};
    float *ys[2] = {y0, y1};
    const hipError_t e = launch_kernel_rows(ws, ns, ys, 2, k, x, xf32, order, s);
    if (e != hipErrorNotSupported) return e;
    return launch_kernel_a(w0, n0, y0, w1, n1, y1, k, x, xf32, order, s);
}

// Matrices that kernel A would not take anyway (small ones), sharing k, x, x_dtype and order, in one launch.
bool qgemv_q4k_groupable(int64_t n, int64_t k) { return (uint64_t)n * (uint64_t)(k / 256) * 144u < (12ull << 20); }

// A group of small Q4_K matrices followed by one small Q6_K matrix over the same activations (q, k and a Q6_K v): one
// launch.  hipErrorNotSupported when the shapes do not suit it; the caller launches the two kinds one after the other.
hipError_t launch_qgemv_q4k_q6k_group(const uint8_t *const *w, const int64_t *n, float *const *y, int count, const uint8_t *w6, int64_t n6,
                                      float *y6, int64_t k, const void *x, uint32_t x_dtype, uint32_t order, hipStream_t s) {
    uint64_t bytes = (uint64_t)n6 * (uint64_t)(k / 256) * 210u;
    for (int i = 0; i < count; i++) bytes += (uint64_t)n[i] * (uint64_t)(k / 256) * 144u;
    const bool xf32 = x_dtype == kDtypeF32;
    if (bytes >= (8ull << 20)) {  // a large group streams through the row-owner kernel, the Q6_K member as its fourth
        const size_t slots = (size_t)(k / 256) * 8;
        if (slots * 16 * (xf32 ? 6 : 5) + slots * 16 > gemv::kMaxLds) return hipErrorNotSupported;
        return launch_kernel_rows(w, n, y, count, k, x, xf32, order, s, w6, n6, y6);
    }
    return launch_group_mixed(w, n, y, count, w6, n6, y6, k, x, xf32, order, s);
}

hipError_t launch_qgemv_q4k_group(const uint8_t *const *w, const int64_t *n, float *const *y, int count, int64_t k,
                                  const void *x, uint32_t x_dtype, uint32_t order, hipStream_t s) {
    if (count < 1 || count > kMaxGemvGroup) return hipErrorInvalidValue;
    // a group that is large as a whole (q / k / v of an 8B-class model: 14 MB) streams like one large matrix
    uint64_t bytes = 0;
    for (int i = 0; i < count; i++) bytes += (uint64_t)n[i] * (uint64_t)(k / 256) * 144u;
    const size_t slots = (size_t)(k / 256) * 8;
    const bool xf32 = x_dtype == kDtypeF32;
    if (bytes >= (8ull << 20) && slots * 16 * (xf32 ? 6 : 5) + slots * 16 <= gemv::kMaxLds) {
        const hipError_t e = launch_kernel_rows(w, n, y, count, k, x, xf32, order, s);
        if (e != hipErrorNotSupported) return e;
    }
    return launch_group_general(w, n, y, count, k, x, xf32, order, s);
}

}  // namespace pmh
