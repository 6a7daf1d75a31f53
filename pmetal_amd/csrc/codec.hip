// Bit-exact f32 <-> {Q8_0, Q4_K, Q6_K} kernels for gfx950.
//
// The results must equal the reference CPU path bit for bit, so this file is compiled with
// -ffp-contract=off: every `a * b + c` below is two roundings, as in the Rust it follows
// (Rust never fuses).  Divisions are IEEE-correct (hipcc's default
// -fhip-fp32-correctly-rounded-divide-sqrt), rounding is half-away-from-zero done exactly, and
// every float sum of the two scale searches is accumulated sequentially in element order by ONE
// lane -- a tree or cross-lane reduction would change the bits.  Only min/max, which are
// order-independent, are reduced across lanes.
//
// Reference functions followed (paths under crates/pmetal-gguf/src/):
//   quantize.rs:268-300 quantize_q8_0        quantize.rs:583-644 make_qkx1_quants
//   quantize.rs:738-841 make_qx_quants       k_quants.rs:876-955 quantize_q4k
//   k_quants.rs:1056-1134 quantize_q6k       dequant.rs:466-495 dequantize_q8_0
//   k_quants.rs:358-404 dequantize_q4k       k_quants.rs:474-496 dequantize_q6k
#include "internal.hpp"

#pragma clang fp contract(off)

namespace {

typedef uint32_t u32_a2 __attribute__((aligned(2)));  // dword at a 2-byte aligned address
typedef uint32_t u32_a1 __attribute__((aligned(1)));

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// half::f16::from_f32: IEEE round-to-nearest-even (v_cvt_f16_f32; f16 denormals are on by default).
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}

// f32::round: half away from zero.  v - trunc(v) is exact, so this is too.
__device__ __forceinline__ float round_half_away(float v) {
    float t = __builtin_truncf(v);
    float diff = v - t;
    return (__builtin_fabsf(diff) >= 0.5f) ? t + __builtin_copysignf(1.0f, v) : t;
}

// clamp(nearest_int(v), lo, hi) with Rust's `as i32` (NaN -> 0, saturating); needs lo <= 0 <= hi.
__device__ __forceinline__ float clamp_round(float v, float lo, float hi) {
    float r = round_half_away(v);
    r = (r != r) ? 0.0f : r;
    return __builtin_fminf(__builtin_fmaxf(r, lo), hi);
}

// clamp(nearest_int(v), 0, 15) in three instructions: clamp first (the bounds are integers, so clamping commutes with
// rounding; NaN -> 0 as `as i32` does), then add the largest float below 0.5 and truncate.  For every w in [0, 15] the
// rounded sum w + 0.49999997 lies on the same side of each integer as w + 0.5 does exactly (checked over all 2^32
// floats on the CPU), so this is round-half-away without a compare.
template <int NMAX = 15>
__device__ __forceinline__ float clamp_round_0_15(float v) {  // NMAX = 31 for the 5-bit quants of Q5_K
    const float w = __builtin_fminf(__builtin_fmaxf(v, 0.0f), (float)NMAX);
    return __builtin_truncf(w + 0.49999997f);
}

// nearest_int(v) = `v.round() as i32` (half away from zero, saturating, NaN -> 0) in three instructions: add the largest
// float below 0.5 to |v|, put the sign back, convert with truncation (the hardware conversion saturates and maps NaN
// to 0; the asm keeps that out of the compiler's reach, for which an out-of-range cast is undefined).  Equal to the
// reference for all 2^32 floats after any clamp to a range inside i32 (checked on the CPU).
__device__ __forceinline__ int nearest_int_sat(float v) {
    const float a = __builtin_fabsf(v) + 0.49999997f;
    int i;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(i) : "v"(__builtin_copysignf(a, v)));
    return i;
}
__device__ __forceinline__ int clamp_i(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// `v as i32` for f32.
__device__ __forceinline__ int f32_as_i32(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return 2147483647;
    if (v <= -2147483648.0f) return -2147483647 - 1;
    return (int)v;
}

// f32::total_cmp key: integer order of the keys is the total order of the floats.
__device__ __forceinline__ int total_key(float v) {
    int b = __builtin_bit_cast(int, v);
    return b ^ (int)(((unsigned)(b >> 31)) >> 1);
}

// -------------------------------------------------------------------------------------------
// Q8_0 quantize (quantize.rs:268-300).  One lane per 4 elements, 8 lanes per 32-element block.
// -------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_quantize_q8_0(const float *__restrict__ x, size_t n,
                                                        uint8_t *__restrict__ dst, size_t n_blocks) {
    const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t blk = tid >> 3;
    const int j = (int)(tid & 7);
    const size_t e = tid * 4;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (e + 3 < n) {
        float4 t = *reinterpret_cast<const float4 *>(x + e);
        v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
    } else {
#pragma unroll
        for (int c = 0; c < 3; c++)
            if (e + c < n) v[c] = x[e + c];
    }
    // amax = fold(0.0, max(|x|)): order-independent, NaN ignored by fmaxf as by f32::max.
    float a = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v[0]), __builtin_fabsf(v[1])),
                              __builtin_fmaxf(__builtin_fabsf(v[2]), __builtin_fabsf(v[3])));
    a = __builtin_fmaxf(a, 0.0f);  // a block of NaNs only folds to 0.0
    a = __builtin_fmaxf(a, __shfl_xor(a, 1));
    a = __builtin_fmaxf(a, __shfl_xor(a, 2));
    a = __builtin_fmaxf(a, __shfl_xor(a, 4));
    const float scale = a / 127.0f;
    const float iscale = (a == 0.0f) ? 0.0f : 127.0f / a;
    uint32_t packed = 0;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        int q = (int)clamp_round(v[c] * iscale, -127.0f, 127.0f);
        if (e + c >= n) q = 0;  // zero-pad the partial last block (quantize.rs:293)
        packed |= ((uint32_t)q & 0xFFu) << (8 * c);
    }
    if (blk < n_blocks) {
        uint8_t *out = dst + blk * 34;
        *reinterpret_cast<u32_a2 *>(out + 2 + 4 * j) = packed;
        if (j == 0) *reinterpret_cast<uint16_t *>(out) = (uint16_t)f32_to_f16_bits(scale);
    }
}

// Four dequantized values as one 16-byte streaming store: the output of a dequantizer is several times its input and is
// not read again by it, so it should not claim room in the caches (measured at 14336 x 4096, Q4_K: 53.2 -> 39.4 us).
__device__ __forceinline__ void store_stream4(float *dst, const float (&o)[4]) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store((f4){o[0], o[1], o[2], o[3]}, reinterpret_cast<f4 *>(dst));
}

// -------------------------------------------------------------------------------------------
// Q8_0 dequantize (dequant.rs:466-495): out = (q as f32) * f16->f32(d).  One lane per 4 outputs.
// -------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_dequantize_q8_0(const uint8_t *__restrict__ src, size_t n,
                                                          float *__restrict__ dst) {
    const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t e = tid * 4;
    if (e >= n) return;
    const uint8_t *blk = src + (tid >> 3) * 34;
    const float d = f16_bits_to_f32(*reinterpret_cast<const uint16_t *>(blk));
    const uint32_t q = *reinterpret_cast<const u32_a2 *>(blk + 2 + 4 * (tid & 7));
    float o[4];
#pragma unroll
    for (int c = 0; c < 4; c++) o[c] = (float)(int8_t)(q >> (8 * c)) * d;
    if (e + 3 < n) {
        store_stream4(dst + e, o);
    } else {
        for (int c = 0; c < 4 && e + c < n; c++) dst[e + c] = o[c];
    }
}

// -------------------------------------------------------------------------------------------
// The 32-element formats beside Q8_0 (FMT = GGML type id): Q4_0 (2: d, 16 bytes of nibbles), Q4_1 (3: d, m, nibbles),
// Q5_0 (6: d, qh, nibbles), Q5_1 (7: d, m, qh, nibbles), Q8_1 (9: d, s, 32 int8).  Low nibbles are elements 0..15, high
// nibbles 16..31; bit i of qh is the fifth bit of element i.  quantize.rs:93-230, :302-359; dequant.rs:300-463, :505-528.
// Eight lanes per block, lane j holding elements 4 j .. 4 j + 3, as in the Q8_0 kernels.
// -------------------------------------------------------------------------------------------
template <int FMT>
struct Legacy32 {
    static constexpr bool kMin = FMT == 3 || FMT == 7, kHigh = FMT == 6 || FMT == 7, kInt8 = FMT == 9;
    static constexpr int kBytes = FMT == 2 ? 18 : FMT == 3 ? 20 : FMT == 6 ? 22 : FMT == 7 ? 24 : 36;
    static constexpr int kQhOff = kMin ? 4 : 2, kQsOff = kInt8 ? 4 : 2 + (kMin ? 2 : 0) + (kHigh ? 4 : 0);
    static constexpr int kMaxQ = kHigh ? 31 : 15;
};

__device__ __forceinline__ bool finite_f32(float v) { return (__builtin_bit_cast(uint32_t, v) & 0x7F800000u) != 0x7F800000u; }

template <int FMT>
__global__ __launch_bounds__(256) void k_quantize_b32(const float *__restrict__ x, size_t n, uint8_t *__restrict__ dst,
                                                       size_t n_blocks) {
    using F = Legacy32<FMT>;
    const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t blk = tid >> 3;
    const int j = (int)(tid & 7);
    const size_t e = tid * 4;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // an element past the end of the tensor counts as 0.0 when it is quantized ...
    bool have[4];                           // ... but takes no part in the block's minimum / maximum
#pragma unroll
    for (int c = 0; c < 4; c++) {
        have[c] = e + c < n;
        if (have[c]) v[c] = x[e + c];
    }
    float scale, mn = 0.0f;
    if (F::kInt8) {  // amax = fold(0.0, max(|x|)), NaN ignored
        float a = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v[0]), __builtin_fabsf(v[1])),
                                  __builtin_fmaxf(__builtin_fabsf(v[2]), __builtin_fabsf(v[3])));
        a = __builtin_fmaxf(a, 0.0f);
        a = __builtin_fmaxf(a, __shfl_xor(a, 1));
        a = __builtin_fmaxf(a, __shfl_xor(a, 2));
        a = __builtin_fmaxf(a, __shfl_xor(a, 4));
        scale = a / 127.0f;
        const float iscale = (a == 0.0f) ? 0.0f : 127.0f / a;
        uint32_t packed = 0;
        int sum = 0;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const int q = (int)clamp_round(v[c] * iscale, -127.0f, 127.0f);
            sum += q;
            packed |= ((uint32_t)q & 0xFFu) << (8 * c);
        }
        sum += __shfl_xor(sum, 1);
        sum += __shfl_xor(sum, 2);
        sum += __shfl_xor(sum, 4);
        if (blk < n_blocks) {
            uint8_t *out = dst + blk * F::kBytes;
            *reinterpret_cast<uint32_t *>(out + 4 + 4 * j) = packed;  // 36-byte blocks: dwords stay aligned
            if (j == 0) {
                *reinterpret_cast<uint16_t *>(out) = (uint16_t)f32_to_f16_bits(scale);
                *reinterpret_cast<uint16_t *>(out + 2) = (uint16_t)f32_to_f16_bits((float)sum * scale);
            }
        }
        return;
    }
    float q[4];
    if (F::kMin) {
        // block_min_max: over the finite elements; (0, 0) if there is none.  Total-order keys, so that of equal zeros the
        // negative one is the minimum and the positive one the maximum.
        int klo = 0x7FFFFFFF, khi = (int)0x80000000;
#pragma unroll
        for (int c = 0; c < 4; c++)
            if (have[c] && finite_f32(v[c])) {
                const int key = total_key(v[c]);
                klo = key < klo ? key : klo;
                khi = key > khi ? key : khi;
            }
#pragma unroll
        for (int off = 1; off < 8; off <<= 1) {
            const int ol = __shfl_xor(klo, off), oh = __shfl_xor(khi, off);
            klo = ol < klo ? ol : klo;
            khi = oh > khi ? oh : khi;
        }
        float mx = 0.0f;
        if (klo <= khi) {  // at least one finite element
            mn = __builtin_bit_cast(float, klo ^ (int)(((unsigned)(klo >> 31)) >> 1));
            mx = __builtin_bit_cast(float, khi ^ (int)(((unsigned)(khi >> 31)) >> 1));
        }
        scale = (mx - mn) / (float)F::kMaxQ;
        const float iscale = scale == 0.0f ? 0.0f : 1.0f / scale;
#pragma unroll
        for (int c = 0; c < 4; c++) q[c] = clamp_round((v[c] - mn) * iscale, 0.0f, (float)F::kMaxQ);
    } else {
        // the element of largest magnitude, the first one among equals (Q5_0: among the finite ones), with its sign
        float amax = 0.0f, smax = 0.0f;
        int idx = 0;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const float ax = __builtin_fabsf(v[c]);
            if (have[c] && (FMT == 2 || finite_f32(v[c])) && ax > amax) amax = ax, smax = v[c], idx = 4 * j + c;
        }
#pragma unroll
        for (int off = 1; off < 8; off <<= 1) {
            const float oa = __shfl_xor(amax, off), os = __shfl_xor(smax, off);
            const int oi = __shfl_xor(idx, off);
            if (oa > amax || (oa == amax && oa > 0.0f && oi < idx)) amax = oa, smax = os, idx = oi;
        }
        scale = smax / (FMT == 2 ? -8.0f : -16.0f);
        const float iscale = scale == 0.0f ? 0.0f : 1.0f / scale;
        const float half_up = FMT == 2 ? 8.5f : 16.5f;
#pragma unroll
        for (int c = 0; c < 4; c++) q[c] = clamp_round(v[c] * iscale + half_up, 0.0f, (float)F::kMaxQ);
    }
    uint32_t nib = 0, hi = 0;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const uint32_t qi = (uint32_t)q[c];
        nib |= (qi & 0xFu) << (8 * c);
        hi |= (qi >> 4) << (4 * j + c);
    }
    const uint32_t other = (uint32_t)__shfl_xor((int)nib, 4);  // lanes 0..3 hold the low, lanes 4..7 the high nibbles
    if (F::kHigh) {
        hi |= (uint32_t)__shfl_xor((int)hi, 1);
        hi |= (uint32_t)__shfl_xor((int)hi, 2);
        hi |= (uint32_t)__shfl_xor((int)hi, 4);
    }
    if (blk < n_blocks) {
        uint8_t *out = dst + blk * F::kBytes;
        if (j < 4) *reinterpret_cast<u32_a2 *>(out + F::kQsOff + 4 * j) = nib | (other << 4);
        if (j == 4) *reinterpret_cast<uint16_t *>(out) = (uint16_t)f32_to_f16_bits(scale);
        if (F::kMin && j == 5) *reinterpret_cast<uint16_t *>(out + 2) = (uint16_t)f32_to_f16_bits(mn);
        if (F::kHigh && j == 6) *reinterpret_cast<u32_a2 *>(out + F::kQhOff) = hi;
    }
}

// One lane per 4 outputs: lane j of a block decodes elements 4 j .. 4 j + 3.
template <int FMT>
__global__ __launch_bounds__(256) void k_dequantize_b32(const uint8_t *__restrict__ src, size_t n, float *__restrict__ dst) {
    using F = Legacy32<FMT>;
    const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t e = tid * 4;
    if (e >= n) return;
    const uint8_t *blk = src + (tid >> 3) * F::kBytes;
    const int j = (int)(tid & 7);
    const float d = f16_bits_to_f32(*reinterpret_cast<const uint16_t *>(blk));
    float o[4];
    if (F::kInt8) {
        const uint32_t q = *reinterpret_cast<const uint32_t *>(blk + 4 + 4 * j);
#pragma unroll
        for (int c = 0; c < 4; c++) o[c] = (float)(int8_t)(q >> (8 * c)) * d;
    } else {
        const float m = F::kMin ? f16_bits_to_f32(*reinterpret_cast<const uint16_t *>(blk + 2)) : 0.0f;
        const uint32_t qs = *reinterpret_cast<const u32_a2 *>(blk + F::kQsOff + 4 * (j & 3)) >> (4 * (j >> 2));
        const uint32_t qh = F::kHigh ? *reinterpret_cast<const u32_a2 *>(blk + F::kQhOff) >> (4 * j) : 0u;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const int q = (int)((qs >> (8 * c)) & 0xFu) | (int)(((qh >> c) & 1u) << 4);
            if (F::kMin) o[c] = (float)q * d + m;
            else o[c] = (float)(q - (F::kHigh ? 16 : 8)) * d;
        }
    }
    if (e + 3 < n) {
        store_stream4(dst + e, o);
    } else {
        for (int c = 0; c < 4 && e + c < n; c++) dst[e + c] = o[c];
    }
}

// get_scale_min_k4 (quantize.rs:844-855) on the 12 scale bytes held as three dwords.
__device__ __forceinline__ void scale_min_k4(int j, uint32_t s0, uint32_t s1, uint32_t s2, uint32_t &sc,
                                             uint32_t &m) {
    const int sh = 8 * (j & 3);
    const uint32_t a = (s0 >> sh) & 0xFFu, b = (s1 >> sh) & 0xFFu, c = (s2 >> sh) & 0xFFu;
    if (j < 4) {
        sc = a & 63u;
        m = b & 63u;
    } else {
        sc = (c & 0xFu) | ((a >> 6) << 4);
        m = (c >> 4) | ((b >> 6) << 4);
    }
}

// -------------------------------------------------------------------------------------------
// Dequantizers of the k-quant formats.  A decoder describes one format: lane i (0..63) of a wave loads its share
// of a super-block (`load`) and turns it into elements 4 i .. 4 i + 3 (`values`), with every operation rounded as
// the reference rounds it.  k_dequantize_kq stores the values; k_kl_sums_kq compares them with the original
// tensor without storing them.  A wave handles kDeqUnroll super-blocks per step and requests the bytes of all of
// them before it computes, so that it has several kilobytes of output per memory round trip.
// ORDER 0: the reference dequantizer's emission order; ORDER 1: the inverse of the quantizer's packing (they differ
// for Q4_K and Q5_K only).
// -------------------------------------------------------------------------------------------
constexpr int kDeqUnroll = 4;

// Q4_K (k_quants.rs:358-404 + :515-560): out = (d*sc) * nibble - (dmin*m).
template <int ORDER>
struct DecQ4K {
    static constexpr int kBytes = 144;
    struct Raw {
        uint4 hdr;
        uint32_t q;
    };
    static __device__ __forceinline__ void where(int i, int &byte, int &hi, int &sb) {
        const int c = i >> 4;        // 64-element chunk
        const int p = (i & 15) * 4;  // position inside the chunk
        if (ORDER == 0) {
            byte = 32 * c + (p & 15) + 16 * (p >> 5);
            hi = (p >> 4) & 1;
        } else {
            byte = 32 * c + (p & 31);
            hi = p >> 5;
        }
        sb = 2 * c + (p >> 5);
    }
    static __device__ __forceinline__ Raw load(const uint8_t *blk, int i) {
        int byte, hi, sb;
        where(i, byte, hi, sb);
        return {*reinterpret_cast<const uint4 *>(blk), *reinterpret_cast<const uint32_t *>(blk + 16 + byte)};
    }
    static __device__ __forceinline__ void values(const Raw &r, int i, float (&o)[4]) {
        int byte, hi, sb;
        where(i, byte, hi, sb);
        const float d = f16_bits_to_f32(r.hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(r.hdr.x >> 16);
        uint32_t sc, m;
        scale_min_k4(sb, r.hdr.y, r.hdr.z, r.hdr.w, sc, m);
        const float d1 = d * (float)sc;
        const float dm1 = dmin * (float)m;
        const uint32_t qq = hi ? (r.q >> 4) : r.q;
#pragma unroll
        for (int t = 0; t < 4; t++) o[t] = d1 * (float)((qq >> (8 * t)) & 0xFu) - dm1;
    }
};

// Q5_K (k_quants.rs:407-462 + :663-710): 176-byte blocks {d, dmin, scales[12], qh[32], qs[128]};
// out = (d*sc) * q - (dmin*m) with q = nibble | fifth bit << 4.
// ORDER 0: output l of the first / second half of chunk c takes nibble l % 2 of qs[32 c + 16 half + l / 2] and bit
// l % 8 of qh[8 c + 4 half + l / 8].  ORDER 1 (the inverse of k_quants.rs:1027-1047): nibble `half` of qs[32 c + l] and
// bit 2 c + half of qh[l].
template <int ORDER>
struct DecQ5K {
    static constexpr int kBytes = 176;
    struct Raw {
        uint4 hdr;
        uint32_t q, h;
    };
    static __device__ __forceinline__ Raw load(const uint8_t *blk, int i) {
        const int c = i >> 4, p = (i & 15) * 4, half = p >> 5, l = p & 31;
        Raw r;
        r.hdr = *reinterpret_cast<const uint4 *>(blk);
        if (ORDER == 0) {
            r.q = *reinterpret_cast<const uint16_t *>(blk + 48 + 32 * c + 16 * half + (l >> 1));
            r.h = (uint32_t)blk[16 + 8 * c + 4 * half + (l >> 3)] >> (l & 7);
        } else {
            r.q = *reinterpret_cast<const uint32_t *>(blk + 48 + 32 * c + l);
            r.h = *reinterpret_cast<const uint32_t *>(blk + 16 + l) >> (2 * c + half);
        }
        return r;
    }
    static __device__ __forceinline__ void values(const Raw &r, int i, float (&o)[4]) {
        const int c = i >> 4, p = (i & 15) * 4, half = p >> 5;
        const float d = f16_bits_to_f32(r.hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(r.hdr.x >> 16);
        uint32_t sc, m;
        scale_min_k4(2 * c + half, r.hdr.y, r.hdr.z, r.hdr.w, sc, m);
        const float d1 = d * (float)sc;
        const float dm1 = dmin * (float)m;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            uint32_t v;
            if (ORDER == 0) v = ((r.q >> (4 * t)) & 0xFu) | (((r.h >> t) & 1u) << 4);
            else v = (((half ? r.q >> 4 : r.q) >> (8 * t)) & 0xFu) | (((r.h >> (8 * t)) & 1u) << 4);
            o[t] = d1 * (float)v - dm1;
        }
    }
    // the same elements as integers: value = d * sc * q[t] - dmin * m
    static constexpr bool kHasMin = true;
    static __device__ __forceinline__ void ints(const Raw &r, int i, int (&q)[4], int &sc_out, int &m_out) {
        const int c = i >> 4, p = (i & 15) * 4, half = p >> 5;
        uint32_t sc, m;
        scale_min_k4(2 * c + half, r.hdr.y, r.hdr.z, r.hdr.w, sc, m);
        sc_out = (int)sc, m_out = (int)m;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            if (ORDER == 0) q[t] = (int)(((r.q >> (4 * t)) & 0xFu) | (((r.h >> t) & 1u) << 4));
            else q[t] = (int)((((half ? r.q >> 4 : r.q) >> (8 * t)) & 0xFu) | (((r.h >> (8 * t)) & 1u) << 4));
        }
    }
    static __device__ __forceinline__ uint32_t d_bits(const uint8_t *blk) { return *reinterpret_cast<const uint16_t *>(blk); }
    static __device__ __forceinline__ uint32_t dmin_bits(const uint8_t *blk) { return *reinterpret_cast<const uint16_t *>(blk + 2); }
};

// Q6_K (k_quants.rs:474-496 + :614-660): out = (d * sc) * q, left-associated.  Blocks are 2-byte aligned.
struct DecQ6K {
    static constexpr int kBytes = 210;
    struct Raw {
        uint32_t ql, qh, d;
        int sc;
    };
    static __device__ __forceinline__ Raw load(const uint8_t *blk, int i) {
        const int h = i >> 5;        // 128-element half
        const int g = (i >> 3) & 3;  // 32-element group inside the half
        const int l = (i & 7) * 4;   // 0..28
        return {*reinterpret_cast<const u32_a2 *>(blk + 64 * h + 32 * (g & 1) + l), *reinterpret_cast<const u32_a2 *>(blk + 128 + 32 * h + l),
                *reinterpret_cast<const uint16_t *>(blk + 208), (int)(int8_t)blk[192 + 8 * h + 2 * g + (l >> 4)]};
    }
    static __device__ __forceinline__ void values(const Raw &r, int i, float (&o)[4]) {
        const int g = (i >> 3) & 3;
        const float dsc = f16_bits_to_f32(r.d) * (float)r.sc;
        const uint32_t nib = (g >= 2) ? (r.ql >> 4) : r.ql;
        const uint32_t hi2 = r.qh >> (2 * g);
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int q = (int)(((nib >> (8 * t)) & 0xFu) | (((hi2 >> (8 * t)) & 3u) << 4)) - 32;
            o[t] = dsc * (float)q;
        }
    }
};

// Q2_K and Q3_K have sixteen 16-element sub-blocks per super-block and pack the low two bits of element e into
// qs[32 (e / 128) + e % 32] at bit 2 ((e % 128) / 32).
// Q2_K (k_quants.rs:230-266 + :762-810): out = (d * (sc & 15)) * q - dmin * (sc >> 4).  84-byte blocks: scales[16],
// qs[64], d, dmin.
struct DecQ2K {
    static constexpr int kBytes = 84;
    struct Raw {
        uint32_t q, sc, dd;
    };
    static __device__ __forceinline__ Raw load(const uint8_t *blk, int i) {
        const int h = i >> 5, l = (i & 7) * 4;
        return {*reinterpret_cast<const uint32_t *>(blk + 16 + 32 * h + l), blk[i >> 2], *reinterpret_cast<const uint32_t *>(blk + 80)};
    }
    static __device__ __forceinline__ void values(const Raw &r, int i, float (&o)[4]) {
        const int p = (i >> 3) & 3;
        const float dl = f16_bits_to_f32(r.dd & 0xFFFFu) * (float)(r.sc & 0xFu);
        const float ml = f16_bits_to_f32(r.dd >> 16) * (float)(r.sc >> 4);
#pragma unroll
        for (int t = 0; t < 4; t++) o[t] = dl * (float)((r.q >> (8 * t + 2 * p)) & 3u) - ml;
    }
    static constexpr bool kHasMin = true;
    static __device__ __forceinline__ void ints(const Raw &r, int i, int (&q)[4], int &sc_out, int &m_out) {
        const int p = (i >> 3) & 3;
        sc_out = (int)(r.sc & 0xFu), m_out = (int)(r.sc >> 4);
#pragma unroll
        for (int t = 0; t < 4; t++) q[t] = (int)((r.q >> (8 * t + 2 * p)) & 3u);
    }
    static __device__ __forceinline__ uint32_t d_bits(const uint8_t *blk) { return *reinterpret_cast<const uint16_t *>(blk + 80); }
    static __device__ __forceinline__ uint32_t dmin_bits(const uint8_t *blk) { return *reinterpret_cast<const uint16_t *>(blk + 82); }
};

// Q3_K (k_quants.rs:281-355 + :713-760): out = (d * (sc6 - 32)) * (q2 - (hbit ? 0 : 4)).  110-byte blocks: hmask[32],
// qs[64], scales[12], d; the high bit of element e is bit e / 32 of hmask[e % 32]; the sixteen 6-bit scales are four low
// bits in the nibbles of scales[0..8] and two high bits in scales[8..12].
struct DecQ3K {
    static constexpr int kBytes = 110;
    struct Raw {
        uint32_t q, h, lo, hi, d;
    };
    static __device__ __forceinline__ Raw load(const uint8_t *blk, int i) {
        const int h = i >> 5, l = (i & 7) * 4, is = i >> 2;
        return {*reinterpret_cast<const u32_a2 *>(blk + 32 + 32 * h + l), *reinterpret_cast<const u32_a2 *>(blk + l), blk[96 + (is & 7)],
                blk[104 + (is & 3)], *reinterpret_cast<const uint16_t *>(blk + 108)};
    }
    static __device__ __forceinline__ void values(const Raw &r, int i, float (&o)[4]) {
        const int h = i >> 5, p = (i >> 3) & 3, is = i >> 2;
        const uint32_t sc6 = ((is < 8 ? r.lo : r.lo >> 4) & 0xFu) | (((r.hi >> (2 * (is >> 2))) & 3u) << 4);
        const float dl = f16_bits_to_f32(r.d) * (float)((int)sc6 - 32);
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int q = (int)((r.q >> (8 * t + 2 * p)) & 3u) - (((r.h >> (8 * t + 4 * h + p)) & 1u) ? 0 : 4);
            o[t] = dl * (float)q;
        }
    }
    static constexpr bool kHasMin = false;
    static __device__ __forceinline__ void ints(const Raw &r, int i, int (&q)[4], int &sc_out, int &m_out) {
        const int h = i >> 5, p = (i >> 3) & 3, is = i >> 2;
        const uint32_t sc6 = ((is < 8 ? r.lo : r.lo >> 4) & 0xFu) | (((r.hi >> (2 * (is >> 2))) & 3u) << 4);
        sc_out = (int)sc6 - 32, m_out = 0;
#pragma unroll
        for (int t = 0; t < 4; t++) q[t] = (int)((r.q >> (8 * t + 2 * p)) & 3u) - (((r.h >> (8 * t + 4 * h + p)) & 1u) ? 0 : 4);
    }
    static __device__ __forceinline__ uint32_t d_bits(const uint8_t *blk) { return *reinterpret_cast<const uint16_t *>(blk + 108); }
    static __device__ __forceinline__ uint32_t dmin_bits(const uint8_t *) { return 0; }
};

// Q8_K (k_quants.rs:498-506): out = d * q, one rounding.  292-byte blocks: d f32, qs[256] i8, bsums[16] i16.
struct DecQ8K {
    static constexpr int kBytes = 292;
    struct Raw {
        float d;
        uint32_t q;
    };
    static __device__ __forceinline__ Raw load(const uint8_t *blk, int i) {
        return {*reinterpret_cast<const float *>(blk), *reinterpret_cast<const uint32_t *>(blk + 4 + 4 * i)};
    }
    static __device__ __forceinline__ void values(const Raw &r, int, float (&o)[4]) {
#pragma unroll
        for (int t = 0; t < 4; t++) o[t] = r.d * (float)(int8_t)(r.q >> (8 * t));
    }
};

template <class D>
__global__ __launch_bounds__(256) void k_dequantize_kq(const uint8_t *__restrict__ src, size_t n, float *__restrict__ dst) {
    const size_t wave = ((size_t)blockIdx.x * 256 + threadIdx.x) >> 6;
    const int i = (int)(threadIdx.x & 63);
    typename D::Raw raw[kDeqUnroll];
#pragma unroll
    for (int u = 0; u < kDeqUnroll; u++) {
        const size_t blk_i = wave * kDeqUnroll + u;
        const bool live = blk_i * 256 + (size_t)i * 4 < n;
        raw[u] = D::load(src + (live ? blk_i : 0) * D::kBytes, i);  // lanes past the end re-read the first block
    }
#pragma unroll
    for (int u = 0; u < kDeqUnroll; u++) {
        const size_t e = (wave * kDeqUnroll + u) * 256 + (size_t)i * 4;
        if (e >= n) continue;
        float o[4];
        D::values(raw[u], i, o);
        if (e + 3 < n) {
            store_stream4(dst + e, o);
        } else {
            for (int t = 0; t < 4 && e + t < n; t++) dst[e + t] = o[t];
        }
    }
}

// Exact re-blocking of Q5_K, Q3_K and Q2_K super-blocks into Q6_K ones, for the matrix-matrix product: the fused GEMM
// kernels exist for Q4_K, Q6_K and Q8_0, and Q6_K (value d * sc * (q - 32), sixteen int8 scales, q - 32 in [-32, 31])
// holds the other formats' elements without loss.  With the decoder's integers (value = d * s * q - dmin * m):
//   block A: d, scale s per 16 elements, stored quant q + 32      (Q5_K: s <= 63, q <= 31; Q3_K: s in [-32, 31], q in
//            [-4, 3]; Q2_K: s <= 15, q <= 3)
//   block B (formats with mins): dmin as d, scale m, stored quant 31, i.e. -1 * dmin * m for every element.
// W x = A x + B x then, every product exact.  One wave per super-block: lane i decodes elements 4 i .. 4 i + 3 into
// LDS, then assembles ql bytes 2 i and 2 i + 1 and qh byte i of the Q6_K layout (k_quants.rs:1116-1130).
template <class D>
__device__ __forceinline__ void reblock_one(const uint8_t *__restrict__ src, size_t blk_i, bool live, int w, int i, uint8_t (&quants)[4][256],
                                            int8_t (&scales)[4][2][16], uint8_t (&outbuf)[2][840]) {
    const uint8_t *blk = src + (live ? blk_i : 0) * D::kBytes;
    const typename D::Raw raw = D::load(blk, i);
    int q[4], sc, m;
    D::ints(raw, i, q, sc, m);
    *reinterpret_cast<uint32_t *>(&quants[w][4 * i]) =
        (uint32_t)(q[0] + 32) | ((uint32_t)(q[1] + 32) << 8) | ((uint32_t)(q[2] + 32) << 16) | ((uint32_t)(q[3] + 32) << 24);
    if ((i & 3) == 0) scales[w][0][i >> 2] = (int8_t)sc, scales[w][1][i >> 2] = (int8_t)m;
    __syncthreads();
    if (!live) return;
    const uint8_t *qv = quants[w];
    uint32_t ql = 0;
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int b = 2 * i + t, lo = 128 * (b >> 6) + (b & 63);  // ql byte b: low nibble of element lo, high of lo + 64
        ql |= ((uint32_t)(qv[lo] & 15u) | ((uint32_t)(qv[lo + 64] & 15u) << 4)) << (8 * t);
    }
    const int e0 = 128 * (i >> 5) + (i & 31);  // qh byte i: bits 2 g .. 2 g + 1 from element e0 + 32 g
    const uint32_t qh = (uint32_t)(qv[e0] >> 4) | ((uint32_t)(qv[e0 + 32] >> 4) << 2) | ((uint32_t)(qv[e0 + 64] >> 4) << 4) |
                        ((uint32_t)(qv[e0 + 96] >> 4) << 6);
    // the four super-blocks of the workgroup are 840 contiguous bytes of the output: assemble them in LDS, store dwords
    uint8_t *oa = outbuf[0] + w * 210, *ob = outbuf[1] + w * 210;
    *reinterpret_cast<uint16_t *>(oa + 2 * i) = (uint16_t)ql;
    oa[128 + i] = (uint8_t)qh;
    if (i < 16) oa[192 + i] = (uint8_t)scales[w][0][i];
    if (i == 0) *reinterpret_cast<uint16_t *>(oa + 208) = (uint16_t)D::d_bits(blk);
    if (D::kHasMin) {
        *reinterpret_cast<uint16_t *>(ob + 2 * i) = 0xFFFFu;  // 31 = nibble 15, top bits 01
        ob[128 + i] = 0x55u;
        if (i < 16) ob[192 + i] = (uint8_t)scales[w][1][i];
        if (i == 0) *reinterpret_cast<uint16_t *>(ob + 208) = (uint16_t)D::dmin_bits(blk);
    }
}

template <class D>
__global__ __launch_bounds__(256) void k_reblock_q6k(const uint8_t *__restrict__ src, size_t n_blocks, uint8_t *__restrict__ dst_a,
                                                     uint8_t *__restrict__ dst_b) {
    __shared__ __align__(16) uint8_t quants[4][256];
    __shared__ int8_t scales[4][2][16];
    __shared__ __align__(16) uint8_t outbuf[2][840];
    const size_t blk0 = (size_t)blockIdx.x * 4;
    const int w = (int)(threadIdx.x >> 6), i = (int)(threadIdx.x & 63);
    const bool live = blk0 + w < n_blocks;  // wave-uniform
    reblock_one<D>(src, blk0 + w, live, w, i, quants, scales, outbuf);
    __syncthreads();
    const size_t left = n_blocks - blk0;
    const unsigned bytes = (unsigned)(left < 4 ? left : 4) * 210u;  // a multiple of 4 except for one or three blocks (then of 2)
    const unsigned t = threadIdx.x;
    for (int part = 0; part < (D::kHasMin ? 2 : 1); part++) {
        uint8_t *dst = (part ? dst_b : dst_a) + blk0 * 210;  // 840 bytes per workgroup: 8-byte aligned
        const uint8_t *from = outbuf[part];
        if (4 * t + 4 <= bytes) *reinterpret_cast<uint32_t *>(dst + 4 * t) = *reinterpret_cast<const uint32_t *>(from + 4 * t);
        else if (4 * t + 2 <= bytes) *reinterpret_cast<uint16_t *>(dst + 4 * t) = *reinterpret_cast<const uint16_t *>(from + 4 * t);
    }
}

// y = a + b (f32), stored as f32 or as bf16 rounded to nearest even
__global__ __launch_bounds__(256) void k_add_store(const float *__restrict__ a, const float *__restrict__ b, size_t n, void *__restrict__ y,
                                                   int y_bf16) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const float v = a[idx] + b[idx];
    if (y_bf16) {
        const uint32_t u = __builtin_bit_cast(uint32_t, v);
        reinterpret_cast<uint16_t *>(y)[idx] =
            (uint16_t)(((u & 0x7FFFFFFFu) > 0x7F800000u) ? ((u >> 16) | 0x40u) : ((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16));
    } else {
        reinterpret_cast<float *>(y)[idx] = v;
    }
}

// The four f64 sums of compute_kl_divergence (crates/pmetal-gguf/src/dynamic.rs:140-180) between the first n elements
// of the original tensor and of the dequantized blocks, which are decoded in registers and never stored: sum (a - b)^2
// with the difference taken in f32, sum a^2, sum a b, sum b^2.  Waves walk the super-blocks with a grid stride; every
// workgroup writes its four partial sums, the caller adds the workgroups' sums in order.
template <class D>
__global__ __launch_bounds__(256) void k_kl_sums_kq(const uint8_t *__restrict__ src, const float *__restrict__ a, size_t n,
                                                    double *__restrict__ partial) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const int i = (int)(threadIdx.x & 63);
    const size_t n_waves = (size_t)gridDim.x * 4, wave0 = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const size_t n_blocks = (n + 255) / 256;
    double s_err = 0.0, s_aa = 0.0, s_ab = 0.0, s_bb = 0.0;
    for (size_t b0 = wave0 * kDeqUnroll; b0 < n_blocks; b0 += n_waves * kDeqUnroll) {
        typename D::Raw raw[kDeqUnroll];
        f4 av[kDeqUnroll];
#pragma unroll
        for (int u = 0; u < kDeqUnroll; u++) {
            const size_t e = (b0 + u) * 256 + (size_t)i * 4;
            raw[u] = D::load(src + (e < n ? b0 + u : 0) * D::kBytes, i);
            av[u] = (f4){0.f, 0.f, 0.f, 0.f};
            if (e + 3 < n) {
                av[u] = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(a + e));
            } else {
                for (int t = 0; t < 4 && e + t < n; t++) av[u][t] = a[e + t];
            }
        }
#pragma unroll
        for (int u = 0; u < kDeqUnroll; u++) {
            const size_t e = (b0 + u) * 256 + (size_t)i * 4;
            float o[4];
            D::values(raw[u], i, o);
#pragma unroll
            for (int t = 0; t < 4; t++) {
                if (e + t < n) {
                    const double diff = (double)(av[u][t] - o[t]), x = (double)av[u][t], y = (double)o[t];
                    s_err += diff * diff, s_aa += x * x, s_ab += x * y, s_bb += y * y;
                }
            }
        }
    }
    __shared__ double red[4][4];
    double v[4] = {s_err, s_aa, s_ab, s_bb};
#pragma unroll
    for (int k = 0; k < 4; k++) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v[k] += __shfl_xor(v[k], off);
    }
    const int wave = threadIdx.x >> 6;
    if (i == 0)
        for (int k = 0; k < 4; k++) red[wave][k] = v[k];
    __syncthreads();
    if (threadIdx.x < 4) partial[(size_t)blockIdx.x * 4 + threadIdx.x] = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
}

// -------------------------------------------------------------------------------------------
// Q4_K quantize (k_quants.rs:876-955).  One wave per 8 super-blocks: lane L owns sub-block L
// (32 elements) of the 64 sub-blocks, runs make_qkx1_quants (quantize.rs:583-644) sequentially in
// registers, then the 8 lanes of a super-block agree on d/dmin, pack the 6-bit scales, requantize
// and emit 16 bytes of nibbles each.
// -------------------------------------------------------------------------------------------
constexpr int kQ4kLdsStride = 33;  // 32 floats + 1 pad: lanes read column-wise without bank conflicts

// NMAX = 15: Q4_K (k_quants.rs:876-955).  NMAX = 31: Q5_K (k_quants.rs:960-1051), the same search and scale packing with
// 5-bit quants: 176-byte blocks, the low four bits packed like Q4_K behind 32 bytes qh, where bit j of qh[l] is the
// fifth bit of element l of sub-block j.
// The super-block part of quantize_q4k / quantize_q5k for the 8 super-blocks from sb0 on: lane L holds the 32 elements of
// sub-block L and make_qkx1_quants' (scale, -min) for it.
template <int NMAX>
__device__ __forceinline__ void q4k_finish(const float (&xv)[32], const float scale, const float neg_min, const int lane, const size_t sb0,
                                           const size_t n_sb, uint8_t *__restrict__ dst) {
    constexpr bool Q5 = NMAX == 31;
    constexpr int kBytes = Q5 ? 176 : 144, kQsOff = Q5 ? 48 : 16;
    // ---- super-block level (k_quants.rs:904-929): the 8 lanes of a super-block cooperate ----
    float max_scale = scale, max_min = neg_min;
#pragma unroll
    for (int off = 1; off < 8; off <<= 1) {
        max_scale = __builtin_fmaxf(max_scale, __shfl_xor(max_scale, off));
        max_min = __builtin_fmaxf(max_min, __shfl_xor(max_min, off));
    }
    // fold(0.0, max): the fold starts from +0.0, and +0.0 orders above -0.0 on the reference's target
    max_scale = __builtin_fmaxf(max_scale, 0.0f);
    max_min = __builtin_fmaxf(max_min, 0.0f);
    if (max_scale == 0.0f) max_scale = 0.0f;
    if (max_min == 0.0f) max_min = 0.0f;
    const float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    const float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    int a = f32_as_i32(round_half_away(inv_scale * scale));
    int b = f32_as_i32(round_half_away(inv_min * neg_min));
    const uint32_t ls8 = (uint32_t)(a < 63 ? a : 63) & 0xFFu;  // `.min(63) as u8`
    const uint32_t lm8 = (uint32_t)(b < 63 ? b : 63) & 0xFFu;
    const int j = lane & 7;
    // partner sub-block j^4 supplies / receives the two high bits
    const uint32_t ls8_p = __shfl_xor(ls8, 4), lm8_p = __shfl_xor(lm8, 4);
    // bytes of the 12-byte scale field this lane produces (k_quants.rs:915-926)
    //   j < 4 : scales[j]   = ls_j | (ls_{j+4} >> 4) << 6 ; scales[j+4] = lm_j | (lm_{j+4} >> 4) << 6
    //   j >= 4: scales[j+4] = (ls_j & 0xF) | (lm_j & 0xF) << 4
    uint32_t byte_a, byte_b = 0;
    uint32_t sc, m;  // get_scale_min_k4(j, scales)
    if (j < 4) {
        byte_a = (ls8 | ((ls8_p >> 4) << 6)) & 0xFFu;
        byte_b = (lm8 | ((lm8_p >> 4) << 6)) & 0xFFu;
        sc = byte_a & 63u;
        m = byte_b & 63u;
    } else {
        byte_a = ((ls8 & 0xFu) | ((lm8 & 0xFu) << 4)) & 0xFFu;
        const uint32_t lo_a = (ls8_p | ((ls8 >> 4) << 6)) & 0xFFu;  // scales[j-4]
        const uint32_t lo_b = (lm8_p | ((lm8 >> 4) << 6)) & 0xFFu;  // scales[j]
        sc = (byte_a & 0xFu) | ((lo_a >> 6) << 4);
        m = (byte_a >> 4) | ((lo_b >> 6) << 4);
    }
    const uint32_t d16 = f32_to_f16_bits(max_scale / 63.0f);
    const uint32_t dmin16 = f32_to_f16_bits(max_min / 63.0f);

    // ---- requantize with the decoded f16 scales (k_quants.rs:932-943) ----
    // L = clamp(nearest_int((x + dm) / dq), 0, 15).  Only the integer matters, so the IEEE division (ten instructions)
    // is replaced by a multiplication with 1 / dq wherever that provably gives the same integer: the product differs
    // from the correctly rounded quotient by less than 3e-6 for quotients below 32, so if it stays 8e-6 away from every
    // rounding boundary n + 0.5 both round alike.  A lane that sees a product closer than that (or a dq outside the
    // range where 1 / dq and the product are normal numbers) redoes its sub-block with the division.
    uint32_t lb[8] = {0, 0, 0, 0, 0, 0, 0, 0};  // 32 quants, one per byte
    const float dq = f16_bits_to_f32(d16) * (float)sc;
    if (dq != 0.0f) {
        const float dm = f16_bits_to_f32(dmin16) * (float)m;
        const float rinv = 1.0f / dq;
        bool exact_needed = !(dq > 1e-20f && dq < 1e20f);
#pragma unroll
        for (int w = 0; w < 8; w++) {
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const float q = __builtin_fminf(__builtin_fmaxf((xv[4 * w + c] + dm) * rinv, 0.0f), (float)NMAX);
                const float r = __builtin_truncf(q + 0.49999997f);
                exact_needed |= !(__builtin_fabsf(__builtin_fabsf(q - r) - 0.5f) >= 8e-6f);
                lb[w] = __builtin_amdgcn_cvt_pk_u8_f32(r, c, lb[w]);  // r is an integer in [0, NMAX]
            }
        }
        if (exact_needed) {
#pragma unroll
            for (int w = 0; w < 8; w++) {
                lb[w] = 0;
#pragma unroll
                for (int c = 0; c < 4; c++) lb[w] |= (uint32_t)clamp_round_0_15<NMAX>((xv[4 * w + c] + dm) / dq) << (8 * c);
            }
        }
    }
    // ---- pack (k_quants.rs:946-951): qs[32c + l] = L[64c + l] | L[64c + l + 32] << 4 ----
    // Even sub-block 2c supplies the low nibbles, odd 2c+1 the high ones.  The even lane emits bytes
    // l = 0..15 of the pair, the odd lane bytes 16..31.
    const bool odd = lane & 1;
    uint32_t qh_word = 0;
    if (Q5) {
        // qh[l] |= 1 << j where L_j[l] > 15 (k_quants.rs:1027-1047): this lane's fifth bits at bit j of every byte, ored
        // over the eight lanes of the super-block; lane j then keeps dword j (bytes 4 j .. 4 j + 3)
#pragma unroll
        for (int w = 0; w < 8; w++) {
            uint32_t h = ((lb[w] >> 4) & 0x01010101u) << j;
            h |= __shfl_xor(h, 1);
            h |= __shfl_xor(h, 2);
            h |= __shfl_xor(h, 4);
            qh_word = j == w ? h : qh_word;
            lb[w] &= 0x0F0F0F0Fu;
        }
    }
    uint32_t outw[4];
#pragma unroll
    for (int w = 0; w < 4; w++) {
        const uint32_t send = odd ? lb[w] : lb[4 + w];
        const uint32_t recv = __shfl_xor(send, 1);
        outw[w] = odd ? (recv | (lb[4 + w] << 4)) : (lb[w] | (recv << 4));
    }
    const size_t sb = sb0 + (lane >> 3);
    if (sb < n_sb) {
        uint8_t *blk = dst + sb * kBytes;
        *reinterpret_cast<uint4 *>(blk + kQsOff + 16 * j) = make_uint4(outw[0], outw[1], outw[2], outw[3]);
        if (Q5) *reinterpret_cast<uint32_t *>(blk + 16 + 4 * j) = qh_word;
        if (j < 4) {
            blk[4 + j] = (uint8_t)byte_a;
            blk[8 + j] = (uint8_t)byte_b;
        } else {
            blk[8 + j] = (uint8_t)byte_a;
        }
        if (j == 0) *reinterpret_cast<uint32_t *>(blk) = d16 | (dmin16 << 16);
    }
}

template <int NMAX>
__global__ __launch_bounds__(64) void k_quantize_q4k(const float *__restrict__ x, size_t n_sb,
                                                      uint8_t *__restrict__ dst) {
    __shared__ float xs[64 * kQ4kLdsStride];
    const int lane = threadIdx.x;
    const size_t sb0 = (size_t)blockIdx.x * 8;
    const size_t n_valid = (n_sb - sb0 < 8 ? n_sb - sb0 : 8) * 256;  // floats this wave may read
    const float *src = x + sb0 * 256;
#pragma unroll
    for (int it = 0; it < 8; it++) {
        const int idx = it * 64 + lane;  // float4 index inside the 2048-float tile
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if ((size_t)idx * 4 < n_valid) v = *reinterpret_cast<const float4 *>(src + idx * 4);
        float *p = xs + (idx >> 3) * kQ4kLdsStride + (idx & 7) * 4;
        p[0] = v.x, p[1] = v.y, p[2] = v.z, p[3] = v.w;
    }
    __syncthreads();
    float xv[32];
#pragma unroll
    for (int i = 0; i < 32; i++) xv[i] = xs[lane * kQ4kLdsStride + i];

    // ---- make_qkx1_quants(NMAX, 5, xv) ----
    // min_by / max_by with total_cmp: equal keys are identical floats, so integer min / max of the keys will do
    int kmn = total_key(xv[0]), kmx = kmn;
#pragma unroll
    for (int i = 1; i < 32; i++) {
        const int key = total_key(xv[i]);
        kmn = key < kmn ? key : kmn;
        kmx = key > kmx ? key : kmx;
    }
    const float mn = __builtin_bit_cast(float, kmn ^ (int)(((unsigned)(kmn >> 31)) >> 1));
    const float mx = __builtin_bit_cast(float, kmx ^ (int)(((unsigned)(kmx >> 31)) >> 1));
    float scale = 0.0f, neg_min = 0.0f;  // returned (scale, -min)
    if (!(mx == mn)) {
        float minv = __builtin_fminf(mn, 0.0f);
        float iscale = (float)NMAX / (mx - minv);
        scale = 1.0f / iscale;
        // Of the previous try's quants only whether any of them changes is asked: they are kept one per byte and compared
        // four at a time (a conversion that packs in place of a move, 8 comparisons per try instead of 32).
        float lf[32];
        uint32_t lp[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 5; t++) {
            float sumlx = 0.0f, suml2 = 0.0f;  // suml2 is an integer <= 32 NMAX^2 < 2^24: exact in f32, with or without fusing
            bool changed = false;
            uint32_t np[8];
#pragma unroll
            for (int i = 0; i < 32; i++) {
                const float xm = xv[i] - minv;
                const float r = clamp_round_0_15<NMAX>(iscale * xm);
                np[i >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(r, i & 3, (i & 3) ? np[i >> 2] : 0u);
                lf[i] = r;
                sumlx += xm * r;
                suml2 = __builtin_fmaf(r, r, suml2);
            }
#pragma unroll
            for (int w = 0; w < 8; w++) {
                changed |= np[w] != lp[w];
                lp[w] = np[w];
            }
            if (suml2 == 0.0f) break;
            scale = sumlx / suml2;
            float sum = -0.0f;  // Iterator::sum::<f32> folds from -0.0
#pragma unroll
            for (int i = 0; i < 32; i++) sum += xv[i] - scale * lf[i];
            minv = sum / 32.0f;
            if (minv > 0.0f) minv = 0.0f;
            iscale = 1.0f / scale;
            if (!changed) break;
        }
        neg_min = -minv;
    }

    q4k_finish<NMAX>(xv, scale, neg_min, lane, sb0, n_sb, dst);
}

// -------------------------------------------------------------------------------------------
// Q6_K quantize (k_quants.rs:1056-1134).  One wave per 4 super-blocks: lane L owns the 16-element
// sub-block L of the 64, runs make_qx_quants(16, 32, x, 1) (quantize.rs:738-841) sequentially,
// then the 16 lanes of a super-block pick max_scale, requantize and assemble ql/qh through LDS.
// -------------------------------------------------------------------------------------------
constexpr int kQ6kLdsStride = 17;

__global__ __launch_bounds__(64) void k_quantize_q6k(const float *__restrict__ x, size_t n_sb,
                                                      uint8_t *__restrict__ dst) {
    __shared__ float xs[64 * kQ6kLdsStride];
    __shared__ uint32_t lbuf[4 * 64];   // final 6-bit values, one per byte, 256 per super-block
    __shared__ __attribute__((aligned(16))) uint16_t obuf[4 * 105];  // the 4 output blocks (210 bytes each)
    const int lane = threadIdx.x;
    const size_t sb0 = (size_t)blockIdx.x * 4;
    const size_t n_here = n_sb - sb0 < 4 ? n_sb - sb0 : 4;
    const size_t n_valid = n_here * 256;
    const float *src = x + sb0 * 256;
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int idx = it * 64 + lane;  // float4 index inside the 1024-float tile
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if ((size_t)idx * 4 < n_valid) v = *reinterpret_cast<const float4 *>(src + idx * 4);
        float *p = xs + (idx >> 2) * kQ6kLdsStride + (idx & 3) * 4;
        p[0] = v.x, p[1] = v.y, p[2] = v.z, p[3] = v.w;
    }
    __syncthreads();
    float xv[16], wx[16], w[16];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        xv[i] = xs[lane * kQ6kLdsStride + i];
        w[i] = xv[i] * xv[i];
        wx[i] = w[i] * xv[i];
    }

    // ---- make_qx_quants(16, 32, xv, rmse_type = 1) ----
    float l[16];  // signed quants l in [-32, 31]; ls = l + 32
    float maxv = 0.0f, amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float ax = __builtin_fabsf(xv[i]);
        if (ax > amax) {
            amax = ax;
            maxv = xv[i];
        }
    }
    float scale = 0.0f;
    bool zero_block = (amax == 0.0f);  // returns (0.0, ls = all zero): l + 32 == 0
#pragma unroll
    for (int i = 0; i < 16; i++) l[i] = -32.0f;
    if (!zero_block) {
        const float iscale0 = -32.0f / maxv;
        float sumlx = 0.0f, suml2 = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            l[i] = (float)clamp_i(nearest_int_sat(iscale0 * xv[i]), -32, 31);
            sumlx += wx[i] * l[i];
            suml2 += w[i] * (l[i] * l[i]);
        }
        scale = sumlx / suml2;
        float best = scale * sumlx;
        for (int t = 0; t < 3; t++) {
            const float isc = 1.0f / scale;
            float slx = 0.0f, sl2 = 0.0f;
            bool changed = false;
            float nl[16];
#pragma unroll
            for (int i = 0; i < 16; i++) {
                nl[i] = (float)clamp_i(nearest_int_sat(isc * xv[i]), -32, 31);
                changed |= (nl[i] != l[i]);
                slx += wx[i] * nl[i];
                sl2 += w[i] * (nl[i] * nl[i]);
            }
            if (!changed || sl2 == 0.0f || slx * slx <= best * sl2) break;
#pragma unroll
            for (int i = 0; i < 16; i++) l[i] = nl[i];
            sumlx = slx;
            suml2 = sl2;
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
        // Coordinate descent (quantize.rs:813-838), branch-free: every element computes its candidate and the test, and
        // takes them by select.  The candidate clamp(nearest_int(x sl2 / slx)) comes from a multiplication with an
        // approximate reciprocal: it differs from the correctly rounded quotient by less than 8e-6 for |quotient| < 33
        // (one ulp of the reciprocal, half an ulp each for the product and the quotient), so a product that stays
        // 2e-5 away from every rounding boundary rounds like the quotient; the rare lane closer than that, or with an
        // slx outside the range where the reciprocal is a normal number, takes the IEEE division.  The returned scale
        // is sumlx / suml2 of the last accepted change, so one division after the loop replaces one per change.
        bool any_change = false;
        for (int t = 0; t < 5; t++) {
            bool changed = false;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float li = l[i];
                const float slx = sumlx - wx[i] * li;
                const float sl2 = suml2 - w[i] * (li * li);
                const float p = xv[i] * sl2;
                const bool pos = slx > 0.0f;
                // The candidate is the current quant whenever the quotient lies within 0.5 of it, i.e. |x sl2 - l slx| < slx / 2:
                // two products and a difference, each correctly rounded, put that difference within 6e-6 slx of its exact
                // value for |quotient| < 33, and the reference's rounded quotient lies within 4e-6 of the exact one, so a
                // difference below 0.49998 slx settles it.  98 % of the elements that reach this point are settled this
                // way; the others (and every slx outside the range where the products are normal numbers) take the
                // quotient -- a whole wave, when one of its lanes has such an element.
                const float dd = p - li * slx;
                const bool same = slx > 1e-30f && slx < 1e30f && __builtin_fabsf(dd) < 0.49998f * slx;
                if (__builtin_amdgcn_ballot_w64(pos && !same) != 0) {
                    const float qf = p * __builtin_amdgcn_rcpf(slx);
                    float nl = (float)clamp_i(nearest_int_sat(qf), -32, 31);
                    const bool sure = slx > 1e-30f && slx < 1e30f && __builtin_fabsf(__builtin_fabsf(qf - nl) - 0.5f) >= 2e-5f;
                    if (pos && !sure) nl = (float)clamp_i(nearest_int_sat(p / slx), -32, 31);
                    const bool differs = pos & (nl != li);
                    // a new candidate is rare: skip the test when no lane has one
                    if (__builtin_amdgcn_ballot_w64(differs) != 0) {
                        const float slx2 = slx + wx[i] * nl;
                        const float sl22 = sl2 + w[i] * (nl * nl);
                        const bool take = differs & (sl22 > 0.0f) & (slx2 * slx2 * suml2 > sumlx * sumlx * sl22);
                        l[i] = take ? nl : li;
                        sumlx = take ? slx2 : sumlx;
                        suml2 = take ? sl22 : suml2;
                        changed |= take;
                    }
                }
            }
            if (!changed) break;
            any_change = true;
        }
        if (any_change) scale = sumlx / suml2;
    }

    // ---- super-block level (k_quants.rs:1082-1102) ----
    // max_scale = scale of the first sub-block attaining the largest |scale| (strict > in a forward
    // scan); |scale| of NaN never wins.
    const float abs_scale = __builtin_fabsf(scale);
    float gmax = (abs_scale == abs_scale) ? abs_scale : 0.0f;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) gmax = __builtin_fmaxf(gmax, __shfl_xor(gmax, off));
    const unsigned long long hit = __ballot(abs_scale == gmax && gmax > 0.0f);
    const int grp = lane & ~15;
    const unsigned long long ghit = (hit >> grp) & 0xFFFFull;
    const int first = ghit ? (__builtin_ctzll(ghit) + grp) : lane;
    float max_scale = __shfl(scale, first);
    if (!ghit) max_scale = 0.0f;
    const float iscale = -128.0f / max_scale;
    const uint32_t d16 = f32_to_f16_bits(1.0f / iscale);
    int sq = f32_as_i32(round_half_away(iscale * scale));
    sq = sq < 127 ? sq : 127;
    const int8_t s8 = (int8_t)(uint8_t)(uint32_t)sq;  // `.min(127) as i8` wraps

    // ---- requantize (k_quants.rs:1105-1113) ----
    // clamp(nearest_int(x / dq), -32, 31) by multiplication with 1 / dq where that provably rounds alike (see the Q4_K
    // kernel), by the division for the lanes that come within 8e-6 of a rounding boundary.
    const float dq = f16_bits_to_f32(d16) * (float)s8;
    uint32_t lw[4] = {0, 0, 0, 0};
    if (dq != 0.0f) {
        const float rinv = 1.0f / dq;
        bool exact_needed = !(__builtin_fabsf(dq) > 1e-20f && __builtin_fabsf(dq) < 1e20f);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float qf = xv[i] * rinv;
            const int ll = clamp_i(nearest_int_sat(qf), -32, 31);
            exact_needed |= !(__builtin_fabsf(__builtin_fabsf(qf - (float)ll) - 0.5f) >= 8e-6f);
            lw[i >> 2] |= (uint32_t)(ll + 32) << (8 * (i & 3));
        }
        if (exact_needed) {
#pragma unroll
            for (int q = 0; q < 4; q++) lw[q] = 0;
#pragma unroll
            for (int i = 0; i < 16; i++)
                lw[i >> 2] |= (uint32_t)(clamp_i(nearest_int_sat(xv[i] / dq), -32, 31) + 32) << (8 * (i & 3));
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float keep = zero_block ? 0.0f : l[i] + 32.0f;  // make_qx_quants' own ls
            lw[i >> 2] |= (uint32_t)(int)keep << (8 * (i & 3));
        }
    }
#pragma unroll
    for (int q = 0; q < 4; q++) lbuf[lane * 4 + q] = lw[q];
    __syncthreads();

    // ---- pack ql / qh (k_quants.rs:1116-1130) into obuf; 16 lanes per super-block ----
    const int sbl = lane >> 4;  // local super-block
    const int t = lane & 15;
    const uint32_t *L32 = lbuf + sbl * 64;
    uint16_t *ob = obuf + sbl * 105;
#pragma unroll
    for (int r = 0; r < 2; r++) {
        const int q = t * 2 + r;  // ql dword 0..31: bytes 4q..4q+3
        const int base = 32 * (q >> 4) + (q & 15);
        const uint32_t lo = L32[base], hi = L32[base + 16];
        const uint32_t v = (lo & 0x0F0F0F0Fu) | ((hi & 0x0F0F0F0Fu) << 4);
        ob[2 * q] = (uint16_t)v;
        ob[2 * q + 1] = (uint16_t)(v >> 16);
    }
    {
        const int p = t;  // qh dword 0..15
        const int base = 32 * (p >> 3) + (p & 7);
        const uint32_t a4 = (L32[base] >> 4) & 0x03030303u, b4 = (L32[base + 8] >> 4) & 0x03030303u;
        const uint32_t c4 = (L32[base + 16] >> 4) & 0x03030303u, e4 = (L32[base + 24] >> 4) & 0x03030303u;
        const uint32_t v = a4 | (b4 << 2) | (c4 << 4) | (e4 << 6);
        ob[64 + 2 * p] = (uint16_t)v;
        ob[64 + 2 * p + 1] = (uint16_t)(v >> 16);
    }
    {
        // scales: 16 signed bytes; two lanes share a u16
        const uint32_t mine = (uint32_t)(uint8_t)s8;
        const uint32_t other = __shfl_xor(mine, 1);
        if ((t & 1) == 0) ob[96 + (t >> 1)] = (uint16_t)(mine | (other << 8));
        if (t == 0) ob[104] = (uint16_t)d16;
    }
    __syncthreads();
    // ---- coalesced store of the n_here * 210 bytes (the tile starts 8-byte aligned) ----
    uint8_t *out = dst + sb0 * 210;
    const uint32_t *ob32 = reinterpret_cast<const uint32_t *>(obuf);
    const int n_u16 = (int)n_here * 105;
    for (int i = lane; i < n_u16 / 2; i += 64) reinterpret_cast<uint32_t *>(out)[i] = ob32[i];
    if ((n_u16 & 1) && lane == 0) reinterpret_cast<uint16_t *>(out)[n_u16 - 1] = obuf[n_u16 - 1];
}

inline unsigned grid_for(size_t work_items, size_t per_block) {
    return (unsigned)((work_items + per_block - 1) / per_block);
}

// -------------------------------------------------------------------------------------------
// Q2_K and Q3_K quantizers.  Both formats have sixteen 16-element sub-blocks per super-block and pack the low two bits
// of element e into qs[32 (e / 128) + e % 32] at bit 2 ((e % 128) / 32); both reference dequantizers are the inverses of
// that packing, so there is one element order.
// -------------------------------------------------------------------------------------------

// The 1024-float tile of four super-blocks, one 16-element sub-block per lane: staged through LDS with a row stride
// of 17 floats so that the lanes' column-wise reads do not collide.
constexpr int kSub16Stride = 17;
__device__ __forceinline__ void load_sub16(const float *__restrict__ x, size_t n_sb, size_t sb0, float *xs, float (&xv)[16]) {
    const int lane = threadIdx.x;
    const size_t n_valid = (n_sb - sb0 < 4 ? n_sb - sb0 : 4) * 256;  // floats this wave may read
    const float *src = x + sb0 * 256;
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int idx = it * 64 + lane;  // float4 index inside the tile
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if ((size_t)idx * 4 < n_valid) v = *reinterpret_cast<const float4 *>(src + idx * 4);
        float *q = xs + (idx >> 2) * kSub16Stride + (idx & 3) * 4;
        q[0] = v.x, q[1] = v.y, q[2] = v.z, q[3] = v.w;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; i++) xv[i] = xs[lane * kSub16Stride + i];
}

// Sub-block j = 8 h + 2 p + s of a super-block holds the elements whose low bits go to qs[32 h + 16 s + i] at bit 2 p.
// The four lanes of one (h, s) or their sixteen bytes together and lane p stores dword p of them.
__device__ __forceinline__ void store_qs2(const uint32_t (&q)[16], int j, uint8_t *qs) {
    const int p = (j >> 1) & 3;
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        w[k] = (q[4 * k] | (q[4 * k + 1] << 8) | (q[4 * k + 2] << 16) | (q[4 * k + 3] << 24)) << (2 * p);
        w[k] |= __shfl_xor(w[k], 2);
        w[k] |= __shfl_xor(w[k], 4);
    }
    const uint32_t mine = p == 0 ? w[0] : (p == 1 ? w[1] : (p == 2 ? w[2] : w[3]));
    if (qs) *reinterpret_cast<u32_a2 *>(qs + 32 * (j >> 3) + 16 * (j & 1) + 4 * p) = mine;
}

// Q2_K quantize (k_quants.rs:1242-1321): make_qkx1_quants(3, 5) (quantize.rs:583-644) per 16-element sub-block, 4-bit
// scales and mins against d = max_scale / 15 and dmin = max_min / 15, requantization with the decoded f16 values.
__global__ __launch_bounds__(64) void k_quantize_q2k(const float *__restrict__ x, size_t n_sb, uint8_t *__restrict__ dst) {
    __shared__ float xs[64 * kSub16Stride];
    const int lane = threadIdx.x, j = lane & 15;
    const size_t sb0 = (size_t)blockIdx.x * 4;
    float xv[16];
    load_sub16(x, n_sb, sb0, xs, xv);

    // ---- make_qkx1_quants(3, 5, xv) ----
    int kmn = total_key(xv[0]), kmx = kmn;
#pragma unroll
    for (int i = 1; i < 16; i++) {
        const int key = total_key(xv[i]);
        kmn = key < kmn ? key : kmn;
        kmx = key > kmx ? key : kmx;
    }
    const float mn = __builtin_bit_cast(float, kmn ^ (int)(((unsigned)(kmn >> 31)) >> 1));
    const float mx = __builtin_bit_cast(float, kmx ^ (int)(((unsigned)(kmx >> 31)) >> 1));
    float scale = 0.0f, neg_min = 0.0f;
    if (!(mx == mn)) {
        float minv = __builtin_fminf(mn, 0.0f);
        float iscale = 3.0f / (mx - minv);
        scale = 1.0f / iscale;
        float lf[16];
        uint32_t lp[4] = {0, 0, 0, 0};  // the previous try's quants, one per byte (as in the Q4_K kernel)
#pragma unroll
        for (int t = 0; t < 5; t++) {
            float sumlx = 0.0f, suml2 = 0.0f;  // suml2 <= 16 * 9: exact in f32
            bool changed = false;
            uint32_t np[4];
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float xm = xv[i] - minv;
                const float r = clamp_round_0_15<3>(iscale * xm);
                np[i >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(r, i & 3, (i & 3) ? np[i >> 2] : 0u);
                lf[i] = r;
                sumlx += xm * r;
                suml2 = __builtin_fmaf(r, r, suml2);
            }
#pragma unroll
            for (int w = 0; w < 4; w++) {
                changed |= np[w] != lp[w];
                lp[w] = np[w];
            }
            if (suml2 == 0.0f) break;
            scale = sumlx / suml2;
            float sum = -0.0f;  // Iterator::sum::<f32> folds from -0.0
#pragma unroll
            for (int i = 0; i < 16; i++) sum += xv[i] - scale * lf[i];
            minv = sum / 16.0f;
            if (minv > 0.0f) minv = 0.0f;
            iscale = 1.0f / scale;
            if (!changed) break;
        }
        neg_min = -minv;
    }

    // ---- super-block level (k_quants.rs:1273-1296): the 16 lanes of a super-block cooperate ----
    float max_scale = scale, max_min = neg_min;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        max_scale = __builtin_fmaxf(max_scale, __shfl_xor(max_scale, off));
        max_min = __builtin_fmaxf(max_min, __shfl_xor(max_min, off));
    }
    max_scale = __builtin_fmaxf(max_scale, 0.0f);  // fold(0.0, max): NaNs drop out, +0.0 wins over -0.0
    max_min = __builtin_fmaxf(max_min, 0.0f);
    uint32_t byte = 0, d16 = 0, dmin16 = 0;
    if (max_scale > 0.0f) {
        byte = (uint32_t)f32_as_i32(round_half_away((15.0f / max_scale) * scale)) & 0xFFu;  // `as u8`
        d16 = f32_to_f16_bits(max_scale / 15.0f);
    }
    if (max_min > 0.0f) {
        const uint32_t lm = (uint32_t)f32_as_i32(round_half_away((15.0f / max_min) * neg_min)) & 0xFFu;
        byte |= (lm << 4) & 0xFFu;
        dmin16 = f32_to_f16_bits(max_min / 15.0f);
    }

    // ---- requantize (k_quants.rs:1299-1310) ----
    uint32_t q[16];
#pragma unroll
    for (int i = 0; i < 16; i++) q[i] = 0;
    const float dq = f16_bits_to_f32(d16) * (float)(byte & 0xFu);
    if (dq != 0.0f) {
        const float dm = f16_bits_to_f32(dmin16) * (float)(byte >> 4);
        // by multiplication with 1 / dq where that provably rounds like the division (see the Q4_K kernel), by the division
        // for the lanes that come within 8e-6 of a rounding boundary
        const float rinv = 1.0f / dq;
        bool exact_needed = !(dq > 1e-20f && dq < 1e20f);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float qf = __builtin_fminf(__builtin_fmaxf((xv[i] + dm) * rinv, 0.0f), 3.0f);
            const float r = __builtin_truncf(qf + 0.49999997f);
            exact_needed |= !(__builtin_fabsf(__builtin_fabsf(qf - r) - 0.5f) >= 8e-6f);
            q[i] = (uint32_t)r;
        }
        if (exact_needed) {
#pragma unroll
            for (int i = 0; i < 16; i++) q[i] = (uint32_t)clamp_round_0_15<3>((xv[i] + dm) / dq);
        }
    }
    const size_t sb = sb0 + (lane >> 4);
    uint8_t *blk = sb < n_sb ? dst + sb * 84 : nullptr;
    store_qs2(q, j, blk ? blk + 16 : nullptr);
    if (blk) {
        blk[j] = (uint8_t)byte;
        if (j == 0) *reinterpret_cast<uint32_t *>(blk + 80) = d16 | (dmin16 << 16);
    }
}

// Q3_K quantize (k_quants.rs:1139-1237): make_q3_quants(x, 4, true) (quantize.rs:655-719) per 16-element sub-block,
// 6-bit signed scales against d = 1 / iscale with iscale = -32 / (the scale of largest magnitude, the first of equals),
// requantization with the decoded f16 value.
__global__ __launch_bounds__(64) void k_quantize_q3k(const float *__restrict__ x, size_t n_sb, uint8_t *__restrict__ dst) {
    __shared__ float xs[64 * kSub16Stride];
    const int lane = threadIdx.x, j = lane & 15;
    const size_t sb0 = (size_t)blockIdx.x * 4;
    float xv[16];
    load_sub16(x, n_sb, sb0, xs, xv);

    // ---- make_q3_quants(xv, 4, true) ----
    float maxv = 0.0f, amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float ax = __builtin_fabsf(xv[i]);
        if (ax > amax) amax = ax, maxv = xv[i];
    }
    float scale = 0.0f;
    if (amax != 0.0f) {
        const float iscale = -4.0f / maxv;
        float l[16], w[16], wx[16];  // the quants as floats: small integers, every product with them as in integer form
        float sumlx = 0.0f, suml2 = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            l[i] = (float)clamp_i(nearest_int_sat(iscale * xv[i]), -4, 3);
            w[i] = xv[i] * xv[i];
            wx[i] = w[i] * xv[i];
            sumlx += wx[i] * l[i];
            suml2 += w[i] * (l[i] * l[i]);
        }
        // The sweeps (quantize.rs:680-713), branch-free as in the Q6_K kernel: every element computes its candidate and the
        // test and takes them by select; the candidate clamp(nearest_int(x sl2 / slx)) comes from a multiplication with an
        // approximate reciprocal where that provably rounds like the quotient (within 8e-6 of it for |quotient| < 33, so
        // 2e-5 away from every rounding boundary is safe), from the IEEE division otherwise.
        for (int sweep = 0; sweep < 5; sweep++) {
            bool any = false;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float li = l[i];
                const float slx = sumlx - wx[i] * li;
                const float sl2 = suml2 - w[i] * (li * li);
                const float p = xv[i] * sl2;
                const bool pos = slx > 0.0f;
                const float qf = p * __builtin_amdgcn_rcpf(slx);
                float nl = (float)clamp_i(nearest_int_sat(qf), -4, 3);
                const bool sure = slx > 1e-30f && slx < 1e30f && __builtin_fabsf(__builtin_fabsf(qf - nl) - 0.5f) >= 2e-5f;
                if (pos && !sure) nl = (float)clamp_i(nearest_int_sat(p / slx), -4, 3);
                const bool differs = pos & (nl != li);
                if (sweep == 0 || __builtin_amdgcn_ballot_w64(differs) != 0) {  // later sweeps: rarely a candidate anywhere
                    const float slx2 = slx + wx[i] * nl;
                    const float sl22 = sl2 + w[i] * (nl * nl);
                    const bool take = differs & (sl22 > 0.0f) & (slx2 * slx2 * suml2 > sumlx * sumlx * sl22);
                    l[i] = take ? nl : li;
                    sumlx = take ? slx2 : sumlx;
                    suml2 = take ? sl22 : suml2;
                    any |= take;
                }
            }
            if (!any) break;
        }
        scale = sumlx / suml2;
    }

    // ---- super-block level (k_quants.rs:1165-1186) ----
    // `if scale.abs() > max_scale.abs()` in order: the first of the largest magnitudes; NaN never compares greater
    const float mag = scale == scale ? __builtin_fabsf(scale) : 0.0f;
    float big = mag;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) big = __builtin_fmaxf(big, __shfl_xor(big, off));
    const unsigned long long hit = __ballot(mag == big);
    const int first = __builtin_ctzll(((hit >> (lane & 48)) & 0xFFFFull) | 0x10000ull) & 15;
    const float max_scale = big > 0.0f ? __shfl(scale, (lane & 48) + first) : 0.0f;
    int lv = 0;
    uint32_t d16 = 0;
    if (max_scale != 0.0f) {
        const float iscale = -32.0f / max_scale;
        lv = clamp_i(nearest_int_sat(iscale * scale), -32, 31) + 32;
        d16 = f32_to_f16_bits(1.0f / iscale);
    }
    // scales[j] = (l_j & 15) | (l_{j+8} & 15) << 4 for j < 8; scales[8 + i] = sum_k (l_{i+4k} >> 4) << 2k
    const uint32_t lo = (uint32_t)lv & 0xFu, lo_hi = __shfl_xor(lo, 8);
    uint32_t top = ((uint32_t)lv >> 4) << (2 * (j >> 2));
    top |= __shfl_xor(top, 4);
    top |= __shfl_xor(top, 8);

    // ---- requantize (k_quants.rs:1192-1206), high bits (:1209-1224) ----
    uint32_t q[16];
#pragma unroll
    for (int i = 0; i < 16; i++) q[i] = 0;
    const float dq = f16_bits_to_f32(d16) * (float)(lv - 32);
    if (max_scale != 0.0f && dq != 0.0f) {
        const float rinv = 1.0f / dq;
        bool exact_needed = !(__builtin_fabsf(dq) > 1e-20f && __builtin_fabsf(dq) < 1e20f);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float qf = xv[i] * rinv;
            const int ll = clamp_i(nearest_int_sat(qf), -4, 3);
            exact_needed |= !(__builtin_fabsf(__builtin_fabsf(qf - (float)ll) - 0.5f) >= 8e-6f);
            q[i] = (uint32_t)(ll + 4);
        }
        if (exact_needed) {
#pragma unroll
            for (int i = 0; i < 16; i++) q[i] = (uint32_t)(clamp_i(nearest_int_sat(xv[i] / dq), -4, 3) + 4);
        }
    }
    // element 16 j + i has its high bit at bit j / 2 of hmask[16 (j % 2) + i]: the eight lanes of one parity or theirs
    uint32_t hw[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        hw[k] = ((q[4 * k] >> 2) | ((q[4 * k + 1] >> 2) << 8) | ((q[4 * k + 2] >> 2) << 16) | ((q[4 * k + 3] >> 2) << 24)) << (j >> 1);
        hw[k] |= __shfl_xor(hw[k], 2);
        hw[k] |= __shfl_xor(hw[k], 4);
        hw[k] |= __shfl_xor(hw[k], 8);
    }
#pragma unroll
    for (int i = 0; i < 16; i++) q[i] &= 3u;
    const size_t sb = sb0 + (lane >> 4);
    uint8_t *blk = sb < n_sb ? dst + sb * 110 : nullptr;
    store_qs2(q, j, blk ? blk + 32 : nullptr);
    if (blk) {
        const int k = j >> 1;  // lanes 0..7 of a super-block store the hmask dwords: parity j & 1, dword k & 3
        if (k < 4) {
            const uint32_t mine = k == 0 ? hw[0] : (k == 1 ? hw[1] : (k == 2 ? hw[2] : hw[3]));
            *reinterpret_cast<u32_a2 *>(blk + 16 * (j & 1) + 4 * k) = mine;
        }
        if (j < 8) blk[96 + j] = (uint8_t)(lo | (lo_hi << 4));
        if (j < 4) blk[104 + j] = (uint8_t)top;
        if (j == 0) *reinterpret_cast<uint16_t *>(blk + 108) = (uint16_t)d16;
    }
}

}  // namespace

namespace pmh {

hipError_t launch_quantize_q8_0(const float *x, size_t n, uint8_t *dst, hipStream_t s) {
    const size_t n_blocks = (n + 31) / 32;
    if (n_blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(k_quantize_q8_0, dim3(grid_for(n_blocks * 8, 256)), dim3(256), 0, s, x, n, dst, n_blocks);
    return hipGetLastError();
}

// Q4_0, Q4_1, Q5_0, Q5_1, Q8_1 (GGML type ids 2, 3, 6, 7, 9)
hipError_t launch_quantize_legacy32(uint32_t type, const float *x, size_t n, uint8_t *dst, hipStream_t s) {
    const size_t n_blocks = (n + 31) / 32;
    if (n_blocks == 0) return hipSuccess;
    const dim3 grid(grid_for(n_blocks * 8, 256)), block(256);
    switch (type) {
    case 2: hipLaunchKernelGGL(k_quantize_b32<2>, grid, block, 0, s, x, n, dst, n_blocks); break;
    case 3: hipLaunchKernelGGL(k_quantize_b32<3>, grid, block, 0, s, x, n, dst, n_blocks); break;
    case 6: hipLaunchKernelGGL(k_quantize_b32<6>, grid, block, 0, s, x, n, dst, n_blocks); break;
    case 7: hipLaunchKernelGGL(k_quantize_b32<7>, grid, block, 0, s, x, n, dst, n_blocks); break;
    case 9: hipLaunchKernelGGL(k_quantize_b32<9>, grid, block, 0, s, x, n, dst, n_blocks); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
hipError_t launch_dequantize_legacy32(uint32_t type, const uint8_t *src, size_t n, float *dst, hipStream_t s) {
    if (n == 0) return hipSuccess;
    const dim3 grid(grid_for((n + 3) / 4, 256)), block(256);
    switch (type) {
    case 2: hipLaunchKernelGGL(k_dequantize_b32<2>, grid, block, 0, s, src, n, dst); break;
    case 3: hipLaunchKernelGGL(k_dequantize_b32<3>, grid, block, 0, s, src, n, dst); break;
    case 6: hipLaunchKernelGGL(k_dequantize_b32<6>, grid, block, 0, s, src, n, dst); break;
    case 7: hipLaunchKernelGGL(k_dequantize_b32<7>, grid, block, 0, s, src, n, dst); break;
    case 9: hipLaunchKernelGGL(k_dequantize_b32<9>, grid, block, 0, s, src, n, dst); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_quantize_q4k(const float *x, size_t n, uint8_t *dst, hipStream_t s) {
    const size_t n_sb = n / 256;  // full super-blocks; a trailing partial one is zero bytes
    if (n % 256) {
        hipError_t e = launch_zero_bytes(dst + n_sb * 144, 144, s);
        if (e != hipSuccess) return e;
    }
    if (n_sb == 0) return hipSuccess;
    hipLaunchKernelGGL(k_quantize_q4k<15>, dim3(grid_for(n_sb, 8)), dim3(64), 0, s, x, n_sb, dst);
    return hipGetLastError();
}

hipError_t launch_quantize_q5k(const float *x, size_t n, uint8_t *dst, hipStream_t s) {
    const size_t n_sb = n / 256;  // full super-blocks; a trailing partial one is zero bytes
    if (n % 256) {
        hipError_t e = launch_zero_bytes(dst + n_sb * 176, 176, s);
        if (e != hipSuccess) return e;
    }
    if (n_sb == 0) return hipSuccess;
    hipLaunchKernelGGL(k_quantize_q4k<31>, dim3(grid_for(n_sb, 8)), dim3(64), 0, s, x, n_sb, dst);
    return hipGetLastError();
}

hipError_t launch_quantize_q6k(const float *x, size_t n, uint8_t *dst, hipStream_t s) {
    const size_t n_sb = n / 256;
    if (n % 256) {
        hipError_t e = launch_zero_bytes(dst + n_sb * 210, 210, s);
        if (e != hipSuccess) return e;
    }
    if (n_sb == 0) return hipSuccess;
    hipLaunchKernelGGL(k_quantize_q6k, dim3(grid_for(n_sb, 4)), dim3(64), 0, s, x, n_sb, dst);
    return hipGetLastError();
}

hipError_t launch_quantize_q2k(const float *x, size_t n, uint8_t *dst, hipStream_t s) {
    const size_t n_sb = n / 256;
    if (n % 256) {
        hipError_t e = launch_zero_bytes(dst + n_sb * 84, 84, s);
        if (e != hipSuccess) return e;
    }
    if (n_sb == 0) return hipSuccess;
    hipLaunchKernelGGL(k_quantize_q2k, dim3(grid_for(n_sb, 4)), dim3(64), 0, s, x, n_sb, dst);
    return hipGetLastError();
}

hipError_t launch_quantize_q3k(const float *x, size_t n, uint8_t *dst, hipStream_t s) {
    const size_t n_sb = n / 256;
    if (n % 256) {
        hipError_t e = launch_zero_bytes(dst + n_sb * 110, 110, s);
        if (e != hipSuccess) return e;
    }
    if (n_sb == 0) return hipSuccess;
    hipLaunchKernelGGL(k_quantize_q3k, dim3(grid_for(n_sb, 4)), dim3(64), 0, s, x, n_sb, dst);
    return hipGetLastError();
}

hipError_t launch_dequantize_q2k(const uint8_t *src, size_t n, float *dst, hipStream_t s) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_dequantize_kq<DecQ2K>, dim3(grid_for((n + 4 * kDeqUnroll - 1) / (4 * kDeqUnroll), 256)), dim3(256), 0, s, src, n, dst);
    return hipGetLastError();
}

hipError_t launch_dequantize_q3k(const uint8_t *src, size_t n, float *dst, hipStream_t s) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_dequantize_kq<DecQ3K>, dim3(grid_for((n + 4 * kDeqUnroll - 1) / (4 * kDeqUnroll), 256)), dim3(256), 0, s, src, n, dst);
    return hipGetLastError();
}

hipError_t launch_dequantize_q8_0(const uint8_t *src, size_t n, float *dst, hipStream_t s) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_dequantize_q8_0, dim3(grid_for((n + 3) / 4, 256)), dim3(256), 0, s, src, n, dst);
    return hipGetLastError();
}

hipError_t launch_dequantize_q5k(const uint8_t *src, size_t n, float *dst, uint32_t order, hipStream_t s) {
    if (n == 0) return hipSuccess;
    const dim3 grid = dim3(grid_for((n + 4 * kDeqUnroll - 1) / (4 * kDeqUnroll), 256));
    if (order == kOrderRef) hipLaunchKernelGGL(k_dequantize_kq<DecQ5K<0>>, grid, dim3(256), 0, s, src, n, dst);
    else hipLaunchKernelGGL(k_dequantize_kq<DecQ5K<1>>, grid, dim3(256), 0, s, src, n, dst);
    return hipGetLastError();
}

hipError_t launch_dequantize_q4k(const uint8_t *src, size_t n, float *dst, uint32_t order, hipStream_t s) {
    if (n == 0) return hipSuccess;
    const dim3 grid = dim3(grid_for((n + 4 * kDeqUnroll - 1) / (4 * kDeqUnroll), 256));  // one lane per 4 outputs of kDeqUnroll super-blocks
    if (order == kOrderRef) hipLaunchKernelGGL(k_dequantize_kq<DecQ4K<0>>, grid, dim3(256), 0, s, src, n, dst);
    else hipLaunchKernelGGL(k_dequantize_kq<DecQ4K<1>>, grid, dim3(256), 0, s, src, n, dst);
    return hipGetLastError();
}

hipError_t launch_dequantize_q6k(const uint8_t *src, size_t n, float *dst, hipStream_t s) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_dequantize_kq<DecQ6K>, dim3(grid_for((n + 4 * kDeqUnroll - 1) / (4 * kDeqUnroll), 256)), dim3(256), 0, s, src, n, dst);
    return hipGetLastError();
}

hipError_t launch_dequantize_q8k(const uint8_t *src, size_t n, float *dst, hipStream_t s) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_dequantize_kq<DecQ8K>, dim3(grid_for((n + 4 * kDeqUnroll - 1) / (4 * kDeqUnroll), 256)), dim3(256), 0, s, src, n, dst);
    return hipGetLastError();
}

// Workgroups of the fused dequantize-and-compare kernel: every wave gets at least two steps of kDeqUnroll super-blocks.
int kl_sums_quantized_workgroups(size_t n) {
    const size_t want = (n + 256 * kDeqUnroll * 8 - 1) / (256 * kDeqUnroll * 8);
    return (int)(want < 1 ? 1 : (want > 2048 ? 2048 : want));
}

// type: one of the k-quants (Q2_K .. Q6_K, Q8_K); n > 0 elements of `original` against the first n decoded elements.
hipError_t launch_kl_sums_quantized(uint32_t type, const uint8_t *src, const float *original, size_t n, uint32_t order, double *partial,
                                    hipStream_t s) {
    const dim3 grid((unsigned)kl_sums_quantized_workgroups(n)), block(256);
    const bool ref = order == kOrderRef;
    switch (type) {
    case kTypeQ2K: hipLaunchKernelGGL(k_kl_sums_kq<DecQ2K>, grid, block, 0, s, src, original, n, partial); break;
    case kTypeQ3K: hipLaunchKernelGGL(k_kl_sums_kq<DecQ3K>, grid, block, 0, s, src, original, n, partial); break;
    case kTypeQ4K:
        if (ref) hipLaunchKernelGGL(k_kl_sums_kq<DecQ4K<0>>, grid, block, 0, s, src, original, n, partial);
        else hipLaunchKernelGGL(k_kl_sums_kq<DecQ4K<1>>, grid, block, 0, s, src, original, n, partial);
        break;
    case kTypeQ5K:
        if (ref) hipLaunchKernelGGL(k_kl_sums_kq<DecQ5K<0>>, grid, block, 0, s, src, original, n, partial);
        else hipLaunchKernelGGL(k_kl_sums_kq<DecQ5K<1>>, grid, block, 0, s, src, original, n, partial);
        break;
    case kTypeQ6K: hipLaunchKernelGGL(k_kl_sums_kq<DecQ6K>, grid, block, 0, s, src, original, n, partial); break;
    case kTypeQ8K: hipLaunchKernelGGL(k_kl_sums_kq<DecQ8K>, grid, block, 0, s, src, original, n, partial); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

int reblock_q6k_parts(uint32_t type) {
    return type == kTypeQ3K ? 1 : (type == kTypeQ5K || type == kTypeQ2K) ? 2 : 0;
}

hipError_t launch_reblock_q6k(uint32_t type, const uint8_t *src, size_t n_blocks, uint32_t order, uint8_t *dst_a, uint8_t *dst_b,
                              hipStream_t s) {
    if (n_blocks == 0) return hipSuccess;
    const dim3 grid((unsigned)((n_blocks + 3) / 4)), block(256);
    if (type == kTypeQ5K) {
        if (order == kOrderRef) hipLaunchKernelGGL(k_reblock_q6k<DecQ5K<0>>, grid, block, 0, s, src, n_blocks, dst_a, dst_b);
        else hipLaunchKernelGGL(k_reblock_q6k<DecQ5K<1>>, grid, block, 0, s, src, n_blocks, dst_a, dst_b);
    } else if (type == kTypeQ3K) {
        hipLaunchKernelGGL(k_reblock_q6k<DecQ3K>, grid, block, 0, s, src, n_blocks, dst_a, dst_b);
    } else if (type == kTypeQ2K) {
        hipLaunchKernelGGL(k_reblock_q6k<DecQ2K>, grid, block, 0, s, src, n_blocks, dst_a, dst_b);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_add_store(const float *a, const float *b, size_t n, void *y, bool y_bf16, hipStream_t s) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_add_store, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, a, b, n, y, y_bf16 ? 1 : 0);
    return hipGetLastError();
}

}  // namespace pmh
