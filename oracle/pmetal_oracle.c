/*
 * pmetal_oracle.c -- CPU restatement of PMetal's GGUF block-quantized weight
 * path (Q8_0, Q4_K, Q6_K).  TEST INFRASTRUCTURE ONLY: see pmetal_oracle.h.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math (see Makefile).  Every float
 * operation below is a single IEEE binary32 operation in the order the
 * reference performs it; Rust never contracts a*b+c into an fma, so neither
 * may the compiler here.
 *
 * Parity status per function (what pins it without running the Rust):
 *   f16/bf16 conversion ... numpy float16 (all 65536 f16 values, sampled and
 *                           boundary f32 values); IEEE definition.
 *   nearest_int ........... reference KATs quantize.rs:862-868.
 *   get_scale_min_k4 ...... reference KATs quantize.rs:1035-1047,
 *                           k_quants.rs:1386-1396; pack/unpack identity.
 *   make_qkx1_quants, make_qx_quants, make_q3_quants
 *                           a restatement of the same Rust in rational arithmetic
 *                           (tests/exact_ref.py: fractions.Fraction, one IEEE-754
 *                           rounding per operation) gives the expected bits for
 *                           tests/golden/exact_cases.json: inputs whose sums are exact
 *                           in any order (2, 3, 4 and 5 tries; rescale passes taken
 *                           and refused; single-element moves taken and refused;
 *                           every exit) and Gaussian inputs in the reference's order.
 *                           Also the reference's closed forms (quantize.rs:998-1032).
 *   quantize_q8_0 ......... rational expected bytes (same fixture): a short last block, a
 *                           zero block, a negative maximum, blocks where 127 / amax and
 *                           1 / (amax / 127) round an element differently; numpy twin.
 *   quantize_q4k/q5k/q6k/q3k/q2k
 *                           whole super-blocks built from those inputs with bytes
 *                           derived by the rational restatement (same fixture), and
 *                           blocks that single out one step each: max_min folded from
 *                           +0.0, two scales of equal magnitude and opposite sign, a
 *                           scale code of 128, scale code 0, all-zero blocks, Gaussian
 *                           blocks whose bytes change when d / dmin are not the decoded
 *                           f16 values or the quotient is not an IEEE division, tensors
 *                           with a partial last super-block; block sizes, reference
 *                           round-trip bounds (k_quants.rs:1446-1553).
 *                           tests/test_oracle_mutations.py edits this file one line at a
 *                           time (one edit or more per item of the bit-exactness checklist)
 *                           and checks that the fixture alone notices each edit.
 *                           These are two restatements of the Rust by reading, pinned
 *                           against each other; the Rust itself was never run (no
 *                           toolchain here).
 *   dequantize_* .......... rational expected values for random block bytes (same fixture);
 *                           reference KATs (dequant.rs:1016-1036,
 *                           k_quants.rs:1368-1383) + hand-built blocks + numpy.
 *   quantize_q4_0/q4_1/q5_0/q5_1/q8_1, dequantize_legacy
 *                           the reference's block tests (dequant.rs:935-1053), every code
 *                           at every position of hand-written blocks, and quantized bytes
 *                           derived by hand for inputs on power-of-two grids (no operation
 *                           rounds), zero / short / non-finite blocks: tests/test_legacy32.py.
 *   recipe ................ reference KATs commands/quantize.rs:1561-1608.
 */
#include "pmetal_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define QK_K 256
#define K_SCALE_SIZE 12

/* ------------------------------------------------------------------------- */
/* half 2.7.1: f16::from_f32 / to_f32, bf16::from_f32 / to_f32               */
/* (call sites k_quants.rs:928-929, :1097, :359-360, :475; quantize.rs:285;  */
/*  dequant.rs:482).  IEEE round-to-nearest-even, subnormals kept,           */
/*  overflow -> inf, NaN kept as a quiet NaN.                                */
/* ------------------------------------------------------------------------- */

static uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

static float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

uint16_t pmo_f32_to_f16(float f) {
    uint32_t x = f32_bits(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x007FFFFFu;
    if (exp == 0xFFu) {
        uint32_t nan_bit = man ? 0x0200u : 0u;
        return (uint16_t)(sign | 0x7C00u | nan_bit | (man >> 13));
    }
    int32_t half_exp = (int32_t)exp - 127 + 15;
    if (half_exp >= 0x1F) return (uint16_t)(sign | 0x7C00u);
    if (half_exp <= 0) {
        if (14 - half_exp > 24) return (uint16_t)sign;
        uint32_t m = man | 0x00800000u;
        uint32_t shift = (uint32_t)(14 - half_exp);
        uint32_t half_man = m >> shift;
        uint32_t round_bit = 1u << (shift - 1);
        /* round to nearest, ties to even */
        if ((m & round_bit) && (m & (3u * round_bit - 1u))) half_man += 1;
        return (uint16_t)(sign | half_man);
    }
    uint32_t out = sign | ((uint32_t)half_exp << 10) | (man >> 13);
    uint32_t round_bit = 0x00001000u;
    if ((man & round_bit) && (man & (3u * round_bit - 1u))) out += 1; /* may carry into exp: correct */
    return (uint16_t)out;
}

float pmo_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = ((uint32_t)h >> 10) & 0x1Fu;
    uint32_t man = (uint32_t)h & 0x03FFu;
    if (exp == 0x1Fu) return bits_f32(sign | 0x7F800000u | (man ? (0x00400000u | (man << 13)) : 0u));
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: value = man * 2^-24, exact in f32 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t pmo_f32_to_bf16(float f) {
    uint32_t x = f32_bits(f);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x0040u);
    uint32_t round_bit = 0x00008000u;
    if ((x & round_bit) && (x & (3u * round_bit - 1u))) return (uint16_t)((x >> 16) + 1u);
    return (uint16_t)(x >> 16);
}

float pmo_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* ------------------------------------------------------------------------- */
/* Rust core semantics                                                       */
/* ------------------------------------------------------------------------- */

/* `v as i32` for f32: saturating, NaN -> 0. */
static int32_t f32_as_i32(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}

/* f32::total_cmp: -1, 0, +1 */
static int total_cmp(float a, float b) {
    int32_t l = (int32_t)f32_bits(a);
    int32_t r = (int32_t)f32_bits(b);
    l ^= (int32_t)(((uint32_t)(l >> 31)) >> 1);
    r ^= (int32_t)(((uint32_t)(r >> 31)) >> 1);
    return (l > r) - (l < r);
}

/* f32::max / f32::min (IEEE 754-2008 maxNum / minNum: a NaN operand is ignored).  For the pair
 * (-0.0, +0.0) IEEE leaves the result open; the reference only runs on Apple Silicon (MLX/Metal),
 * whose FMAXNM / FMINNM order -0.0 below +0.0, so that is what is restated here (the C library's
 * own max would return its first argument instead). */
static float rust_max(float a, float b) {
    if (a != a) return b;
    if (b != b) return a;
    if (a == b) return bits_f32(f32_bits(a) & f32_bits(b)); /* +0 wins over -0 */
    return a > b ? a : b;
}

static float rust_min(float a, float b) {
    if (a != a) return b;
    if (b != b) return a;
    if (a == b) return bits_f32(f32_bits(a) | f32_bits(b)); /* -0 wins over +0 */
    return a < b ? a : b;
}

static int32_t clamp_i32(int32_t v, int32_t lo, int32_t hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* quantize.rs:566-570: `v.round() as i32` -- half away from zero, saturating. */
int32_t pmo_nearest_int(float v) { return f32_as_i32(roundf(v)); }

/* ------------------------------------------------------------------------- */
/* quantize.rs:583-644 make_qkx1_quants                                      */
/* ------------------------------------------------------------------------- */
void pmo_make_qkx1_quants(int32_t nmax, int32_t ntry, const float *x, int32_t n, float *scale_out,
                          float *min_out) {
    uint8_t l[QK_K];
    memset(l, 0, sizeof l);

    /* :588-593 min_by/max_by with total_cmp (first minimum, last maximum). */
    float min = x[0], max = x[0];
    for (int32_t i = 1; i < n; i++) {
        if (total_cmp(min, x[i]) > 0) min = x[i];
        if (total_cmp(max, x[i]) <= 0) max = x[i];
    }
    /* :596 */
    if (max == min) {
        *scale_out = 0.0f;
        *min_out = 0.0f;
        return;
    }
    /* :601 */
    min = rust_min(min, 0.0f);
    /* :604-605 */
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;

    for (int32_t t = 0; t < ntry; t++) {
        float sumlx = 0.0f;
        int32_t suml2 = 0;
        int did_change = 0;
        /* :612-621 */
        for (int32_t i = 0; i < n; i++) {
            int32_t li = clamp_i32(pmo_nearest_int(iscale * (x[i] - min)), 0, nmax);
            uint8_t cl = (uint8_t)li;
            if (cl != l[i]) {
                l[i] = cl;
                did_change = 1;
            }
            sumlx += (x[i] - min) * (float)li;
            suml2 += li * li;
        }
        /* :622-624 */
        if (suml2 == 0) break;
        /* :625 */
        scale = sumlx / (float)suml2;
        /* :627-632 Iterator::sum::<f32>: sequential; Rust >= 1.83 (the reference
         * pins rust-version 1.89) folds from -0.0. */
        float sum = -0.0f;
        for (int32_t i = 0; i < n; i++) sum += x[i] - scale * (float)l[i];
        /* :634-637 */
        min = sum / (float)n;
        if (min > 0.0f) min = 0.0f;
        /* :638-641 */
        iscale = 1.0f / scale;
        if (!did_change) break;
    }
    *scale_out = scale;
    *min_out = -min;
}

/* ------------------------------------------------------------------------- */
/* quantize.rs:738-841 make_qx_quants                                        */
/* ------------------------------------------------------------------------- */
float pmo_make_qx_quants(int32_t n, int32_t nmax, const float *x, int32_t rmse_type, int8_t *ls) {
    memset(ls, 0, (size_t)n);

    /* :742-750 */
    float max = 0.0f, amax = 0.0f;
    for (int32_t i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) {
            amax = ax;
            max = x[i];
        }
    }
    /* :752-754 */
    if (amax == 0.0f) return 0.0f;
    /* :756 */
    float iscale = -(float)nmax / max;

    /* :758-764 */
    if (rmse_type == 0) {
        for (int32_t i = 0; i < n; i++) {
            int32_t l = pmo_nearest_int(iscale * x[i]);
            ls[i] = (int8_t)(nmax + clamp_i32(l, -nmax, nmax - 1));
        }
        return 1.0f / iscale;
    }

    int32_t weight_type = rmse_type % 2;
    float sumlx = 0.0f, suml2 = 0.0f;
    /* :770-776 */
    for (int32_t i = 0; i < n; i++) {
        int32_t l = clamp_i32(pmo_nearest_int(iscale * x[i]), -nmax, nmax - 1);
        ls[i] = (int8_t)(l + nmax);
        float w = weight_type == 1 ? x[i] * x[i] : 1.0f;
        sumlx += w * x[i] * (float)l;
        suml2 += w * (float)(l * l);
    }
    /* :778-779 */
    float scale = sumlx / suml2;
    float best = scale * sumlx;

    /* :782-810 */
    for (int32_t t = 0; t < 3; t++) {
        float iscale2 = 1.0f / scale;
        float slx = 0.0f, sl2 = 0.0f;
        int changed = 0;
        for (int32_t i = 0; i < n; i++) {
            int32_t l = clamp_i32(pmo_nearest_int(iscale2 * x[i]), -nmax, nmax - 1);
            if (l + nmax != (int32_t)ls[i]) changed = 1;
            float w = weight_type == 1 ? x[i] * x[i] : 1.0f;
            slx += w * x[i] * (float)l;
            sl2 += w * (float)(l * l);
        }
        if (!changed || sl2 == 0.0f || slx * slx <= best * sl2) break;
        for (int32_t i = 0; i < n; i++) {
            int32_t l = pmo_nearest_int(iscale2 * x[i]);
            ls[i] = (int8_t)(nmax + clamp_i32(l, -nmax, nmax - 1));
        }
        sumlx = slx;
        suml2 = sl2;
        scale = sumlx / suml2;
        best = scale * sumlx;
    }

    /* :813-838 */
    for (int32_t t = 0; t < 5; t++) {
        int32_t n_changed = 0;
        for (int32_t i = 0; i < n; i++) {
            float w = weight_type == 1 ? x[i] * x[i] : 1.0f;
            int32_t l = (int32_t)ls[i] - nmax;
            float slx = sumlx - w * x[i] * (float)l;
            if (slx > 0.0f) {
                float sl2 = suml2 - w * (float)(l * l);
                int32_t new_l = clamp_i32(pmo_nearest_int(x[i] * sl2 / slx), -nmax, nmax - 1);
                if (new_l != l) {
                    slx += w * x[i] * (float)new_l;
                    sl2 += w * (float)(new_l * new_l);
                    if (sl2 > 0.0f && slx * slx * suml2 > sumlx * sumlx * sl2) {
                        ls[i] = (int8_t)(nmax + new_l);
                        sumlx = slx;
                        suml2 = sl2;
                        scale = sumlx / suml2;
                        n_changed += 1;
                    }
                }
            }
        }
        if (n_changed == 0) break;
    }
    return scale;
}

/* quantize.rs:844-855 */
void pmo_get_scale_min_k4(int32_t j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* ------------------------------------------------------------------------- */
/* types.rs:102-187                                                          */
/* ------------------------------------------------------------------------- */
size_t pmo_type_size(uint32_t t) {
    switch (t) {
    case PMO_TYPE_F32: return 4;
    case PMO_TYPE_F16: return 2;
    case PMO_TYPE_Q4_0: return 18;
    case PMO_TYPE_Q4_1: return 20;
    case PMO_TYPE_Q5_0: return 22;
    case PMO_TYPE_Q5_1: return 24;
    case PMO_TYPE_Q8_0: return 34;
    case PMO_TYPE_Q8_1: return 36;
    case PMO_TYPE_Q2K: return 84;
    case PMO_TYPE_Q3K: return 110;
    case PMO_TYPE_Q4K: return 144;
    case PMO_TYPE_Q5K: return 176;
    case PMO_TYPE_Q6K: return 210;
    case PMO_TYPE_Q8K: return 292;
    default: return 0;
    }
}

size_t pmo_block_size(uint32_t t) {
    switch (t) {
    case PMO_TYPE_F32:
    case PMO_TYPE_F16: return 1;
    case PMO_TYPE_Q4_0:
    case PMO_TYPE_Q4_1:
    case PMO_TYPE_Q5_0:
    case PMO_TYPE_Q5_1:
    case PMO_TYPE_Q8_1:
    case PMO_TYPE_Q8_0: return 32;
    case PMO_TYPE_Q2K:
    case PMO_TYPE_Q3K:
    case PMO_TYPE_Q4K:
    case PMO_TYPE_Q5K:
    case PMO_TYPE_Q6K:
    case PMO_TYPE_Q8K: return 256;
    default: return 0;
    }
}

size_t pmo_tensor_size(uint32_t t, size_t n) {
    size_t bs = pmo_block_size(t);
    if (bs == 0) return 0;
    size_t n_blocks = n / bs + (n % bs != 0);
    return n_blocks * pmo_type_size(t);
}

/* ------------------------------------------------------------------------- */
/* quantize.rs:268-300 quantize_q8_0                                         */
/* ------------------------------------------------------------------------- */
void pmo_quantize_q8_0(const float *x, size_t n, uint8_t *dst) {
    size_t n_blocks = n / 32 + (n % 32 != 0);
    for (size_t b = 0; b < n_blocks; b++) {
        size_t start = b * 32;
        size_t end = start + 32 < n ? start + 32 : n;
        float amax = 0.0f;
        for (size_t i = start; i < end; i++) amax = rust_max(amax, fabsf(x[i])); /* acc.max(x.abs()) */
        float scale = amax / 127.0f;
        float iscale = amax == 0.0f ? 0.0f : 127.0f / amax;
        uint16_t d = pmo_f32_to_f16(scale);
        uint8_t *out = dst + b * 34;
        out[0] = (uint8_t)(d & 0xFF);
        out[1] = (uint8_t)(d >> 8);
        for (size_t i = 0; i < 32; i++) {
            int8_t v = 0;
            if (start + i < end) v = (int8_t)clamp_i32(pmo_nearest_int(x[start + i] * iscale), -127, 127);
            out[2 + i] = (uint8_t)v;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* The 32-element formats beside Q8_0: quantize.rs:93-230, :302-359 and      */
/* dequant.rs:300-463, :505-528.  A short last block is quantized over the   */
/* elements it has (its minimum / maximum are taken over those only) with    */
/* 0.0 standing in for the missing ones.                                     */
/* ------------------------------------------------------------------------- */
static int is_finite_f32(float v) { return (f32_bits(v) & 0x7F800000u) != 0x7F800000u; }

/* quantize.rs:332-342 */
static float signed_absmax(const float *x, size_t n) {
    float s = 0.0f, absmax = 0.0f;
    for (size_t i = 0; i < n; i++)
        if (is_finite_f32(x[i]) && fabsf(x[i]) > absmax) absmax = fabsf(x[i]), s = x[i];
    return s;
}

/* quantize.rs:344-359; f32::min / f32::max over finite values only, so no NaN reaches them */
static void block_min_max(const float *x, size_t n, float *mn, float *mx) {
    float lo = INFINITY, hi = -INFINITY;
    *mn = *mx = 0.0f;
    if (n == 0) return;
    for (size_t i = 0; i < n; i++) {
        if (!is_finite_f32(x[i])) continue;
        /* equal values of opposite-signed zeros: f32::min keeps -0.0 over +0.0 and f32::max +0.0 over -0.0 on the
           reference's targets; only the value matters below (min is encoded as f16, where -0.0 and +0.0 differ) */
        if (x[i] < lo || (x[i] == lo && (f32_bits(x[i]) >> 31))) lo = x[i];
        if (x[i] > hi || (x[i] == hi && !(f32_bits(x[i]) >> 31))) hi = x[i];
    }
    if (is_finite_f32(lo) && is_finite_f32(hi)) *mn = lo, *mx = hi;
}

static void put_f16(uint8_t *p, float v) {
    uint16_t h = pmo_f32_to_f16(v);
    p[0] = (uint8_t)(h & 0xFF), p[1] = (uint8_t)(h >> 8);
}
static float get_f16(const uint8_t *p) { return pmo_f16_to_f32((uint16_t)(p[0] | (p[1] << 8))); }
static float at_or_zero(const float *x, size_t len, size_t i) { return i < len ? x[i] : 0.0f; }

/* quantize.rs:93-128 */
void pmo_quantize_q4_0(const float *x, size_t n, uint8_t *dst) {
    size_t n_blocks = n / 32 + (n % 32 != 0);
    for (size_t b = 0; b < n_blocks; b++) {
        const float *blk = x + b * 32;
        size_t len = n - b * 32 < 32 ? n - b * 32 : 32;
        float max = 0.0f, amax = 0.0f;
        for (size_t i = 0; i < len; i++) {
            float ax = fabsf(blk[i]);
            if (ax > amax) amax = ax, max = blk[i];
        }
        float scale = max / -8.0f;
        float iscale = scale == 0.0f ? 0.0f : 1.0f / scale;
        uint8_t *out = dst + b * 18;
        put_f16(out, scale);
        for (size_t i = 0; i < 16; i++) {
            int32_t q0 = clamp_i32(pmo_nearest_int(at_or_zero(blk, len, i) * iscale + 8.5f), 0, 15);
            int32_t q1 = clamp_i32(pmo_nearest_int(at_or_zero(blk, len, i + 16) * iscale + 8.5f), 0, 15);
            out[2 + i] = (uint8_t)(q0 | (q1 << 4));
        }
    }
}

/* quantize.rs:130-157 */
void pmo_quantize_q4_1(const float *x, size_t n, uint8_t *dst) {
    size_t n_blocks = n / 32 + (n % 32 != 0);
    for (size_t b = 0; b < n_blocks; b++) {
        const float *blk = x + b * 32;
        size_t len = n - b * 32 < 32 ? n - b * 32 : 32;
        float mn, mx;
        block_min_max(blk, len, &mn, &mx);
        float scale = (mx - mn) / 15.0f;
        float iscale = scale == 0.0f ? 0.0f : 1.0f / scale;
        uint8_t *out = dst + b * 20;
        put_f16(out, scale);
        put_f16(out + 2, mn);
        for (size_t i = 0; i < 16; i++) {
            int32_t q0 = clamp_i32(pmo_nearest_int((at_or_zero(blk, len, i) - mn) * iscale), 0, 15);
            int32_t q1 = clamp_i32(pmo_nearest_int((at_or_zero(blk, len, i + 16) - mn) * iscale), 0, 15);
            out[4 + i] = (uint8_t)(q0 | (q1 << 4));
        }
    }
}

/* quantize.rs:159-191 (Q5_0) and :193-230 (Q5_1) */
static void quantize_q5(const float *x, size_t n, uint8_t *dst, int with_min) {
    size_t n_blocks = n / 32 + (n % 32 != 0), bytes = with_min ? 24 : 22;
    for (size_t b = 0; b < n_blocks; b++) {
        const float *blk = x + b * 32;
        size_t len = n - b * 32 < 32 ? n - b * 32 : 32;
        float mn = 0.0f, mx = 0.0f, scale;
        if (with_min) {
            block_min_max(blk, len, &mn, &mx);
            scale = (mx - mn) / 31.0f;
        } else {
            scale = signed_absmax(blk, len) / -16.0f;
        }
        float iscale = scale == 0.0f ? 0.0f : 1.0f / scale;
        uint32_t qh = 0;
        uint8_t qs[16];
        for (size_t i = 0; i < 16; i++) {
            float x0 = at_or_zero(blk, len, i), x1 = at_or_zero(blk, len, i + 16);
            int32_t q0, q1;
            if (with_min) {
                q0 = clamp_i32(pmo_nearest_int((x0 - mn) * iscale), 0, 31);
                q1 = clamp_i32(pmo_nearest_int((x1 - mn) * iscale), 0, 31);
            } else {
                q0 = clamp_i32(pmo_nearest_int(x0 * iscale + 16.5f), 0, 31);
                q1 = clamp_i32(pmo_nearest_int(x1 * iscale + 16.5f), 0, 31);
            }
            qs[i] = (uint8_t)((q0 & 0x0F) | ((q1 & 0x0F) << 4));
            qh |= (uint32_t)((q0 & 0x10) >> 4) << i;
            qh |= (uint32_t)((q1 & 0x10) >> 4) << (i + 16);
        }
        uint8_t *out = dst + b * bytes;
        put_f16(out, scale);
        out += 2;
        if (with_min) put_f16(out, mn), out += 2;
        out[0] = (uint8_t)qh, out[1] = (uint8_t)(qh >> 8), out[2] = (uint8_t)(qh >> 16), out[3] = (uint8_t)(qh >> 24);
        memcpy(out + 4, qs, 16);
    }
}
void pmo_quantize_q5_0(const float *x, size_t n, uint8_t *dst) { quantize_q5(x, n, dst, 0); }
void pmo_quantize_q5_1(const float *x, size_t n, uint8_t *dst) { quantize_q5(x, n, dst, 1); }

/* quantize.rs:302-330 */
void pmo_quantize_q8_1(const float *x, size_t n, uint8_t *dst) {
    size_t n_blocks = n / 32 + (n % 32 != 0);
    for (size_t b = 0; b < n_blocks; b++) {
        const float *blk = x + b * 32;
        size_t len = n - b * 32 < 32 ? n - b * 32 : 32;
        float amax = 0.0f;
        for (size_t i = 0; i < len; i++) amax = rust_max(amax, fabsf(blk[i]));
        float scale = amax / 127.0f;
        float iscale = amax == 0.0f ? 0.0f : 127.0f / amax;
        uint8_t *out = dst + b * 36;
        int32_t sum = 0;
        for (size_t i = 0; i < 32; i++) {
            int32_t q = clamp_i32(pmo_nearest_int(at_or_zero(blk, len, i) * iscale), -127, 127);
            out[4 + i] = (uint8_t)(int8_t)q;
            sum += q;
        }
        put_f16(out, scale);
        put_f16(out + 2, (float)sum * scale);
    }
}

/* dequant.rs:300-334 (Q4_0), :344-371 (Q4_1), :382-414 (Q5_0), :425-463 (Q5_1), :505-528 (Q8_1) */
void pmo_dequantize_legacy(uint32_t t, const uint8_t *src, size_t n, float *dst) {
    size_t n_blocks = n / 32 + (n % 32 != 0), bytes = pmo_type_size(t);
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = src + b * bytes;
        float v[32];
        float scale = get_f16(blk);
        if (t == PMO_TYPE_Q8_1) {
            for (int i = 0; i < 32; i++) v[i] = (float)(int8_t)blk[4 + i] * scale;
        } else if (t == PMO_TYPE_Q4_0) {
            for (int i = 0; i < 16; i++) {
                v[i] = (float)(int8_t)((int8_t)(blk[2 + i] & 0x0F) - 8) * scale;
                v[i + 16] = (float)(int8_t)((int8_t)(blk[2 + i] >> 4) - 8) * scale;
            }
        } else if (t == PMO_TYPE_Q4_1) {
            float mn = get_f16(blk + 2);
            for (int i = 0; i < 16; i++) {
                v[i] = (float)(blk[4 + i] & 0x0F) * scale + mn;
                v[i + 16] = (float)(blk[4 + i] >> 4) * scale + mn;
            }
        } else {
            int with_min = t == PMO_TYPE_Q5_1;
            float mn = with_min ? get_f16(blk + 2) : 0.0f;
            const uint8_t *p = blk + (with_min ? 4 : 2);
            uint32_t qh = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
            const uint8_t *qs = p + 4;
            for (int i = 0; i < 16; i++) {
                int32_t q_lo = (int32_t)(qs[i] & 0x0F) | (int32_t)(((qh >> i) & 1u) << 4);
                int32_t q_hi = (int32_t)(qs[i] >> 4) | (int32_t)(((qh >> (i + 16)) & 1u) << 4);
                if (with_min) {
                    v[i] = (float)q_lo * scale + mn;
                    v[i + 16] = (float)q_hi * scale + mn;
                } else {
                    v[i] = (float)(q_lo - 16) * scale;
                    v[i + 16] = (float)(q_hi - 16) * scale;
                }
            }
        }
        for (size_t i = 0; i < 32 && b * 32 + i < n; i++) dst[b * 32 + i] = v[i];
    }
}

/* ------------------------------------------------------------------------- */
/* k_quants.rs:876-955 quantize_q4k                                          */
/* ------------------------------------------------------------------------- */
void pmo_quantize_q4k(const float *xs, size_t n, uint8_t *dst) {
    size_t n_blocks = n / QK_K + (n % QK_K != 0);
    memset(dst, 0, n_blocks * 144); /* :878-886; f16::from_f32(0.0) = 0x0000 */
    for (size_t b = 0; b < n_blocks; b++) {
        size_t start = b * QK_K;
        if (start + QK_K > n) continue; /* :890-892 trailing partial block stays zero */
        const float *x = xs + start;
        uint8_t *blk = dst + b * 144;
        uint8_t *bscales = blk + 4;
        uint8_t *qs = blk + 16;

        float mins[8], scales[8];
        for (int j = 0; j < 8; j++) pmo_make_qkx1_quants(15, 5, x + 32 * j, 32, &scales[j], &mins[j]);

        /* :904-905 fold(0.0, |max, val| val.max(max)) */
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < 8; j++) max_scale = rust_max(scales[j], max_scale);
        for (int j = 0; j < 8; j++) max_min = rust_max(mins[j], max_min);

        float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
        float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;

        /* :915-926 */
        for (int j = 0; j < 8; j++) {
            int32_t a = pmo_nearest_int(inv_scale * scales[j]);
            int32_t c = pmo_nearest_int(inv_min * mins[j]);
            uint8_t ls = (uint8_t)(a < 63 ? a : 63);
            uint8_t lm = (uint8_t)(c < 63 ? c : 63);
            if (j < 4) {
                bscales[j] = ls;
                bscales[j + 4] = lm;
            } else {
                bscales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                bscales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                bscales[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }

        /* :928-929 */
        uint16_t d16 = pmo_f32_to_f16(max_scale / 63.0f);
        uint16_t dmin16 = pmo_f32_to_f16(max_min / 63.0f);
        blk[0] = (uint8_t)(d16 & 0xFF);
        blk[1] = (uint8_t)(d16 >> 8);
        blk[2] = (uint8_t)(dmin16 & 0xFF);
        blk[3] = (uint8_t)(dmin16 >> 8);
        float df = pmo_f16_to_f32(d16), dminf = pmo_f16_to_f32(dmin16);

        /* :932-943 */
        uint8_t l[QK_K];
        memset(l, 0, sizeof l);
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m;
            pmo_get_scale_min_k4(j, bscales, &sc, &m);
            float d = df * (float)sc;
            if (d != 0.0f) {
                float dm = dminf * (float)m;
                for (int ii = 0; ii < 32; ii++) {
                    int32_t lv = pmo_nearest_int((x[32 * j + ii] + dm) / d);
                    l[32 * j + ii] = (uint8_t)clamp_i32(lv, 0, 15);
                }
            }
        }
        /* :946-951 */
        for (int j = 0; j < QK_K; j += 64)
            for (int lv = 0; lv < 32; lv++)
                qs[(j / 64) * 32 + lv] = (uint8_t)(l[j + lv] | (l[j + lv + 32] << 4));
    }
}

/* ------------------------------------------------------------------------- */
/* k_quants.rs:1056-1134 quantize_q6k                                        */
/* ------------------------------------------------------------------------- */
void pmo_quantize_q6k(const float *xs, size_t n, uint8_t *dst) {
    size_t n_blocks = n / QK_K + (n % QK_K != 0);
    memset(dst, 0, n_blocks * 210);
    for (size_t b = 0; b < n_blocks; b++) {
        size_t start = b * QK_K;
        if (start + QK_K > n) continue; /* :1070-1072 */
        const float *x = xs + start;
        uint8_t *blk = dst + b * 210;
        uint8_t *ql = blk, *qh = blk + 128;
        int8_t *bscales = (int8_t *)(blk + 192);

        int8_t l[QK_K];
        float scales_f[16];
        float max_scale = 0.0f, max_abs_scale = 0.0f;

        /* :1082-1094 */
        for (int ib = 0; ib < 16; ib++) {
            float scale = pmo_make_qx_quants(16, 32, x + 16 * ib, 1, l + 16 * ib);
            scales_f[ib] = scale;
            float abs_scale = fabsf(scale);
            if (abs_scale > max_abs_scale) {
                max_abs_scale = abs_scale;
                max_scale = scale;
            }
        }
        /* :1096-1097 (all-zero block: iscale = -inf, d = f16(-0.0) = 0x8000) */
        float iscale = -128.0f / max_scale;
        uint16_t d16 = pmo_f32_to_f16(1.0f / iscale);
        blk[208] = (uint8_t)(d16 & 0xFF);
        blk[209] = (uint8_t)(d16 >> 8);
        float df = pmo_f16_to_f32(d16);

        /* :1100-1102 `.min(127) as i8` (i32 -> i8 wraps) */
        for (int j = 0; j < 16; j++) {
            int32_t v = pmo_nearest_int(iscale * scales_f[j]);
            if (v > 127) v = 127;
            bscales[j] = (int8_t)(uint8_t)(uint32_t)v;
        }
        /* :1105-1113 */
        for (int j = 0; j < 16; j++) {
            float d = df * (float)bscales[j];
            if (d != 0.0f) {
                for (int ii = 0; ii < 16; ii++) {
                    int32_t ll = clamp_i32(pmo_nearest_int(x[16 * j + ii] / d), -32, 31);
                    l[16 * j + ii] = (int8_t)(ll + 32);
                }
            }
        }
        /* :1116-1130 */
        for (int j = 0; j < QK_K; j += 128) {
            for (int li = 0; li < 32; li++) {
                uint8_t a = (uint8_t)l[j + li], c = (uint8_t)l[j + li + 32];
                uint8_t e = (uint8_t)l[j + li + 64], g = (uint8_t)l[j + li + 96];
                ql[j / 2 + li] = (uint8_t)((a & 0xF) | ((e & 0xF) << 4));
                ql[j / 2 + li + 32] = (uint8_t)((c & 0xF) | ((g & 0xF) << 4));
                qh[j / 4 + li] = (uint8_t)((a >> 4) | ((c >> 4) << 2) | ((e >> 4) << 4) | ((g >> 4) << 6));
            }
        }
    }
}

/* ------------------------------------------------------------------------- */
/* dequant.rs:466-495 dequantize_q8_0 (body)                                 */
/* ------------------------------------------------------------------------- */
void pmo_dequantize_q8_0(const uint8_t *src, size_t n, float *dst) {
    size_t n_blocks = n / 32 + (n % 32 != 0);
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = src + b * 34;
        float scale = pmo_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        for (size_t i = 0; i < 32 && b * 32 + i < n; i++) dst[b * 32 + i] = (float)(int8_t)blk[2 + i] * scale;
    }
}

/* ------------------------------------------------------------------------- */
/* k_quants.rs:358-404 dequantize_q4k + :515-560 dequantize_q4k_bytes        */
/* ------------------------------------------------------------------------- */
static void dequantize_q4k_block(const uint8_t *blk, float *out, uint32_t order) {
    float d = pmo_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
    float dmin = pmo_f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
    const uint8_t *scales = blk + 4;
    const uint8_t *qs = blk + 16;
    int idx = 0, is = 0;
    for (int j = 0; j < QK_K; j += 64) {
        uint8_t sc1, m1, sc2, m2;
        pmo_get_scale_min_k4(is, scales, &sc1, &m1);
        float d1 = d * (float)sc1, dm1 = dmin * (float)m1;
        pmo_get_scale_min_k4(is + 1, scales, &sc2, &m2);
        float d2 = d * (float)sc2, dm2 = dmin * (float)m2;
        const uint8_t *q = qs + j / 2;
        if (order == PMO_ORDER_REF) {
            /* :380-400: 16 low, 16 high of bytes 0..15 with (d1, dm1); then bytes 16..31 with (d2, dm2) */
            for (int l = 0; l < 16; l++) out[idx++] = d1 * (float)(q[l] & 0xF) - dm1;
            for (int l = 0; l < 16; l++) out[idx++] = d1 * (float)(q[l] >> 4) - dm1;
            for (int l = 0; l < 16; l++) out[idx++] = d2 * (float)(q[16 + l] & 0xF) - dm2;
            for (int l = 0; l < 16; l++) out[idx++] = d2 * (float)(q[16 + l] >> 4) - dm2;
        } else {
            /* the inverse of the quantizer's packing, k_quants.rs:946-951 */
            for (int l = 0; l < 32; l++) out[idx++] = d1 * (float)(q[l] & 0xF) - dm1;
            for (int l = 0; l < 32; l++) out[idx++] = d2 * (float)(q[l] >> 4) - dm2;
        }
        is += 2;
    }
}

void pmo_dequantize_q4k(const uint8_t *src, size_t n, float *dst, uint32_t order) {
    size_t n_blocks = n / QK_K + (n % QK_K != 0);
    float tmp[QK_K];
    for (size_t b = 0; b < n_blocks; b++) {
        dequantize_q4k_block(src + b * 144, tmp, order);
        size_t cnt = n - b * QK_K < QK_K ? n - b * QK_K : QK_K;
        memcpy(dst + b * QK_K, tmp, cnt * sizeof(float));
    }
}

/* ------------------------------------------------------------------------- */
/* k_quants.rs:474-496 dequantize_q6k + :614-660 dequantize_q6k_bytes        */
/* ------------------------------------------------------------------------- */
static void dequantize_q6k_block(const uint8_t *blk, float *out) {
    float d = pmo_f16_to_f32((uint16_t)(blk[208] | (blk[209] << 8)));
    for (int n = 0; n < QK_K; n += 128) {
        int c = n / 128;
        float *ys = out + n;
        const int8_t *sc = (const int8_t *)(blk + 192 + 8 * c);
        const uint8_t *ql = blk + 64 * c;
        const uint8_t *qh = blk + 128 + 32 * c;
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            int8_t q1 = (int8_t)((int8_t)((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32);
            int8_t q2 = (int8_t)((int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
            int8_t q3 = (int8_t)((int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
            int8_t q4 = (int8_t)((int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
            ys[l] = d * (float)sc[is] * (float)q1;
            ys[l + 32] = d * (float)sc[is + 2] * (float)q2;
            ys[l + 64] = d * (float)sc[is + 4] * (float)q3;
            ys[l + 96] = d * (float)sc[is + 6] * (float)q4;
        }
    }
}

void pmo_dequantize_q6k(const uint8_t *src, size_t n, float *dst) {
    size_t n_blocks = n / QK_K + (n % QK_K != 0);
    float tmp[QK_K];
    for (size_t b = 0; b < n_blocks; b++) {
        dequantize_q6k_block(src + b * 210, tmp);
        size_t cnt = n - b * QK_K < QK_K ? n - b * QK_K : QK_K;
        memcpy(dst + b * QK_K, tmp, cnt * sizeof(float));
    }
}

/* ------------------------------------------------------------------------- */
/* k_quants.rs:960-1051 quantize_q5k, :407-462 dequantize_q5k                */
/* ------------------------------------------------------------------------- */
void pmo_quantize_q5k(const float *xs, size_t n, uint8_t *dst) {
    size_t n_blocks = n / QK_K + (n % QK_K != 0);
    memset(dst, 0, n_blocks * 176); /* :962-971; a partial last block is skipped (:975-977) */
    for (size_t b = 0; b < n / QK_K; b++) {
        const float *x = xs + b * QK_K;
        uint8_t *blk = dst + b * 176, *sc_bytes = blk + 4, *qh = blk + 16, *qs = blk + 48;
        float mins[8], scales[8];
        for (int j = 0; j < 8; j++) pmo_make_qkx1_quants(31, 5, x + 32 * j, 32, &scales[j], &mins[j]); /* :983-985 */
        float max_scale = 0.0f, max_min = 0.0f; /* :987-988 fold(0.0, |max, val| val.max(max)) */
        for (int j = 0; j < 8; j++) {
            max_scale = rust_max(scales[j], max_scale);
            max_min = rust_max(mins[j], max_min);
        }
        float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f; /* :990-995 */
        float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
        for (int j = 0; j < 8; j++) { /* :997-1008 */
            int32_t a = pmo_nearest_int(inv_scale * scales[j]), c = pmo_nearest_int(inv_min * mins[j]);
            uint8_t ls = (uint8_t)(a < 63 ? a : 63), lm = (uint8_t)(c < 63 ? c : 63);
            if (j < 4) {
                sc_bytes[j] = ls;
                sc_bytes[j + 4] = lm;
            } else {
                sc_bytes[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                sc_bytes[j - 4] |= (uint8_t)((ls >> 4) << 6);
                sc_bytes[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        uint16_t d16 = pmo_f32_to_f16(max_scale / 63.0f), dmin16 = pmo_f32_to_f16(max_min / 63.0f); /* :1010-1011 */
        memcpy(blk, &d16, 2);
        memcpy(blk + 2, &dmin16, 2);
        uint8_t l[QK_K];
        memset(l, 0, sizeof l);
        for (int j = 0; j < 8; j++) { /* :1013-1024 */
            uint8_t sc, m;
            pmo_get_scale_min_k4(j, sc_bytes, &sc, &m);
            float d = pmo_f16_to_f32(d16) * (float)sc;
            if (d != 0.0f) {
                float dm = pmo_f16_to_f32(dmin16) * (float)m;
                for (int ii = 0; ii < 32; ii++)
                    l[32 * j + ii] = (uint8_t)clamp_i32(pmo_nearest_int((x[32 * j + ii] + dm) / d), 0, 31);
            }
        }
        uint8_t m1 = 1, m2 = 2; /* :1027-1047 */
        for (int n0 = 0; n0 < QK_K; n0 += 64) {
            int offset = (n0 / 64) * 32;
            for (int j = 0; j < 32; j++) {
                uint8_t l1 = l[n0 + j], l2 = l[n0 + j + 32];
                if (l1 > 15) {
                    l1 -= 16;
                    qh[j] |= m1;
                }
                if (l2 > 15) {
                    l2 -= 16;
                    qh[j] |= m2;
                }
                qs[offset + j] = (uint8_t)(l1 | (l2 << 4));
            }
            m1 = (uint8_t)(m1 << 2);
            m2 = (uint8_t)(m2 << 2);
        }
    }
}

static void dequantize_q5k_block(const uint8_t *blk, float *out, uint32_t order) {
    uint16_t d16, dmin16;
    memcpy(&d16, blk, 2);
    memcpy(&dmin16, blk + 2, 2);
    const float d = pmo_f16_to_f32(d16), dmin = pmo_f16_to_f32(dmin16);
    const uint8_t *scales = blk + 4, *qh = blk + 16, *qs = blk + 48;
    int idx = 0, is = 0;
    for (int j = 0; j < QK_K; j += 64) { /* :414-459 */
        uint8_t sc1, m1, sc2, m2;
        pmo_get_scale_min_k4(is, scales, &sc1, &m1);
        pmo_get_scale_min_k4(is + 1, scales, &sc2, &m2);
        const float d1 = d * (float)sc1, dm1 = dmin * (float)m1, d2 = d * (float)sc2, dm2 = dmin * (float)m2;
        const int q_start = j / 2, qh_start = j / 8, c = j / 64;
        for (int half = 0; half < 2; half++) {
            for (int l = 0; l < 32; l++) {
                uint8_t nib, bit;
                if (order == PMO_ORDER_REF) { /* :426-438, :442-455 */
                    const uint8_t byte = qs[q_start + 16 * half + l / 2];
                    nib = (l % 2 == 0) ? (uint8_t)(byte & 0xF) : (uint8_t)(byte >> 4);
                    bit = (uint8_t)((qh[qh_start + 4 * half + l / 8] >> (l % 8)) & 1);
                } else { /* inverse of :1030-1047 */
                    const uint8_t byte = qs[32 * c + l];
                    nib = half ? (uint8_t)(byte >> 4) : (uint8_t)(byte & 0xF);
                    bit = (uint8_t)((qh[l] >> (2 * c + half)) & 1);
                }
                const uint8_t q = (uint8_t)(nib | (bit << 4));
                out[idx++] = half ? d2 * (float)q - dm2 : d1 * (float)q - dm1;
            }
        }
        is += 2;
    }
}

void pmo_dequantize_q5k(const uint8_t *src, size_t n, float *dst, uint32_t order) {
    size_t n_blocks = n / QK_K + (n % QK_K != 0);
    float tmp[QK_K];
    for (size_t b = 0; b < n_blocks; b++) {
        dequantize_q5k_block(src + b * 176, tmp, order);
        size_t cnt = n - b * QK_K < QK_K ? n - b * QK_K : QK_K;
        memcpy(dst + b * QK_K, tmp, cnt * sizeof(float));
    }
}

/* ------------------------------------------------------------------------- */
/* k_quants.rs:1242-1321 quantize_q2k, :230-266 dequantize_q2k               */
/* Block (84 bytes): scales[16] (low nibble scale, high nibble min), qs[64],  */
/* d f16, dmin f16.                                                           */
/* ------------------------------------------------------------------------- */
void pmo_quantize_q2k(const float *xs, size_t n, uint8_t *dst) {
    size_t n_blocks = n / QK_K + (n % QK_K != 0);
    memset(dst, 0, n_blocks * 84); /* :1246-1255; a partial last block is skipped (:1259-1261) */
    for (size_t b = 0; b < n / QK_K; b++) {
        const float *x = xs + b * QK_K;
        uint8_t *blk = dst + b * 84, *bscales = blk, *qs = blk + 16;
        float mins[16], scales[16];
        for (int j = 0; j < 16; j++) pmo_make_qkx1_quants(3, 5, x + 16 * j, 16, &scales[j], &mins[j]); /* :1267-1271 */
        float max_scale = 0.0f, max_min = 0.0f; /* :1273-1274 fold(0.0, |max, val| val.max(max)) */
        for (int j = 0; j < 16; j++) max_scale = rust_max(scales[j], max_scale);
        for (int j = 0; j < 16; j++) max_min = rust_max(mins[j], max_min);
        uint16_t d16 = 0, dmin16 = 0;
        if (max_scale > 0.0f) { /* :1276-1285; `as u8` keeps the low eight bits of the i32 */
            float iscale = 15.0f / max_scale;
            for (int j = 0; j < 16; j++) bscales[j] = (uint8_t)(uint32_t)pmo_nearest_int(iscale * scales[j]);
            d16 = pmo_f32_to_f16(max_scale / 15.0f);
        }
        if (max_min > 0.0f) { /* :1287-1296; `l << 4` on a u8 drops the bits shifted out */
            float iscale = 15.0f / max_min;
            for (int j = 0; j < 16; j++) {
                uint8_t l = (uint8_t)(uint32_t)pmo_nearest_int(iscale * mins[j]);
                bscales[j] |= (uint8_t)(l << 4);
            }
            dmin16 = pmo_f32_to_f16(max_min / 15.0f);
        }
        memcpy(blk + 80, &d16, 2);
        memcpy(blk + 82, &dmin16, 2);
        uint8_t l[QK_K];
        memset(l, 0, sizeof l);
        for (int j = 0; j < 16; j++) { /* :1299-1310 */
            float d = pmo_f16_to_f32(d16) * (float)(bscales[j] & 0xF);
            if (d == 0.0f) continue;
            float dm = pmo_f16_to_f32(dmin16) * (float)(bscales[j] >> 4);
            for (int ii = 0; ii < 16; ii++)
                l[16 * j + ii] = (uint8_t)clamp_i32(pmo_nearest_int((x[16 * j + ii] + dm) / d), 0, 3);
        }
        for (int j = 0; j < QK_K; j += 128) /* :1313-1320 */
            for (int ll = 0; ll < 32; ll++)
                qs[j / 4 + ll] = (uint8_t)(l[j + ll] | (l[j + ll + 32] << 2) | (l[j + ll + 64] << 4) | (l[j + ll + 96] << 6));
    }
}

static void dequantize_q2k_block(const uint8_t *blk, float *out) {
    uint16_t d16, dmin16;
    memcpy(&d16, blk + 80, 2);
    memcpy(&dmin16, blk + 82, 2);
    const float d = pmo_f16_to_f32(d16), min = pmo_f16_to_f32(dmin16);
    const uint8_t *scales = blk;
    int idx = 0, is = 0;
    for (int h = 0; h < 2; h++) { /* :237-265 */
        const uint8_t *qs = blk + 16 + 32 * h;
        for (int shift = 0; shift < 8; shift += 2) {
            for (int sub = 0; sub < 2; sub++) {
                const uint8_t sc = scales[is++];
                const float dl = d * (float)(sc & 0xF), ml = min * (float)(sc >> 4);
                for (int i = 0; i < 16; i++) out[idx++] = dl * (float)((qs[16 * sub + i] >> shift) & 3) - ml;
            }
        }
    }
}

void pmo_dequantize_q2k(const uint8_t *src, size_t n, float *dst) {
    size_t n_blocks = n / QK_K + (n % QK_K != 0);
    float tmp[QK_K];
    for (size_t b = 0; b < n_blocks; b++) {
        dequantize_q2k_block(src + b * 84, tmp);
        size_t cnt = n - b * QK_K < QK_K ? n - b * QK_K : QK_K;
        memcpy(dst + b * QK_K, tmp, cnt * sizeof(float));
    }
}

/* ------------------------------------------------------------------------- */
/* quantize.rs:655-727 make_q3_quants; k_quants.rs:1139-1237 quantize_q3k,    */
/* :281-355 dequantize_q3k.  Block (110 bytes): hmask[32], qs[64],            */
/* scales[12], d f16.                                                         */
/* ------------------------------------------------------------------------- */
float pmo_make_q3_quants(const float *x, int32_t n, int32_t nmax, int32_t do_rmse, int8_t *ls) {
    int8_t l[QK_K];
    memset(l, 0, sizeof l);
    float max = 0.0f, amax = 0.0f; /* :659-667 */
    for (int32_t i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) {
            amax = ax;
            max = x[i];
        }
    }
    if (amax == 0.0f) { /* :669-671 */
        if (ls) memset(ls, 0, (size_t)n);
        return 0.0f;
    }
    float iscale = -(float)nmax / max; /* :673 */
    if (do_rmse) {
        float sumlx = 0.0f, suml2 = 0.0f; /* :676-685 */
        for (int32_t i = 0; i < n; i++) {
            int32_t li = clamp_i32(f32_as_i32(roundf(iscale * x[i])), -nmax, nmax - 1);
            l[i] = (int8_t)li;
            float w = x[i] * x[i];
            sumlx += w * x[i] * (float)li;
            suml2 += w * (float)(li * li);
        }
        for (int sweep = 0; sweep < 5; sweep++) { /* :688-713 */
            int n_changed = 0;
            for (int32_t i = 0; i < n; i++) {
                float w = x[i] * x[i];
                float slx = sumlx - w * x[i] * (float)l[i];
                if (slx > 0.0f) {
                    float sl2 = suml2 - w * (float)((int32_t)l[i] * (int32_t)l[i]);
                    int32_t new_l = clamp_i32(f32_as_i32(roundf(x[i] * sl2 / slx)), -nmax, nmax - 1);
                    if (new_l != (int32_t)l[i]) {
                        slx += w * x[i] * (float)new_l;
                        sl2 += w * (float)(new_l * new_l);
                        if (sl2 > 0.0f && slx * slx * suml2 > sumlx * sumlx * sl2) {
                            l[i] = (int8_t)new_l;
                            sumlx = slx;
                            suml2 = sl2;
                            n_changed++;
                        }
                    }
                }
            }
            if (n_changed == 0) break;
        }
        if (ls)
            for (int32_t i = 0; i < n; i++) ls[i] = (int8_t)(l[i] + nmax); /* :715-717 */
        return sumlx / suml2;
    }
    for (int32_t i = 0; i < n; i++) { /* :722-726 */
        int32_t li = clamp_i32(f32_as_i32(roundf(iscale * x[i])), -nmax, nmax - 1);
        if (ls) ls[i] = (int8_t)(li + nmax);
    }
    return 1.0f / iscale;
}

void pmo_quantize_q3k(const float *xs, size_t n, uint8_t *dst) {
    size_t n_blocks = n / QK_K + (n % QK_K != 0);
    memset(dst, 0, n_blocks * 110); /* :1141-1150; a partial last block is skipped (:1154-1156) */
    for (size_t b = 0; b < n / QK_K; b++) {
        const float *x = xs + b * QK_K;
        uint8_t *blk = dst + b * 110, *hmask = blk, *qs = blk + 32, *bscales = blk + 96;
        float scales_f[16];
        for (int j = 0; j < 16; j++) scales_f[j] = pmo_make_q3_quants(x + 16 * j, 16, 4, 1, NULL); /* :1159-1162 */
        float max_scale = 0.0f; /* :1165-1170 */
        for (int j = 0; j < 16; j++)
            if (fabsf(scales_f[j]) > fabsf(max_scale)) max_scale = scales_f[j];
        uint16_t d16 = pmo_f32_to_f16(0.0f);
        if (max_scale != 0.0f) { /* :1174-1186 */
            float iscale = -32.0f / max_scale;
            for (int j = 0; j < 16; j++) {
                int32_t l_val = clamp_i32(pmo_nearest_int(iscale * scales_f[j]), -32, 31) + 32;
                if (j < 8) bscales[j] = (uint8_t)(l_val & 0xF);
                else bscales[j - 8] |= (uint8_t)((l_val & 0xF) << 4);
                l_val >>= 4;
                bscales[j % 4 + 8] |= (uint8_t)(l_val << (2 * (j / 4)));
            }
            d16 = pmo_f32_to_f16(1.0f / iscale);
        }
        memcpy(blk + 108, &d16, 2);
        int8_t l[QK_K];
        memset(l, 0, sizeof l);
        for (int j = 0; j < 16; j++) { /* :1192-1206 */
            uint8_t sc = j < 8 ? (uint8_t)(bscales[j] & 0xF) : (uint8_t)(bscales[j - 8] >> 4);
            int8_t scs = (int8_t)((int8_t)(sc | (((bscales[8 + j % 4] >> (2 * (j / 4))) & 3) << 4)) - 32);
            float d = pmo_f16_to_f32(d16) * (float)scs;
            if (d != 0.0f)
                for (int ii = 0; ii < 16; ii++)
                    l[16 * j + ii] = (int8_t)(clamp_i32(pmo_nearest_int(x[16 * j + ii] / d), -4, 3) + 4);
        }
        int m = 0; /* :1209-1224 */
        uint8_t hm = 1;
        for (int i = 0; i < QK_K; i++) {
            if (l[i] > 3) {
                hmask[m] |= hm;
                l[i] = (int8_t)(l[i] - 4);
            }
            if (++m == QK_K / 8) {
                m = 0;
                hm = (uint8_t)(hm << 1);
            }
        }
        for (int j = 0; j < QK_K; j += 128) /* :1227-1234 */
            for (int ll = 0; ll < 32; ll++)
                qs[j / 4 + ll] = (uint8_t)(l[j + ll] | (l[j + ll + 32] << 2) | (l[j + ll + 64] << 4) | (l[j + ll + 96] << 6));
    }
}

static void dequantize_q3k_block(const uint8_t *blk, float *out) {
    uint16_t d16;
    memcpy(&d16, blk + 108, 2);
    const float d = pmo_f16_to_f32(d16);
    const uint8_t *hmask = blk, *bscales = blk + 96;
    uint32_t aux[4] = {0, 0, 0, 0}; /* :285-314 */
    for (int i = 0; i < 3; i++)
        aux[i] = (uint32_t)bscales[4 * i] | (uint32_t)bscales[4 * i + 1] << 8 | (uint32_t)bscales[4 * i + 2] << 16 |
                 (uint32_t)bscales[4 * i + 3] << 24;
    const uint32_t k1 = 0x03030303u, k2 = 0x0f0f0f0fu, tmp = aux[2];
    aux[2] = ((aux[0] >> 4) & k2) | (((tmp >> 4) & k1) << 4);
    aux[3] = ((aux[1] >> 4) & k2) | (((tmp >> 6) & k1) << 4);
    aux[0] = (aux[0] & k2) | ((tmp & k1) << 4);
    aux[1] = (aux[1] & k2) | (((tmp >> 2) & k1) << 4);
    int8_t scales[16]; /* :317-323 */
    for (int i = 0; i < 4; i++)
        for (int j = 0; j < 4; j++) scales[4 * i + j] = (int8_t)((int8_t)(uint8_t)(aux[i] >> (8 * j)) - 32);
    int is = 0, idx = 0; /* :332-354 */
    uint8_t m = 1;
    for (int h = 0; h < 2; h++) {
        const uint8_t *qs = blk + 32 + 32 * h;
        for (int shift = 0; shift < 8; shift += 2) {
            for (int sub = 0; sub < 2; sub++) {
                const float dl = d * (float)scales[is++];
                for (int i = 0; i < 16; i++) {
                    const int qi = i + 16 * sub;
                    const int8_t q = (int8_t)(((qs[qi] >> shift) & 3) + ((hmask[qi] & m) ? 0 : -4));
                    out[idx++] = dl * (float)q;
                }
            }
            m = (uint8_t)(m << 1);
        }
    }
}

void pmo_dequantize_q3k(const uint8_t *src, size_t n, float *dst) {
    size_t n_blocks = n / QK_K + (n % QK_K != 0);
    float tmp[QK_K];
    for (size_t b = 0; b < n_blocks; b++) {
        dequantize_q3k_block(src + b * 110, tmp);
        size_t cnt = n - b * QK_K < QK_K ? n - b * QK_K : QK_K;
        memcpy(dst + b * QK_K, tmp, cnt * sizeof(float));
    }
}

/* ------------------------------------------------------------------------- */
/* Q8_K: k_quants.rs:815-871 quantize_q8k; vec_dot.rs:617-692 (scalar)        */
/* ------------------------------------------------------------------------- */
size_t pmo_q8k_size(size_t n) { return (n / 256 + (n % 256 != 0)) * 292; }

/* `v as i8` for f32: saturating, NaN -> 0 */
static int8_t f32_as_i8(float v) {
    if (v != v) return 0;
    if (v >= 127.0f) return 127;
    if (v <= -128.0f) return -128;
    return (int8_t)v;
}

void pmo_quantize_q8k(const float *xs, size_t n, uint8_t *dst) {
    size_t n_blocks = n / 256 + (n % 256 != 0);
    memset(dst, 0, n_blocks * 292); /* :818-825; a partial last block is skipped (:829-834) */
    for (size_t b = 0; b + 1 <= n / 256; b++) {
        const float *x = xs + b * 256;
        uint8_t *blk = dst + b * 292;
        /* :837-844 */
        float max = 0.0f, amax = 0.0f;
        for (int i = 0; i < 256; i++) {
            if (fabsf(x[i]) > amax) {
                amax = fabsf(x[i]);
                max = x[i];
            }
        }
        if (amax == 0.0f) continue; /* :846-851 */
        float iscale = -128.0f / max; /* :853 */
        int8_t q[256];
        for (int j = 0; j < 256; j++) { /* :854-857: v.round().min(127.0) as i8; f32::min returns the non-NaN operand */
            float v = roundf(iscale * x[j]);
            v = rust_min(v, 127.0f);
            q[j] = f32_as_i8(v);
        }
        memcpy(blk + 4, q, 256);
        for (int j = 0; j < 16; j++) { /* :860-866 */
            int32_t sum = 0;
            for (int ii = 0; ii < 16; ii++) sum += q[j * 16 + ii];
            int16_t s16 = (int16_t)sum;
            memcpy(blk + 260 + 2 * j, &s16, 2);
        }
        float d = 1.0f / iscale; /* :868 */
        memcpy(blk, &d, 4);
    }
}

/* k_quants.rs:498-506 */
void pmo_dequantize_q8k(const uint8_t *src, size_t n, float *dst) {
    for (size_t i = 0; i < n; i++) {
        const uint8_t *blk = src + (i / 256) * 292;
        float d;
        memcpy(&d, blk, 4);
        dst[i] = d * (float)(int8_t)blk[4 + i % 256];
    }
}

/* dynamic.rs:140-180 */
double pmo_kl_divergence(const float *original, const float *dequantized, size_t n) {
    if (n == 0) return 0.0;
    double sq_err_sum = 0.0, sq_orig_sum = 0.0;
    for (size_t i = 0; i < n; i++) { /* :150-154: the difference is taken in f32, then widened */
        double diff = (double)(original[i] - dequantized[i]);
        sq_err_sum += diff * diff;
        sq_orig_sum += (double)original[i] * (double)original[i];
    }
    double nrmse = sq_orig_sum > 0.0 ? sqrt(sq_err_sum / (double)n) / sqrt(sq_orig_sum / (double)n) : 0.0;
    double dot = 0.0, norm_a = 0.0, norm_b = 0.0;
    for (size_t i = 0; i < n; i++) { /* :163-169 */
        double a = (double)original[i], b = (double)dequantized[i];
        dot += a * b;
        norm_a += a * a;
        norm_b += b * b;
    }
    double cos_sim = (norm_a > 0.0 && norm_b > 0.0) ? dot / (sqrt(norm_a) * sqrt(norm_b)) : 1.0;
    return nrmse + (1.0 - cos_sim);
}

/* vec_dot.rs:617-656 */
float pmo_vec_dot_q4k_q8k(const uint8_t *xs, const uint8_t *ys, size_t n_blocks) {
    float sum = 0.0f;
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *x = xs + b * 144, *y = ys + b * 292;
        uint16_t d16, dmin16;
        float yd;
        memcpy(&d16, x, 2);
        memcpy(&dmin16, x + 2, 2);
        memcpy(&yd, y, 4);
        const uint8_t *scales = x + 4, *qs = x + 16;
        const int8_t *q8 = (const int8_t *)(y + 4);
        float d = pmo_f16_to_f32(d16) * yd;       /* :621 */
        float dmin = pmo_f16_to_f32(dmin16) * yd; /* :622 */
        int32_t mins_sum = 0;                     /* :625-630 */
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m;
            int16_t b0, b1;
            pmo_get_scale_min_k4(j, scales, &sc, &m);
            memcpy(&b0, y + 260 + 2 * (2 * j), 2);
            memcpy(&b1, y + 260 + 2 * (2 * j + 1), 2);
            mins_sum += (int32_t)m * ((int32_t)b0 + (int32_t)b1);
        }
        sum -= dmin * (float)mins_sum; /* :631 */
        int32_t sumi = 0;              /* :633-650 */
        for (int j = 0; j < 4; j++) {
            uint8_t sc0, sc1, m;
            pmo_get_scale_min_k4(j * 2, scales, &sc0, &m);
            pmo_get_scale_min_k4(j * 2 + 1, scales, &sc1, &m);
            for (int k = 0; k < 32; k++) {
                int32_t q4l = qs[j * 32 + k] & 0x0F, q4h = qs[j * 32 + k] >> 4;
                sumi += q4l * (int32_t)q8[j * 64 + k] * (int32_t)sc0;
                sumi += q4h * (int32_t)q8[j * 64 + k + 32] * (int32_t)sc1;
            }
        }
        sum += d * (float)sumi; /* :652 */
    }
    return sum;
}

/* vec_dot.rs:658-692 */
float pmo_vec_dot_q6k_q8k(const uint8_t *xs, const uint8_t *ys, size_t n_blocks) {
    float sum = 0.0f;
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *x = xs + b * 210, *y = ys + b * 292;
        const uint8_t *ql = x, *qh = x + 128;
        const int8_t *scales = (const int8_t *)(x + 192);
        const int8_t *q8 = (const int8_t *)(y + 4);
        uint16_t d16;
        float yd;
        memcpy(&d16, x + 208, 2);
        memcpy(&yd, y, 4);
        float d = pmo_f16_to_f32(d16) * yd; /* :662 */
        int32_t sumi = 0;
        for (int j = 0; j < 16; j++) { /* :665-686 */
            int32_t scale = scales[j];
            for (int k = 0; k < 16; k++) {
                int idx = j * 16 + k;
                uint8_t lo = (idx % 2 == 0) ? (uint8_t)(ql[idx / 2] & 0x0F) : (uint8_t)(ql[idx / 2] >> 4);
                uint8_t hi = (uint8_t)((qh[idx / 4] >> ((idx % 4) * 2)) & 0x03);
                int32_t q6 = (int32_t)(lo | (hi << 4)) - 32;
                sumi += q6 * (int32_t)q8[idx] * scale;
            }
        }
        sum += d * (float)sumi; /* :688 */
    }
    return sum;
}

/* vec_dot.rs:695-737 (scalar): element j of a super-block takes the low (j even) or high nibble of qs[j / 2], bit j % 8 of
 * qh[j / 8] and the scale of sub-block j / 32; the min term as for Q4_K. */
float pmo_vec_dot_q5k_q8k(const uint8_t *xs, const uint8_t *ys, size_t n_blocks) {
    float sum = 0.0f;
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *x = xs + b * 176, *y = ys + b * 292;
        const uint8_t *scales = x + 4, *qh = x + 16, *qs = x + 48;
        const int8_t *q8 = (const int8_t *)(y + 4);
        uint16_t d16, m16;
        float yd;
        memcpy(&d16, x, 2);
        memcpy(&m16, x + 2, 2);
        memcpy(&yd, y, 4);
        float d = pmo_f16_to_f32(d16) * yd, dmin = pmo_f16_to_f32(m16) * yd; /* :699-700 */
        int32_t mins_sum = 0;
        for (int j = 0; j < 8; j++) { /* :703-708 */
            uint8_t sc, m;
            int16_t b0, b1;
            pmo_get_scale_min_k4(j, scales, &sc, &m);
            memcpy(&b0, y + 260 + 4 * j, 2);
            memcpy(&b1, y + 262 + 4 * j, 2);
            mins_sum += (int32_t)m * ((int32_t)b0 + (int32_t)b1);
        }
        sum -= dmin * (float)mins_sum; /* :709 */
        int32_t sumi = 0;
        for (int j = 0; j < 256; j++) { /* :712-731 */
            uint8_t ql = (j % 2 == 0) ? (uint8_t)(qs[j / 2] & 0x0F) : (uint8_t)(qs[j / 2] >> 4);
            uint8_t hi = (uint8_t)(((qh[j / 8] >> (j % 8)) & 0x01) << 4);
            int32_t q5 = (int32_t)(ql | hi);
            uint8_t sc, m;
            pmo_get_scale_min_k4(j / 32, scales, &sc, &m);
            sumi += q5 * (int32_t)q8[j] * (int32_t)sc;
        }
        sum += d * (float)sumi; /* :733 */
    }
    return sum;
}

/* vec_dot.rs:739-777 (scalar): only the first eight scales are unpacked (the low nibbles of scales[0..4], minus 8); the
 * scales of sub-blocks 8..15 stay zero, so the second half of every super-block contributes nothing.  Element j takes
 * bits 2 (j % 4) .. of qs[j / 4] and bit j % 8 of hmask[j / 8] as its third bit, minus 4. */
float pmo_vec_dot_q3k_q8k(const uint8_t *xs, const uint8_t *ys, size_t n_blocks) {
    float sum = 0.0f;
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *x = xs + b * 110, *y = ys + b * 292;
        const uint8_t *hmask = x, *qs = x + 32, *sc12 = x + 96;
        const int8_t *q8 = (const int8_t *)(y + 4);
        uint16_t d16;
        float yd;
        memcpy(&d16, x + 108, 2);
        memcpy(&yd, y, 4);
        float d = pmo_f16_to_f32(d16) * yd; /* :743 */
        int32_t scales[16] = {0};
        int32_t aux0 = (int32_t)((uint32_t)sc12[0] | ((uint32_t)sc12[1] << 8) | ((uint32_t)sc12[2] << 16) | ((uint32_t)sc12[3] << 24));
        for (int i = 0; i < 8; i++) scales[i] = (int32_t)(int8_t)((aux0 >> (4 * i)) & 0xF) - 8; /* :747-755 */
        int32_t sumi = 0;
        for (int j = 0; j < 256; j++) { /* :757-771 */
            uint8_t ql = (uint8_t)((qs[j / 4] >> ((j % 4) * 2)) & 0x03);
            uint8_t hi = (uint8_t)(((hmask[j / 8] >> (j % 8)) & 0x01) << 2);
            int32_t q3 = (int32_t)(ql | hi) - 4;
            sumi += q3 * (int32_t)q8[j] * scales[j / 16];
        }
        sum += d * (float)sumi; /* :773 */
    }
    return sum;
}

/* vec_dot.rs:779-810 (scalar): element j takes bits 2 (j % 4) .. of qs[j / 4] and the low nibble of scales[j / 16]; the
 * min term is the high nibble of scales[j] times bsums[j]. */
float pmo_vec_dot_q2k_q8k(const uint8_t *xs, const uint8_t *ys, size_t n_blocks) {
    float sum = 0.0f;
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *x = xs + b * 84, *y = ys + b * 292;
        const uint8_t *scales = x, *qs = x + 16;
        const int8_t *q8 = (const int8_t *)(y + 4);
        uint16_t d16, m16;
        float yd;
        memcpy(&d16, x + 80, 2);
        memcpy(&m16, x + 82, 2);
        memcpy(&yd, y, 4);
        float d = pmo_f16_to_f32(d16) * yd, dmin = pmo_f16_to_f32(m16) * yd; /* :783-784 */
        int32_t mins_sum = 0;
        for (int j = 0; j < 16; j++) { /* :787-792 */
            int16_t bs;
            memcpy(&bs, y + 260 + 2 * j, 2);
            mins_sum += (int32_t)(scales[j] >> 4) * (int32_t)bs;
        }
        sum -= dmin * (float)mins_sum; /* :793 */
        int32_t sumi = 0;
        for (int j = 0; j < 256; j++) { /* :796-803 */
            int32_t q2 = (int32_t)((qs[j / 4] >> ((j % 4) * 2)) & 0x03);
            sumi += q2 * (int32_t)q8[j] * (int32_t)(scales[j / 16] & 0x0F);
        }
        sum += d * (float)sumi; /* :805 */
    }
    return sum;
}

int32_t pmo_qmatvec_q8k(uint32_t t, const uint8_t *w, size_t n_rows, size_t k, const uint8_t *xq, float *y) {
    float (*dot)(const uint8_t *, const uint8_t *, size_t) = t == PMO_TYPE_Q4K   ? pmo_vec_dot_q4k_q8k
                                                             : t == PMO_TYPE_Q6K ? pmo_vec_dot_q6k_q8k
                                                             : t == PMO_TYPE_Q5K ? pmo_vec_dot_q5k_q8k
                                                             : t == PMO_TYPE_Q3K ? pmo_vec_dot_q3k_q8k
                                                             : t == PMO_TYPE_Q2K ? pmo_vec_dot_q2k_q8k
                                                                                 : NULL;
    if (!dot) return PMO_ERR_UNSUPPORTED_TYPE;
    if (k % 256 != 0) return PMO_ERR_INVALID_SHAPE;
    size_t spr = k / 256, row = spr * pmo_type_size(t);
    for (size_t r = 0; r < n_rows; r++) y[r] = dot(w + r * row, xq, spr);
    return PMO_OK;
}

/* ------------------------------------------------------------------------- */
/* quantize.rs:17-87 and dequant.rs:92-132, :184-216                         */
/* ------------------------------------------------------------------------- */
int32_t pmo_quantize(uint32_t t, const float *x, size_t n, uint8_t *dst, size_t dst_len) {
    int legacy = t == PMO_TYPE_Q4_0 || t == PMO_TYPE_Q4_1 || t == PMO_TYPE_Q5_0 || t == PMO_TYPE_Q5_1 || t == PMO_TYPE_Q8_1;
    if (!legacy && t != PMO_TYPE_Q8_0 && t != PMO_TYPE_Q2K && t != PMO_TYPE_Q3K && t != PMO_TYPE_Q4K && t != PMO_TYPE_Q5K && t != PMO_TYPE_Q6K && t != PMO_TYPE_Q8K)
        return PMO_ERR_UNSUPPORTED_TYPE;
    if (dst_len != pmo_tensor_size(t, n)) return PMO_ERR_INVALID_SIZE;
    if (t == PMO_TYPE_Q4_0) return pmo_quantize_q4_0(x, n, dst), PMO_OK;
    if (t == PMO_TYPE_Q4_1) return pmo_quantize_q4_1(x, n, dst), PMO_OK;
    if (t == PMO_TYPE_Q5_0) return pmo_quantize_q5_0(x, n, dst), PMO_OK;
    if (t == PMO_TYPE_Q5_1) return pmo_quantize_q5_1(x, n, dst), PMO_OK;
    if (t == PMO_TYPE_Q8_1) return pmo_quantize_q8_1(x, n, dst), PMO_OK;
    if (t == PMO_TYPE_Q8K) pmo_quantize_q8k(x, n, dst);
    else if (t == PMO_TYPE_Q2K) pmo_quantize_q2k(x, n, dst);
    else if (t == PMO_TYPE_Q3K) pmo_quantize_q3k(x, n, dst);
    else if (t == PMO_TYPE_Q8_0) pmo_quantize_q8_0(x, n, dst);
    else if (t == PMO_TYPE_Q4K) pmo_quantize_q4k(x, n, dst);
    else if (t == PMO_TYPE_Q5K) pmo_quantize_q5k(x, n, dst);
    else pmo_quantize_q6k(x, n, dst);
    return PMO_OK;
}

int32_t pmo_dequantize(uint32_t t, const uint8_t *src, size_t src_len, const int32_t *shape, size_t ndim,
                       float *dst, size_t dst_cap, uint32_t order) {
    int legacy = t == PMO_TYPE_Q4_0 || t == PMO_TYPE_Q4_1 || t == PMO_TYPE_Q5_0 || t == PMO_TYPE_Q5_1 || t == PMO_TYPE_Q8_1;
    if (!legacy && t != PMO_TYPE_Q8_0 && t != PMO_TYPE_Q2K && t != PMO_TYPE_Q3K && t != PMO_TYPE_Q4K && t != PMO_TYPE_Q5K && t != PMO_TYPE_Q6K && t != PMO_TYPE_Q8K)
        return PMO_ERR_UNSUPPORTED_TYPE;
    /* dequant.rs:193-206 shape_n_elements */
    for (size_t i = 0; i < ndim; i++)
        if (shape[i] < 0) return PMO_ERR_INVALID_SHAPE;
    size_t n = 1;
    for (size_t i = 0; i < ndim; i++) {
        size_t dim = (size_t)shape[i];
        if (dim != 0 && n > SIZE_MAX / dim) return PMO_ERR_SHAPE_TOO_LARGE;
        n *= dim;
    }
    /* dequant.rs:208-216 validate_data_size */
    if (src_len != pmo_tensor_size(t, n)) return PMO_ERR_INVALID_SIZE;
    if (dst_cap < n) return PMO_ERR_INVALID_SIZE;
    if (legacy) pmo_dequantize_legacy(t, src, n, dst);
    else if (t == PMO_TYPE_Q8_0) pmo_dequantize_q8_0(src, n, dst);
    else if (t == PMO_TYPE_Q4K) pmo_dequantize_q4k(src, n, dst, order);
    else if (t == PMO_TYPE_Q5K) pmo_dequantize_q5k(src, n, dst, order);
    else if (t == PMO_TYPE_Q8K) pmo_dequantize_q8k(src, n, dst);
    else if (t == PMO_TYPE_Q2K) pmo_dequantize_q2k(src, n, dst);
    else if (t == PMO_TYPE_Q3K) pmo_dequantize_q3k(src, n, dst);
    else pmo_dequantize_q6k(src, n, dst);
    return PMO_OK;
}

/* ------------------------------------------------------------------------- */
/* crates/pmetal/src/commands/quantize.rs:955-1137 (method q4_k_m)           */
/* ------------------------------------------------------------------------- */
int32_t pmo_use_more_bits(size_t layer, size_t n_layers) {
    if (n_layers == 0) return 0;
    size_t sat = layer >= n_layers / 8 ? layer - n_layers / 8 : 0; /* saturating_sub */
    return layer < n_layers / 8 || layer >= 7 * n_layers / 8 || sat % 3 == 2;
}

static int ends_with(const char *s, const char *suffix) {
    size_t a = strlen(s), b = strlen(suffix);
    return a >= b && memcmp(s + a - b, suffix, b) == 0;
}

int32_t pmo_is_quantizable_gguf_tensor(const char *name, size_t ndim) {
    static const char *const deny[] = {
        "_norm.weight", "norm.weight", "ffn_gate_inp.weight", "router", "altup", "laurel",
        "per_layer_model_proj", "pos_embd", "token_types", "ssm_conv1d", "shortconv.conv.weight",
        "attn_rel_b.weight", ".position_embd", ".rel_pos", ".patch_embd", ".patch_merger"};
    if (!(ndim == 2 || ndim == 3) || !ends_with(name, ".weight")) return 0;
    char lower[512];
    size_t len = strlen(name);
    if (len >= sizeof lower) len = sizeof lower - 1;
    for (size_t i = 0; i < len; i++) {
        char c = name[i];
        lower[i] = (c >= 'A' && c <= 'Z') ? (char)(c + 32) : c;
    }
    lower[len] = 0;
    for (size_t i = 0; i < sizeof deny / sizeof deny[0]; i++)
        if (strstr(lower, deny[i])) return 0;
    return 1;
}

/* parse_layer_from_gguf_name :982-986: "blk.<n>.rest" */
static int parse_layer(const char *name, size_t *layer) {
    if (strncmp(name, "blk.", 4) != 0) return 0;
    const char *p = name + 4;
    const char *dot = strchr(p, '.');
    if (!dot || dot == p) return 0;
    size_t v = 0;
    const char *q = p;
    if (*q == '+') q++; /* usize::from_str accepts a leading '+' */
    if (q == dot) return 0;
    for (; q < dot; q++) {
        if (*q < '0' || *q > '9') return 0;
        v = v * 10 + (size_t)(*q - '0');
    }
    *layer = v;
    return 1;
}

uint32_t pmo_q4km_tensor_type(const char *name, size_t ndim, size_t n_layers) {
    if (!pmo_is_quantizable_gguf_tensor(name, ndim)) return PMO_TYPE_F16; /* :1015-1017 */
    uint32_t dtype = PMO_TYPE_Q4K;                                        /* :1019-1023 */
    size_t layer = 0;
    if (!parse_layer(name, &layer)) layer = 0; /* :1034 */
    if (strcmp(name, "output.weight") == 0 || strcmp(name, "token_embd.weight") == 0)
        return PMO_TYPE_Q6K; /* :1036-1055 */
    if (strstr(name, "attn_v.weight")) { /* :1058-1090, arm Q4KM :1075-1081 */
        if (pmo_use_more_bits(layer, n_layers)) dtype = PMO_TYPE_Q6K;
    } else if (strstr(name, "ffn_down.weight") || strstr(name, "ffn_down_exps.weight")) {
        if (pmo_use_more_bits(layer, n_layers)) dtype = PMO_TYPE_Q6K; /* :1104-1110 */
    } else if (strstr(name, "attn_output.weight")) {
        /* :1120-1126: q4_k_m keeps the default */
    } else if (strstr(name, "attn_qkv.weight")) {
        /* :1127-1133: q4_k_m -> Q5K, a type outside this path; reported as its GgmlType id 13 */
        dtype = 13;
    }
    return dtype;
}

/* ------------------------------------------------------------------------- */
/* dequantize-then-matmul (definition of the fused kernels' expected output) */
/* ------------------------------------------------------------------------- */
static int32_t dequant_row(uint32_t t, const uint8_t *w, size_t row, size_t k, float *tmp, uint32_t order) {
    size_t row_bytes = pmo_tensor_size(t, k);
    if (t == PMO_TYPE_Q8_0) pmo_dequantize_q8_0(w + row * row_bytes, k, tmp);
    else if (t == PMO_TYPE_Q4K) pmo_dequantize_q4k(w + row * row_bytes, k, tmp, order);
    else if (t == PMO_TYPE_Q5K) pmo_dequantize_q5k(w + row * row_bytes, k, tmp, order);
    else if (t == PMO_TYPE_Q2K) pmo_dequantize_q2k(w + row * row_bytes, k, tmp);
    else if (t == PMO_TYPE_Q3K) pmo_dequantize_q3k(w + row * row_bytes, k, tmp);
    else if (t == PMO_TYPE_Q6K) pmo_dequantize_q6k(w + row * row_bytes, k, tmp);
    else return PMO_ERR_UNSUPPORTED_TYPE;
    return PMO_OK;
}

int32_t pmo_qmatvec_f64(uint32_t t, const uint8_t *w, size_t n_rows, size_t k, const float *x, float *y,
                        uint32_t order) {
    size_t bs = pmo_block_size(t);
    if (bs <= 1 || k % bs != 0) return PMO_ERR_INVALID_SHAPE;
    float *tmp = (float *)malloc(k * sizeof(float));
    if (!tmp) return PMO_ERR_SHAPE_TOO_LARGE;
    for (size_t r = 0; r < n_rows; r++) {
        dequant_row(t, w, r, k, tmp, order);
        double acc = 0.0;
        for (size_t i = 0; i < k; i++) acc += (double)tmp[i] * (double)x[i];
        y[r] = (float)acc;
    }
    free(tmp);
    return PMO_OK;
}

int32_t pmo_qmatvec_f32(uint32_t t, const uint8_t *w, size_t n_rows, size_t k, const float *x, float *y,
                        uint32_t order) {
    size_t bs = pmo_block_size(t);
    if (bs <= 1 || k % bs != 0) return PMO_ERR_INVALID_SHAPE;
    float *tmp = (float *)malloc(k * sizeof(float));
    if (!tmp) return PMO_ERR_SHAPE_TOO_LARGE;
    for (size_t r = 0; r < n_rows; r++) {
        dequant_row(t, w, r, k, tmp, order);
        float acc = 0.0f;
        for (size_t i = 0; i < k; i++) acc += tmp[i] * x[i];
        y[r] = acc;
    }
    free(tmp);
    return PMO_OK;
}

int32_t pmo_qmatmul_f64(uint32_t t, const uint8_t *w, size_t n_rows, size_t k, const float *x, size_t m_rows,
                        float *y, uint32_t order) {
    size_t bs = pmo_block_size(t);
    if (bs <= 1 || k % bs != 0) return PMO_ERR_INVALID_SHAPE;
    float *tmp = (float *)malloc(k * sizeof(float));
    if (!tmp) return PMO_ERR_SHAPE_TOO_LARGE;
    for (size_t r = 0; r < n_rows; r++) {
        dequant_row(t, w, r, k, tmp, order);
        for (size_t m = 0; m < m_rows; m++) {
            const float *xr = x + m * k;
            double acc = 0.0;
            for (size_t i = 0; i < k; i++) acc += (double)tmp[i] * (double)xr[i];
            y[m * n_rows + r] = (float)acc;
        }
    }
    free(tmp);
    return PMO_OK;
}

/* ------------------------------------------------------------------------- */
/* The same functions over several host threads.  The reference runs this path */
/* on one thread (no rayon in crates/pmetal-gguf); these exist so that whole    */
/* tensors can be checked in a test's time budget and so that the benchmark can */
/* report an all-cores CPU figure beside the single-thread one.  Every thread   */
/* calls the single-threaded function above on its own range of blocks or rows, */
/* so the results are the single-threaded ones bit for bit.                     */
/* ------------------------------------------------------------------------- */
typedef struct {
    int kind; /* 0 quantize, 1 matvec f32, 2 matvec f64, 3 matmul f64 */
    uint32_t t, order;
    const float *x;
    const uint8_t *w;
    uint8_t *dst;
    float *y;
    size_t lo, hi, n, k, m_rows, n_rows;
} mt_job;

static void *mt_run(void *arg) {
    mt_job *j = (mt_job *)arg;
    if (j->kind == 0) { /* blocks [lo, hi) of a flat tensor of n elements */
        size_t bs = pmo_block_size(j->t), ts = pmo_type_size(j->t);
        size_t e0 = j->lo * bs, e1 = j->hi * bs < j->n ? j->hi * bs : j->n;
        (void)pmo_quantize(j->t, j->x + e0, e1 - e0, j->dst + j->lo * ts, pmo_tensor_size(j->t, e1 - e0));
    } else if (j->kind == 1 || j->kind == 2) { /* rows [lo, hi) */
        size_t row_bytes = pmo_tensor_size(j->t, j->k);
        if (j->kind == 1) (void)pmo_qmatvec_f32(j->t, j->w + j->lo * row_bytes, j->hi - j->lo, j->k, j->x, j->y + j->lo, j->order);
        else (void)pmo_qmatvec_f64(j->t, j->w + j->lo * row_bytes, j->hi - j->lo, j->k, j->x, j->y + j->lo, j->order);
    } else { /* rows [lo, hi) of W against every activation row */
        float *tmp = (float *)malloc(j->k * sizeof(float));
        if (!tmp) return NULL;
        for (size_t r = j->lo; r < j->hi; r++) {
            dequant_row(j->t, j->w, r, j->k, tmp, j->order);
            for (size_t m = 0; m < j->m_rows; m++) {
                const float *xr = j->x + m * j->k;
                double acc = 0.0;
                for (size_t i = 0; i < j->k; i++) acc += (double)tmp[i] * (double)xr[i];
                j->y[m * j->n_rows + r] = (float)acc;
            }
        }
        free(tmp);
    }
    return NULL;
}

static int32_t mt_dispatch(mt_job proto, size_t units, int32_t threads) {
    if (threads < 1) threads = 1;
    if ((size_t)threads > units) threads = units ? (int32_t)units : 1;
    pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)threads);
    mt_job *jobs = (mt_job *)malloc(sizeof(mt_job) * (size_t)threads);
    if (!th || !jobs) {
        free(th);
        free(jobs);
        return PMO_ERR_SHAPE_TOO_LARGE;
    }
    int started = 0;
    for (int i = 0; i < threads; i++) {
        jobs[i] = proto;
        jobs[i].lo = units * (size_t)i / (size_t)threads;
        jobs[i].hi = units * (size_t)(i + 1) / (size_t)threads;
        if (pthread_create(&th[i], NULL, mt_run, &jobs[i]) != 0) break;
        started++;
    }
    for (int i = started; i < threads; i++) { /* could not start: run the rest here */
        jobs[i] = proto;
        jobs[i].lo = units * (size_t)i / (size_t)threads;
        jobs[i].hi = units * (size_t)(i + 1) / (size_t)threads;
        mt_run(&jobs[i]);
    }
    for (int i = 0; i < started; i++) pthread_join(th[i], NULL);
    free(th);
    free(jobs);
    return PMO_OK;
}

int32_t pmo_quantize_mt(uint32_t t, const float *x, size_t n, uint8_t *dst, size_t dst_len, int32_t threads) {
    size_t bs = pmo_block_size(t);
    if (bs == 0 || t == PMO_TYPE_F32 || t == PMO_TYPE_F16) return PMO_ERR_UNSUPPORTED_TYPE;
    if (dst_len != pmo_tensor_size(t, n)) return PMO_ERR_INVALID_SIZE;
    mt_job j;
    memset(&j, 0, sizeof j);
    j.kind = 0, j.t = t, j.x = x, j.dst = dst, j.n = n;
    return mt_dispatch(j, (n + bs - 1) / bs, threads);
}

int32_t pmo_qmatvec_mt(uint32_t t, const uint8_t *w, size_t n_rows, size_t k, const float *x, float *y, uint32_t order,
                       int32_t f64_acc, int32_t threads) {
    size_t bs = pmo_block_size(t);
    if (bs <= 1 || k % bs != 0) return PMO_ERR_INVALID_SHAPE;
    mt_job j;
    memset(&j, 0, sizeof j);
    j.kind = f64_acc ? 2 : 1, j.t = t, j.order = order, j.w = w, j.x = x, j.y = y, j.k = k;
    return mt_dispatch(j, n_rows, threads);
}

int32_t pmo_qmatmul_f64_mt(uint32_t t, const uint8_t *w, size_t n_rows, size_t k, const float *x, size_t m_rows, float *y,
                           uint32_t order, int32_t threads) {
    size_t bs = pmo_block_size(t);
    if (bs <= 1 || k % bs != 0) return PMO_ERR_INVALID_SHAPE;
    mt_job j;
    memset(&j, 0, sizeof j);
    j.kind = 3, j.t = t, j.order = order, j.w = w, j.x = x, j.y = y, j.k = k, j.m_rows = m_rows, j.n_rows = n_rows;
    return mt_dispatch(j, n_rows, threads);
}
