// Q8_K activation blocks and the integer dot products over them, for gfx950.
//
// Reference functions followed (paths under crates/pmetal-gguf/src/):
//   k_quants.rs:140-155   BlockQ8K {f32 d; i8 qs[256]; i16 bsums[16]} = 292 bytes
//   k_quants.rs:815-871   quantize_q8k (a trailing partial block stays all-zero)
//   vec_dot.rs:617-656    scalar vec_dot_q4k_q8k      vec_dot.rs:658-692   scalar vec_dot_q6k_q8k
//
// Results are bit-identical to those functions: the integer sums are exact in any order, and the float chain of a
// row (per block: sum -= dmin * mins, sum += d * sumi, each product and each addition rounded, in block order) is
// run in exactly that order.  This file is compiled without fp contraction.
#include "internal.hpp"

#pragma clang fp contract(off)

namespace {

constexpr int kQ8kBytes = 292;

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) { return (float)__builtin_bit_cast(_Float16, (uint16_t)h); }

// ------------------------------------------------------------------------------------------------
// quantize_q8k: one wave per block, four consecutive elements per lane
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_quantize_q8k(const float *__restrict__ x, size_t n_full, size_t n_blocks,
                                                       uint8_t *__restrict__ dst) {
    const size_t blk = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (blk >= n_blocks) return;
    uint8_t *out = dst + blk * kQ8kBytes;
    uint32_t *out32 = reinterpret_cast<uint32_t *>(out);  // blocks are 4-byte aligned (292 = 4 * 73)
    if (blk >= n_full) {  // the partial last block is left all-zero (k_quants.rs:829-834)
        for (int i = lane; i < kQ8kBytes / 4; i += 64) out32[i] = 0u;
        return;
    }
    const float4 v4 = *reinterpret_cast<const float4 *>(x + blk * 256 + 4 * lane);
    const float v[4] = {v4.x, v4.y, v4.z, v4.w};
    // `if x.abs() > amax { amax = x.abs(); max = x }` scanning forward: the first element that attains the largest
    // magnitude wins; NaN never compares greater.
    float amax = 0.0f, maxv = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const float a = __builtin_fabsf(v[c]);
        if (a > amax) amax = a, maxv = v[c];
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float oa = __shfl_xor(amax, off), om = __shfl_xor(maxv, off);
        // the lower lane holds the earlier elements: it keeps its value on a tie
        const bool other_is_lower = (lane & off) != 0;
        const bool take = other_is_lower ? (oa >= amax) : (oa > amax);
        amax = take ? oa : amax, maxv = take ? om : maxv;
    }
    if (amax == 0.0f) {  // d = 0, qs = 0, bsums = 0 (k_quants.rs:846-851)
        for (int i = lane; i < kQ8kBytes / 4; i += 64) out32[i] = 0u;
        return;
    }
    const float iscale = -128.0f / maxv;
    uint32_t packed = 0;
    int sum = 0;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        // (iscale * x).round().min(127.0) as i8: f32::min returns the other operand for a NaN, the cast saturates
        const float p = iscale * v[c];
        const float t = __builtin_truncf(p);
        float r = (__builtin_fabsf(p - t) >= 0.5f) ? t + __builtin_copysignf(1.0f, p) : t;
        r = (r != r) ? 127.0f : (r < 127.0f ? r : 127.0f);
        r = r < -128.0f ? -128.0f : r;
        const int q = (int)r;
        sum += q;
        packed |= ((uint32_t)q & 0xFFu) << (8 * c);
    }
    out32[1 + lane] = packed;
    sum += __shfl_xor(sum, 1);
    sum += __shfl_xor(sum, 2);
    if ((lane & 3) == 0) reinterpret_cast<int16_t *>(out + 260)[lane >> 2] = (int16_t)sum;
    if (lane == 0) *reinterpret_cast<float *>(out) = 1.0f / iscale;
}

// The four f64 sums of compute_kl_divergence (crates/pmetal-gguf/src/dynamic.rs:140-180) over n pairs (original,
// dequantized): sum (a - b)^2 with the difference taken in f32 as the reference takes it, sum a^2, sum a b, sum b^2.
// Every workgroup writes its four partial sums; the caller adds the workgroups' sums in order.
__global__ __launch_bounds__(256) void k_kl_sums(const float *__restrict__ a, const float *__restrict__ b, size_t n,
                                                  double *__restrict__ partial) {
    double s_err = 0.0, s_aa = 0.0, s_ab = 0.0, s_bb = 0.0;
    auto add = [&](float av, float bv) {
        const double diff = (double)(av - bv), x = (double)av, y = (double)bv;
        s_err += diff * diff, s_aa += x * x, s_ab += x * y, s_bb += y * y;
    };
    // Whole rounds of four float4 pairs per lane (eight loads in flight), then single float4 pairs, then the tail.
    constexpr int kUnroll = 4;
    const size_t lanes = (size_t)gridDim.x * 256, me = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t nvec = n / 4, rounds = nvec / (lanes * kUnroll);
    typedef float f4 __attribute__((ext_vector_type(4)));
    const f4 *a4 = reinterpret_cast<const f4 *>(a), *b4 = reinterpret_cast<const f4 *>(b);
    for (size_t r = 0; r < rounds; r++) {
        f4 x[kUnroll], y[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const size_t v = (r * kUnroll + u) * lanes + me;
            x[u] = __builtin_nontemporal_load(a4 + v), y[u] = __builtin_nontemporal_load(b4 + v);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) add(x[u].x, y[u].x), add(x[u].y, y[u].y), add(x[u].z, y[u].z), add(x[u].w, y[u].w);
    }
    for (size_t v = rounds * kUnroll * lanes + me; v < nvec; v += lanes) {
        const f4 x = a4[v], y = b4[v];
        add(x.x, y.x), add(x.y, y.y), add(x.z, y.z), add(x.w, y.w);
    }
    for (size_t e = nvec * 4 + me; e < n; e += lanes) add(a[e], b[e]);
    __shared__ double red[4][4];
    double v[4] = {s_err, s_aa, s_ab, s_bb};
#pragma unroll
    for (int k = 0; k < 4; k++) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v[k] += __shfl_xor(v[k], off);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0)
        for (int k = 0; k < 4; k++) red[wave][k] = v[k];
    __syncthreads();
    if (threadIdx.x < 4) partial[(size_t)blockIdx.x * 4 + threadIdx.x] = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
}

// ------------------------------------------------------------------------------------------------
// GEMV over Q8_K activations.  The activation blocks are laid out once per workgroup in LDS (qs 16-byte aligned,
// then d, then bsums).
// ------------------------------------------------------------------------------------------------
struct XqLds {
    const uint4 *qs;      // [spr][16] pieces of 16 int8
    const float *d;       // [spr]
    const int16_t *bsum;  // [spr][16]
};

__device__ __forceinline__ void stage_xq(const uint8_t *__restrict__ xq, int spr, uint4 *smem) {
    uint32_t *qs = reinterpret_cast<uint32_t *>(smem);                 // spr * 64 dwords
    uint32_t *d = qs + spr * 64;                                        // spr dwords
    uint32_t *bs = d + ((spr + 3) & ~3);                                // spr * 8 dwords
    const uint32_t *src = reinterpret_cast<const uint32_t *>(xq);       // 73 dwords per block
    for (int i = threadIdx.x; i < spr * 73; i += blockDim.x) {
        const int b = i / 73, o = i - b * 73;
        const uint32_t v = src[i];
        if (o == 0) d[b] = v;
        else if (o <= 64) qs[b * 64 + o - 1] = v;
        else bs[b * 8 + o - 65] = v;
    }
}
__device__ __forceinline__ XqLds xq_view(int spr, const uint4 *smem) {
    const uint32_t *qs = reinterpret_cast<const uint32_t *>(smem);
    const uint32_t *d = qs + spr * 64;
    const uint32_t *bs = d + ((spr + 3) & ~3);
    return XqLds{smem, reinterpret_cast<const float *>(d), reinterpret_cast<const int16_t *>(bs)};
}
size_t xq_lds_bytes(int spr) { return ((size_t)spr * 64 + ((spr + 3) & ~3) + (size_t)spr * 8) * 4; }

__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) { return __builtin_amdgcn_sdot4((int)a, (int)b, c, false); }

// get_scale_min_k4 (crates/pmetal-gguf/src/quantize.rs:844-855) on the 12 scale bytes held as three dwords, without a
// branch: byte j % 4 of the first dword holds sc (j < 4) or the top two bits of sc (j >= 4) in its bits 6-7, the same
// byte of the second dword does that for m, and byte j % 4 of the third dword holds the low nibbles for j >= 4.
__device__ __forceinline__ void scale_min_k4(int j, uint32_t s0, uint32_t s1, uint32_t s2, uint32_t &sc, uint32_t &m) {
    const uint32_t sh = 8u * (uint32_t)(j & 3);
    const uint32_t a = (s0 >> sh) & 0xFFu, b = (s1 >> sh) & 0xFFu, c = (s2 >> sh) & 0xFFu;
    const bool low = j < 4;
    sc = low ? (a & 63u) : ((c & 0xFu) | ((a >> 6) << 4));
    m = low ? (b & 63u) : ((c >> 4) | ((b >> 6) << 4));
}

// Q4_K: 8 lanes per super-block, lane j holds piece j of qs (bytes 16 j .. 16 j + 15): chunk c = j / 2, low nibbles
// against q8[64 c + 16 (j % 2) + i], high nibbles 32 further, scaled by sub-blocks 2 c and 2 c + 1; lane j also
// takes the min term of sub-block j.
struct TaskQ4 {
    uint4 hdr, q;
};
__device__ __forceinline__ void load_q4(const uint8_t *__restrict__ row, int sb, int j, bool live, TaskQ4 &t) {
    const uint8_t *blk = row + (size_t)(live ? sb : 0) * 144;
    t.hdr = *reinterpret_cast<const uint4 *>(blk);
    t.q = *reinterpret_cast<const uint4 *>(blk + 16 + 16 * j);
}
__device__ __forceinline__ void dot_q4(const TaskQ4 &t, const XqLds &xq, int sb, int j, int &sumi, int &mins) {
    const int c = j >> 1, half = j & 1;
    const uint4 lo8 = xq.qs[sb * 16 + 4 * c + half], hi8 = xq.qs[sb * 16 + 4 * c + 2 + half];
    const uint32_t w[4] = {t.q.x, t.q.y, t.q.z, t.q.w};
    const uint32_t l8[4] = {lo8.x, lo8.y, lo8.z, lo8.w}, h8[4] = {hi8.x, hi8.y, hi8.z, hi8.w};
    int sl = 0, sh = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        sl = dot4(w[i] & 0x0F0F0F0Fu, l8[i], sl);
        sh = dot4((w[i] >> 4) & 0x0F0F0F0Fu, h8[i], sh);
    }
    // every lane decodes the scale and min of its own sub-block j; the scales of sub-blocks 2 c and 2 c + 1 sit in the
    // even and the odd lane of the pair
    uint32_t scj, mj;
    scale_min_k4(j, t.hdr.y, t.hdr.z, t.hdr.w, scj, mj);
    const int sc0 = __builtin_amdgcn_mov_dpp((int)scj, 0xA0, 0xF, 0xF, true);  // quad_perm [0, 0, 2, 2]: the even lane's
    const int sc1 = __builtin_amdgcn_mov_dpp((int)scj, 0xF5, 0xF, 0xF, true);  // quad_perm [1, 1, 3, 3]: the odd lane's
    const uint32_t bs = reinterpret_cast<const uint32_t *>(xq.bsum)[sb * 8 + j];  // bsums 2 j and 2 j + 1
    sumi = sc0 * sl + sc1 * sh;
    mins = (int)mj * ((int)(int16_t)(bs & 0xFFFFu) + (int)(int16_t)(bs >> 16));
}

// Sum over the GROUP (8 or 16) consecutive lanes of a group, left in all of them: neighbours in the quad, the other
// pair of the quad, the mirrored half of eight (whose quad holds the other quad's sum), the mirrored row of sixteen.
template <int GROUP>
__device__ __forceinline__ int group_sum(int v) {
    v += __builtin_amdgcn_mov_dpp(v, 0xB1, 0xF, 0xF, true);   // quad_perm [1, 0, 3, 2]
    v += __builtin_amdgcn_mov_dpp(v, 0x4E, 0xF, 0xF, true);   // quad_perm [2, 3, 0, 1]
    v += __builtin_amdgcn_mov_dpp(v, 0x141, 0xF, 0xF, true);  // row_half_mirror
    if (GROUP == 16) v += __builtin_amdgcn_mov_dpp(v, 0x140, 0xF, 0xF, true);  // row_mirror
    return v;
}

// Q6_K in the element order of the reference's dot product: element idx of a super-block takes the low (idx even) or
// high nibble of ql[idx / 2], bits 2 (idx % 4) .. of qh[idx / 4] and scale idx / 16.  16 lanes per super-block, lane g
// holds the 16 elements of scale group g: ql bytes 8 g .. 8 g + 7, qh bytes 4 g .. 4 g + 3.
// sum (q - 32) q8 = sum q q8 - 32 bsum[g].
struct TaskQ6 {
    uint32_t ql0, ql1, qh, sc_d;  // sc_d: the scale byte of the group | d << 16
};
__device__ __forceinline__ uint32_t load_u32_a2(const uint8_t *p) {
    typedef uint32_t u32_a2 __attribute__((aligned(2)));
    return *reinterpret_cast<const u32_a2 *>(p);
}
__device__ __forceinline__ void load_q6(const uint8_t *__restrict__ row, int sb, int g, bool live, TaskQ6 &t) {
    const uint8_t *blk = row + (size_t)(live ? sb : 0) * 210;  // 2-byte aligned
    t.ql0 = load_u32_a2(blk + 8 * g), t.ql1 = load_u32_a2(blk + 8 * g + 4);
    t.qh = load_u32_a2(blk + 128 + 4 * g);
    t.sc_d = (uint32_t)blk[192 + g] | ((uint32_t)*reinterpret_cast<const uint16_t *>(blk + 208) << 16);
}
__device__ __forceinline__ int dot_q6(const TaskQ6 &t, const XqLds &xq, int sb, int g) {
    const uint4 q8 = xq.qs[sb * 16 + g];
    const uint32_t y[4] = {q8.x, q8.y, q8.z, q8.w};
    const uint32_t ql[2] = {t.ql0, t.ql1};
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        // elements 4 i .. 4 i + 3 of the group: ql bytes 2 i, 2 i + 1 (low then high nibble of each), qh byte i
        const uint32_t two = (ql[i >> 1] >> (16 * (i & 1))) & 0xFFFFu;
        const uint32_t lo = two & 0x0F0Fu, hi = (two >> 4) & 0x0F0Fu;  // (e0, e2) and (e1, e3)
        const uint32_t nib = (lo & 0xFFu) | ((hi & 0xFFu) << 8) | ((lo >> 8) << 16) | ((hi >> 8) << 24);
        const uint32_t h = (t.qh >> (8 * i)) & 0xFFu;
        // byte e of `top` = bits 2 e, 2 e + 1 of h: fields 0 and 2 move by 0 and 12 bits, fields 1 and 3 by 6 and 18 (the
        // two copies of each product do not overlap, so the multiplications are plain shifts and ors)
        const uint32_t top = (((h & 0x33u) * 0x1001u) & 0x00030003u) | (((h & 0xCCu) * 0x40040u) & 0x03000300u);
        s = dot4(nib | (top << 4), y[i], s);
    }
    const int scale = (int)(int8_t)(t.sc_d & 0xFFu);
    return scale * (s - 32 * (int)xq.bsum[sb * 16 + g]);
}

// Byte e of the result = bits 2 e, 2 e + 1 of the byte h: fields 0 and 2 move by 0 and 12 bits, fields 1 and 3 by 6 and 18
// (the two copies of each product do not overlap, so the multiplications are plain shifts and ors).
__device__ __forceinline__ uint32_t spread_fields2(uint32_t h) {
    return (((h & 0x33u) * 0x1001u) & 0x00030003u) | (((h & 0xCCu) * 0x40040u) & 0x03000300u);
}
// Byte e of the result = bit e of the nibble b (bit e moves by 7 e; the stray copies fall outside the mask).
__device__ __forceinline__ uint32_t spread_bits4(uint32_t b) { return (b * 0x00204081u) & 0x01010101u; }
// Byte e of the result = nibble e of the 16-bit value x.
__device__ __forceinline__ uint32_t spread_nibbles4(uint32_t x) {
    x = (x | (x << 8)) & 0x00FF00FFu;
    return (x | (x << 4)) & 0x0F0F0F0Fu;
}

// Q5_K in the element order of the reference's dot product (crates/pmetal-gguf/src/vec_dot.rs:695-737): element j takes
// the low (j even) or high nibble of qs[j / 2], bit j % 8 of qh[j / 8] and the scale of sub-block j / 32.  8 lanes per
// super-block, lane j holds sub-block j: qs bytes 16 j .. 16 j + 15, qh bytes 4 j .. 4 j + 3; it also takes the min term
// of sub-block j.
struct TaskQ5 {
    uint4 hdr, q;
    uint32_t qh;
};
__device__ __forceinline__ void load_q5(const uint8_t *__restrict__ row, int sb, int j, bool live, TaskQ5 &t) {
    const uint8_t *blk = row + (size_t)(live ? sb : 0) * 176;
    t.hdr = *reinterpret_cast<const uint4 *>(blk);
    t.qh = *reinterpret_cast<const uint32_t *>(blk + 16 + 4 * j);
    t.q = *reinterpret_cast<const uint4 *>(blk + 48 + 16 * j);
}
__device__ __forceinline__ void dot_q5(const TaskQ5 &t, const XqLds &xq, int sb, int j, int &sumi, int &mins) {
    const uint4 ya = xq.qs[sb * 16 + 2 * j], yb = xq.qs[sb * 16 + 2 * j + 1];
    const uint32_t y[8] = {ya.x, ya.y, ya.z, ya.w, yb.x, yb.y, yb.z, yb.w};
    const uint32_t w[4] = {t.q.x, t.q.y, t.q.z, t.q.w};
    int s = 0;
#pragma unroll
    for (int m = 0; m < 8; m++) {  // elements 4 m .. 4 m + 3 of the sub-block: qs bytes 2 m, 2 m + 1, bits 4 m .. of qh
        const uint32_t nib = spread_nibbles4((w[m >> 1] >> (16 * (m & 1))) & 0xFFFFu);
        const uint32_t top = spread_bits4((t.qh >> (4 * m)) & 0xFu) << 4;
        s = dot4(nib | top, y[m], s);
    }
    uint32_t scj, mj;
    scale_min_k4(j, t.hdr.y, t.hdr.z, t.hdr.w, scj, mj);
    const uint32_t bs = reinterpret_cast<const uint32_t *>(xq.bsum)[sb * 8 + j];  // bsums 2 j and 2 j + 1
    sumi = (int)scj * s;
    mins = (int)mj * ((int)(int16_t)(bs & 0xFFFFu) + (int)(int16_t)(bs >> 16));
}

// Q2_K (crates/pmetal-gguf/src/vec_dot.rs:779-810): element j takes bits 2 (j % 4) .. of qs[j / 4] and the low nibble of
// scales[j / 16]; the min term is the high nibble of scales[g] times bsums[g].  16 lanes per super-block, lane g holds
// the 16 elements of group g: qs bytes 4 g .. 4 g + 3.  Blocks are 84 bytes: dwords stay aligned.
struct TaskQ2 {
    uint32_t q, sc, hdr;  // sc: scales[g]; hdr: d | dmin << 16
};
__device__ __forceinline__ void load_q2(const uint8_t *__restrict__ row, int sb, int g, bool live, TaskQ2 &t) {
    const uint8_t *blk = row + (size_t)(live ? sb : 0) * 84;
    t.sc = blk[g];
    t.q = *reinterpret_cast<const uint32_t *>(blk + 16 + 4 * g);
    t.hdr = *reinterpret_cast<const uint32_t *>(blk + 80);
}
__device__ __forceinline__ void dot_q2(const TaskQ2 &t, const XqLds &xq, int sb, int g, int &sumi, int &mins) {
    const uint4 q8 = xq.qs[sb * 16 + g];
    const uint32_t y[4] = {q8.x, q8.y, q8.z, q8.w};
    int s = 0;
#pragma unroll
    for (int m = 0; m < 4; m++) s = dot4(spread_fields2((t.q >> (8 * m)) & 0xFFu), y[m], s);
    sumi = (int)(t.sc & 0xFu) * s;
    mins = (int)(t.sc >> 4) * (int)xq.bsum[sb * 16 + g];
}

// Q3_K (crates/pmetal-gguf/src/vec_dot.rs:739-777): element j takes bits 2 (j % 4) .. of qs[j / 4], bit j % 8 of
// hmask[j / 8] as its third bit, minus 4; that routine unpacks only the first eight scales (nibble g of the first four
// scale bytes, minus 8) and leaves the scales of groups 8..15 at zero.  16 lanes per super-block, lane g holds group g:
// qs bytes 4 g .. 4 g + 3, hmask bytes 2 g, 2 g + 1.  Blocks are 110 bytes: only 2-byte aligned.
// sum (q - 4) q8 = sum q q8 - 4 bsum[g].
struct TaskQ3 {
    uint32_t q, hm, aux0, d;
};
__device__ __forceinline__ void load_q3(const uint8_t *__restrict__ row, int sb, int g, bool live, TaskQ3 &t) {
    const uint8_t *blk = row + (size_t)(live ? sb : 0) * 110;
    t.hm = *reinterpret_cast<const uint16_t *>(blk + 2 * g);
    t.q = load_u32_a2(blk + 32 + 4 * g);
    t.aux0 = load_u32_a2(blk + 96);
    t.d = *reinterpret_cast<const uint16_t *>(blk + 108);
}
__device__ __forceinline__ int dot_q3(const TaskQ3 &t, const XqLds &xq, int sb, int g) {
    const uint4 q8 = xq.qs[sb * 16 + g];
    const uint32_t y[4] = {q8.x, q8.y, q8.z, q8.w};
    int s = 0;
#pragma unroll
    for (int m = 0; m < 4; m++)
        s = dot4(spread_fields2((t.q >> (8 * m)) & 0xFFu) | (spread_bits4((t.hm >> (4 * m)) & 0xFu) << 2), y[m], s);
    const int scale = g < 8 ? (int)((t.aux0 >> (4 * g)) & 0xFu) - 8 : 0;
    return scale * (s - 4 * (int)xq.bsum[sb * 16 + g]);
}

// What the row walker below needs to know about a weight type.
struct Q4Traits {
    using Task = TaskQ4;
    static constexpr int kGroup = 8, kBlockBytes = 144;  // lanes per super-block
    static constexpr bool kHasMin = true;
    static __device__ __forceinline__ void load(const uint8_t *row, int sb, int l, bool live, Task &t) { load_q4(row, sb, l, live, t); }
    static __device__ __forceinline__ void dot(const Task &t, const XqLds &xq, int sb, int l, int &sumi, int &mins) { dot_q4(t, xq, sb, l, sumi, mins); }
    static __device__ __forceinline__ uint32_t header(const Task &t) { return t.hdr.x; }  // d | dmin << 16
};
struct Q6Traits {
    using Task = TaskQ6;
    static constexpr int kGroup = 16, kBlockBytes = 210;
    static constexpr bool kHasMin = false;
    static __device__ __forceinline__ void load(const uint8_t *row, int sb, int l, bool live, Task &t) { load_q6(row, sb, l, live, t); }
    static __device__ __forceinline__ void dot(const Task &t, const XqLds &xq, int sb, int l, int &sumi, int &mins) {
        sumi = dot_q6(t, xq, sb, l), mins = 0;
    }
    static __device__ __forceinline__ uint32_t header(const Task &t) { return t.sc_d >> 16;  }  // d
};

struct Q5Traits {
    using Task = TaskQ5;
    static constexpr int kGroup = 8, kBlockBytes = 176;
    static constexpr bool kHasMin = true;
    static __device__ __forceinline__ void load(const uint8_t *row, int sb, int l, bool live, Task &t) { load_q5(row, sb, l, live, t); }
    static __device__ __forceinline__ void dot(const Task &t, const XqLds &xq, int sb, int l, int &sumi, int &mins) { dot_q5(t, xq, sb, l, sumi, mins); }
    static __device__ __forceinline__ uint32_t header(const Task &t) { return t.hdr.x; }  // d | dmin << 16
};
struct Q2Traits {
    using Task = TaskQ2;
    static constexpr int kGroup = 16, kBlockBytes = 84;
    static constexpr bool kHasMin = true;
    static __device__ __forceinline__ void load(const uint8_t *row, int sb, int l, bool live, Task &t) { load_q2(row, sb, l, live, t); }
    static __device__ __forceinline__ void dot(const Task &t, const XqLds &xq, int sb, int l, int &sumi, int &mins) { dot_q2(t, xq, sb, l, sumi, mins); }
    static __device__ __forceinline__ uint32_t header(const Task &t) { return t.hdr; }  // d | dmin << 16
};
struct Q3Traits {
    using Task = TaskQ3;
    static constexpr int kGroup = 16, kBlockBytes = 110;
    static constexpr bool kHasMin = false;
    static __device__ __forceinline__ void load(const uint8_t *row, int sb, int l, bool live, Task &t) { load_q3(row, sb, l, live, t); }
    static __device__ __forceinline__ void dot(const Task &t, const XqLds &xq, int sb, int l, int &sumi, int &mins) {
        sumi = dot_q3(t, xq, sb, l), mins = 0;
    }
    static __device__ __forceinline__ uint32_t header(const Task &t) { return t.d; }
};

// A wave multiplies 64 / kGroup rows at once: lane group g walks row g of the wave's rows super-block by
// super-block, so the float sum of a row (per block: sum -= (dmin yd) mins, sum += (d yd) sumi, every product and
// every addition rounded, in block order) is two instructions per step for all the wave's rows together.  kDepth
// super-blocks are requested per round, then multiplied in order; every request is unconditional (a block past the
// end re-reads the last one).
constexpr int kDepth = 8;
constexpr int kWaves = 4;  // per workgroup

template <typename TR>
__global__ __launch_bounds__(64 * kWaves) void k_qgemv_q8k(const uint8_t *__restrict__ W, const uint8_t *__restrict__ xqg,
                                                            float *__restrict__ y, int n_rows, int spr) {
    constexpr int G = TR::kGroup, RPW = 64 / G;
    extern __shared__ uint4 smem[];
    stage_xq(xqg, spr, smem);
    __syncthreads();
    const XqLds xq = xq_view(spr, smem);
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int l = lane & (G - 1), g = lane / G;
    const int row0 = (blockIdx.x * kWaves + wave) * RPW;
    if (row0 >= n_rows) return;
    const int row = row0 + g < n_rows ? row0 + g : n_rows - 1;  // a group past the end repeats the last row
    const uint8_t *rowp = W + (size_t)row * (size_t)spr * TR::kBlockBytes;
    float sum = 0.0f;
    for (int b0 = 0; b0 < spr; b0 += kDepth) {
        typename TR::Task ring[kDepth];
#pragma unroll
        for (int i = 0; i < kDepth; i++) TR::load(rowp, b0 + i < spr ? b0 + i : spr - 1, l, true, ring[i]);
#pragma unroll
        for (int i = 0; i < kDepth; i++) {
            if (b0 + i < spr) {  // the same for the whole wave
                const int sb = b0 + i;
                int sumi, mins;
                TR::dot(ring[i], xq, sb, l, sumi, mins);
                sumi = group_sum<G>(sumi);
                const uint32_t hd = TR::header(ring[i]);
                const float yd = xq.d[sb];
                if (TR::kHasMin) {
                    mins = group_sum<G>(mins);
                    sum -= (f16_bits_to_f32(hd >> 16) * yd) * (float)mins;
                }
                sum += (f16_bits_to_f32(hd & 0xFFFFu) * yd) * (float)sumi;
            }
        }
    }
    if (l == 0 && row0 + g < n_rows) y[row0 + g] = sum;
}

}  // namespace

namespace pmh {

hipError_t launch_quantize_q8k(const float *x, size_t n, uint8_t *dst, hipStream_t s) {
    const size_t n_blocks = n / 256 + (n % 256 != 0), n_full = n / 256;
    if (n_blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(k_quantize_q8k, dim3((unsigned)((n_blocks + 3) / 4)), dim3(256), 0, s, x, n_full, n_blocks, dst);
    return hipGetLastError();
}

int kl_sums_workgroups(size_t n) {
    const size_t want = (n + 4095) / 4096;  // at least four float4 pairs per lane
    return (int)(want < 1 ? 1 : (want > 2048 ? 2048 : want));
}
hipError_t launch_kl_sums(const float *a, const float *b, size_t n, double *partial, hipStream_t s) {
    hipLaunchKernelGGL(k_kl_sums, dim3((unsigned)kl_sums_workgroups(n)), dim3(256), 0, s, a, b, n, partial);
    return hipGetLastError();
}

// k must be a multiple of 256 with the activation blocks fitting in LDS (k <= 32768); type Q4_K, Q6_K, Q5_K, Q3_K or Q2_K.
template <typename TR>
static hipError_t launch_q8k_rows(const uint8_t *w, int64_t n, int spr, size_t lds, const uint8_t *xq, float *y, hipStream_t s) {
    const int rows_per_wg = kWaves * 64 / TR::kGroup;
    const dim3 grid((unsigned)((n + rows_per_wg - 1) / rows_per_wg)), block(64 * kWaves);
    hipLaunchKernelGGL(k_qgemv_q8k<TR>, grid, block, lds, s, w, xq, y, (int)n, spr);
    return hipGetLastError();
}
hipError_t launch_qgemv_q8k(uint32_t type, const uint8_t *w, int64_t n, int64_t k, const uint8_t *xq, float *y, hipStream_t s) {
    const int spr = (int)(k / 256);
    const size_t lds = xq_lds_bytes(spr);
    if (lds > 64 * 1024) return hipErrorInvalidValue;
    switch (type) {
    case kTypeQ4K: return launch_q8k_rows<Q4Traits>(w, n, spr, lds, xq, y, s);
    case kTypeQ5K: return launch_q8k_rows<Q5Traits>(w, n, spr, lds, xq, y, s);
    case kTypeQ3K: return launch_q8k_rows<Q3Traits>(w, n, spr, lds, xq, y, s);
    case kTypeQ2K: return launch_q8k_rows<Q2Traits>(w, n, spr, lds, xq, y, s);
    default: return launch_q8k_rows<Q6Traits>(w, n, spr, lds, xq, y, s);
    }
}

}  // namespace pmh
