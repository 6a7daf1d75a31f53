// Dequant-fused GEMM  Y[m,n] = sum_k X[m,k] * W[n,k]  (prefill) on the gfx950 matrix cores, large-tile design:
// one dequantized weight tile per workgroup, shared through LDS.  It serves Q6_K, and Q4_K shapes outside the
// limits of the kernel in gemm_rowwave.hip (where every wave owns its weight rows), which is the faster one.
// The text below describes Q4_K; the Q6_K differences are noted at dequant16_q6.
//
// W is the packed GGUF stream [n, k] of 144-byte super-blocks; a weight's value is what the reference's
// dequantize_q4k yields (crates/pmetal-gguf/src/k_quants.rs:358-404; element order REF or GGML as for the
// GEMV).  The reference has no fused kernel (it dequantizes on the CPU at load,
// crates/pmetal-models/src/weight_format.rs:299-303, and multiplies densely); this kernel is checked
// against exactly that, dequantize-then-matmul, to 1e-3.
//
// Why the tiles are exact integers in f16 and not rounded bf16 weights: rounding d*sc*q - dmin*m to bf16
// (8 significant bits) leaves a relative error of about 1e-3 per product, which fails the 1e-3 gate.
// Instead the MFMA multiplies quantities that are exact in f16:
//     B tile  = sc * q             an integer <= 63 * 15 = 945          (f16 holds integers to 2048)
//     A tile  = x * 2^-e_m         bf16 activations are exact in f16 once a per-row power of two keeps
//                                  them below 2^10 (a pre-pass does that and sums x per 32-element block)
// and the per-super-block factor d is applied to the fp32 partial sums:
//     Y[m,n] = 2^e_m * sum_SB ( d[n,SB] * P_SB[m,n] + R_SB[m,n] )
//     P_SB = sum_{k in SB} A[m,k] * B[n,k]              16 x v_mfma_f32_32x32x16_f16 per 32x32 block
//     R_SB = - sum_{j<8} (dmin[n,SB] * m[n,j]) * xsum[m,j]
// R_SB also runs on the matrix core, straight into the accumulators: dmin * m (17 significant bits) and the
// block sums xsum are each split exactly into an f16 head and tail, and the four cross products of the
// eight sub-blocks make one K = 32 product (two more MFMAs per block and super-block).  The only roundings
// are the fp32 accumulations.
//
// Tiling: a workgroup of 8, 4 or 2 waves computes a 256 x 128, 128 x 128 or 64 x 32 tile of Y (by the number
// of activation rows); every wave owns 2 x 2 (or one) MFMA blocks.  K advances 64 elements per stage.  The pre-pass
// stores the activations as 16-byte items (8 consecutive k of one row) in [k / 8][m] order, so that a wave
// copies 64 consecutive items from global memory to LDS: coalesced reads, conflict-free writes, and the
// items lie in LDS exactly as the MFMA A operand wants them ([k-step][k-group][row]).  The B tile is
// dequantized by the whole workgroup once per stage into the same operand order.  Global loads run two
// stages ahead in registers, the LDS stages are double buffered, one barrier per stage.
#include "internal.hpp"

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // 16 bytes in registers

constexpr int kMPad = 256; // the pre-pass pads the activation rows to a multiple of this

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return __builtin_bit_cast(float, h << 16); }

// ------------------------------------------------------------------------------------------------
// Pre-pass 1: one wave per row m (rows up to Mp, a multiple of 4): rowscale[m] = 2^e_m with the row maximum * 2^-e_m in [2^9, 2^10),
// so that block sums (< 2^15) fit f16 and small rows stay out of the f16 subnormal range.
// ------------------------------------------------------------------------------------------------
template <bool XF32>
__global__ __launch_bounds__(256) void k_prep_scale(const void *__restrict__ xg, int64_t k, int M,
                                                     float *__restrict__ rowscale) {
    // one wave per row, 16-byte loads (k is a multiple of 256)
    const int64_t m = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    float amax = 0.0f;
    if (m < M) {
        if (XF32) {
            const float4 *row = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(xg) + m * k);
            for (int64_t i = lane; i < k / 4; i += 64) {
                const float4 v = row[i];
                amax = __builtin_fmaxf(__builtin_fmaxf(amax, __builtin_fmaxf(__builtin_fabsf(v.x), __builtin_fabsf(v.y))),
                                       __builtin_fmaxf(__builtin_fabsf(v.z), __builtin_fabsf(v.w)));
            }
        } else {
            const uint4 *row = reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(xg) + m * k);
            for (int64_t i = lane; i < k / 8; i += 64) {
                const uint4 v = row[i];
                const uint32_t r[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int q = 0; q < 4; q++)
                    amax = __builtin_fmaxf(amax, __builtin_fmaxf(__builtin_fabsf(bf16_to_f32(r[q] & 0xFFFFu)),
                                                                 __builtin_fabsf(bf16_to_f32(r[q] >> 16))));
            }
        }
    }
    for (int off = 32; off > 0; off >>= 1) amax = __builtin_fmaxf(amax, __shfl_xor(amax, off));
    const int eb = (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xFFu);  // amax in [2^(eb-127), 2^(eb-126))
    int e = eb - 126 - 10;
    e = e < -126 ? -126 : (e > 126 ? 126 : e);
    if (eb == 255) e = 0;  // inf / NaN: let them through
    if (lane == 0) rowscale[m] = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
}

// ------------------------------------------------------------------------------------------------
// Pre-pass 2: grid (Mp / 32, k / 256), 256 threads.  Thread (row = tid / 8, c8 = tid % 8) converts the 8
// activations of chunk c8 of every 64-element group of the super-block: 8 lanes read 128 contiguous bytes
// of a row, and for one chunk the 8 rows of a wave write 128 contiguous bytes.
//   xs   [k / 8][Mp]               items of 8 f16: x[m][8c .. 8c+7] * 2^-e_m   (rows >= M are zero)
//   xsum [k / 256][2][2][Mp]       items of 8 f16 for the R_SB product, item (t, g) of row m =
//                                  (h_j, l_j, h_j, l_j, h_j+1, l_j+1, h_j+1, l_j+1),  j = 4 t + 2 g,
//                                  h + l = sum of the 32 scaled activations of sub-block j (exact split)
// ------------------------------------------------------------------------------------------------
template <bool XF32>
__global__ __launch_bounds__(256) void k_prep_tiles(const void *__restrict__ xg, int64_t k, int M, int Mp,
                                                     const float *__restrict__ rowscale, uint4 *__restrict__ xs,
                                                     uint4 *__restrict__ xsum) {
    const int c8 = threadIdx.x & 7;
    const int m = blockIdx.x * 32 + (threadIdx.x >> 3);
    const int64_t sb = blockIdx.y;
    const bool live = m < M;
    const float down = live ? 1.0f / rowscale[m] : 0.0f;  // exact: a power of two
#pragma unroll
    for (int it = 0; it < 4; it++) {  // 64 elements per trip: sub-blocks 2 it (c8 < 4) and 2 it + 1
        const int64_t k0 = sb * 256 + it * 64 + c8 * 8;
        float v[8];
        if (!live) {
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = 0.0f;
        } else if (XF32) {
            const float4 a = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(xg) + (int64_t)m * k + k0);
            const float4 b = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(xg) + (int64_t)m * k + k0 + 4);
            v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
        } else {
            const uint4 u = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(xg) + (int64_t)m * k + k0);
            const uint32_t r[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
            for (int i = 0; i < 4; i++) v[2 * i] = bf16_to_f32(r[i] & 0xFFFFu), v[2 * i + 1] = bf16_to_f32(r[i] >> 16);
        }
        half8_t h;
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            h[i] = (_Float16)(v[i] * down);
            sum += (float)h[i];
        }
        xs[(size_t)(k0 / 8) * Mp + m] = __builtin_bit_cast(uint4, h);
        // sub-block sums: over the 4 lanes of a chunk quad (exact: every partial sum is a multiple of the
        // row's f16 grid and stays below 2^15 of it), then the pair (2 it, 2 it + 1) meets in lane c8 = 0
        sum += __shfl_xor(sum, 1);
        sum += __shfl_xor(sum, 2);
        const float other = __shfl_down(sum, 4);
        if (c8 == 0) {
            const _Float16 h0 = (_Float16)sum, h1 = (_Float16)other;
            const _Float16 l0 = (_Float16)(sum - (float)h0), l1 = (_Float16)(other - (float)h1);
            const half8_t item = {h0, l0, h0, l0, h1, l1, h1, l1};
            xsum[((size_t)sb * 4 + it) * Mp + m] = __builtin_bit_cast(uint4, item);  // j = 2 it = 4 t + 2 g
        }
    }
}

// ------------------------------------------------------------------------------------------------
// main kernel
// ------------------------------------------------------------------------------------------------
// 16 nibbles (one plane of a 16-byte piece) times the integer scale -> 16 exact f16 values.
// 0x6400 | q is the f16 1024 + q; (1024 + q) * sc - 1024 * sc is exact in a packed f16 fma.
__device__ __forceinline__ void dequant16(const uint4 piece, const int plane, const uint32_t sc, uint4 &lo8, uint4 &hi8) {
    const _Float16 s = (_Float16)(float)sc;
    const half2_t sc2 = {s, s};
    const _Float16 o = (_Float16)(-1024.0f * (float)sc);  // exact: sc <= 63
    const half2_t off2 = {o, o};
    const uint32_t w[4] = {piece.x, piece.y, piece.z, piece.w};
    uint32_t out[8];
#pragma unroll
    for (int d = 0; d < 4; d++) {
        const uint32_t nib = (plane ? (w[d] >> 4) : w[d]) & 0x0F0F0F0Fu;  // 4 quants, one per byte
        // bytes (b0, b1) and (b2, b3) -> f16 pairs 0x64bb
        const uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, nib, 0x04010400u);
        const uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, nib, 0x04030402u);
        // must be a fused multiply-add: the product alone is not representable in f16
        const half2_t r0 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, p0), sc2, off2);
        const half2_t r1 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, p1), sc2, off2);
        out[2 * d] = __builtin_bit_cast(uint32_t, r0);
        out[2 * d + 1] = __builtin_bit_cast(uint32_t, r1);
    }
    lo8 = make_uint4(out[0], out[1], out[2], out[3]);
    hi8 = make_uint4(out[4], out[5], out[6], out[7]);
}

// (scale, min) of sub-block j from the 12 scale bytes (quantize.rs:844-855); j is a compile-time constant
// wherever this is called, so the branch folds.
__device__ __forceinline__ void scale_min_u(const uint4 hdr, const int j, uint32_t &sc, uint32_t &mn) {
    const int sh = 8 * (j & 3);
    if (j < 4) {
        sc = (hdr.y >> sh) & 63u;
        mn = (hdr.z >> sh) & 63u;
    } else {
        const uint32_t c = hdr.w >> sh;
        sc = (c & 0xFu) | (((hdr.y >> (sh + 6)) & 3u) << 4);
        mn = ((c >> 4) & 0xFu) | (((hdr.z >> (sh + 6)) & 3u) << 4);
    }
}

// 16 bytes / 4 bytes / 2 bytes at an address that is only 2-byte aligned (Q6_K super-blocks are 210 bytes)
struct __attribute__((packed, aligned(2))) u32x4_a2 {
    uint32_t x, y, z, w;
};
struct __attribute__((packed, aligned(2))) u32_a2 {
    uint32_t v;
};
typedef uint16_t u16_a2 __attribute__((aligned(2)));

__device__ __forceinline__ u32x4 load16_a2(const uint8_t *p) {
    const u32x4_a2 t = *reinterpret_cast<const u32x4_a2 *>(p);
    return u32x4{t.x, t.y, t.z, t.w};
}

// Q6_K: 16 six-bit quants (low nibbles in ql shifted by ql_shift, top two bits in qh at qh_shift) of one
// 16-element scale group.  sc * (q - 32) can reach 4096 and would not always be exact in f16, so the value is
// split where the storage splits it, q - 32 = 16 (hi2 - 2) + nib, into two exact tiles:
//     B1 = (16 sc) * (hi2 - 2)   |.| <= 2048 * 2, a multiple of 16        B2 = sc * nib   |.| <= 1920
// multiplied one after the other into the same accumulator.  (0x6400 | v is the f16 1024 + v.)
__device__ __forceinline__ void dequant16_q6(const u32x4 ql, const u32x4 qh, const int ql_shift, const int qh_shift,
                                             const int sc, uint4 &b1lo, uint4 &b1hi, uint4 &b2lo, uint4 &b2hi) {
    const _Float16 s1 = (_Float16)(float)(16 * sc), s2 = (_Float16)(float)sc;  // exact: |sc| <= 128
    const half2_t s1v = {s1, s1}, s2v = {s2, s2};
    const half2_t m1026 = {(_Float16)-1026.0f, (_Float16)-1026.0f}, m1024 = {(_Float16)-1024.0f, (_Float16)-1024.0f};
    const uint32_t lw[4] = {ql.x, ql.y, ql.z, ql.w}, hw[4] = {qh.x, qh.y, qh.z, qh.w};
    uint32_t o1[8], o2[8];
#pragma unroll
    for (int d = 0; d < 4; d++) {
        const uint32_t nib = (lw[d] >> ql_shift) & 0x0F0F0F0Fu;
        const uint32_t hi2 = (hw[d] >> qh_shift) & 0x03030303u;
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const uint32_t sel = half ? 0x04030402u : 0x04010400u;  // bytes (b0, b1) resp. (b2, b3) -> 0x64bb pairs
            const half2_t n2 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, nib, sel));
            const half2_t h2 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, hi2, sel));
            o2[2 * d + half] = __builtin_bit_cast(uint32_t, (n2 + m1024) * s2v);  // both steps exact
            o1[2 * d + half] = __builtin_bit_cast(uint32_t, (h2 + m1026) * s1v);
        }
    }
    b1lo = make_uint4(o1[0], o1[1], o1[2], o1[3]);
    b1hi = make_uint4(o1[4], o1[5], o1[6], o1[7]);
    b2lo = make_uint4(o2[0], o2[1], o2[2], o2[3]);
    b2hi = make_uint4(o2[4], o2[5], o2[6], o2[7]);
}

// -(dmin * mn) split exactly into an f16 head and tail (dmin has 11 significant bits, mn 6).
__device__ __forceinline__ void neg_min_split(const float dmin, const uint32_t mn, _Float16 &h, _Float16 &l) {
    const float p = -(dmin * (float)mn);  // exact in fp32
    h = (_Float16)p;
    l = (_Float16)(p - (float)h);
}

// Workgroup = WM x WN waves, every wave owns NB x NB MFMA blocks of 32 x 32:
//   <4, 2, 2>: 256 x 128 tile, 512 threads      <2, 2, 2>: 128 x 128, 256 threads      <2, 1, 1>: 64 x 32, 128 threads
template <int QT, int WM, int WN, int NB>
struct Tile {
    static constexpr int BM = 32 * NB * WM, BN = 32 * NB * WN, kThreads = 64 * WM * WN;
    static constexpr int kUnits = kThreads / BN;   // threads per weight row
    static constexpr int kBTasks = 4 / kUnits;     // (piece, plane) tasks per thread and stage
    // 16-byte pieces of weight data per thread and stage: Q4_K one or two quant pieces; Q6_K ql + qh per task
    static constexpr int kPieces = QT == 14 ? 2 * kBTasks : (kBTasks == 4 ? 2 : 1);
    static constexpr int kBItems = (QT == 14 ? 16 : 8) * BN;  // items of one B stage (Q6_K: two tiles)
    static constexpr int kBlockBytes = QT == 14 ? 210 : 144;
    static constexpr int kAItems = 8 * BM / kThreads;  // A items per thread and stage
    static constexpr size_t kLdsBytes = (size_t)(2 * 8 * BM + 2 * kBItems + 4 * BN) * 16 + BN * 4;
    static_assert(kUnits == 1 || kUnits == 2 || kUnits == 4, "a weight row is staged by 1, 2 or 4 threads");
    static_assert(8 * BM % kThreads == 0, "the A tile must divide among the threads");
};

template <int QT, int ORDER, bool YBF16, int WM, int WN, int NB>
__global__ __launch_bounds__(64 * WM * WN, NB == 1 ? 2 : 512 / (64 * WM * WN)) void k_qgemm(
    const uint8_t *__restrict__ W, const uint4 *__restrict__ xs, const uint4 *__restrict__ xsum,
    const float *__restrict__ rowscale, void *__restrict__ yg, int M, int Mp, int N, int spr) {
    using TL = Tile<QT, WM, WN, NB>;
    constexpr int BM = TL::BM, BN = TL::BN, kThreads = TL::kThreads, kUnits = TL::kUnits, kBTasks = TL::kBTasks,
                  kPieces = TL::kPieces, kAItems = TL::kAItems, kBItems = TL::kBItems;
    constexpr bool kQ6 = QT == 14;
    // LDS: two stages of the A tile [8 chunks][BM] and the B tile [4 k-steps][2 k-groups][BN] (16-byte items),
    // the B operand of the R product [2][2][BN] and d [BN] of the current super-block.
    extern __shared__ uint4 smem[];
    uint4 *lds_a = smem;
    uint4 *lds_b = lds_a + 2 * 8 * BM;
    uint4 *lds_r = lds_b + 2 * kBItems;
    float *lds_d = reinterpret_cast<float *>(lds_r + 4 * BN);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;  // wave position in the WM x WN grid
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const size_t row_bytes = (size_t)spr * TL::kBlockBytes;

    // ---- loader roles ----
    // A: item idx = tid + i * kThreads (i < kAItems) -> chunk = idx / BM, row = idx % BM: a wave copies 64
    //    consecutive items.
    // B: weight row bn = tid % BN, unit bu = tid / BN; (piece, plane) task q = bu * kBTasks + t,
    //    piece = q / 2, plane = q % 2.
    const int bn = tid % BN, bu = tid / BN;
    const uint8_t *wrow = W + (size_t)(n0 + bn < N ? n0 + bn : N - 1) * row_bytes;

    // One stage's global data in registers: the A items of this thread, and for B the super-block header and
    // one or two 16-byte pieces.  Steps past the end re-read the last one, so every load is unconditional.
    const int last_step = spr * 4 - 1;
    auto fetch_a = [&](int step, u32x4 (&fa)[kAItems]) __attribute__((always_inline)) {
        step = step < last_step ? step : last_step;
#pragma unroll
        for (int i = 0; i < kAItems; i++) {
            const int idx = tid + i * kThreads;
            fa[i] = *reinterpret_cast<const u32x4 *>(xs + (size_t)(step * 8 + idx / BM) * Mp + m0 + idx % BM);
        }
    };
    auto fetch_b = [&](int step, u32x4 &fhdr, u32x4 (&fpc)[kPieces]) __attribute__((always_inline)) {
        step = step < last_step ? step : last_step;
        const uint8_t *blk = wrow + (size_t)(step >> 2) * TL::kBlockBytes;
        const int c = step & 3;
        if constexpr (kQ6) {
            // stage c covers elements 64 c .. + 63 of the super-block: half h = c / 2, the low (c even) or high
            // nibbles of ql bytes 64 h .. + 63 in natural order, qh bytes 32 h + (k % 32) at bit 2 (2 (c % 2) + k / 32),
            // scales 4 c .. 4 c + 3 (crates/pmetal-gguf/src/k_quants.rs:484-494).  Task = one 16-element scale group.
            const int h = c >> 1;
#pragma unroll
            for (int t = 0; t < kBTasks; t++) {
                const int ks = bu * kBTasks + t;
                fpc[t] = load16_a2(blk + 64 * h + 16 * ks);
                fpc[kBTasks + t] = load16_a2(blk + 128 + 32 * h + 16 * (ks & 1));
            }
            fhdr = u32x4{reinterpret_cast<const u32_a2 *>(blk + 192 + 4 * c)->v, *reinterpret_cast<const u16_a2 *>(blk + 208), 0u, 0u};
        } else {
            fhdr = *reinterpret_cast<const u32x4 *>(blk);
            // the stage covers sub-blocks 2c and 2c+1, which are pieces 2c and 2c+1 in both orders
            if (kPieces == 2) {
#pragma unroll
                for (int q = 0; q < kPieces; q++) fpc[q] = *reinterpret_cast<const u32x4 *>(blk + 16 + 16 * (2 * c + q));
            } else {
                const int pc = (bu * kBTasks) >> 1;
                fpc[0] = *reinterpret_cast<const u32x4 *>(blk + 16 + 16 * (2 * c + pc));
            }
        }
    };
    auto stage_a = [&](int stage, const u32x4 (&fa)[kAItems]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kAItems; i++) *reinterpret_cast<u32x4 *>(lds_a + stage * 8 * BM + tid + i * kThreads) = fa[i];
    };
    // c = step % 4 is a compile-time constant at every call
    auto stage_b = [&](int stage, int c, const u32x4 &fhdr, const u32x4 (&fpc)[kPieces]) __attribute__((always_inline)) {
        if constexpr (kQ6) {
            uint4 *dst1 = lds_b + stage * kBItems, *dst2 = dst1 + 8 * BN;
#pragma unroll
            for (int t = 0; t < kBTasks; t++) {
                const int ks = bu * kBTasks + t;
                const int sc = (int)(int8_t)(fhdr.x >> (8 * ks));
                uint4 b1lo, b1hi, b2lo, b2hi;
                dequant16_q6(fpc[t], fpc[kBTasks + t], 4 * (c & 1), 2 * (2 * (c & 1) + (ks >> 1)), sc, b1lo, b1hi, b2lo, b2hi);
                dst1[(ks * 2 + 0) * BN + bn] = b1lo;
                dst1[(ks * 2 + 1) * BN + bn] = b1hi;
                dst2[(ks * 2 + 0) * BN + bn] = b2lo;
                dst2[(ks * 2 + 1) * BN + bn] = b2hi;
            }
            if (c == 1 && bu == 0) lds_d[bn] = f16_bits_to_f32(fhdr.y);
        } else {
            uint4 *dst = lds_b + stage * kBItems;
            const uint4 hdr4 = make_uint4(fhdr.x, fhdr.y, fhdr.z, fhdr.w);
            uint32_t sc0, sc1, mn;
            scale_min_u(hdr4, 2 * c, sc0, mn);
            scale_min_u(hdr4, 2 * c + 1, sc1, mn);
    #pragma unroll
            for (int t = 0; t < kBTasks; t++) {
                const int q = bu * kBTasks + t;
                const int bw = q >> 1, p = q & 1;
                // nibble plane p of piece bw:
                //   REF : elements 16 p .. + 15 of sub-block 2c + bw  -> k = 32 bw + 16 p + b, scale 2c + bw
                //   GGML: elements 16 bw .. + 15 of sub-block 2c + p  -> k = 32 p + 16 bw + b, scale 2c + p
                const int ks = ORDER == 0 ? 2 * bw + p : 2 * p + bw;
                const uint32_t sc = (ORDER == 0 ? bw : p) ? sc1 : sc0;
                const u32x4 pc4 = fpc[kPieces == 2 ? bw : 0];
                uint4 b0, b1;
                dequant16(make_uint4(pc4.x, pc4.y, pc4.z, pc4.w), p, sc, b0, b1);
                dst[(ks * 2 + 0) * BN + bn] = b0;
                dst[(ks * 2 + 1) * BN + bn] = b1;
            }
            if (c == 1) {
                // once per super-block (while its second stage is being staged, one barrier after the previous
                // super-block's R product has been issued): d and the B operand of the R product for this column.
                // item (t, g) = (-h_j, -h_j, -l_j, -l_j, -h_j+1, -h_j+1, -l_j+1, -l_j+1), j = 4 t + 2 g, against
                // the activations' (h, l, h, l, ...): all four cross products.
                const float dmin = f16_bits_to_f32(hdr4.x >> 16);
                if (bu == 0) lds_d[bn] = f16_bits_to_f32(hdr4.x & 0xFFFFu);
    #pragma unroll
                for (int r = 0; r < 4; r++) {
                    if (r % kUnits == bu) {
                        uint32_t sc, mn0, mn1;
                        scale_min_u(hdr4, 2 * r, sc, mn0);
                        scale_min_u(hdr4, 2 * r + 1, sc, mn1);
                        _Float16 h0, l0, h1, l1;
                        neg_min_split(dmin, mn0, h0, l0);
                        neg_min_split(dmin, mn1, h1, l1);
                        const half8_t item = {h0, h0, l0, l0, h1, h1, l1, l1};
                        lds_r[r * BN + bn] = __builtin_bit_cast(uint4, item);
                    }
                }
            }
        }
    };

    // ---- accumulators: NB x NB blocks of 32 x 32 per wave ----
    float16_t acc[NB][NB], part[NB][NB];
#pragma unroll
    for (int i = 0; i < NB; i++)
#pragma unroll
        for (int jx = 0; jx < NB; jx++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][jx][r] = 0.0f, part[i][jx][r] = 0.0f;

    const int col = lane & 31, kgrp = lane >> 5;

    // A operand of the R product: requested one step before it is used
    u32x4 xsv[2][NB];
    auto fetch_xsum = [&](int sb) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < NB; i++)
                xsv[t][i] = *reinterpret_cast<const u32x4 *>(xsum + ((size_t)sb * 4 + t * 2 + kgrp) * Mp + m0 + (wm * NB + i) * 32 + col);
    };

    // c = step % 4 is a compile-time constant at every call
    auto compute = [&](int stage, int c, int sb) __attribute__((always_inline)) {
        const uint4 *sa = lds_a + stage * 8 * BM, *sbp = lds_b + stage * kBItems;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            half8_t av[NB], bv[NB], bw[NB];
#pragma unroll
            for (int i = 0; i < NB; i++) av[i] = __builtin_bit_cast(half8_t, sa[(ks * 2 + kgrp) * BM + (wm * NB + i) * 32 + col]);
#pragma unroll
            for (int jx = 0; jx < NB; jx++) {
                bv[jx] = __builtin_bit_cast(half8_t, sbp[(ks * 2 + kgrp) * BN + (wn * NB + jx) * 32 + col]);
                if (kQ6) bw[jx] = __builtin_bit_cast(half8_t, sbp[8 * BN + (ks * 2 + kgrp) * BN + (wn * NB + jx) * 32 + col]);
            }
#pragma unroll
            for (int i = 0; i < NB; i++)
#pragma unroll
                for (int jx = 0; jx < NB; jx++) {
                    if (c == 0 && ks == 0) {  // first product of a super-block starts from zero
                        float16_t z;
#pragma unroll
                        for (int r = 0; r < 16; r++) z[r] = 0.0f;
                        part[i][jx] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[i], bv[jx], z, 0, 0, 0);
                    } else {
                        part[i][jx] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[i], bv[jx], part[i][jx], 0, 0, 0);
                    }
                    if (kQ6) part[i][jx] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[i], bw[jx], part[i][jx], 0, 0, 0);
                }
        }
        if (c == 3) {
            // ---- end of a super-block: R product into the accumulators (Q4_K), then acc += d * P ----
#pragma unroll
            for (int t = 0; t < (kQ6 ? 0 : 2); t++) {
                half8_t sv[NB], mv[NB];
#pragma unroll
                for (int i = 0; i < NB; i++) sv[i] = __builtin_bit_cast(half8_t, xsv[t][i]);
#pragma unroll
                for (int jx = 0; jx < NB; jx++) mv[jx] = __builtin_bit_cast(half8_t, lds_r[(t * 2 + kgrp) * BN + (wn * NB + jx) * 32 + col]);
#pragma unroll
                for (int i = 0; i < NB; i++)
#pragma unroll
                    for (int jx = 0; jx < NB; jx++)
                        acc[i][jx] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sv[i], mv[jx], acc[i][jx], 0, 0, 0);
            }
#pragma unroll
            for (int jx = 0; jx < NB; jx++) {
                const float dd = lds_d[(wn * NB + jx) * 32 + col];
#pragma unroll
                for (int i = 0; i < NB; i++)
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[i][jx][r] = __builtin_fmaf(dd, part[i][jx][r], acc[i][jx][r]);
            }
        }
    };

    // Global loads run ahead of the LDS staging in register sets; with four steps per loop trip the set a step
    // uses is a compile-time constant.  Large tiles (registers are scarce): B two steps ahead in two sets, A
    // requested at the start of a step and stored to LDS at its end, behind the MFMAs.  The small tile (short
    // steps, few waves per compute unit to hide latency): both four steps ahead in four sets.
    // Two LDS stages; one barrier per step; c = step % 4 and the LDS stage are compile-time constants.
    constexpr int DA = NB == 1 ? 4 : 1, DB = NB == 1 ? 4 : 2;
    u32x4 fa[DA][kAItems], fh[DB], fp[DB][kPieces];
#pragma unroll
    for (int i = 0; i < DA; i++) fetch_a(i, fa[i]);
#pragma unroll
    for (int i = 0; i < DB; i++) fetch_b(i, fh[i], fp[i]);
    stage_a(0, fa[0]);
    stage_b(0, 0, fh[0], fp[0]);
    if (DA > 1) fetch_a(DA, fa[0]);
    fetch_b(DB, fh[0], fp[0]);
    __syncthreads();
#define PMH_STEP(C)                                                                                      \
    if ((C) == 2 && !kQ6) fetch_xsum(sb);                                                                        \
    if (DA == 1) {                                                                                       \
        fetch_a(step + (C) + 1, fa[0]);                                                                  \
        __builtin_amdgcn_sched_barrier(0); /* keep the requests a whole step ahead of their use */       \
    }                                                                                                    \
    stage_b(((C) + 1) & 1, ((C) + 1) & 3, fh[((C) + 1) % DB], fp[((C) + 1) % DB]);                       \
    fetch_b(step + (C) + 1 + DB, fh[((C) + 1) % DB], fp[((C) + 1) % DB]);                                \
    compute((C) & 1, C, sb);                                                                             \
    stage_a(((C) + 1) & 1, fa[((C) + 1) % DA]);                                                          \
    if (DA > 1) fetch_a(step + (C) + 1 + DA, fa[((C) + 1) % DA]);                                        \
    __syncthreads();
    for (int sb = 0; sb < spr; sb++) {
        const int step = sb * 4;
        PMH_STEP(0)
        PMH_STEP(1)
        PMH_STEP(2)
        PMH_STEP(3)
    }
#undef PMH_STEP

    // ---- epilogue: C layout of v_mfma_f32_32x32x*: lane holds column (lane & 31), rows 8 (r / 4) + 4 (lane / 32) + r % 4
#pragma unroll
    for (int i = 0; i < NB; i++)
#pragma unroll
        for (int jx = 0; jx < NB; jx++) {
            const int n = n0 + (wn * NB + jx) * 32 + col;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + (wm * NB + i) * 32 + 8 * (r >> 2) + 4 * kgrp + (r & 3);
                if (m < M && n < N) {
                    const float v = acc[i][jx][r] * rowscale[m];
                    if (YBF16) {
                        uint32_t u = __builtin_bit_cast(uint32_t, v);
                        u = ((u & 0x7FFFFFFFu) > 0x7F800000u) ? ((u >> 16) | 0x40u) : ((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
                        reinterpret_cast<uint16_t *>(yg)[(size_t)m * N + n] = (uint16_t)u;
                    } else {
                        reinterpret_cast<float *>(yg)[(size_t)m * N + n] = v;
                    }
                }
            }
        }
}

}  // namespace

namespace pmh {

// workspace: xs [k/8][Mp] items, xsum [k/256][4][Mp] items, rowscale [Mp] f32 (each 256-byte aligned)
static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }
static int64_t padded_rows(int64_t m) { return (m + kMPad - 1) / kMPad * kMPad; }

size_t qgemm_workspace_bytes(int64_t m, int64_t k) {
    const size_t mp = (size_t)padded_rows(m);
    return align256(mp * (size_t)k * 2) + align256(mp * (size_t)(k / 256) * 4 * 16) + align256(mp * 4);
}

template <int QT, int ORDER, bool YBF16, int WM, int WN, int NB>
static hipError_t launch_tile(hipStream_t s, const uint8_t *w, const uint4 *xs, const uint4 *xsum, const float *rowscale,
                              void *y, int64_t m, int64_t mp, int64_t n, int spr) {
    using TL = Tile<QT, WM, WN, NB>;
    auto kern = k_qgemm<QT, ORDER, YBF16, WM, WN, NB>;
    if (TL::kLdsBytes > 64 * 1024) {
        hipError_t a = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)TL::kLdsBytes);
        if (a != hipSuccess) return a;
    }
    const dim3 grid((unsigned)((n + TL::BN - 1) / TL::BN), (unsigned)((m + TL::BM - 1) / TL::BM));
    hipLaunchKernelGGL(kern, grid, dim3(TL::kThreads), TL::kLdsBytes, s, w, xs, xsum, rowscale, y, (int)m, (int)mp, (int)n, spr);
    return hipGetLastError();
}

template <int QT, int ORDER, bool YBF16>
static hipError_t launch_shape(hipStream_t s, const uint8_t *w, const uint4 *xs, const uint4 *xsum, const float *rowscale,
                               void *y, int64_t m, int64_t mp, int64_t n, int spr) {
    // tile by m: short activation batches use small tiles, so that less of the MFMA work is padding and the
    // weight matrix spreads over enough workgroups to pull it from HBM at speed
    if (m <= 64) return launch_tile<QT, ORDER, YBF16, 2, 1, 1>(s, w, xs, xsum, rowscale, y, m, mp, n, spr);
    if (m <= 256) return launch_tile<QT, ORDER, YBF16, 2, 2, 2>(s, w, xs, xsum, rowscale, y, m, mp, n, spr);
    return launch_tile<QT, ORDER, YBF16, 4, 2, 2>(s, w, xs, xsum, rowscale, y, m, mp, n, spr);
}

hipError_t launch_qgemm(uint32_t type, const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype,
                        int64_t m, void *y, uint32_t y_dtype, uint32_t order, void *workspace, hipStream_t s) {
    if (type != kTypeQ4K && type != kTypeQ6K) return hipErrorNotSupported;
    if (k % 256 != 0 || m <= 0 || n <= 0) return hipErrorInvalidValue;
    const int64_t mp = padded_rows(m);
    uint8_t *ws = reinterpret_cast<uint8_t *>(workspace);
    uint4 *xs = reinterpret_cast<uint4 *>(ws);
    uint4 *xsum = reinterpret_cast<uint4 *>(ws + align256((size_t)mp * k * 2));
    float *rowscale = reinterpret_cast<float *>(ws + align256((size_t)mp * k * 2) + align256((size_t)mp * (k / 256) * 64));
    const dim3 pgrid((unsigned)(mp / 32), (unsigned)(k / 256));
    if (x_dtype == kDtypeF32) {
        hipLaunchKernelGGL(k_prep_scale<true>, dim3((unsigned)((mp + 3) / 4)), dim3(256), 0, s, x, k, (int)m, rowscale);
        hipLaunchKernelGGL(k_prep_tiles<true>, pgrid, dim3(256), 0, s, x, k, (int)m, (int)mp, rowscale, xs, xsum);
    } else {
        hipLaunchKernelGGL(k_prep_scale<false>, dim3((unsigned)((mp + 3) / 4)), dim3(256), 0, s, x, k, (int)m, rowscale);
        hipLaunchKernelGGL(k_prep_tiles<false>, pgrid, dim3(256), 0, s, x, k, (int)m, (int)mp, rowscale, xs, xsum);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int spr = (int)(k / 256);
    const bool ybf = y_dtype == kDtypeBf16;
    if (type == kTypeQ6K)  // one element order
        return ybf ? launch_shape<14, 0, true>(s, w, xs, xsum, rowscale, y, m, mp, n, spr)
                   : launch_shape<14, 0, false>(s, w, xs, xsum, rowscale, y, m, mp, n, spr);
    if (order == kOrderRef)
        return ybf ? launch_shape<12, 0, true>(s, w, xs, xsum, rowscale, y, m, mp, n, spr)
                   : launch_shape<12, 0, false>(s, w, xs, xsum, rowscale, y, m, mp, n, spr);
    return ybf ? launch_shape<12, 1, true>(s, w, xs, xsum, rowscale, y, m, mp, n, spr)
               : launch_shape<12, 1, false>(s, w, xs, xsum, rowscale, y, m, mp, n, spr);
}

}  // namespace pmh
