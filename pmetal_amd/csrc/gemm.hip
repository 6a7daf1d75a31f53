// Dequant-fused Q4_K GEMM  Y[m,n] = sum_k X[m,k] * W[n,k]  (prefill) on the gfx950 matrix cores.
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
// and the per-super-block factors are applied to the fp32 partial sums:
//     Y[m,n] = 2^e_m * sum_SB ( d[n,SB] * P_SB[m,n] - dmin[n,SB] * Q_SB[m,n] )
//     P_SB = sum_{k in SB} A[m,k] * B[n,k]            16 x v_mfma_f32_32x32x16_f16 per 32x32 block
//     Q_SB = sum_{j<8} m[n,j] * xsum[m,j]             one more MFMA: xsum as f16 hi + lo, m exact
// so the only roundings are the fp32 accumulations.
//
// Tiling: a workgroup of 256 threads (4 waves) computes a BM x 128 tile of Y (BM = 128, or 64 / 32 for
// short activation batches); for BM = 128 the waves form a 2 x 2 grid and each owns 2 x 2 MFMA blocks.  K advances two 32-element sub-blocks per stage: every thread dequantizes
// 32 weights (one 16-byte piece, both nibble planes) into the B tile and copies 4 x 8 activations into the
// A tile (a wave reads 8 rows x 128 contiguous bytes per load); both tiles are stored in LDS in MFMA
// operand order ([k-step][k-group][row] items of 16 bytes) so the operand reads are conflict-free
// ds_read_b128.  Global loads run two stages ahead in registers, the LDS stages are double buffered.
#include "internal.hpp"

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int BN = 128;  // workgroup tile width (weight rows); the height BM is a template parameter
constexpr int kThreads = 256;

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return __builtin_bit_cast(float, h << 16); }

// ------------------------------------------------------------------------------------------------
// Pre-pass over the activations: one workgroup per row m.
//   xs[m][k]            = f16( x[m][k] * 2^-e_m )          exact
//   xsum[m][sb][0 / 1]  = hi / lo f16 split of sum_{k in 32-block sb} xs[m][k]
//   rowscale[m]         = 2^e_m
// e_m normalises the row maximum into [2^9, 2^10): block sums (< 2^15) fit f16 and small rows stay out of
// the f16 subnormal range.
// ------------------------------------------------------------------------------------------------
template <bool XF32>
__global__ __launch_bounds__(256) void k_prep_x(const void *__restrict__ xg, int64_t k, _Float16 *__restrict__ xs,
                                                 _Float16 *__restrict__ xsum, float *__restrict__ rowscale) {
    __shared__ float red[4];
    const int64_t m = blockIdx.x;
    const int tid = threadIdx.x;
    auto load = [&](int64_t i) -> float {
        if (XF32) return reinterpret_cast<const float *>(xg)[m * k + i];
        return bf16_to_f32(reinterpret_cast<const uint16_t *>(xg)[m * k + i]);
    };
    float amax = 0.0f;
    for (int64_t i = tid; i < k; i += 256) amax = __builtin_fmaxf(amax, __builtin_fabsf(load(i)));
    for (int off = 32; off > 0; off >>= 1) amax = __builtin_fmaxf(amax, __shfl_xor(amax, off));
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = __builtin_fmaxf(__builtin_fmaxf(red[0], red[1]), __builtin_fmaxf(red[2], red[3]));
    // 2^e with amax * 2^-e < 2^10, so that the sum of a 32-element block (< 2^15) also fits f16
    const int eb = (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xFFu);  // amax in [2^(eb-127), 2^(eb-126))
    int e = eb - 126 - 10;  // also scales small rows up, out of the f16 subnormal range
    e = e < -126 ? -126 : (e > 126 ? 126 : e);
    if (eb == 255) e = 0;  // inf / NaN: let them through
    const float down = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);
    if (tid == 0) rowscale[m] = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
    // 32-element blocks: 8 lanes per block, 4 elements per lane
    const int64_t n_sb = k / 32;
    for (int64_t blk = tid >> 3; blk < n_sb; blk += 32) {
        const int part = tid & 7;
        float s = 0.0f;
        _Float16 out[4];
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const _Float16 h = (_Float16)(load(blk * 32 + part * 4 + c) * down);
            out[c] = h;
            s += (float)h;
        }
        *reinterpret_cast<uint2 *>(xs + m * k + blk * 32 + part * 4) = *reinterpret_cast<const uint2 *>(out);
        s += __shfl_xor(s, 1);
        s += __shfl_xor(s, 2);
        s += __shfl_xor(s, 4);
        if (part == 0) {
            const _Float16 hi = (_Float16)s;
            const _Float16 lo = (_Float16)(s - (float)hi);
            xsum[(m * n_sb + blk) * 2] = hi;
            xsum[(m * n_sb + blk) * 2 + 1] = lo;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// main kernel
// ------------------------------------------------------------------------------------------------
// K advances 64 elements (two sub-blocks) per stage.  LDS stage: A then B tile, each
// [4 MFMA k-steps][2 k-groups][128 rows] items of 8 f16 (16 bytes) = 16 KiB; two stages.
constexpr int BK = 64;
constexpr int kItemsB = 4 * 2 * BN;  // uint4 items of the B tile per stage

// 16 nibbles (one plane of a 16-byte piece) times the integer scale -> 16 exact f16 values.
// 0x6400 | q is the f16 1024 + q; (1024 + q) * sc - 1024 * sc is exact in a packed f16 fma.
__device__ __forceinline__ void dequant16(const uint4 piece, const int plane, const float sc, uint4 &lo8, uint4 &hi8) {
    const half2_t sc2 = {(_Float16)sc, (_Float16)sc};
    const half2_t off2 = {(_Float16)(-1024.0f * sc), (_Float16)(-1024.0f * sc)};  // exact: sc <= 63
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

// (scale, min) of sub-block j from the 12 scale bytes (quantize.rs:844-855).
__device__ __forceinline__ void scale_min_u(const uint4 hdr, const int j, uint32_t &sc, uint32_t &mn) {
    const int sh = 8 * (j & 3);
    const uint32_t a = (hdr.y >> sh) & 0xFFu, b = (hdr.z >> sh) & 0xFFu, c = (hdr.w >> sh) & 0xFFu;
    if (j < 4) {
        sc = a & 63u;
        mn = b & 63u;
    } else {
        sc = (c & 0xFu) | ((a >> 6) << 4);
        mn = (c >> 4) | ((b >> 6) << 4);
    }
}

// The 4 waves form a WAVES_M x (4 / WAVES_M) grid; each wave owns BLK_M x BLK_N MFMA blocks of 32 x 32:
//   BM = 128: 2 x 2 waves of 2 x 2 blocks      BM = 64: 1 x 4 waves of 2 x 1      BM = 32: 1 x 4 waves of 1 x 1
template <int ORDER, bool YBF16, int WAVES_M, int BLK_M>
__global__ __launch_bounds__(kThreads, 2) void k_qgemm_q4k(const uint8_t *__restrict__ W,
                                                            const _Float16 *__restrict__ xs,
                                                            const _Float16 *__restrict__ xsum,
                                                            const float *__restrict__ rowscale, void *__restrict__ yg,
                                                            int M, int N, int spr) {
    constexpr int WAVES_N = 4 / WAVES_M;
    constexpr int BLK_N = BN / 32 / WAVES_N;
    constexpr int BM = WAVES_M * BLK_M * 32;
    constexpr int RA = BM / 32;  // A-tile rows copied per thread and stage
    __shared__ uint4 lds_a[2][8 * BM];  // [stage][(k-step, k-group) = chunk][row]
    __shared__ uint4 lds_b[2][kItemsB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;  // wave position in the grid
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int K = spr * 256;
    const size_t row_bytes = (size_t)spr * 144;

    // ---- loader roles ----
    // A: thread (row = tid / 8 + 32 r, chunk c = tid % 8) copies 8 f16 at k = 8 c: a wave reads 8 rows x 128 B
    const int ac = tid & 7, ar = tid >> 3;
    const _Float16 *xrow[RA];
#pragma unroll
    for (int r = 0; r < RA; r++) {
        const int row = m0 + ar + 32 * r;
        xrow[r] = xs + (size_t)(row < M ? row : M - 1) * K + 8 * ac;  // rows past M are computed and dropped
    }
    // B: thread (n = tid / 2, w = tid % 2) dequantizes both nibble planes of one 16-byte piece per stage
    const int bn = tid >> 1, bw = tid & 1;
    const uint8_t *wrow = W + (size_t)(n0 + bn < N ? n0 + bn : N - 1) * row_bytes;

    struct Fetch {
        uint4 a[RA], hdr, piece;
    };
    auto fetch = [&](int step, Fetch &f) {
#pragma unroll
        for (int r = 0; r < RA; r++) f.a[r] = *reinterpret_cast<const uint4 *>(xrow[r] + (size_t)step * BK);
        const uint8_t *blk = wrow + (size_t)(step >> 2) * 144;
        f.hdr = *reinterpret_cast<const uint4 *>(blk);
        // the stage covers sub-blocks 2c and 2c+1, c = step % 4, which are pieces 2c and 2c+1 in both orders
        f.piece = *reinterpret_cast<const uint4 *>(blk + 16 + 16 * (2 * (step & 3) + bw));
    };
    auto stage_in = [&](int stage, int step, const Fetch &f) {
#pragma unroll
        for (int r = 0; r < RA; r++) lds_a[stage][ac * BM + ar + 32 * r] = f.a[r];  // item [ks = c / 2][g = c % 2][row]
        const int c = step & 3;
#pragma unroll
        for (int p = 0; p < 2; p++) {
            // nibble plane p of this piece:
            //   REF : elements 16 p .. + 15 of sub-block 2c + bw  -> k = 32 bw + 16 p + b, scale 2c + bw
            //   GGML: elements 16 bw .. + 15 of sub-block 2c + p  -> k = 32 p + 16 bw + b, scale 2c + p
            const int sub = ORDER == 0 ? 2 * c + bw : 2 * c + p;
            const int ks = ORDER == 0 ? 2 * bw + p : 2 * p + bw;
            uint32_t sc, mn;
            scale_min_u(f.hdr, sub, sc, mn);
            uint4 b0, b1;
            dequant16(f.piece, p, (float)sc, b0, b1);
            lds_b[stage][(ks * 2 + 0) * BN + bn] = b0;
            lds_b[stage][(ks * 2 + 1) * BN + bn] = b1;
        }
    };

    // ---- accumulators: BLK_M x BLK_N blocks of 32 x 32 per wave ----
    float16_t acc[BLK_M][BLK_N], part[BLK_M][BLK_N];
#pragma unroll
    for (int i = 0; i < BLK_M; i++)
#pragma unroll
        for (int jx = 0; jx < BLK_N; jx++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][jx][r] = 0.0f, part[i][jx][r] = 0.0f;

    const int col = lane & 31, kgrp = lane >> 5;
    // columns this lane owns in the two n-blocks of its wave, and their weight rows (for d, dmin, mins)
    int ncol[BLK_N];
    const uint8_t *nrow[BLK_N];
#pragma unroll
    for (int jx = 0; jx < BLK_N; jx++) {
        ncol[jx] = n0 + (wn * BLK_N + jx) * 32 + col;
        nrow[jx] = W + (size_t)(ncol[jx] < N ? ncol[jx] : N - 1) * row_bytes;
    }
    // rows this lane feeds as A operand in the min-term MFMA
    int mrow[BLK_M];
#pragma unroll
    for (int i = 0; i < BLK_M; i++) {
        const int r = m0 + (wm * BLK_M + i) * 32 + col;
        mrow[i] = r < M ? r : M - 1;
    }

    // Global loads run two stages ahead of the MFMAs (two register sets), the dequantization into LDS one
    // stage ahead (two LDS stages).
    const int n_steps = spr * 4;
    Fetch f0, f1;
    fetch(0, f0);
    if (1 < n_steps) fetch(1, f1);
    stage_in(0, 0, f0);
    if (2 < n_steps) fetch(2, f0);
    __syncthreads();

    auto compute = [&](int step) {
        const int stage = step & 1;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            half8_t av[BLK_M], bv[BLK_N];
#pragma unroll
            for (int i = 0; i < BLK_M; i++)
                av[i] = __builtin_bit_cast(half8_t, lds_a[stage][(ks * 2 + kgrp) * BM + (wm * BLK_M + i) * 32 + col]);
#pragma unroll
            for (int jx = 0; jx < BLK_N; jx++)
                bv[jx] = __builtin_bit_cast(half8_t, lds_b[stage][(ks * 2 + kgrp) * BN + (wn * BLK_N + jx) * 32 + col]);
#pragma unroll
            for (int i = 0; i < BLK_M; i++)
#pragma unroll
                for (int jx = 0; jx < BLK_N; jx++)
                    part[i][jx] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[i], bv[jx], part[i][jx], 0, 0, 0);
        }
        if ((step & 3) == 3) {
            // ---- end of a super-block: fold P and the min term into the accumulators ----
            const int sb = step >> 2;
            float dd[BLK_N], dm[BLK_N];
            half8_t mv[BLK_N];
#pragma unroll
            for (int jx = 0; jx < BLK_N; jx++) {
                const uint4 h = *reinterpret_cast<const uint4 *>(nrow[jx] + (size_t)sb * 144);
                dd[jx] = f16_bits_to_f32(h.x & 0xFFFFu);
                dm[jx] = f16_bits_to_f32(h.x >> 16);
                // B' operand of the min term: column n, k' = 8 kgrp .. + 7 -> mins m_0..m_7 (hi and lo half)
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    uint32_t sc, mn;
                    scale_min_u(h, t, sc, mn);
                    mv[jx][t] = (_Float16)(float)mn;
                }
            }
            half8_t sv[BLK_M];  // A' operand: row m; k-group 0 -> hi parts of the 8 sums, k-group 1 -> lo parts
#pragma unroll
            for (int i = 0; i < BLK_M; i++) {
                const _Float16 *p = xsum + ((size_t)mrow[i] * (spr * 8) + (size_t)sb * 8) * 2;
                const half8_t a = *reinterpret_cast<const half8_t *>(p);      // hi0 lo0 hi1 lo1 hi2 lo2 hi3 lo3
                const half8_t b = *reinterpret_cast<const half8_t *>(p + 8);  // hi4 lo4 ...
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    sv[i][t] = kgrp ? a[2 * t + 1] : a[2 * t];
                    sv[i][4 + t] = kgrp ? b[2 * t + 1] : b[2 * t];
                }
            }
#pragma unroll
            for (int i = 0; i < BLK_M; i++)
#pragma unroll
                for (int jx = 0; jx < BLK_N; jx++) {
                    float16_t q;
#pragma unroll
                    for (int r = 0; r < 16; r++) q[r] = 0.0f;
                    q = __builtin_amdgcn_mfma_f32_32x32x16_f16(sv[i], mv[jx], q, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        acc[i][jx][r] += dd[jx] * part[i][jx][r] - dm[jx] * q[r];
                        part[i][jx][r] = 0.0f;
                    }
                }
        }
    };

    for (int step = 0; step < n_steps; step += 2) {
        // even step: stage step + 1 comes from f1, then f1 is refilled for step + 3
        if (step + 1 < n_steps) stage_in(1, step + 1, f1);
        if (step + 3 < n_steps) fetch(step + 3, f1);
        compute(step);
        __syncthreads();
        if (step + 1 < n_steps) {
            if (step + 2 < n_steps) stage_in(0, step + 2, f0);
            if (step + 4 < n_steps) fetch(step + 4, f0);
            compute(step + 1);
            __syncthreads();
        }
    }

    // ---- epilogue: C layout of v_mfma_f32_32x32x*: lane holds column (lane & 31), rows 8 (r / 4) + 4 (lane / 32) + r % 4
#pragma unroll
    for (int i = 0; i < BLK_M; i++)
#pragma unroll
        for (int jx = 0; jx < BLK_N; jx++) {
            const int n = ncol[jx];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + (wm * BLK_M + i) * 32 + 8 * (r >> 2) + 4 * kgrp + (r & 3);
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

// workspace: xs [m, k] f16, xsum [m, k/32, 2] f16, rowscale [m] f32 (each 256-byte aligned)
static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

size_t qgemm_workspace_bytes(int64_t m, int64_t k) {
    return align256((size_t)m * k * 2) + align256((size_t)m * (k / 32) * 4) + align256((size_t)m * 4);
}

hipError_t launch_qgemm(uint32_t type, const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype,
                        int64_t m, void *y, uint32_t y_dtype, uint32_t order, void *workspace, hipStream_t s) {
    if (type != kTypeQ4K) return hipErrorNotSupported;
    if (k % 256 != 0 || m <= 0 || n <= 0) return hipErrorInvalidValue;
    uint8_t *ws = reinterpret_cast<uint8_t *>(workspace);
    _Float16 *xs = reinterpret_cast<_Float16 *>(ws);
    _Float16 *xsum = reinterpret_cast<_Float16 *>(ws + align256((size_t)m * k * 2));
    float *rowscale = reinterpret_cast<float *>(ws + align256((size_t)m * k * 2) + align256((size_t)m * (k / 32) * 4));
    if (x_dtype == kDtypeF32) hipLaunchKernelGGL(k_prep_x<true>, dim3((unsigned)m), dim3(256), 0, s, x, k, xs, xsum, rowscale);
    else hipLaunchKernelGGL(k_prep_x<false>, dim3((unsigned)m), dim3(256), 0, s, x, k, xs, xsum, rowscale);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int spr = (int)(k / 256);
    const bool ybf = y_dtype == kDtypeBf16;
    auto go = [&](auto kern, int bm) {
        const dim3 grid((unsigned)((n + BN - 1) / BN), (unsigned)((m + bm - 1) / bm));
        hipLaunchKernelGGL(kern, grid, dim3(kThreads), 0, s, w, xs, xsum, rowscale, y, (int)m, (int)n, spr);
    };
    // tile height by m: short activation batches use a flatter tile so that less of the MFMA work is padding
    const int shape = m <= 32 ? 0 : (m <= 64 ? 1 : 2);
    if (order == kOrderRef) {
        if (ybf) {
            if (shape == 0) go(k_qgemm_q4k<0, true, 1, 1>, 32);
            else if (shape == 1) go(k_qgemm_q4k<0, true, 1, 2>, 64);
            else go(k_qgemm_q4k<0, true, 2, 2>, 128);
        } else {
            if (shape == 0) go(k_qgemm_q4k<0, false, 1, 1>, 32);
            else if (shape == 1) go(k_qgemm_q4k<0, false, 1, 2>, 64);
            else go(k_qgemm_q4k<0, false, 2, 2>, 128);
        }
    } else {
        if (ybf) {
            if (shape == 0) go(k_qgemm_q4k<1, true, 1, 1>, 32);
            else if (shape == 1) go(k_qgemm_q4k<1, true, 1, 2>, 64);
            else go(k_qgemm_q4k<1, true, 2, 2>, 128);
        } else {
            if (shape == 0) go(k_qgemm_q4k<1, false, 1, 1>, 32);
            else if (shape == 1) go(k_qgemm_q4k<1, false, 1, 2>, 64);
            else go(k_qgemm_q4k<1, false, 2, 2>, 128);
        }
    }
    return hipGetLastError();
}

}  // namespace pmh
