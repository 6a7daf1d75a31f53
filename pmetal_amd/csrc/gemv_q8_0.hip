// Dequant-fused GEMV for large Q8_0 matrices on gfx950: rows staged through LDS, integer dot products.
//
// y[n] = sum_k W[n,k] * x[k], W the GGUF Q8_0 block stream (34 bytes per 32 weights: d f16, qs[32] i8; value d * q,
// dequant.rs:466-495).  A 34-byte block is aligned to two bytes only, and a lane that reads its own block from
// global memory touches a different cache line than its neighbours with every load.  Here a wave copies 2176
// contiguous, 16-byte aligned bytes of a row (64 blocks) into LDS with whole-wave 16-byte loads, and each lane then
// takes its block out of LDS as aligned dwords which one funnel shift per dword puts into place.
//
//  * The activations are converted once per workgroup to fixed point: every 32-element group (one block) gets a
//    power-of-two scale that puts its largest magnitude below 2^22, and the 23-bit signed integers are written as
//    three balanced base-256 digits in [-128, 127].  sum q x over a block is then 2^e * (65536 dot(q, d2) + 256
//    dot(q, d1) + dot(q, d0)) with v_dot4_i32_i8 on the quant dwords: integer arithmetic, exact up to the fixed-point
//    resolution of x (22 bits under the group maximum).
//  * One workgroup per compute unit; a row is ks = (k / 32) / 64 chunks of 64 blocks.  Wave (g, h) takes chunk h of the
//    rows of row group g, lane l block 64 h + l, so that a lane's digits (24 registers) never change.  Up to kDepth
//    rows are in flight per wave; every load is issued unconditionally (rows past the end read the first bytes of
//    W) so that the number of outstanding loads is known at every wait.  Lane partial sums go to LDS; after a barrier
//    the workgroup adds up each of its rows and stores y.
//
//  * A row whose last chunk is short (k a multiple of 256 but not of 2048) is handled by the RAGGED variant (see there).
//
// Matrices below 12 MiB, rows shorter than one chunk and k that is not a multiple of 256 stay with the kernel in gemv.hip.
#include "gemv_chunk.hpp"
#include "internal.hpp"

namespace {

using namespace pmh::gemv;

typedef uint32_t u4v __attribute__((ext_vector_type(4)));  // a 16-byte piece

constexpr int kDepth = 5;  // rows in flight per wave
constexpr int kPre = 2;    // of which this many are requested before x is converted
constexpr int kPlanes = 3;
constexpr int kChunkBytes = 64 * 34;          // 2176 = 136 pieces of 16 bytes
constexpr int kStageBytes = kChunkBytes + 16;  // the ninth dword of the last lane lies past the chunk

// Activations -> LDS.  Thread idx converts elements 16 idx .. 16 idx + 15; two consecutive threads hold one block.
// xd[(plane * 8 + dword) * slots + block]: four digits; xm[block] = the block's scale.
// Blocks past the end of a row (its last chunk may hold fewer than 64 blocks) get zero digits and a zero scale.
template <bool XF32>
__device__ __forceinline__ void stage_x(const void *__restrict__ xg, int slots, int k_quads, int nthreads, uint32_t *xd, float *xm) {
    // a thread converts half a block (16 elements: dwords 4 hf .. 4 hf + 3 of the block's digits); the two threads of a
    // block are neighbours in a wave and exchange their largest magnitudes
    const int total = slots * 2, k_halves = k_quads >> 2;  // half blocks, padded to whole chunks; k_halves of them exist
    for (int idx0 = 0; idx0 < total; idx0 += nthreads) {
        const int idx = idx0 + (int)threadIdx.x;
        const bool live = idx < total;
        const int id = live ? idx : total - 1;
        float v[4][4];
        if (id >= k_halves) {
#pragma unroll
            for (int q = 0; q < 4; q++) v[q][0] = v[q][1] = v[q][2] = v[q][3] = 0.f;
        } else if (XF32) {
            const float4 *src = reinterpret_cast<const float4 *>(xg) + (size_t)id * 4;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 f = src[q];
                v[q][0] = f.x, v[q][1] = f.y, v[q][2] = f.z, v[q][3] = f.w;
            }
        } else {
            const uint4 *src = reinterpret_cast<const uint4 *>(xg) + (size_t)id * 2;
            const uint4 a = src[0], b = src[1];
            const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int q = 0; q < 4; q++) {
                v[q][0] = __builtin_bit_cast(float, w[2 * q] << 16), v[q][1] = __builtin_bit_cast(float, w[2 * q] & 0xFFFF0000u);
                v[q][2] = __builtin_bit_cast(float, w[2 * q + 1] << 16), v[q][3] = __builtin_bit_cast(float, w[2 * q + 1] & 0xFFFF0000u);
            }
        }
        // largest magnitude of the block, as bits (the order of non-negative floats is that of their bits)
        uint32_t mb = 0;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t o = max_magnitude_bits(v[q]);
            mb = o > mb ? o : mb;
        }
        const uint32_t o = (uint32_t)__shfl_xor((int)mb, 1);
        mb = o > mb ? o : mb;
        const GroupScale gs = group_scale(mb);
        const int blk = id >> 1, hf = id & 1;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            uint32_t dig[kPlanes];
            to_digits(v[q], gs, dig);
            if (live) {
#pragma unroll
                for (int p = 0; p < kPlanes; p++) xd[(p * 8 + 4 * hf + q) * slots + blk] = dig[p];
            }
        }
        if (live && hf == 0) xm[blk] = gs.scale;
    }
}

// RAGGED: rows whose last chunk is short (k / 32 not a multiple of 64; k is a multiple of 256, so rows and chunks still
// start on 16-byte boundaries).  The copy must not pass the tensor's last piece, and the lanes without a block
// contribute zero.
template <bool XF32, bool SINGLE, bool RAGGED>
__global__ __launch_bounds__(1024) void k_qgemv_q8_0_chunk(const uint8_t *__restrict__ W, const void *__restrict__ xg,
                                                            float *__restrict__ y, int n_rows, int bpr, int rows_per_wg,
                                                            int rows_per_wave, int n_nominal, int nthreads,
                                                            uint32_t w_last) {
    extern __shared__ uint4 smem[];
    const int ks = (bpr + 63) >> 6;
    const int slots = ks * 64;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int n_waves = nthreads >> 6;
    uint32_t *stage = reinterpret_cast<uint32_t *>(smem) + wave * (kStageBytes / 4);  // this wave's row chunk
    uint32_t *xd = reinterpret_cast<uint32_t *>(smem) + n_waves * (kStageBytes / 4);  // [kPlanes * 8][slots]
    float *xm = reinterpret_cast<float *>(xd + kPlanes * 8 * slots);                  // [slots]
    float *part = xm + slots;                                                         // [group][n_nominal][ks]
    const int h = wave % ks, g = wave / ks;
    const int wg_r0 = blockIdx.x * rows_per_wg;
    const int wg_r1 = wg_r0 + rows_per_wg < n_rows ? wg_r0 + rows_per_wg : n_rows;
    const int wave_r0 = wg_r0 + g * rows_per_wave;
    const int wave_r1 = wave_r0 + rows_per_wave < wg_r1 ? wave_r0 + rows_per_wave : wg_r1;
    const int nt_wave = wave_r1 > wave_r0 ? wave_r1 - wave_r0 : 0;  // real tasks of this wave (wave-uniform)

    const uint32_t rowbytes = (uint32_t)bpr * 34u;
    const uint32_t off_a = (uint32_t)h * kChunkBytes + 16u * (uint32_t)lane;
    const uint32_t off_c = (uint32_t)h * kChunkBytes + 2048u + 16u * (uint32_t)(lane & 7);
    // a wave's 136 pieces of a row chunk: lane l takes pieces l and 64 + l, lanes 0..7 also piece 128 + l
    auto issue = [&](int i, u4v &a, u4v &b, u4v &c) {
        const bool real = i < nt_wave;  // wave-uniform
        const uint32_t ro = real ? (uint32_t)(wave_r0 + i) * rowbytes : 0u;
        uint32_t pa = ro + (real ? off_a : 0u), pb = ro + (real ? off_a + 1024u : 0u), pc = ro + (real ? off_c : 0u);
        if (RAGGED) pa = pa < w_last ? pa : w_last, pb = pb < w_last ? pb : w_last, pc = pc < w_last ? pc : w_last;
        a = *reinterpret_cast<const u4v *>(W + pa);
        b = *reinterpret_cast<const u4v *>(W + pb);
        c = *reinterpret_cast<const u4v *>(W + pc);
    };

    u4v ra[kDepth], rb[kDepth], rc[kDepth];
#pragma unroll
    for (int i = 0; i < kPre; i++) issue(i, ra[i], rb[i], rc[i]);
    stage_x<XF32>(xg, slots, bpr * 8, nthreads, xd, xm);
    __syncthreads();

    const int slot = h * 64 + lane;
    uint32_t xr[kPlanes][8];
#pragma unroll
    for (int p = 0; p < kPlanes; p++)
#pragma unroll
        for (int k = 0; k < 8; k++) xr[p][k] = xd[(p * 8 + k) * slots + slot];
    const float xscale = xm[slot];

    // Block `lane` of the chunk starts at byte 34 lane: on a dword boundary for an even lane (the scale is the low half
    // of that dword, the quants follow two bytes in), two bytes past one for an odd lane (the scale is the high half of
    // the dword below, the quants start on a dword boundary).
    const int odd = lane & 1;
    const uint32_t *sp = stage + ((34 * lane) >> 2);       // the dword that holds the scale
    const uint32_t *qp = stage + ((34 * lane + 2) >> 2);   // the dword that holds the first quant
    const uint32_t d_shift = odd ? 16u : 0u, q_shift = odd ? 0u : 16u;
    const bool lane_valid = !RAGGED || slot < bpr;  // the last chunk of a ragged row is short

    float *pp = part + (size_t)(g * n_nominal) * ks + h;
    auto consume = [&](int i, const u4v a, const u4v b, const u4v c) {
        if (i < nt_wave) {  // wave-uniform
        u4v *st4 = reinterpret_cast<u4v *>(stage);
        st4[lane] = a;
        st4[64 + lane] = b;
        if (lane < 8) st4[128 + lane] = c;
        // LDS executes a wave's instructions in order: the reads below see the writes above, and the next row's writes
        // come after these reads
        const uint32_t dw = *sp;
        uint32_t w[9];
#pragma unroll
        for (int k = 0; k < 9; k++) w[k] = qp[k];
        int acc[kPlanes] = {0, 0, 0};
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const uint32_t q = __builtin_amdgcn_alignbit(w[k + 1], w[k], q_shift);
#pragma unroll
            for (int p = 0; p < kPlanes; p++) acc[p] = sdot4(q, xr[p][k], acc[p]);
        }
        float f = (float)acc[kPlanes - 1];
#pragma unroll
        for (int p = kPlanes - 2; p >= 0; p--) f = __builtin_fmaf(f, 256.0f, (float)acc[p]);
        store_chunk_sum(pp + (size_t)i * ks, lane_valid ? (f16_bits_to_f32((dw >> d_shift) & 0xFFFFu) * xscale) * f : 0.0f, lane);
        }
    };

    int issued = kPre;
#pragma unroll
    for (int i = 0; i < kDepth; i++) {
        consume(i, ra[i], rb[i], rc[i]);
        const int upto = SINGLE ? (kPre + 2 * (i + 1) < kDepth ? kPre + 2 * (i + 1) : kDepth)
                                : (kPre + 2 * (i + 1) < kDepth + i + 1 ? kPre + 2 * (i + 1) : kDepth + i + 1);
#pragma unroll
        for (; issued < upto; issued++) issue(issued, ra[issued % kDepth], rb[issued % kDepth], rc[issued % kDepth]);
    }
    if (!SINGLE) {
        int base = kDepth;
        for (; base + kDepth < n_nominal; base += kDepth) {
#pragma unroll
            for (int i = 0; i < kDepth; i++) {
                consume(base + i, ra[i], rb[i], rc[i]);
                issue(base + kDepth + i, ra[i], rb[i], rc[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < kDepth; i++) consume(base + i, ra[i], rb[i], rc[i]);
    }
    __syncthreads();

    reduce_rows(part, ks, wg_r0, wg_r1 - wg_r0, rows_per_wave, n_nominal, nthreads, y);
}

}  // namespace

namespace pmh {

// Runs the row-staging kernel when the shape suits it and returns true; otherwise leaves *err untouched and returns
// false (the caller falls back to the general Q8_0 kernel).  Preconditions as for launch_qgemv.
bool try_launch_qgemv_q8_0_chunk(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y,
                                 hipStream_t s, hipError_t *err) {
    const int bpr = (int)(k / 32);
    if (bpr < 64 || bpr % 8) return false;  // rows of at least one chunk that start on 16-byte boundaries
    const bool ragged = bpr % 64 != 0;
    const int ks = (bpr + 63) / 64;
    const uint64_t w_bytes = (uint64_t)n * (uint64_t)bpr * 34u;
    if (ks > 16 || w_bytes >= (1ull << 32)) return false;
    if (w_bytes < (12ull << 20)) return false;  // measured crossover with the general kernel
    const size_t slots = (size_t)ks * 64;
    const gemv::ChunkPlan plan = gemv::plan_chunks(n, ks, kStageBytes, slots * 4 * (kPlanes * 8) + slots * 4);
    const int64_t n_wg = plan.n_wg, rows_per_wg = plan.rows_per_wg, rows_per_wave = plan.rows_per_wave, n_nominal = plan.n_nominal,
                  threads = plan.threads;
    const size_t lds = plan.lds;
    if (lds > 128 * 1024) return false;
    const bool single = n_nominal <= kDepth;
    const bool xf32 = x_dtype == kDtypeF32;
    auto go = [&](auto kern) {
        if (lds > 64 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kern, dim3((unsigned)n_wg), dim3((unsigned)threads), lds, s, w, x, y, (int)n, bpr, (int)rows_per_wg,
                           (int)rows_per_wave, (int)n_nominal, (int)threads, (uint32_t)((w_bytes - 1) & ~(uint64_t)15));
        return hipGetLastError();
    };
    if (ragged) {
        if (xf32) *err = single ? go(k_qgemv_q8_0_chunk<true, true, true>) : go(k_qgemv_q8_0_chunk<true, false, true>);
        else *err = single ? go(k_qgemv_q8_0_chunk<false, true, true>) : go(k_qgemv_q8_0_chunk<false, false, true>);
    } else {
        if (xf32) *err = single ? go(k_qgemv_q8_0_chunk<true, true, false>) : go(k_qgemv_q8_0_chunk<true, false, false>);
        else *err = single ? go(k_qgemv_q8_0_chunk<false, true, false>) : go(k_qgemv_q8_0_chunk<false, false, false>);
    }
    return true;
}

}  // namespace pmh
