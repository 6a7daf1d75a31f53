// Dequant-fused GEMV for large Q6_K matrices on gfx950: integer dot products over the packed bytes.
//
// y[n] = sum_k W[n,k] * x[k], W the GGUF Q6_K block stream (210 bytes per 256 weights: ql[128], qh[64],
// scales[16] i8, d f16; value d * sc * (q - 32) with q = nibble | two high bits << 4, k_quants.rs:474-496).
//
//  * The activations are converted once per workgroup to fixed point: every 16-element group (one Q6_K
//    sub-block) gets a power-of-two scale that puts its largest magnitude below 2^22, and the 23-bit signed
//    integers are written as three balanced base-256 digits in [-128, 127].  sum q x over a sub-block is then
//    2^e * (65536 dot(q, d2) + 256 dot(q, d1) + dot(q, d0)) with v_dot4_i32_i8 on four stored 6-bit values per
//    dword: integer arithmetic, exact up to the fixed-point resolution of x (22 bits under the group maximum).
//    The stored values are q + 32; the offset is removed with the group's sum of x, computed with the digits.
//  * One workgroup per compute unit; a row is ks = (k / 256) / 8 chunks of eight super-blocks.  Wave (g, h) takes
//    chunk h of the rows of row group g: eight lanes per super-block, lane t owning the two sub-blocks that
//    share the ql bytes 16 (t % 4) .. + 15 of half t / 4, so that a lane's digits (24 registers) never change.
//  * Blocks are only 2-byte aligned, and dword loads at such addresses are slow.  A wave therefore copies the 1680
//    contiguous, 16-byte aligned bytes of its chunk of a row into its own piece of LDS with whole-wave 16-byte loads
//    (up to kDepth rows in flight, every load issued unconditionally so that the number of outstanding loads is known
//    at every wait; rows past the end read the first bytes of W), and each lane takes its pieces out of LDS as
//    aligned dwords which one funnel shift per dword puts into place for the odd super-blocks.  LDS executes a
//    wave's instructions in order, so the copy needs no barrier.
//  * Lane partial sums go to LDS; after a barrier the workgroup adds up each of its rows and stores y.
//
//  * Rows of k / 256 super-blocks that are not whole chunks are handled by the RAGGED variant of the kernel (see there).
//
//  * Rows shorter than a chunk (k < 2048) are handled by the FOLD variant: a wave's task is 8 / (k / 256) whole rows.
//
// Matrices below 12 MiB stay with the bf16 kernel in gemv.hip.
#include "gemv_chunk.hpp"
#include "internal.hpp"

namespace {

using namespace pmh::gemv;

typedef uint32_t u4v __attribute__((ext_vector_type(4)));  // a 16-byte piece

constexpr int kDepth = 6;      // tasks in flight per wave
constexpr int kDepthLong = 8;  // ... for the variant that holds all of a wave's seven or eight tasks at once (DEEP)
constexpr int kPre = 2;    // of which this many are requested before x is converted
constexpr int kPlanes = 3;
constexpr int kChunkBytes = 8 * 210;           // 1680 = 105 pieces of 16 bytes
constexpr int kStageBytes = kChunkBytes + 32;  // a chunk that starts up to 14 bytes into its first piece, plus one dword for the shifted reads

// Activations -> LDS.  A thread converts one 16-element group (one Q6_K sub-block): the group's largest magnitude and
// the sum of its fixed-point values stay inside the thread, and the index arithmetic is done once per group.
// Element e = 256 sb + 128 hh + 32 g + l belongs to lane t = 4 hh + 2 (g & 1) + l / 16 of its super-block
// (slot 8 sb + t), sub-block s = g >> 1 of that lane, dword (l % 16) / 4.
// xd[(plane * 8 + 4 s + dword) * slots + slot]: four digits; xm[slot] = (scale s = 0, scale s = 1, sum s = 0, sum s = 1).
// Slots past the end of a row (its last chunk may hold fewer than eight super-blocks) get zero digits and a zero scale.
template <bool XF32>
__device__ __forceinline__ void stage_x(const void *__restrict__ xg, int slots, int k_quads, int nthreads, uint32_t *xd, float *xm) {
    const int total = slots * 2, k_groups = k_quads >> 2;  // groups, padded to whole chunks; k_groups of them exist
    for (int grp = (int)threadIdx.x; grp < total; grp += nthreads) {
        float v[4][4];
        if (grp >= k_groups) {
#pragma unroll
            for (int q = 0; q < 4; q++) v[q][0] = v[q][1] = v[q][2] = v[q][3] = 0.f;
        } else if (XF32) {
            const float4 *src = reinterpret_cast<const float4 *>(xg) + (size_t)grp * 4;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 f = src[q];
                v[q][0] = f.x, v[q][1] = f.y, v[q][2] = f.z, v[q][3] = f.w;
            }
        } else {
            const uint4 *src = reinterpret_cast<const uint4 *>(xg) + (size_t)grp * 2;
            const uint4 a = src[0], b = src[1];
            const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int q = 0; q < 4; q++) {
                v[q][0] = __builtin_bit_cast(float, w[2 * q] << 16), v[q][1] = __builtin_bit_cast(float, w[2 * q] & 0xFFFF0000u);
                v[q][2] = __builtin_bit_cast(float, w[2 * q + 1] << 16), v[q][3] = __builtin_bit_cast(float, w[2 * q + 1] & 0xFFFF0000u);
            }
        }
        // largest magnitude of the group, as bits (the order of non-negative floats is that of their bits)
        uint32_t mb = 0;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t o = max_magnitude_bits(v[q]);
            mb = o > mb ? o : mb;
        }
        const GroupScale gs = group_scale(mb);
        const int e = grp * 16, sb = e >> 8, r = e & 255;
        const int hh = r >> 7, g = (r >> 5) & 3;
        const int slot = sb * 8 + 4 * hh + 2 * (g & 1) + ((r >> 4) & 1), s = g >> 1;
        int sum = 0;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            uint32_t dig[kPlanes];
            sum += to_digits(v[q], gs, dig);
#pragma unroll
            for (int p = 0; p < kPlanes; p++) xd[(p * 8 + 4 * s + q) * slots + slot] = dig[p];
        }
        xm[slot * 4 + s] = gs.scale;
        xm[slot * 4 + 2 + s] = (float)sum;
    }
}

// One lane's share of a super-block, as it lies in memory.
struct Task {
    uint32_t ql[4], qh[4], sc[2], d;
};

// The two sub-blocks of a lane: A = low nibbles (group ga = tq >> 1), B = high nibbles (group ga + 2).
template <int PLANES>
__device__ __forceinline__ float lane_dot(const Task &t, const uint32_t (&xr)[kPlanes][8], const float4 xm, int sh_a, int sh_b,
                                          int sc_up) {
    const uint32_t(&ql)[4] = t.ql, (&qh)[4] = t.qh;
    int acc_a[PLANES], acc_b[PLANES];
#pragma unroll
    for (int p = 0; p < PLANES; p++) acc_a[p] = acc_b[p] = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const uint32_t va = (ql[k] & 0x0F0F0F0Fu) | ((qh[k] << sh_a) & 0x30303030u);
        const uint32_t vb = ((ql[k] >> 4) & 0x0F0F0F0Fu) | ((qh[k] >> sh_b) & 0x30303030u);
#pragma unroll
        for (int p = 0; p < PLANES; p++) {
            acc_a[p] = sdot4(va, xr[p][k], acc_a[p]);
            acc_b[p] = sdot4(vb, xr[p][4 + k], acc_b[p]);
        }
    }
    float fa = (float)acc_a[PLANES - 1], fb = (float)acc_b[PLANES - 1];
#pragma unroll
    for (int p = PLANES - 2; p >= 0; p--) {
        fa = __builtin_fmaf(fa, 256.0f, (float)acc_a[p]);
        fb = __builtin_fmaf(fb, 256.0f, (float)acc_b[p]);
    }
    fa = __builtin_fmaf(-32.0f, xm.z, fa);  // the stored quants are q + 32
    fb = __builtin_fmaf(-32.0f, xm.w, fb);
    const float sa = (float)((int)(t.sc[0] << sc_up) >> 24), sb = (float)((int)(t.sc[1] << sc_up) >> 24);  // the lane's two i8 scales
    return f16_bits_to_f32(t.d) * __builtin_fmaf(sa * xm.x, fa, (sb * xm.y) * fb);
}

// RAGGED: rows that are not whole chunks (k / 256 not a multiple of 8).  Such rows start at any even address, so a
// chunk starts `delta` bytes into its first 16-byte piece, delta and the odd / even position of the super-blocks
// change from row to row, the last chunk of a row is short, and the last pieces of the tensor must not be passed.
// DEEP: a ring of kDepthLong tasks for waves with seven or eight rows, all of which are then in flight at once (measured
// against the ring of six, same machine: 4096 x 14336 13.98 -> 13.24 us, 14336 x 4096 12.08 -> 11.72, 8192 x 8192 14.1 ->
// 13.4; waves with more rows, or fewer, are better off with six: 18944 x 3584 15.3 against 15.7, 4096 x 4096 6.15 against 6.25).
// FOLD (with RAGGED): rows of fold_spr < 8 super-blocks.  Rows follow one another in memory, so rpc = 8 / fold_spr of them
// are one task: the kernel sees a matrix of ceil(n_real / rpc) rows of spr = rpc * fold_spr super-blocks, every lane
// group takes the activations of its super-block's place in its own row, and the lane sums are added per row inside
// the wave and stored straight to y (a task's rows past the end of the matrix are loaded from clamped addresses and
// dropped).
template <bool XF32, bool SINGLE, bool RAGGED, bool DEEP = false, bool FOLD = false>
__global__ __launch_bounds__(1024) void k_qgemv_q6k_chunk(const uint8_t *__restrict__ W, const void *__restrict__ xg,
                                                           float *__restrict__ y, int n_rows, int spr, int rows_per_wg,
                                                           int rows_per_wave, int n_nominal, int nthreads,
                                                           uint32_t w_last, int fold_spr, int n_real) {
    static_assert(!FOLD || RAGGED, "folded rows start at any even address");
    constexpr int kDepth = DEEP ? kDepthLong : ::kDepth;
    extern __shared__ uint4 smem[];
    const int ks = (spr + 7) >> 3;
    const int slots = ks * 64;
    const int n_waves = nthreads >> 6;
    const int wave_id = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    uint32_t *stage = reinterpret_cast<uint32_t *>(smem) + wave_id * (kStageBytes / 4);  // this wave's row chunk
    uint32_t *xd = reinterpret_cast<uint32_t *>(smem) + n_waves * (kStageBytes / 4);     // [kPlanes * 8][slots]
    float *xm = reinterpret_cast<float *>(xd + kPlanes * 8 * slots);  // [slots][4]
    float *part = xm + 4 * slots;                              // [group][n_nominal][ks]
    const int lane = threadIdx.x & 63;
    const int t = lane & 7, hh = t >> 2, tq = t & 3;
    const int wave = wave_id;
    const int h = wave % ks, g = wave / ks;
    const int wg_r0 = blockIdx.x * rows_per_wg;
    const int wg_r1 = wg_r0 + rows_per_wg < n_rows ? wg_r0 + rows_per_wg : n_rows;
    const int wave_r0 = wg_r0 + g * rows_per_wave;
    const int wave_r1 = wave_r0 + rows_per_wave < wg_r1 ? wave_r0 + rows_per_wave : wg_r1;
    const int nt_wave = wave_r1 > wave_r0 ? wave_r1 - wave_r0 : 0;  // real tasks of this wave (wave-uniform)

    const uint32_t rowbytes = (uint32_t)spr * 210u;
    // a wave's 105 pieces of a row chunk (106 when the chunk may start inside a piece): lane l takes piece l, the first
    // 41 (42) lanes also piece 64 + l
    const uint32_t off_a = (uint32_t)h * kChunkBytes + 16u * (uint32_t)lane;
    constexpr int kTail = RAGGED ? 42 : 41;  // lanes that take a second piece
    const uint32_t off_b = (uint32_t)h * kChunkBytes + 1024u + 16u * (uint32_t)(lane < kTail ? lane : kTail - 1);
    auto issue = [&](int i, u4v &a, u4v &b) {
        const bool real = i < nt_wave;  // wave-uniform
        const uint32_t ro = real ? (uint32_t)(wave_r0 + i) * rowbytes : 0u;
        uint32_t pa = ro + (real ? off_a : 0u), pb = ro + (real ? off_b : 0u);
        if (RAGGED) {  // from the 16-byte boundary below the chunk, never past the piece that holds the tensor's last byte
            pa = (pa & ~15u) < w_last ? (pa & ~15u) : w_last;
            pb = (pb & ~15u) < w_last ? (pb & ~15u) : w_last;
        }
        a = *reinterpret_cast<const u4v *>(W + pa);
        b = *reinterpret_cast<const u4v *>(W + pb);
    };

    u4v ra[kDepth], rb[kDepth];
#pragma unroll
    for (int i = 0; i < kPre; i++) issue(i, ra[i], rb[i]);
    stage_x<XF32>(xg, slots, (FOLD ? fold_spr : spr) * 64, nthreads, xd, xm);
    __syncthreads();

    const int row_lanes = FOLD ? fold_spr * 8 : 64;   // lanes that share a row of the matrix
    const int row_in_task = FOLD ? lane / row_lanes : 0;
    const int slot = FOLD ? lane - row_in_task * row_lanes : h * 64 + lane;
    uint32_t xr[kPlanes][8];
#pragma unroll
    for (int p = 0; p < kPlanes; p++)
#pragma unroll
        for (int k = 0; k < 8; k++) xr[p][k] = xd[(p * 8 + k) * slots + slot];
    const float4 xmr = *reinterpret_cast<const float4 *>(xm + 4 * slot);
    const int ga = tq >> 1;
    const int sh_a = 4 - 2 * ga, sh_b = 2 * ga;      // group ga: bits 2 ga of a qh byte -> bits 4..5; group ga + 2: bits 4 + 2 ga
    const int sc_up = 24 - 8 * (2 * ga + (tq & 1));  // scale bytes 2 g + l / 16 of the half (word x for A, word y for B): shift to the top byte

    // Super-block sb of the chunk starts at byte delta + 210 sb of the staged pieces (delta = 0 unless RAGGED): on a dword
    // boundary or two bytes past one.  Every piece is read from the dword boundary at or below it and shifted down by
    // `mis` bytes.
    const uint32_t sb_byte = (uint32_t)(lane >> 3) * 210u;
    const uint32_t c_ql = 16u * hh + 4u * tq, c_qh = 32u + 8u * hh + 4u * (tq & 1), c_sc = 48u + 2u * hh, c_d = 52u;  // dwords into the block
    const bool lane_valid = !RAGGED || h * 8 + (lane >> 3) < spr;  // the last chunk of a ragged row is short

    float *pp = part + (size_t)(g * n_nominal) * ks + h;
    auto consume = [&](int i, const u4v a, const u4v b) {
        if (i < nt_wave) {  // wave-uniform
            u4v *st4 = reinterpret_cast<u4v *>(stage);
            st4[lane] = a;
            if (lane < kTail) st4[64 + lane] = b;
            // LDS executes a wave's instructions in order: the reads below see the writes above, and the next row's
            // writes come after these reads
            const uint32_t delta = RAGGED ? ((uint32_t)(wave_r0 + i) * rowbytes) & 15u : 0u;  // wave-uniform
            const uint32_t t0 = delta + sb_byte, mis = t0 & 2u, sh = 8u * mis;
            const uint32_t *blk = stage + ((t0 - mis) >> 2);
            const uint32_t *p_ql = blk + c_ql, *p_qh = blk + c_qh, *p_sc = blk + c_sc;
            uint32_t wl[5], wh[5], ws[3];
#pragma unroll
            for (int k = 0; k < 5; k++) wl[k] = p_ql[k], wh[k] = p_qh[k];
#pragma unroll
            for (int k = 0; k < 3; k++) ws[k] = p_sc[k];
            Task tk;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                tk.ql[k] = __builtin_amdgcn_alignbit(wl[k + 1], wl[k], sh);
                tk.qh[k] = __builtin_amdgcn_alignbit(wh[k + 1], wh[k], sh);
            }
            tk.sc[0] = __builtin_amdgcn_alignbit(ws[1], ws[0], sh);
            tk.sc[1] = __builtin_amdgcn_alignbit(ws[2], ws[1], sh);
            tk.d = (blk[c_d] >> sh) & 0xFFFFu;
            const float val = lane_dot<kPlanes>(tk, xr, xmr, sh_a, sh_b, sc_up);
            if (FOLD) {
                float tot;
                if ((fold_spr & (fold_spr - 1)) == 0) {
                    tot = team_sum_rt(val, row_lanes);
                } else {  // 3, 5, 6 or 7 lane groups: the group totals, then the row's groups one by one
                    const float grp = team_sum<8>(val);
                    tot = grp;
                    for (int j = 1; j < fold_spr; j++) tot += __shfl(grp, (lane + 8 * j) & 63);
                }
                const int row = (wave_r0 + i) * (spr / fold_spr) + row_in_task;
                if (lane_valid && lane == row_in_task * row_lanes && row < n_real) y[row] = tot;
            } else {
                store_chunk_sum(pp + (size_t)i * ks, lane_valid ? val : 0.0f, lane);
            }
        }
    };

    int issued = kPre;
#pragma unroll
    for (int i = 0; i < kDepth; i++) {
        consume(i, ra[i], rb[i]);
        const int upto = SINGLE ? (kPre + 2 * (i + 1) < kDepth ? kPre + 2 * (i + 1) : kDepth)
                                : (kPre + 2 * (i + 1) < kDepth + i + 1 ? kPre + 2 * (i + 1) : kDepth + i + 1);
#pragma unroll
        for (; issued < upto; issued++) issue(issued, ra[issued % kDepth], rb[issued % kDepth]);
    }
    if (!SINGLE) {
        int base = kDepth;
        for (; base + kDepth < n_nominal; base += kDepth) {
#pragma unroll
            for (int i = 0; i < kDepth; i++) {
                consume(base + i, ra[i], rb[i]);
                issue(base + kDepth + i, ra[i], rb[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < kDepth; i++) consume(base + i, ra[i], rb[i]);
    }
    if (FOLD) return;
    __syncthreads();

    reduce_rows(part, ks, wg_r0, wg_r1 - wg_r0, rows_per_wave, n_nominal, nthreads, y);
}

}  // namespace

namespace pmh {

// Runs the chunk kernel when the shape suits it and returns true; otherwise leaves *err untouched and returns
// false (the caller falls back to the general Q6_K kernel).  Preconditions as for launch_qgemv.
bool try_launch_qgemv_q6k_chunk(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y,
                                hipStream_t s, hipError_t *err) {
    const int spr_real = (int)(k / 256);
    // Short rows: 8 / spr_real of them are one row of the kernel.  Rows of 5 or 6 super-blocks would leave three or two
    // of a wave's eight lane groups idle and are faster in the general kernel (128256 x 1536: 40.9 against 48.9 us), as are
    // matrices below 24 MiB (16000 x 1024: 6.1 against 7.0 us; 32000 x 1024: 10.0 against 9.6).
    const bool fold = spr_real < 8;
    if (fold && (spr_real == 5 || spr_real == 6 || (uint64_t)n * (uint64_t)spr_real * 210u < (24ull << 20))) return false;
    const int rpc = fold ? 8 / spr_real : 1;
    const int spr = spr_real * rpc;
    const int64_t n_real = n;
    if (fold) n = (n + rpc - 1) / rpc;
    const bool ragged = fold || spr % 8 != 0;
    const int ks = (spr + 7) / 8;
    const uint64_t w_bytes = (uint64_t)n_real * (uint64_t)spr_real * 210u;
    if (ks > 16 || w_bytes >= (1ull << 32)) return false;
    if (w_bytes < (12ull << 20)) return false;  // measured crossover with the general kernel
    const size_t slots = (size_t)ks * 64;
    const size_t lds_x = slots * 4 * (kPlanes * 8) + slots * 16;
    const gemv::ChunkPlan plan = gemv::plan_chunks(n, ks, kStageBytes, lds_x);
    const int64_t n_wg = plan.n_wg, rows_per_wg = plan.rows_per_wg, rows_per_wave = plan.rows_per_wave, n_nominal = plan.n_nominal,
                  threads = plan.threads;
    const size_t lds = plan.lds;
    if (lds > 128 * 1024) return false;
    const bool deep = n_nominal > kDepth && n_nominal <= kDepthLong;
    const bool single = n_nominal <= kDepth;
    const bool xf32 = x_dtype == kDtypeF32;
    auto go = [&](auto kern) {
        if (lds > 64 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kern, dim3((unsigned)n_wg), dim3((unsigned)threads), lds, s, w, x, y, (int)n, spr, (int)rows_per_wg,
                           (int)rows_per_wave, (int)n_nominal, (int)threads, (uint32_t)((w_bytes - 1) & ~(uint64_t)15), spr_real, (int)n_real);
        return hipGetLastError();
    };
    if (fold) {
        if (deep) *err = xf32 ? go(k_qgemv_q6k_chunk<true, true, true, true, true>) : go(k_qgemv_q6k_chunk<false, true, true, true, true>);
        else if (xf32) *err = single ? go(k_qgemv_q6k_chunk<true, true, true, false, true>) : go(k_qgemv_q6k_chunk<true, false, true, false, true>);
        else *err = single ? go(k_qgemv_q6k_chunk<false, true, true, false, true>) : go(k_qgemv_q6k_chunk<false, false, true, false, true>);
    } else if (deep) {  // all tasks of a wave fit the longer ring: the SINGLE form of it
        if (ragged) *err = xf32 ? go(k_qgemv_q6k_chunk<true, true, true, true>) : go(k_qgemv_q6k_chunk<false, true, true, true>);
        else *err = xf32 ? go(k_qgemv_q6k_chunk<true, true, false, true>) : go(k_qgemv_q6k_chunk<false, true, false, true>);
    } else if (ragged) {
        if (xf32) *err = single ? go(k_qgemv_q6k_chunk<true, true, true>) : go(k_qgemv_q6k_chunk<true, false, true>);
        else *err = single ? go(k_qgemv_q6k_chunk<false, true, true>) : go(k_qgemv_q6k_chunk<false, false, true>);
    } else {
        if (xf32) *err = single ? go(k_qgemv_q6k_chunk<true, true, false>) : go(k_qgemv_q6k_chunk<true, false, false>);
        else *err = single ? go(k_qgemv_q6k_chunk<false, true, false>) : go(k_qgemv_q6k_chunk<false, false, false>);
    }
    return true;
}

}  // namespace pmh
