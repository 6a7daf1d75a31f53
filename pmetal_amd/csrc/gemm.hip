// Dequant-fused Q4_K, Q5_K, Q6_K and Q8_0 GEMM  Y[m,n] = sum_k X[m,k] * W[n,k]  on the gfx950 matrix cores, every wave
// owning its weight rows.  The text below describes Q4_K (Q5_K is the same kernel with the fifth bit of every quant
// taken from the block's qh bytes: FMT = 1); the Q6_K and Q8_0 kernels further down note their differences.
//
// W is the packed GGUF stream [n, k] of 144-byte super-blocks; a weight's value is what the reference's
// dequantize_q4k yields (crates/pmetal-gguf/src/k_quants.rs:358-404; element order REF or GGML as for the
// GEMV).  The reference has no fused kernel (it dequantizes on the CPU at load,
// crates/pmetal-models/src/weight_format.rs:299-303, and multiplies densely); this kernel is checked against
// exactly that, dequantize-then-matmul, to 1e-3.
//
// A wave owns 32 weight rows and dequantizes them straight into MFMA operand registers (no shared weight tile
// in LDS, no LDS writes by the waves at all); only the activations are shared by the waves of a workgroup.  A
// launch is cut along N, M and, for short activation batches, K into enough workgroups to fill the machine.
// The arithmetic is exact up to the fp32 accumulation: rounding d*sc*q - dmin*m to f16 or bf16 leaves a relative
// error per product that fails the element-wise 1e-3 gate on small outputs, so the MFMA multiplies integer tiles
// sc * q in f16 (<= 63 * 15 = 945; f16 holds integers to 2048) with activations scaled per row by a power of two
// into the f16 range (bf16 activations are exact there), the per-super-block factor d is applied to the fp32
// partial sums, and the min term is a K = 32 MFMA product of exact head + tail splits.
//
// Data movement uses direct global -> LDS loads only (no staging registers, no ds_write):
//   * activations: a pre-pass writes 16-byte items (8 f16) in the order the MFMA wants them,
//     xs[(2 sb + h) * 18 + grp][Mp], per half super-block h 16 operand groups (k-step t, lane half g) and two
//     groups of sub-block sums; a workgroup copies the 18 x BM items of a half super-block into one of two
//     LDS stages while it computes on the other (one barrier per half super-block);
//   * weights: each wave copies the 64 quant bytes per row of a half super-block (coalesced: four lanes per
//     row) two half super-blocks ahead, and the 16-byte headers one super-block ahead, into its private LDS
//     region; then every lane (row n = lane % 32, half g = lane / 32) reads back the 32 bytes it multiplies:
//     dword t of them holds the eight 4-bit quants of MFMA k-step t.  Which k they are is a property of the
//     element order, matched by the pre-pass:
//         GGML: k = 64 (2h + g) + 4t + e (low nibbles, sub-block 4h+2g), + 32 (high nibbles, sub-block 4h+2g+1)
//         REF : k = 32 (4h + 2g + t/4) + 4 (t%4) + e (low), + 16 (high), both sub-block 4h + 2g + t/4
// With a K split (grid.z > 1) the workgroups write fp32 partial tiles and a small kernel adds them in a fixed
// order, so the result does not depend on scheduling.
//
// What bounds it: every matrix instruction reads its 1 KiB activation fragment from LDS (a wave cannot reuse a
// fragment for a second group of weight rows without doubling the dequantization work per matrix instruction,
// which measured slower, as did one wave per SIMD with a 128 x 64 tile), so a 128-row workgroup is bound by the
// LDS read rate at about 60 % of the matrix peak.
#include "internal.hpp"

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kGroups = 18;    // 16-byte items per activation row and half super-block
constexpr int kBlockBytes = 144;
// FMT 0: Q4_K (144 bytes: d, dmin, 12 scale bytes, 128 quant bytes); FMT 1: Q5_K (176 bytes: the same header, then 32 bytes
// qh with the fifth bits, then the 128 quant bytes; crates/pmetal-gguf/src/k_quants.rs:407-462)
template <int FMT>
struct BlockFmt {
    static constexpr int kBytes = FMT ? 176 : 144, kQs = FMT ? 48 : 16;
};

#define PMH_GPTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define PMH_LPTR(p) ((__attribute__((address_space(3))) void *)(p))

// 16 bytes per lane from global memory to LDS: lane l lands at dst + 16 l (dst is wave-uniform).
__device__ __forceinline__ void dma16(const void *src, uint4 *dst) {
    __builtin_amdgcn_global_load_lds(PMH_GPTR(src), PMH_LPTR(dst), 16, 0, 0);
}

// Workgroup barrier that leaves the newest `keep` vector-memory requests in flight.  (__syncthreads() carries a
// release fence, which waits for every direct-to-LDS copy.)  The copies that the other waves will read are older
// than those, and this wave's own LDS reads have returned (lgkmcnt(0)) before another wave may refill a stage.
template <int KEEP>
__device__ __forceinline__ void barrier_keep() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0070 | KEEP);  // vmcnt(KEEP) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}
__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return __builtin_bit_cast(float, h << 16); }

// ------------------------------------------------------------------------------------------------
// Pre-pass: a workgroup takes R activation rows m < Mp (R = 1: 512 threads on one row, for few rows; R = 4: 256 threads
// per row with the row index fastest across lanes, so that four lanes write 64 contiguous bytes of every item row).  rowscale[m] = 2^e with the row maximum * 2^-e in
// [2^9, 2^10) (bf16 activations are then exact in f16 and block sums stay below 2^15); rows >= M are zero.
// One thread per operand item: chunk u = 64 elements = sub-blocks 2u, 2u+1 (u = 4 sb + 2 h + g), k-step t.
// ORDER 0 / 1: Q4_K element orders REF / GGML (1 is also Q5_K's GGML order); ORDER 2: the Q6_K layout, ORDER 3: the
// natural order (Q8_0), both without block sums; ORDER 4: Q5_K's REF order, whose sub-block j holds its 32 elements as
// consecutive nibbles of 16 bytes, so k-step t of a chunk is elements 8 t .. 8 t + 7, the even ones (low nibbles) first;
// ORDER 5: Q2_K / Q3_K, whose qs byte 32 h + l holds elements 128 h + l + 32 s at bit 2 s: k-step t of lane half g is dword
// t / 2 of the bytes 16 g .. 16 g + 15 of a half with the shifts s = 2 (t % 2) (first run) and 2 (t % 2) + 1 (second run), and
// the sums are those of the four 16-element sub-blocks 4 (t % 2) + 2 (run) + g of the half: 20 items per half.
// ------------------------------------------------------------------------------------------------
template <bool XF32, int ORDER, int R>
__global__ __launch_bounds__(R == 1 ? 512 : 1024) void k_prep_rw(const void *__restrict__ xg, int64_t k, int M, int Mp,
                                                                  float *__restrict__ rowscale, uint4 *__restrict__ xs) {
    constexpr int NT = R == 1 ? 512 : 1024, JN = NT / R, NWV = NT / 64;
    constexpr int kGroups = ORDER == 5 ? 20 : 18;  // items per half super-block and row (shadows the Q4_K constant)
    const int tid = threadIdx.x, lane = tid & 63, r = tid % R, j = tid / R;
    const int m = blockIdx.x * R + r;
    const bool live = m < M;
    __shared__ float red[NWV][R];
    float amax = 0.0f;
    if (live) {
        if (XF32) {
            const float4 *row = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(xg) + (int64_t)m * k);
            for (int64_t i = j; i < k / 4; i += JN) {
                const float4 v = row[i];
                amax = __builtin_fmaxf(__builtin_fmaxf(amax, __builtin_fmaxf(__builtin_fabsf(v.x), __builtin_fabsf(v.y))),
                                       __builtin_fmaxf(__builtin_fabsf(v.z), __builtin_fabsf(v.w)));
            }
        } else {
            const uint4 *row = reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(xg) + (int64_t)m * k);
            for (int64_t i = j; i < k / 8; i += JN) {
                const uint4 v = row[i];
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int q = 0; q < 4; q++)
                    amax = __builtin_fmaxf(amax, __builtin_fmaxf(__builtin_fabsf(bf16_to_f32(w[q] & 0xFFFFu)),
                                                                 __builtin_fabsf(bf16_to_f32(w[q] >> 16))));
            }
        }
    }
    for (int off = 32; off >= R; off >>= 1) amax = __builtin_fmaxf(amax, __shfl_xor(amax, off));
    if (lane < R) red[tid >> 6][lane] = amax;
    __syncthreads();
    amax = red[0][r];
#pragma unroll
    for (int w = 1; w < NWV; w++) amax = __builtin_fmaxf(amax, red[w][r]);
    const int eb = (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xFFu);  // amax in [2^(eb-127), 2^(eb-126))
    int e = eb - 126 - 10;
    e = e < -126 ? -126 : (e > 126 ? 126 : e);
    if (eb == 255) e = 0;  // inf / NaN: let them through
    const float up = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
    if (j == 0) rowscale[m] = up;
    const float down = live ? 1.0f / up : 0.0f;  // exact: a power of two

    for (int64_t q = j; q < k / 8; q += JN) {
        // the item's two runs of four elements (lo, hi), its half super-block and its operand group
        int64_t lo, hi, half;
        int t, g;
        if (ORDER == 2 || ORDER == 3) {  // half = 128 elements, 16 items
            half = q >> 4;
            t = (int)(q & 15) >> 1, g = (int)q & 1;
            if (ORDER == 2) {  // Q6_K: low nibbles at 32 g + 4 t, high nibbles 64 further
                lo = 128 * half + 32 * g + 4 * t;
                hi = lo + 64;
            } else {  // Q8_0: the natural order, 8 consecutive elements
                lo = 128 * half + 16 * t + 8 * g;
                hi = lo + 4;
            }
        } else {
            const int64_t u = q >> 3;
            t = (int)(q & 7), g = (int)u & 1;
            half = u >> 1;
            lo = ORDER == 5   ? 128 * half + 64 * (t & 1) + 16 * g + 4 * (t >> 1)
                 : ORDER == 4 ? 64 * u + 8 * t
                              : (ORDER == 0 ? 64 * u + 32 * (t >> 2) + 4 * (t & 3) : 64 * u + 4 * t);
            hi = lo + (ORDER == 4 ? 4 : (ORDER == 0 ? 16 : 32));
        }
        float v[8];
        if (!live) {
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = 0.0f;
        } else if (XF32) {
            const float *row = reinterpret_cast<const float *>(xg) + (int64_t)m * k;
            const float4 a = *reinterpret_cast<const float4 *>(row + lo), b = *reinterpret_cast<const float4 *>(row + hi);
            v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
        } else {
            const uint16_t *row = reinterpret_cast<const uint16_t *>(xg) + (int64_t)m * k;
            const uint2 a = *reinterpret_cast<const uint2 *>(row + lo), b = *reinterpret_cast<const uint2 *>(row + hi);
            v[0] = bf16_to_f32(a.x & 0xFFFFu), v[1] = bf16_to_f32(a.x >> 16), v[2] = bf16_to_f32(a.y & 0xFFFFu), v[3] = bf16_to_f32(a.y >> 16);
            v[4] = bf16_to_f32(b.x & 0xFFFFu), v[5] = bf16_to_f32(b.x >> 16), v[6] = bf16_to_f32(b.y & 0xFFFFu), v[7] = bf16_to_f32(b.y >> 16);
        }
        if (ORDER == 4) {  // eight consecutive elements: the even ones, then the odd ones
            const float e[8] = {v[0], v[2], v[4], v[6], v[1], v[3], v[5], v[7]};
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = e[i];
        }
        half8_t h;
        float slo = 0.0f, shi = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            h[i] = (_Float16)(v[i] * down);
            if (i < 4) slo += (float)h[i];
            else shi += (float)h[i];
        }
        const size_t base = (size_t)(half * kGroups) * Mp + m;
        xs[base + (size_t)(t * 2 + g) * Mp] = __builtin_bit_cast(uint4, h);
        if (ORDER == 2 || ORDER == 3) continue;  // Q6_K and Q8_0 have no min term: no block sums
        // sums of the two sub-blocks of the chunk over its 8 k-steps (8 lanes, R apart)
        float s0, s1;
        if (ORDER == 5) {
            // the first runs of the k-steps of one parity are one 16-element sub-block, their second runs another:
            // k-step 0 ends up with the sums for t % 2 == 0 (item 16 + g), k-step 1 with those for t % 2 == 1 (item 18 + g)
            slo += __shfl_xor(slo, 2 * R), shi += __shfl_xor(shi, 2 * R);
            slo += __shfl_xor(slo, 4 * R), shi += __shfl_xor(shi, 4 * R);
            if (t < 2) {
                const _Float16 h0 = (_Float16)slo, h1 = (_Float16)shi;
                const _Float16 l0 = (_Float16)(slo - (float)h0), l1 = (_Float16)(shi - (float)h1);
                const half8_t item = {h0, l0, h0, l0, h1, l1, h1, l1};
                xs[base + (size_t)(16 + 2 * t + g) * Mp] = __builtin_bit_cast(uint4, item);
            }
            continue;
        }
        if (ORDER == 0 || ORDER == 4) {  // sub-block 2u: k-steps 0..3 (low and high nibbles), 2u+1: k-steps 4..7
            float s = slo + shi;
            s += __shfl_xor(s, R);
            s += __shfl_xor(s, 2 * R);
            s0 = s;
            s1 = __shfl_down(s, 4 * R);
        } else {  // sub-block 2u: the low nibbles of all k-steps, 2u+1: the high nibbles
            slo += __shfl_xor(slo, R), shi += __shfl_xor(shi, R);
            slo += __shfl_xor(slo, 2 * R), shi += __shfl_xor(shi, 2 * R);
            slo += __shfl_xor(slo, 4 * R), shi += __shfl_xor(shi, 4 * R);
            s0 = slo, s1 = shi;
        }
        if (t == 0) {  // exact head + tail split of each sum; item (H0, L0, H0, L0, H1, L1, H1, L1)
            const _Float16 h0 = (_Float16)s0, h1 = (_Float16)s1;
            const _Float16 l0 = (_Float16)(s0 - (float)h0), l1 = (_Float16)(s1 - (float)h1);
            const half8_t item = {h0, l0, h0, l0, h1, l1, h1, l1};
            xs[base + (size_t)(16 + g) * Mp] = __builtin_bit_cast(uint4, item);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// main kernel
// ------------------------------------------------------------------------------------------------
// Epilogue shared by the kernels below: a workgroup's BM x 32 NW tile of Y (256 columns for 8 waves) goes through LDS so that it leaves as
// whole rows (16 bytes per lane, 512 bytes or 1 KiB contiguous per row) instead of 2- or 4-byte pieces per lane.
// Every wave holds 32 columns (lane % 32) of all BM rows: C layout of v_mfma_f32_32x32x*: rows
// 8 (r / 4) + 4 (lane / 32) + r % 4 of block i.  mode 0: y f32, 1: y bf16 (both scaled by rowscale), 2: fp32
// partial tile of split z.  Must be reached by all threads of the workgroup, with no copies into LDS in flight.
constexpr int kTilePad = 16;  // bytes added to an LDS row: rows 4 apart (the two lane halves) then lie in different banks
template <int MB, int NW = 8>
constexpr size_t tile_lds_bytes() {
    return (size_t)32 * MB * (32 * NW * 4 + kTilePad);
}

__device__ __forceinline__ uint32_t bf16_rne_bits(const float v) {
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    return ((u & 0x7FFFFFFFu) > 0x7F800000u) ? ((u >> 16) | 0x40u) : ((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

template <int MB, int NW = 8>
__device__ __forceinline__ void store_tile(const float16_t (&acc)[MB], uint4 *smem, const int wave, const int col, const int g,
                                           const int m0, const int n0, const int M, const int N, const int Mp,
                                           const float *__restrict__ rowscale, void *__restrict__ yg,
                                           float *__restrict__ partial, const int mode, const int z) {
    constexpr int BM = 32 * MB;
    constexpr int kCols = 32 * NW;                    // weight rows of the workgroup = columns of its tile of Y
    constexpr int kRowStride = kCols * 4 + kTilePad;  // the LDS tile is fp32, not yet scaled
    uint8_t *tile = reinterpret_cast<uint8_t *>(smem);
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int ml = 32 * i + 8 * (r >> 2) + 4 * g + (r & 3);
            *reinterpret_cast<float *>(tile + ml * kRowStride + (32 * wave + col) * 4) = acc[i][r];
        }
    __syncthreads();
    // one 16-byte store per trip and lane: 4 (fp32) or 8 (bf16) consecutive outputs of one row
    const int per = mode == 1 ? 8 : 4, chunks = kCols / per, esize = mode == 1 ? 2 : 4;
    uint8_t *out = mode == 2 ? reinterpret_cast<uint8_t *>(partial) + (size_t)z * Mp * N * 4 : reinterpret_cast<uint8_t *>(yg);
    const bool rows_aligned = ((size_t)N * esize) % 16 == 0;
    for (int idx = threadIdx.x; idx < BM * chunks; idx += blockDim.x) {
        const int ml = idx / chunks, c = idx % chunks;
        const int m = m0 + ml, n = n0 + c * per;
        if (m >= M || n >= N) continue;
        const float scale = mode == 2 ? 1.0f : rowscale[m];
        const float4 *src = reinterpret_cast<const float4 *>(tile + ml * kRowStride + c * per * 4);
        float v[8];
        const float4 lo = src[0];
        v[0] = lo.x * scale, v[1] = lo.y * scale, v[2] = lo.z * scale, v[3] = lo.w * scale;
        uint4 pack;
        if (mode == 1) {
            const float4 hi = src[1];
            v[4] = hi.x * scale, v[5] = hi.y * scale, v[6] = hi.z * scale, v[7] = hi.w * scale;
            pack = make_uint4(bf16_rne_bits(v[0]) | (bf16_rne_bits(v[1]) << 16), bf16_rne_bits(v[2]) | (bf16_rne_bits(v[3]) << 16),
                              bf16_rne_bits(v[4]) | (bf16_rne_bits(v[5]) << 16), bf16_rne_bits(v[6]) | (bf16_rne_bits(v[7]) << 16));
        } else {
            pack = make_uint4(__builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[1]),
                              __builtin_bit_cast(uint32_t, v[2]), __builtin_bit_cast(uint32_t, v[3]));
        }
        uint8_t *dst = out + ((size_t)m * N + n) * esize;
        if (rows_aligned && n + per <= N) {
            // Y is not read again by this launch: a streaming store keeps it from pushing the activation items and the
            // other row blocks' weights out of the caches (a partial tile is read back by the reduction: an ordinary store)
            if (mode == 2) *reinterpret_cast<uint4 *>(dst) = pack;
            else __builtin_nontemporal_store(u32x4{pack.x, pack.y, pack.z, pack.w}, reinterpret_cast<u32x4 *>(dst));
        } else {
            for (int e = 0; e < per && n + e < N; e++) {
                if (mode == 1) reinterpret_cast<uint16_t *>(dst)[e] = (uint16_t)bf16_rne_bits(v[e]);
                else reinterpret_cast<float *>(dst)[e] = v[e];
            }
        }
    }
}

// per-thread constants of the copy roles; a wave owns NR groups of 32 weight rows
template <int MB, int NR, int NW>
struct Lane {
    static constexpr int BM = 32 * MB, kThreads = 64 * NW;
    static constexpr int kARounds = (kGroups * BM + kThreads - 1) / kThreads;
    int wave, col, g;
    uint32_t q_off[NR][2];     // byte offset of this lane's quant piece of round r from the workgroup's first row
    uint32_t h_off[NR];        // ... of this lane's header
    uint32_t qh_off[NR];       // ... of this lane's piece of the fifth bits (Q5_K: row lane / 2, piece lane % 2)
    uint32_t a_off[kARounds];  // item offset of this lane's activation item of round i from (group 0, row m0)
};

template <int MB, int NR>
struct Acc {
    float16_t acc[NR][MB], part[NR][MB];
    u32x4 hdr[NR];  // headers of the current super-block: d | dmin << 16, then the 12 scale bytes
    uint32_t qh[NR][8];  // Q5_K: the 32 qh bytes of the current super-block of this lane's row
};

// 8 quants of one dword (low nibbles, then high nibbles) times their integer scales -> 8 exact f16 values:
// 0x6400 | q is the f16 1024 + q, and (1024 + q) * sc - 1024 * sc is exact in a packed f16 fma.  Built in four
// pieces, so that the pieces can be placed between matrix instructions.  k-step t selects the
// scales: GGML order multiplies the low nibbles by the first and the high nibbles by the second sub-block scale,
// REF order both by the scale of sub-block t / 4.
struct Dq {
    uint32_t lo, hi;
    half2_t r[4];
    __device__ __forceinline__ half8_t value() const { return half8_t{r[0][0], r[0][1], r[1][0], r[1][1], r[2][0], r[2][1], r[3][0], r[3][1]}; }
};
// Q5_K (FMT 1): bit 4 of every quant comes from `hq`.  GGML order: hq is the qh dword of the same four bytes, shifted so
// that bits 0 and 1 of each of its bytes belong to the low and the high nibble of the quant byte at the same place.  REF
// order: hq is the one qh byte whose bits 0..7 belong to the eight consecutive elements of this k-step (even elements =
// low nibbles): a multiplication spreads bits 0, 2, 4, 6 to bit 4 of bytes 0..3 (bit 2 i lands on 2 i + 4 + 6 i; the
// other partial products meet at most in pairs on bits that the mask drops, and their carries stop there).  Values up to
// 31 times scales up to 63 stay below 2048: exact in f16 like Q4_K's.
template <int ORDER, int FMT = 0>
__device__ __forceinline__ void dq_chunk(const int c, const int t, const uint32_t w, const half2_t (&sc2)[2], const half2_t (&off2)[2], Dq &d,
                                         const uint32_t hq = 0) {
    const int lo_s = ORDER == 0 ? (t >> 2) : 0, hi_s = ORDER == 0 ? (t >> 2) : 1;
    if (FMT == 1 && c == 0) {
        const uint32_t bit = ORDER == 0 ? ((hq & 0x55u) * 0x00410410u) & 0x10101010u : (hq & 0x01010101u) << 4;
        d.lo = (w & 0x0F0F0F0Fu) | bit;
        d.r[0] = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, d.lo, 0x04010400u)), sc2[lo_s], off2[lo_s]);
    } else if (FMT == 1 && c == 1) {
        d.r[1] = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, d.lo, 0x04030402u)), sc2[lo_s], off2[lo_s]);
        const uint32_t bit = ORDER == 0 ? (((hq >> 1) & 0x55u) * 0x00410410u) & 0x10101010u : (hq & 0x02020202u) << 3;
        d.hi = ((w >> 4) & 0x0F0F0F0Fu) | bit;
    } else if (c == 0) {
        d.lo = w & 0x0F0F0F0Fu;
        d.r[0] = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, d.lo, 0x04010400u)), sc2[lo_s], off2[lo_s]);
    } else if (c == 1) {
        d.r[1] = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, d.lo, 0x04030402u)), sc2[lo_s], off2[lo_s]);
        d.hi = (w >> 4) & 0x0F0F0F0Fu;
    } else if (c == 2) {
        d.r[2] = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, d.hi, 0x04010400u)), sc2[hi_s], off2[hi_s]);
    } else {
        d.r[3] = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, d.hi, 0x04030402u)), sc2[hi_s], off2[hi_s]);
    }
}

// -(dmin * mn) split exactly into an f16 head and tail (dmin has 11 significant bits, mn 6).
__device__ __forceinline__ void neg_min_split(const float dmin, const uint32_t mn, _Float16 &h, _Float16 &l) {
    const float p = -(dmin * (float)mn);  // exact in fp32
    h = (_Float16)p;
    l = (_Float16)(p - (float)h);
}

// One half super-block H of one wave.  The restrict qualifiers say what the copies in flight cannot touch:
// operand reads from a_cur / q_cur need not wait for the direct loads into a_nxt / q_nxt / hb.
//   a_cur / a_nxt: activation stages (18 x BM items)      q_cur / q_nxt: this wave's quant pieces (NR x 128 items)
//   hb: this wave's headers (NR x 64 items)       qhs: Q5_K, this wave's fifth bits (NR x 32 rows x 2 items)
//   xs_nxt: item (group 0, row m0) of the next half super-block    wq_nxt / wh_nxt: first row of the workgroup at
//   the next half's quant bytes / the next super-block's header
template <int ORDER, int MB, int NR, int NW, int H, int FMT>
__device__ __forceinline__ void rw_half(const uint4 *__restrict__ a_cur, uint4 *__restrict__ a_nxt,
                                        const uint4 *__restrict__ q_cur, uint4 *__restrict__ q_nxt, uint4 *__restrict__ hb,
                                        uint4 *__restrict__ qhs, const uint4 *__restrict__ xs_nxt, const uint8_t *__restrict__ wq_nxt,
                                        const uint8_t *__restrict__ wh_nxt, const Lane<MB, NR, NW> &L, Acc<MB, NR> &R) {
    constexpr int BM = 32 * MB, kThreads = 64 * NW;
    const int col = L.col, g = L.g;
    if (H == 0) {
#pragma unroll
        for (int rg = 0; rg < NR; rg++) {
            const uint4 hv = hb[rg * 64 + col];
            R.hdr[rg] = u32x4{hv.x, hv.y, hv.z, hv.w};
            if (FMT == 1) {  // both halves of the super-block take their fifth bits from these registers
                const uint4 ha = qhs[rg * 64 + 2 * col], hb2 = qhs[rg * 64 + 2 * col + 1];
                R.qh[rg][0] = ha.x, R.qh[rg][1] = ha.y, R.qh[rg][2] = ha.z, R.qh[rg][3] = ha.w;
                R.qh[rg][4] = hb2.x, R.qh[rg][5] = hb2.y, R.qh[rg][6] = hb2.z, R.qh[rg][7] = hb2.w;
            }
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the headers are in registers before their buffer is refilled
#pragma unroll
        for (int rg = 0; rg < NR; rg++) {
            dma16(wh_nxt + L.h_off[rg], hb + rg * 64);
            if (FMT == 1) dma16(wh_nxt + L.qh_off[rg], qhs + rg * 64);
        }
    }
    // copies for the next half super-block
#pragma unroll
    for (int i = 0; i < Lane<MB, NR, NW>::kARounds; i++)
        if (i * kThreads + L.wave * 64 < kGroups * BM) dma16(xs_nxt + L.a_off[i], a_nxt + i * kThreads + L.wave * 64);
    // the quant copies must be the newest requests of this half: the barrier at its end waits for all but them
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int rg = 0; rg < NR; rg++)
#pragma unroll
        for (int r = 0; r < 2; r++) dma16(wq_nxt + L.q_off[rg][r], q_nxt + rg * 128 + r * 64);
    __builtin_amdgcn_sched_barrier(0);  // the copies are requested before anything else of this half

    // scales and mins of sub-blocks j0 = 4 H + 2 g and j0 + 1 (6-bit fields, crates/pmetal/src/commands/quantize.rs:844-855)
    const uint32_t sh = 16u * (uint32_t)g;
    half2_t sc2[NR][2], off2[NR][2];
    uint32_t mn[NR][2];
    uint32_t qd[NR][8];
    // this lane's 32 quant bytes per row group: pieces 2g and 2g+1 of row col (the copy swizzles the four pieces of
    // a row by (row / 4) % 4 so that 16 consecutive rows read conflict-free)
    const int sw = (col >> 2) & 3;
#pragma unroll
    for (int rg = 0; rg < NR; rg++) {
        const uint4 qa = q_cur[rg * 128 + col * 4 + ((2 * g) ^ sw)], qb = q_cur[rg * 128 + col * 4 + ((2 * g + 1) ^ sw)];
        qd[rg][0] = qa.x, qd[rg][1] = qa.y, qd[rg][2] = qa.z, qd[rg][3] = qa.w;
        qd[rg][4] = qb.x, qd[rg][5] = qb.y, qd[rg][6] = qb.z, qd[rg][7] = qb.w;
        uint32_t sc0, sc1;
        if (H == 0) {
            const uint32_t yv = R.hdr[rg].y >> sh, zv = R.hdr[rg].z >> sh;
            sc0 = yv & 63u, sc1 = (yv >> 8) & 63u;
            mn[rg][0] = zv & 63u, mn[rg][1] = (zv >> 8) & 63u;
        } else {
            const uint32_t wv = R.hdr[rg].w >> sh, yv = R.hdr[rg].y >> sh, zv = R.hdr[rg].z >> sh;
            sc0 = (wv & 0xFu) | ((yv >> 2) & 0x30u), sc1 = ((wv >> 8) & 0xFu) | ((yv >> 10) & 0x30u);
            mn[rg][0] = ((wv >> 4) & 0xFu) | ((zv >> 2) & 0x30u), mn[rg][1] = ((wv >> 12) & 0xFu) | ((zv >> 10) & 0x30u);
        }
        const _Float16 s0 = (_Float16)(float)sc0, s1 = (_Float16)(float)sc1;
        const _Float16 o0 = (_Float16)(-1024.0f * (float)sc0), o1 = (_Float16)(-1024.0f * (float)sc1);  // exact: sc <= 63
        sc2[rg][0] = half2_t{s0, s0}, sc2[rg][1] = half2_t{s1, s1};
        off2[rg][0] = half2_t{o0, o0}, off2[rg][1] = half2_t{o1, o1};
    }

    // Q5_K: where k-step t finds its fifth bits.  GGML order: qh dword t (the same four bytes as quant dword t), bits
    // j0 = 4 H + 2 g (low nibbles) and j0 + 1 (high nibbles) of every byte.  REF order: byte 4 j0 + t of qh.
    auto fifth = [&](int rg, int t) -> uint32_t {
        if (FMT == 0) return 0u;
        if (ORDER == 1) return R.qh[rg][t] >> (uint32_t)(4 * H + 2 * g);
        const uint32_t dw = g ? R.qh[rg][4 * H + 2 + (t >> 2)] : R.qh[rg][4 * H + (t >> 2)];
        return dw >> (8 * (t & 3));  // (the decoder masks the byte)
    };

    // min term of sub-blocks j0, j0 + 1: (-h, -h, -l, -l) against the activations' (H, L, H, L): all four cross
    // products of the exact head + tail splits, straight into the accumulators (after the eight k-steps)
    half8_t br[NR];
#pragma unroll
    for (int rg = 0; rg < NR; rg++) {
        const float dmin = f16_bits_to_f32(R.hdr[rg].x >> 16);
        _Float16 h0, l0, h1, l1;
        neg_min_split(dmin, mn[rg][0], h0, l0);
        neg_min_split(dmin, mn[rg][1], h1, l1);
        br[rg] = half8_t{h0, h0, l0, l0, h1, h1, l1, l1};
    }

    // Software pipeline, written in issue order (a wave issues in order, so the order here is the schedule):
    // the activation fragments of k-step t + 1 are requested before the products of k-step t, and the weights of
    // k-step t + 1 are dequantized in pieces between those products.
    constexpr int kSlots = MB * NR, kChunks = 4 * NR;
    half8_t af[2][MB];
    Dq dq[NR];
#pragma unroll
    for (int i = 0; i < MB; i++) af[0][i] = __builtin_bit_cast(half8_t, a_cur[g * BM + 32 * i + col]);
#pragma unroll
    for (int rg = 0; rg < NR; rg++)
#pragma unroll
        for (int c = 0; c < 4; c++) dq_chunk<ORDER, FMT>(c, 0, qd[rg][0], sc2[rg], off2[rg], dq[rg], fifth(rg, 0));
#pragma unroll
    for (int t = 0; t < 8; t++) {
        half8_t b[NR];
#pragma unroll
        for (int rg = 0; rg < NR; rg++) b[rg] = dq[rg].value();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < MB; i++)
#pragma unroll
            for (int rg = 0; rg < NR; rg++) {
                const half8_t a = af[t & 1][i];
                if (H == 0 && t == 0) {  // first product of a super-block starts from zero
                    float16_t z;
#pragma unroll
                    for (int r = 0; r < 16; r++) z[r] = 0.0f;
                    R.part[rg][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b[rg], z, 0, 0, 0);
                } else {
                    R.part[rg][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b[rg], R.part[rg][i], 0, 0, 0);
                }
                if (t < 7) {
                    const int slot = i * NR + rg;
#pragma unroll
                    for (int ch = slot * kChunks / kSlots; ch < (slot + 1) * kChunks / kSlots; ch++)
                        dq_chunk<ORDER, FMT>(ch % 4, t + 1, qd[ch / 4][t + 1], sc2[ch / 4], off2[ch / 4], dq[ch / 4], fifth(ch / 4, t + 1));
                }
                if (i == 0 && rg == 0) {
                    // the next step's fragments are requested behind the first product of this step: the wait in
                    // front of that product then covers only fragments requested a whole step ago
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int ii = 0; ii < MB; ii++)
                        af[(t + 1) & 1][ii] = __builtin_bit_cast(half8_t, a_cur[(t < 7 ? (t + 1) * 2 + g : 16 + g) * BM + 32 * ii + col]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
    }
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int rg = 0; rg < NR; rg++) R.acc[rg][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[0][i], br[rg], R.acc[rg][i], 0, 0, 0);
    if (H == 1) {
#pragma unroll
        for (int rg = 0; rg < NR; rg++) {
            const float d = f16_bits_to_f32(R.hdr[rg].x & 0xFFFFu);
#pragma unroll
            for (int i = 0; i < MB; i++)
#pragma unroll
                for (int r = 0; r < 16; r++) R.acc[rg][i][r] = __builtin_fmaf(d, R.part[rg][i][r], R.acc[rg][i][r]);
        }
    }
}

// grid (ceil(N / (32 NR NW)), Mp / BM, splits); workgroup z works on super-blocks [z * chunk, min(spr, (z + 1) * chunk)).
// mode 0: y f32 [M][N], 1: y bf16, 2: fp32 partial tiles [splits][Mp][N] (not yet scaled by rowscale)
//
// Copies in flight: the activation stage of the next half super-block (it comes from L2) and the quant pieces of
// the next two (they come from HBM): three quant stages per wave, rotated.  Within a half super-block the
// activation copies are requested before the quant copies, so waiting until only the 2 NR newest requests are
// outstanding leaves exactly the quant copies for the half after next in flight.
template <int ORDER, int MB, int NR, int NW, int FMT = 0>
__global__ __launch_bounds__(64 * NW, MB * NR <= 1 && NW <= 8 ? 2 : 1) void k_qgemm_rw(
    const uint8_t *__restrict__ W, const uint4 *__restrict__ xs, const float *__restrict__ rowscale, void *__restrict__ yg,
    float *__restrict__ partial, int M, int Mp, int N, int spr, int chunk, int mode) {
    constexpr int BM = 32 * MB, kThreads = 64 * NW, kRows = 32 * NR * NW;
    constexpr int kBlockBytes = BlockFmt<FMT>::kBytes, kQs = BlockFmt<FMT>::kQs;
    extern __shared__ uint4 smem[];
    uint4 *a0 = smem, *a1 = a0 + kGroups * BM, *qbase = a1 + kGroups * BM, *hb = qbase + 3 * NW * NR * 128;
    uint4 *qhb = hb + NW * NR * 64;  // Q5_K only
    const int tid = threadIdx.x;
    Lane<MB, NR, NW> L;
    L.wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    L.col = lane & 31, L.g = lane >> 5;
    const int n0 = blockIdx.x * kRows, m0 = blockIdx.y * BM;
    const int nw0 = n0 + 32 * NR * L.wave;  // first weight row of this wave
    const int sb0 = blockIdx.z * chunk;
    const int cnt = spr - sb0 < chunk ? spr - sb0 : chunk;
    const uint32_t row_bytes = (uint32_t)spr * kBlockBytes;
    auto row_off = [&](int row) {  // byte offset of a row of this wave from the workgroup's first row; rows past N repeat the last
        int n = nw0 + row;
        n = n < N ? n : N - 1;
        return (uint32_t)(n - n0) * row_bytes;
    };
#pragma unroll
    for (int rg = 0; rg < NR; rg++) {
#pragma unroll
        for (int r = 0; r < 2; r++) {
            const int row = 16 * r + (lane >> 2);
            L.q_off[rg][r] = row_off(32 * rg + row) + 16u * (uint32_t)((lane & 3) ^ ((row >> 2) & 3));
        }
        L.h_off[rg] = row_off(32 * rg + (lane & 31));
        L.qh_off[rg] = row_off(32 * rg + (lane >> 1)) + 16u + 16u * (uint32_t)(lane & 1);
    }
#pragma unroll
    for (int i = 0; i < Lane<MB, NR, NW>::kARounds; i++) {
        const int idx = tid + i * kThreads;
        L.a_off[i] = (uint32_t)((idx / BM) * Mp + idx % BM);
    }
    // this wave's three quant stages (rotated: qa is read, qb is next, qc receives the copies) and its headers
    uint4 *qa = qbase + L.wave * (NR * 128), *qb = qa + NW * NR * 128, *qc = qb + NW * NR * 128;
    uint4 *hw = hb + L.wave * (NR * 64), *qhw = qhb + L.wave * (NR * 64);
    const uint8_t *wblk = W + (size_t)n0 * row_bytes;

    Acc<MB, NR> R;
#pragma unroll
    for (int rg = 0; rg < NR; rg++)
#pragma unroll
        for (int i = 0; i < MB; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) R.acc[rg][i][r] = 0.0f, R.part[rg][i][r] = 0.0f;

    // prologue: headers, both halves' quant pieces and the first activation stage of super-block sb0
    {
        const uint8_t *blk = wblk + (size_t)sb0 * kBlockBytes;
#pragma unroll
        for (int rg = 0; rg < NR; rg++) {
            dma16(blk + L.h_off[rg], hw + rg * 64);
            if (FMT == 1) dma16(blk + L.qh_off[rg], qhw + rg * 64);
#pragma unroll
            for (int r = 0; r < 2; r++) {
                dma16(blk + kQs + L.q_off[rg][r], qa + rg * 128 + r * 64);
                dma16(blk + kQs + 64 + L.q_off[rg][r], qb + rg * 128 + r * 64);
            }
        }
        const uint4 *xa = xs + (size_t)(sb0 * 2 * kGroups) * Mp + m0;
#pragma unroll
        for (int i = 0; i < Lane<MB, NR, NW>::kARounds; i++)
            if (i * kThreads + L.wave * 64 < kGroups * BM) dma16(xa + L.a_off[i], a0 + i * kThreads + L.wave * 64);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();

    for (int s = 0; s < cnt; s++) {
        const int sb = sb0 + s;
        const int sbn = sb + 1 < spr ? sb + 1 : spr - 1;  // the copies for "the next super-block" stay inside the matrix
        const uint8_t *blkn = wblk + (size_t)sbn * kBlockBytes;
        rw_half<ORDER, MB, NR, NW, 0, FMT>(a0, a1, qa, qc, hw, qhw, xs + (size_t)((sb * 2 + 1) * kGroups) * Mp + m0, blkn + kQs, blkn, L, R);
        barrier_keep<2 * NR>();
        rw_half<ORDER, MB, NR, NW, 1, FMT>(a1, a0, qb, qa, hw, qhw, xs + (size_t)(sbn * 2 * kGroups) * Mp + m0, blkn + kQs + 64, nullptr, L, R);
        barrier_keep<2 * NR>();
        // two half super-blocks on: (qa, qb, qc) <- (qc, qa, qb)
        uint4 *t = qc;
        qc = qb, qb = qa, qa = t;
    }
    // the last copies (for a half super-block past the end) have landed and every wave is done with the stages
    static_assert(NR == 1, "the tile store takes one group of weight rows per wave");
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    store_tile<MB, NW>(R.acc[0], smem, L.wave, L.col, L.g, m0, n0, M, N, Mp, rowscale, yg, partial, mode, blockIdx.z);
}

// ------------------------------------------------------------------------------------------------
// Q2_K and Q3_K (crates/pmetal-gguf/src/k_quants.rs:230-266, :281-355): sixteen 16-element sub-blocks per super-block,
// two-bit quants, qs byte 32 h + l = elements 128 h + l + 32 s at bit 2 s.  The Q4_K kernel's structure with these
// differences:
//   * a half super-block of a row is 32 bytes of qs: lane (n, g) takes bytes 16 g .. 16 g + 15; dword t / 2 of them gives
//     k-step t its eight values, four at shift 4 (t % 2) (sub-block 8 h + 4 (t % 2) + g) and four at 4 (t % 2) + 2
//     (sub-block 8 h + 4 (t % 2) + 2 + g): four scales per lane and half, one quant copy per wave and half;
//   * Q2_K: value d (sc & 15) q - dmin (sc >> 4), q in 0..3: the B tile is (sc & 15) q, and the min terms of the lane's
//     four sub-blocks are two K = 16 products of exact head + tail splits (activation items 16 + g and 18 + g);
//   * Q3_K: value d s' (q3 - 4) with s' = sc6 - 32 and q3 = q | hbit << 2, hbit = bit 4 h + s of hmask[l]: the B tile is
//     s' q3 = (1024 + q3) s' - 1024 s' (1028 s' would not be an f16 number), and the - 4 d s' of every element leaves with the
//     sub-block sums of the activations, exactly as Q2_K's mins do (coefficient 4 d s' in place of dmin m);
//   * blocks are 84 / 110 bytes, so rows start at 4- / 2-byte aligned addresses (the direct-to-LDS loads take them); the
//     header pieces of a row are Q2_K: bytes 0..15 (scales) and 68..83 (d, dmin in the last dword); Q3_K: 0..31 (hmask) and
//     94..109 (scales in bytes 2..13 of the piece, d in 14..15).
// ------------------------------------------------------------------------------------------------
constexpr int kGroups16 = 20;  // activation items per row and half super-block: 16 operands and four of sub-block sums
template <int FMT>
struct Block16 {  // FMT 2: Q3_K, 3: Q2_K
    static constexpr int kBytes = FMT == 3 ? 84 : 110, kQs = FMT == 3 ? 16 : 32;
    static constexpr int kHdrPieces = FMT == 3 ? 2 : 3;           // per row and super-block
    static constexpr int kHdrRounds = (32 * kHdrPieces + 63) / 64;  // whole-wave copies
    static constexpr int kHdrStage = 64 * kHdrRounds;              // items of a wave's header stage
    static __device__ __forceinline__ uint32_t piece_off(int p) { return FMT == 3 ? (p == 0 ? 0u : 68u) : (p == 2 ? 94u : 16u * (uint32_t)p); }
};

template <int FMT, int MB, int H>
__device__ __forceinline__ void rw16_half(const uint4 *__restrict__ a_cur, uint4 *__restrict__ a_nxt, const uint4 *__restrict__ q_cur,
                                          uint4 *__restrict__ q_nxt, uint4 *__restrict__ hs, const uint4 *__restrict__ xs_nxt,
                                          const uint8_t *__restrict__ wq_nxt, const uint8_t *__restrict__ wh_nxt, const int wave,
                                          const int col, const int g, const uint32_t q_off, const uint32_t (&h_off)[Block16<FMT>::kHdrRounds],
                                          const uint32_t *a_off, float16_t (&acc)[MB], float16_t (&part)[MB], uint32_t (&hdr)[8],
                                          uint32_t (&hm)[4], uint32_t &dbits) {
    using B = Block16<FMT>;
    constexpr int BM = 32 * MB, kThreads = 512, kARounds = (kGroups16 * BM + kThreads - 1) / kThreads;
    if (H == 0) {
        // this row's header pieces into registers, then their stage is refilled with the next super-block's
        if (FMT == 3) {
            const uint4 sc = hs[col * 2], dd = hs[col * 2 + 1];
            hdr[0] = sc.x, hdr[1] = sc.y, hdr[2] = sc.z, hdr[3] = sc.w;
            dbits = dd.w;  // d | dmin << 16
        } else {
            const uint4 m0 = hs[col * 3], m1 = hs[col * 3 + 1], sd = hs[col * 3 + 2];
            // the lane's hmask bytes 16 g + 4 dw .. + 3 (both halves of the super-block use them)
            hm[0] = g ? m1.x : m0.x, hm[1] = g ? m1.y : m0.y, hm[2] = g ? m1.z : m0.z, hm[3] = g ? m1.w : m0.w;
            // the twelve scale bytes as three dwords (they start two bytes into the piece), d behind them
            hdr[0] = __builtin_amdgcn_alignbit(sd.y, sd.x, 16), hdr[1] = __builtin_amdgcn_alignbit(sd.z, sd.y, 16);
            hdr[2] = __builtin_amdgcn_alignbit(sd.w, sd.z, 16);
            dbits = sd.w >> 16;
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
#pragma unroll
        for (int r = 0; r < B::kHdrRounds; r++) dma16(wh_nxt + h_off[r], hs + 64 * r);
    }
#pragma unroll
    for (int i = 0; i < kARounds; i++)
        if (i * kThreads + wave * 64 < kGroups16 * BM) dma16(xs_nxt + a_off[i], a_nxt + i * kThreads + wave * 64);
    // the quant copy must be the newest request of this half: the barrier at its end waits for all but it
    __builtin_amdgcn_sched_barrier(0);
    dma16(wq_nxt + q_off, q_nxt);
    __builtin_amdgcn_sched_barrier(0);

    // this lane's 16 quant bytes: piece g of row col
    const uint4 qv = q_cur[col * 2 + g];
    const uint32_t qd[4] = {qv.x, qv.y, qv.z, qv.w};
    // scales (and mins) of the lane's four sub-blocks j = 8 H + 4 sp + 2 lh + g, index 2 sp + lh
    half2_t sc2[4], off2[4];
    float nm[4];  // what a sub-block subtracts per unit of its activation sum, negated: -dmin m (Q2_K), -4 d s' (Q3_K); exact in fp32
#pragma unroll
    for (int sp = 0; sp < 2; sp++)
#pragma unroll
        for (int lh = 0; lh < 2; lh++) {
            float scf;
            if (FMT == 3) {  // byte j of the sixteen: low nibble scale, high nibble min
                const uint32_t b = (hdr[2 * H + sp] >> (8u * (uint32_t)g + 16u * lh)) & 0xFFu;
                scf = (float)(b & 15u);
                nm[2 * sp + lh] = -(f16_bits_to_f32(dbits >> 16) * (float)(b >> 4));
            } else {
                // sc6 of sub-block j: low nibble (j < 8) or high nibble (j >= 8) of byte j % 8, bits 4..5 = bits
                // 2 (j / 4) of byte 8 + j % 4
                const uint32_t lo4 = (hdr[sp] >> (8u * (uint32_t)g + 16u * lh + 4u * H)) & 15u;
                const uint32_t hi2 = (hdr[2] >> (8u * (uint32_t)g + 16u * lh + 2u * (2 * H + sp))) & 3u;
                scf = (float)((int)(lo4 | (hi2 << 4)) - 32);
                nm[2 * sp + lh] = -(f16_bits_to_f32(dbits & 0xFFFFu) * (4.0f * scf));
            }
            const _Float16 sh = (_Float16)scf, oh = (_Float16)(-1024.0f * scf);  // exact: |sc| <= 32
            sc2[2 * sp + lh] = half2_t{sh, sh}, off2[2 * sp + lh] = half2_t{oh, oh};
        }
    // operand of k-step t: dword t / 2, the two-bit fields at 4 (t % 2) and 4 (t % 2) + 2 (Q3_K: bit 2 from hmask)
    auto operand = [&](int t) -> half8_t {
        const int dw = t >> 1, sp = t & 1;
        uint32_t lo = (qd[dw] >> (4 * sp)) & 0x03030303u, hi = (qd[dw] >> (4 * sp + 2)) & 0x03030303u;
        if (FMT == 2) {
            const uint32_t m = hm[dw] >> (4 * H + 2 * sp);
            lo |= (m & 0x01010101u) << 2, hi |= (m & 0x02020202u) << 1;
        }
        const half2_t r0 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, lo, 0x04010400u)), sc2[2 * sp], off2[2 * sp]);
        const half2_t r1 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, lo, 0x04030402u)), sc2[2 * sp], off2[2 * sp]);
        const half2_t r2 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, hi, 0x04010400u)), sc2[2 * sp + 1], off2[2 * sp + 1]);
        const half2_t r3 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, hi, 0x04030402u)), sc2[2 * sp + 1], off2[2 * sp + 1]);
        return half8_t{r0[0], r0[1], r1[0], r1[1], r2[0], r2[1], r3[0], r3[1]};
    };
    half8_t af[2][MB];
#pragma unroll
    for (int i = 0; i < MB; i++) af[0][i] = __builtin_bit_cast(half8_t, a_cur[g * BM + 32 * i + col]);
    half8_t b = operand(0);
#pragma unroll
    for (int t = 0; t < 8; t++) {
        const half8_t bt = b;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < MB; i++) {
            const half8_t a = af[t & 1][i];
            if (H == 0 && t == 0) {  // first product of a super-block starts from zero
                float16_t z;
#pragma unroll
                for (int r = 0; r < 16; r++) z[r] = 0.0f;
                part[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bt, z, 0, 0, 0);
            } else {
                part[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bt, part[i], 0, 0, 0);
            }
            if (i == 0) {
                // the next step's fragments (after the last step: the first sums item) and its operand
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ii = 0; ii < MB; ii++)
                    af[(t + 1) & 1][ii] = __builtin_bit_cast(half8_t, a_cur[(t < 7 ? (t + 1) * 2 + g : 16 + g) * BM + 32 * ii + col]);
                if (t < 7) b = operand(t + 1);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    {
        // sum terms of the lane's four sub-blocks: exact head + tail splits (h, h, l, l) against the sums' (H, L, H, L), pairs
        // (sp, 0), (sp, 1)
#pragma unroll
        for (int sp = 0; sp < 2; sp++) {
            const _Float16 h0 = (_Float16)nm[2 * sp], h1 = (_Float16)nm[2 * sp + 1];
            const _Float16 l0 = (_Float16)(nm[2 * sp] - (float)h0), l1 = (_Float16)(nm[2 * sp + 1] - (float)h1);
            const half8_t br = half8_t{h0, h0, l0, l0, h1, h1, l1, l1};
#pragma unroll
            for (int i = 0; i < MB; i++) {
                const half8_t a = sp == 0 ? af[0][i] : __builtin_bit_cast(half8_t, a_cur[(18 + g) * BM + 32 * i + col]);
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, br, acc[i], 0, 0, 0);
            }
        }
    }
    if (H == 1) {
        const float d = f16_bits_to_f32(dbits & 0xFFFFu);
#pragma unroll
        for (int i = 0; i < MB; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][r] = __builtin_fmaf(d, part[i][r], acc[i][r]);
    }
}

// grid and modes as k_qgemm_rw; eight waves of 32 weight rows
template <int FMT, int MB>
__global__ __launch_bounds__(512, MB <= 1 ? 2 : 1) void k_qgemm_rw16(const uint8_t *__restrict__ W, const uint4 *__restrict__ xs,
                                                                      const float *__restrict__ rowscale, void *__restrict__ yg,
                                                                      float *__restrict__ partial, int M, int Mp, int N, int spr, int chunk,
                                                                      int mode) {
    using B = Block16<FMT>;
    constexpr int BM = 32 * MB, NW = 8, kThreads = 512, kRows = 256, kARounds = (kGroups16 * BM + kThreads - 1) / kThreads;
    extern __shared__ uint4 smem[];
    uint4 *a0 = smem, *a1 = a0 + kGroups16 * BM, *qbase = a1 + kGroups16 * BM, *hb = qbase + 3 * NW * 64;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, col = lane & 31, g = lane >> 5;
    const int n0 = blockIdx.x * kRows, m0 = blockIdx.y * BM;
    const int nw0 = n0 + 32 * wave;  // first weight row of this wave
    const int sb0 = blockIdx.z * chunk;
    const int cnt = spr - sb0 < chunk ? spr - sb0 : chunk;
    const uint32_t row_bytes = (uint32_t)spr * B::kBytes;
    auto row_off = [&](int row) {  // byte offset of a row of this wave from the workgroup's first row; rows past N repeat the last
        int n = nw0 + row;
        n = n < N ? n : N - 1;
        return (uint32_t)(n - n0) * row_bytes;
    };
    // quant copy: lane -> (row lane / 2, piece lane % 2); header copies: item lane + 64 r -> (row item / P, piece item % P)
    const uint32_t q_off = row_off(lane >> 1) + 16u * (uint32_t)(lane & 1);
    uint32_t h_off[B::kHdrRounds];
#pragma unroll
    for (int r = 0; r < B::kHdrRounds; r++) {
        int item = lane + 64 * r;
        item = item < 32 * B::kHdrPieces ? item : 32 * B::kHdrPieces - 1;  // (the copies past the last item repeat it into the stage's padding)
        h_off[r] = row_off(item / B::kHdrPieces) + B::piece_off(item % B::kHdrPieces);
    }
    uint32_t a_off[kARounds];
#pragma unroll
    for (int i = 0; i < kARounds; i++) {
        const int idx = tid + i * kThreads;
        a_off[i] = (uint32_t)((idx / BM) * Mp + idx % BM);
    }
    uint4 *qa = qbase + wave * 64, *qb = qa + NW * 64, *qc = qb + NW * 64;
    uint4 *hw = hb + wave * B::kHdrStage;
    const uint8_t *wblk = W + (size_t)n0 * row_bytes;

    float16_t acc[MB], part[MB];
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.0f, part[i][r] = 0.0f;
    uint32_t hdr[8] = {0, 0, 0, 0, 0, 0, 0, 0}, hm[4] = {0, 0, 0, 0}, dbits = 0;

    {  // prologue: headers, both halves' quant pieces and the first activation stage of super-block sb0
        const uint8_t *blk = wblk + (size_t)sb0 * B::kBytes;
#pragma unroll
        for (int r = 0; r < B::kHdrRounds; r++) dma16(blk + h_off[r], hw + 64 * r);
        dma16(blk + B::kQs + q_off, qa);
        dma16(blk + B::kQs + 32 + q_off, qb);
        const uint4 *xa = xs + (size_t)(sb0 * 2 * kGroups16) * Mp + m0;
#pragma unroll
        for (int i = 0; i < kARounds; i++)
            if (i * kThreads + wave * 64 < kGroups16 * BM) dma16(xa + a_off[i], a0 + i * kThreads + wave * 64);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();

    for (int s = 0; s < cnt; s++) {
        const int sb = sb0 + s;
        const int sbn = sb + 1 < spr ? sb + 1 : spr - 1;  // the copies for "the next super-block" stay inside the matrix
        const uint8_t *blkn = wblk + (size_t)sbn * B::kBytes;
        rw16_half<FMT, MB, 0>(a0, a1, qa, qc, hw, xs + (size_t)((sb * 2 + 1) * kGroups16) * Mp + m0, blkn + B::kQs, blkn, wave, col, g, q_off,
                              h_off, a_off, acc, part, hdr, hm, dbits);
        barrier_keep<1>();
        rw16_half<FMT, MB, 1>(a1, a0, qb, qa, hw, xs + (size_t)(sbn * 2 * kGroups16) * Mp + m0, blkn + B::kQs + 32, nullptr, wave, col, g, q_off,
                              h_off, a_off, acc, part, hdr, hm, dbits);
        barrier_keep<1>();
        uint4 *t = qc;  // two half super-blocks on: (qa, qb, qc) <- (qc, qa, qb)
        qc = qb, qb = qa, qa = t;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    store_tile<MB, NW>(acc, smem, wave, col, g, m0, n0, M, N, Mp, rowscale, yg, partial, mode, blockIdx.z);
}

template <int FMT, int MB>
constexpr size_t rw16_lds_bytes() {
    const size_t stages = (size_t)(2 * kGroups16 * 32 * MB + 8 * (3 * 64 + Block16<FMT>::kHdrStage)) * 16;
    return stages > tile_lds_bytes<MB, 8>() ? stages : tile_lds_bytes<MB, 8>();
}

// ------------------------------------------------------------------------------------------------
// Q6_K (crates/pmetal-gguf/src/k_quants.rs:474-496: 210-byte super-blocks: ql[128] low nibbles, qh[64] top two
// bits, 16 int8 scales, f16 d; value d * sc * (q - 32)).  Same structure as the Q4_K kernel, with these differences:
//   * sc * (q - 32) can reach 4096 and is not always exact in f16, so it is split where the storage splits it,
//     q - 32 = 16 (hi2 - 2) + nib, into two exact tiles  B1 = (16 sc) (hi2 - 2)  and  B2 = sc * nib  that multiply
//     the same activation fragment one after the other (a fragment read from LDS feeds two matrix instructions);
//   * no min term; one scale per 16 elements;
//   * a half super-block of a row is 64 bytes of ql and 32 of qh; lane (n, g) multiplies ql bytes 32 g .. 32 g + 31
//     (dword t: low nibbles = elements 32 g + 4 t + e of the half, high nibbles 64 further) with the qh bytes
//     4 t + e (two-bit field g for the low, 2 + g for the high nibbles);
//   * super-blocks are only 2-byte aligned; the direct-to-LDS loads take such addresses.
// ------------------------------------------------------------------------------------------------
constexpr int kQ6Bytes = 210, kQ6Groups = 16, kQ6Stage = 192;  // LDS items of a wave's quant stage: 128 ql + 64 qh

template <int MB>
struct LaneQ6 {
    static constexpr int BM = 32 * MB, kThreads = 512;
    static constexpr int kARounds = kQ6Groups * BM / kThreads;
    static_assert(kQ6Groups * BM % kThreads == 0, "the activation stage must divide among the threads");
    int wave, col, g;
    uint32_t ql_off[2], qh_off, h_off;  // byte offsets of this lane's pieces from the workgroup's first row
    uint32_t a_off[kARounds];
};

template <int MB>
struct AccQ6 {
    float16_t acc[MB], part[MB];
    u32x4 sc;    // the 16 int8 scales of the current super-block
    uint32_t d;  // f16 bits of d
};

// The two operands of one k-step, built in eight pieces that are placed between matrix instructions.
struct Dq6 {
    uint32_t nlo, nhi, hlo, hhi;
    half2_t r1[4], r2[4];
    __device__ __forceinline__ half8_t b1() const { return half8_t{r1[0][0], r1[0][1], r1[1][0], r1[1][1], r1[2][0], r1[2][1], r1[3][0], r1[3][1]}; }
    __device__ __forceinline__ half8_t b2() const { return half8_t{r2[0][0], r2[0][1], r2[1][0], r2[1][1], r2[2][0], r2[2][1], r2[3][0], r2[3][1]}; }
};
// qlw: the ql dword of the k-step; qhw: its qh dword already shifted by 2 g; s2 / s1: (sc, sc) and (16 sc, 16 sc)
// of the low-nibble and of the high-nibble elements.  0x6400 | v is the f16 1024 + v; both steps of each value are exact.
__device__ __forceinline__ void dq6_chunk(const int c, const uint32_t qlw, const uint32_t qhw, const half2_t (&s2)[2],
                                          const half2_t (&s1)[2], Dq6 &d) {
    const half2_t m1024 = {(_Float16)-1024.0f, (_Float16)-1024.0f}, m1026 = {(_Float16)-1026.0f, (_Float16)-1026.0f};
    const uint32_t sel = (c & 1) ? 0x04030402u : 0x04010400u;  // bytes (b0, b1) resp. (b2, b3) -> 0x64bb pairs
    if (c == 0) d.nlo = qlw & 0x0F0F0F0Fu;
    if (c == 2) d.nhi = (qlw >> 4) & 0x0F0F0F0Fu;
    if (c == 4) d.hlo = qhw & 0x03030303u;
    if (c == 6) d.hhi = (qhw >> 4) & 0x03030303u;
    if (c < 4) {
        const uint32_t v = c < 2 ? d.nlo : d.nhi;
        d.r2[c] = (__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, sel)) + m1024) * s2[c >> 1];
    } else {
        const uint32_t v = c < 6 ? d.hlo : d.hhi;
        d.r1[c - 4] = (__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, sel)) + m1026) * s1[(c - 4) >> 1];
    }
}

template <int MB, int H>
__device__ __forceinline__ void rw_half_q6(const uint4 *__restrict__ a_cur, uint4 *__restrict__ a_nxt,
                                           const uint4 *__restrict__ q_cur, uint4 *__restrict__ q_nxt, uint4 *__restrict__ hb,
                                           const uint4 *__restrict__ xs_nxt, const uint8_t *__restrict__ wq_nxt,
                                           const uint8_t *__restrict__ wh_nxt, const LaneQ6<MB> &L, AccQ6<MB> &R) {
    constexpr int BM = 32 * MB, kThreads = 512;
    const int col = L.col, g = L.g;
    if (H == 0) {
        const uint4 sv = hb[col], dv = hb[32 + col];  // bytes 192..207 and 194..209 of the super-block
        R.sc = u32x4{sv.x, sv.y, sv.z, sv.w};
        R.d = dv.w >> 16;
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the header is in registers before its buffer is refilled
        dma16(wh_nxt + L.h_off, hb);
    }
#pragma unroll
    for (int i = 0; i < LaneQ6<MB>::kARounds; i++) dma16(xs_nxt + L.a_off[i], a_nxt + i * kThreads + L.wave * 64);
    __builtin_amdgcn_sched_barrier(0);  // the three quant copies stay the newest requests (see barrier_keep)
    // quant pieces two half super-blocks ahead: ql bytes 64 H .., qh bytes 128 + 32 H .. of that super-block
#pragma unroll
    for (int r = 0; r < 2; r++) dma16(wq_nxt + 64 * H + L.ql_off[r], q_nxt + r * 64);
    dma16(wq_nxt + 32 * H + L.qh_off, q_nxt + 128);
    __builtin_amdgcn_sched_barrier(0);  // the copies are requested before anything else of this half

    // this lane's 32 ql bytes and the 32 qh bytes of its row (pieces swizzled by the copy for conflict-free reads)
    const int sw = (col >> 2) & 3, sw2 = (col >> 3) & 1;
    const uint4 qa = q_cur[col * 4 + ((2 * g) ^ sw)], qb = q_cur[col * 4 + ((2 * g + 1) ^ sw)];
    const uint4 ha = q_cur[128 + col * 2 + sw2], hc = q_cur[128 + col * 2 + (1 ^ sw2)];
    const uint32_t qd[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
    const uint32_t hs = 2u * (uint32_t)g;
    const uint32_t hd[8] = {ha.x >> hs, ha.y >> hs, ha.z >> hs, ha.w >> hs, hc.x >> hs, hc.y >> hs, hc.z >> hs, hc.w >> hs};
    // scales 8 H + 2 g + t / 4 (low nibbles) and 8 H + 4 + 2 g + t / 4 (high nibbles)
    const uint32_t wlo = (H == 0 ? R.sc.x : R.sc.z) >> (16u * (uint32_t)g), whi = (H == 0 ? R.sc.y : R.sc.w) >> (16u * (uint32_t)g);
    half2_t s2[2][2], s1[2][2];  // [k-step / 4][low, high]
#pragma unroll
    for (int th = 0; th < 2; th++) {
        const float fl = (float)(int)(int8_t)(wlo >> (8 * th)), fh = (float)(int)(int8_t)(whi >> (8 * th));
        const _Float16 l2 = (_Float16)fl, h2 = (_Float16)fh, l1 = (_Float16)(16.0f * fl), h1 = (_Float16)(16.0f * fh);  // exact: |sc| <= 128
        s2[th][0] = half2_t{l2, l2}, s2[th][1] = half2_t{h2, h2};
        s1[th][0] = half2_t{l1, l1}, s1[th][1] = half2_t{h1, h1};
    }

    // software pipeline in issue order, as in the Q4_K kernel; every fragment feeds two matrix instructions
    constexpr int kSlots = 2 * MB;
    half8_t af[2][MB];
    Dq6 dq;
#pragma unroll
    for (int i = 0; i < MB; i++) af[0][i] = __builtin_bit_cast(half8_t, a_cur[g * BM + 32 * i + col]);
#pragma unroll
    for (int c = 0; c < 8; c++) dq6_chunk(c, qd[0], hd[0], s2[0], s1[0], dq);
#pragma unroll
    for (int t = 0; t < 8; t++) {
        const half8_t b1 = dq.b1(), b2 = dq.b2();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int slot = 0; slot < kSlots; slot++) {
            const int i = slot >> 1;
            const half8_t a = af[t & 1][i];
            if (H == 0 && t == 0 && (slot & 1) == 0) {  // first product of a super-block starts from zero
                float16_t z;
#pragma unroll
                for (int r = 0; r < 16; r++) z[r] = 0.0f;
                R.part[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b1, z, 0, 0, 0);
            } else {
                R.part[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, (slot & 1) ? b2 : b1, R.part[i], 0, 0, 0);
            }
            if (t < 7) {
#pragma unroll
                for (int ch = slot * 8 / kSlots; ch < (slot + 1) * 8 / kSlots; ch++)
                    dq6_chunk(ch, qd[t + 1], hd[t + 1], s2[(t + 1) >> 2], s1[(t + 1) >> 2], dq);
                if (slot == 0) {
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int ii = 0; ii < MB; ii++)
                        af[(t + 1) & 1][ii] = __builtin_bit_cast(half8_t, a_cur[((t + 1) * 2 + g) * BM + 32 * ii + col]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if (H == 1) {
        const float d = f16_bits_to_f32(R.d);
#pragma unroll
        for (int i = 0; i < MB; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) R.acc[i][r] = __builtin_fmaf(d, R.part[i][r], R.acc[i][r]);
    }
}

// grid and modes as for k_qgemm_rw; 8 waves = 256 weight rows per workgroup
template <int MB>
__global__ __launch_bounds__(512, 1) void k_qgemm_rw_q6(const uint8_t *__restrict__ W, const uint4 *__restrict__ xs,
                                                         const float *__restrict__ rowscale, void *__restrict__ yg,
                                                         float *__restrict__ partial, int M, int Mp, int N, int spr, int chunk,
                                                         int mode) {
    constexpr int BM = 32 * MB, kThreads = 512, NW = 8;
    extern __shared__ uint4 smem[];
    uint4 *a0 = smem, *a1 = a0 + kQ6Groups * BM, *qbase = a1 + kQ6Groups * BM, *hb = qbase + 3 * NW * kQ6Stage;
    const int tid = threadIdx.x;
    LaneQ6<MB> L;
    L.wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    L.col = lane & 31, L.g = lane >> 5;
    const int n0 = blockIdx.x * 256, m0 = blockIdx.y * BM;
    const int nw0 = n0 + 32 * L.wave;
    const int sb0 = blockIdx.z * chunk;
    const int cnt = spr - sb0 < chunk ? spr - sb0 : chunk;
    const uint32_t row_bytes = (uint32_t)spr * kQ6Bytes;
    auto row_off = [&](int row) {  // rows past N repeat the last
        int n = nw0 + row;
        n = n < N ? n : N - 1;
        return (uint32_t)(n - n0) * row_bytes;
    };
#pragma unroll
    for (int r = 0; r < 2; r++) {
        const int row = 16 * r + (lane >> 2);
        L.ql_off[r] = row_off(row) + 16u * (uint32_t)((lane & 3) ^ ((row >> 2) & 3));
    }
    {
        const int row = lane >> 1;
        L.qh_off = row_off(row) + 128u + 16u * (uint32_t)((lane & 1) ^ ((row >> 3) & 1));
    }
    L.h_off = row_off(lane & 31) + (lane < 32 ? 192u : 194u);
#pragma unroll
    for (int i = 0; i < LaneQ6<MB>::kARounds; i++) {
        const int idx = tid + i * kThreads;
        L.a_off[i] = (uint32_t)((idx / BM) * Mp + idx % BM);
    }
    uint4 *qa = qbase + L.wave * kQ6Stage, *qb = qa + NW * kQ6Stage, *qc = qb + NW * kQ6Stage;
    uint4 *hw = hb + L.wave * 64;
    const uint8_t *wblk = W + (size_t)n0 * row_bytes;

    AccQ6<MB> R;
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) R.acc[i][r] = 0.0f, R.part[i][r] = 0.0f;

    {
        const uint8_t *blk = wblk + (size_t)sb0 * kQ6Bytes;
        dma16(blk + L.h_off, hw);
#pragma unroll
        for (int r = 0; r < 2; r++) {
            dma16(blk + L.ql_off[r], qa + r * 64);
            dma16(blk + 64 + L.ql_off[r], qb + r * 64);
        }
        dma16(blk + L.qh_off, qa + 128);
        dma16(blk + 32 + L.qh_off, qb + 128);
        const uint4 *xa = xs + (size_t)(sb0 * 2 * kGroups) * Mp + m0;
#pragma unroll
        for (int i = 0; i < LaneQ6<MB>::kARounds; i++) dma16(xa + L.a_off[i], a0 + i * kThreads + L.wave * 64);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();

    for (int s = 0; s < cnt; s++) {
        const int sb = sb0 + s;
        const int sbn = sb + 1 < spr ? sb + 1 : spr - 1;
        const uint8_t *blkn = wblk + (size_t)sbn * kQ6Bytes;
        rw_half_q6<MB, 0>(a0, a1, qa, qc, hw, xs + (size_t)((sb * 2 + 1) * kGroups) * Mp + m0, blkn, blkn, L, R);
        barrier_keep<3>();
        rw_half_q6<MB, 1>(a1, a0, qb, qa, hw, xs + (size_t)(sbn * 2 * kGroups) * Mp + m0, blkn, nullptr, L, R);
        barrier_keep<3>();
        uint4 *t = qc;
        qc = qb, qb = qa, qa = t;
    }

    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the last copies (past the end) have landed
    __syncthreads();
    store_tile<MB>(R.acc, smem, L.wave, L.col, L.g, m0, n0, M, N, Mp, rowscale, yg, partial, mode, blockIdx.z);
}

// ------------------------------------------------------------------------------------------------
// Q8_0 (crates/pmetal-gguf/src/quantize.rs:268-300: 34-byte blocks of 32: f16 d, 32 int8; value d * q).  The int8
// quants are exact in f16, so the B tile is q itself and d, one per 32 elements, multiplies the fp32 partial
// sum of two k-steps.  That is 16 fp32 FMAs per matrix instruction pair and output block: this kernel is bound
// by its VALU work, not by the matrix pipe.  A block is 34 bytes, so nothing in a row is aligned to more than
// 2 bytes: every lane (row n, half g) loads its own 8 quants per k-step and the scales straight from global
// memory into registers, one half super-block (four blocks) ahead; the activations go through LDS as in the
// kernels above (natural element order).
// ------------------------------------------------------------------------------------------------
struct __attribute__((packed, aligned(2))) q8_u32x2 {
    uint32_t x, y;
};
typedef uint16_t q8_u16 __attribute__((aligned(2)));

struct Q8Half {       // one lane's share of four blocks
    uint32_t q[4][2][2];  // [block][k-step of the block][dword]
    uint32_t d[4];        // f16 bits
};

__device__ __forceinline__ void q8_load(const uint8_t *p, const int g, Q8Half &h) {  // p: the lane's row at the half
#pragma unroll
    for (int b = 0; b < 4; b++) {
        h.d[b] = *reinterpret_cast<const q8_u16 *>(p + 34 * b);
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
            const q8_u32x2 v = *reinterpret_cast<const q8_u32x2 *>(p + 34 * b + 2 + 16 * tt + 8 * g);
            h.q[b][tt][0] = v.x, h.q[b][tt][1] = v.y;
        }
    }
}

// 8 int8 -> 8 exact f16: q + 128 as an unsigned byte b, 0x6400 | b is the f16 1024 + b, minus 1152.
__device__ __forceinline__ half8_t q8_operand(const uint32_t w0, const uint32_t w1) {
    const half2_t m1152 = {(_Float16)-1152.0f, (_Float16)-1152.0f};
    const uint32_t u0 = w0 ^ 0x80808080u, u1 = w1 ^ 0x80808080u;
    const half2_t r0 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, u0, 0x04010400u)) + m1152;
    const half2_t r1 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, u0, 0x04030402u)) + m1152;
    const half2_t r2 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, u1, 0x04010400u)) + m1152;
    const half2_t r3 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, u1, 0x04030402u)) + m1152;
    return half8_t{r0[0], r0[1], r1[0], r1[1], r2[0], r2[1], r3[0], r3[1]};
}

template <int MB>
__device__ __forceinline__ void rw_half_q8(const uint4 *__restrict__ a_cur, uint4 *__restrict__ a_nxt,
                                           const uint4 *__restrict__ xs_nxt, const uint8_t *w_nxt, const Q8Half &cur,
                                           Q8Half &nxt, const LaneQ6<MB> &L, float16_t (&acc)[MB]) {
    constexpr int BM = 32 * MB, kThreads = 512;
    const int col = L.col, g = L.g;
    // `cur` was requested a whole half super-block ago and is the only thing still outstanding; waiting for it
    // here, before the new requests go out, keeps that wait from covering them too
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
#pragma unroll
    for (int i = 0; i < LaneQ6<MB>::kARounds; i++) dma16(xs_nxt + L.a_off[i], a_nxt + i * kThreads + L.wave * 64);
    __builtin_amdgcn_sched_barrier(0);  // the 12 register loads below stay the newest requests (see barrier_keep)
    q8_load(w_nxt, g, nxt);
    __builtin_amdgcn_sched_barrier(0);

    half8_t af[2][MB];
#pragma unroll
    for (int i = 0; i < MB; i++) af[0][i] = __builtin_bit_cast(half8_t, a_cur[g * BM + 32 * i + col]);
#pragma unroll
    for (int b = 0; b < 4; b++) {
        float16_t part[MB];
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
            const int t = 2 * b + tt;
            const half8_t bop = q8_operand(cur.q[b][tt][0], cur.q[b][tt][1]);
#pragma unroll
            for (int i = 0; i < MB; i++) {
                if (tt == 0) {
                    float16_t z;
#pragma unroll
                    for (int r = 0; r < 16; r++) z[r] = 0.0f;
                    part[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[t & 1][i], bop, z, 0, 0, 0);
                } else {
                    part[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[t & 1][i], bop, part[i], 0, 0, 0);
                }
                if (i == 0 && t < 7) {  // the next step's fragments, behind the first product of this step
#pragma unroll
                    for (int ii = 0; ii < MB; ii++)
                        af[(t + 1) & 1][ii] = __builtin_bit_cast(half8_t, a_cur[((t + 1) * 2 + g) * BM + 32 * ii + col]);
                }
            }
        }
        const float d = f16_bits_to_f32(cur.d[b]);
#pragma unroll
        for (int i = 0; i < MB; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][r] = __builtin_fmaf(d, part[i][r], acc[i][r]);
    }
}

// grid and modes as for k_qgemm_rw; 8 waves = 256 weight rows per workgroup; LDS holds the two activation stages
template <int MB>
__global__ __launch_bounds__(512, 1) void k_qgemm_rw_q8(const uint8_t *__restrict__ W, const uint4 *__restrict__ xs,
                                                         const float *__restrict__ rowscale, void *__restrict__ yg,
                                                         float *__restrict__ partial, int M, int Mp, int N, int spr, int chunk,
                                                         int mode) {
    constexpr int BM = 32 * MB, kThreads = 512;
    extern __shared__ uint4 smem[];
    uint4 *a0 = smem, *a1 = a0 + kQ6Groups * BM;
    const int tid = threadIdx.x;
    LaneQ6<MB> L;
    L.wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    L.col = lane & 31, L.g = lane >> 5;
    const int n0 = blockIdx.x * 256, m0 = blockIdx.y * BM;
    const int n = n0 + 32 * L.wave + L.col;
    const int sb0 = blockIdx.z * chunk;
    const int cnt = spr - sb0 < chunk ? spr - sb0 : chunk;
    const size_t row_bytes = (size_t)spr * 272;
    // this lane's row (rows past N repeat the last) at the first block of super-block sb0, and at its last half
    const uint8_t *wp = W + (size_t)(n < N ? n : N - 1) * row_bytes + (size_t)sb0 * 272;
    const uint8_t *wlast = W + (size_t)(n < N ? n : N - 1) * row_bytes + (size_t)(spr * 2 - 1) * 136;
#pragma unroll
    for (int i = 0; i < LaneQ6<MB>::kARounds; i++) {
        const int idx = tid + i * kThreads;
        L.a_off[i] = (uint32_t)((idx / BM) * Mp + idx % BM);
    }
    float16_t acc[MB];
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.0f;

    Q8Half ha, hb;
    q8_load(wp, L.g, ha);
    {
        const uint4 *xa = xs + (size_t)(sb0 * 2 * kGroups) * Mp + m0;
#pragma unroll
        for (int i = 0; i < LaneQ6<MB>::kARounds; i++) dma16(xa + L.a_off[i], a0 + i * kThreads + L.wave * 64);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();

    for (int s = 0; s < cnt; s++) {
        const int sb = sb0 + s;
        const int sbn = sb + 1 < spr ? sb + 1 : spr - 1;  // the copies for "the next super-block" stay inside the matrix
        const uint8_t *w1 = wp + 136, *w2 = wp + 272;
        rw_half_q8<MB>(a0, a1, xs + (size_t)((sb * 2 + 1) * kGroups) * Mp + m0, w1, ha, hb, L, acc);
        barrier_keep<12>();
        rw_half_q8<MB>(a1, a0, xs + (size_t)(sbn * 2 * kGroups) * Mp + m0, w2 < wlast ? w2 : wlast, hb, ha, L, acc);
        barrier_keep<12>();
        wp = w2;
    }

    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the last register loads and copies (past the end) are done
    __syncthreads();
    store_tile<MB>(acc, smem, L.wave, L.col, L.g, m0, n0, M, N, Mp, rowscale, yg, partial, mode, blockIdx.z);
}

// ------------------------------------------------------------------------------------------------
// Q4_K with at most 16 activation rows (a decode batch, a speculative window) and rows of at most 16 super-blocks: the
// weights are read once, at the pace of the GEMV, and nothing but the pre-pass runs before or after this kernel.
//   * v_mfma_f32_16x16x32_f16: 16 activation rows x 16 weight rows x 32 k.  Lane (r = lane % 16, kg = lane / 16) holds
//     the eight k of k-group kg for activation row r (first operand) resp. weight row r (second operand); the output
//     tile has column lane % 16 (weight row) and rows 4 (lane / 16) + 0..3 (activation rows).
//   * A wave owns one or two super-block columns of W (wave w: super-blocks w and w + 8) and walks the row tiles of its
//     workgroup.  Its activation operands for those super-blocks -- per super-block eight items (k-step t, k-group kg)
//     and the item of sub-block sums, exactly the items the pre-pass writes -- are loaded once and stay in registers.
//   * Per row tile the wave copies its one or two super-blocks of the 16 rows (144 or 288 contiguous bytes per row)
//     through registers into its own piece of LDS with whole-wave 16-byte loads, a row tile ahead (every load
//     unconditional, so the outstanding loads are counted exactly); a lane then takes the 16-byte header of its weight
//     row and the 32 quant bytes of sub-blocks 2 kg and 2 kg + 1 (dword t of them is its operand of k-step t) out of
//     LDS.  LDS executes a wave's instructions in order, so the copy needs no barrier.  (Each lane loading its own three
//     pieces from global memory -- 16-byte pieces 32 bytes apart, 16 rows per request -- was 4 % slower per call.)
//     Arithmetic as in the large kernel: exact integer tiles sc * q, d on the fp32 sum of a super-block, the min term as
//     one more matrix instruction over exact head + tail splits.
//   * The waves' 16 x 16 partial tiles (one per super-block column) are added through LDS in wave order by the first
//     wave (one barrier per row tile, no partial tiles in global memory, no reduction kernel; the result does not
//     depend on scheduling) and collected in LDS; the workgroup stores its columns of y after its last row tile, scaled
//     by the rows' powers of two.  No store and no other load is issued inside the streaming loop: on this target stores
//     share the loads' counter, and one of them in flight turns every counted wait into a wait for everything.
// ------------------------------------------------------------------------------------------------
typedef float float4_t __attribute__((ext_vector_type(4)));
constexpr int kSmallWaves = 8;  // waves per workgroup (fewer when a row has fewer super-blocks); 16 waves of one super-block each run alike
constexpr int kSmallDepth = 2;  // row tiles in flight per wave (four are slower: 16.5 against 12.7 us at 14336 x 4096)
constexpr int kSmallMaxM = 16, kSmallMaxSpr = 16;
constexpr int kSmallMaxM2 = 32;  // Q4_K and Q5_K: two 16-row blocks of activations per weight operand

// The two steps the short-batch kernels share.  A row tile's 16 x 16 partial tiles, one per wave: every wave leaves its
// own in LDS, and after one barrier the first wave adds them in wave order and keeps the sum as finished tile `ti` (the
// next tile writes the other buffer; the one after that comes behind the next barrier).
//
// A workgroup with few tiles (at most kSmallKeepTiles) keeps every wave's partial tile of every row tile instead
// (`keep`, [tile][wave][lane]) and adds them after the last one, in the same wave order: its waves then meet at one
// barrier, not at one per tile.
constexpr int kSmallKeepTiles = 8;
__device__ __forceinline__ void small_add_waves(float4_t (&red)[2][kSmallWaves][64], float4_t *keep, int ti, int wave, int nwaves,
                                                int lane, const float4_t acc, float4_t *out_tiles) {
    if (keep) {  // workgroup-uniform
        keep[(ti * nwaves + wave) * 64 + lane] = acc;
        return;
    }
    const int buf = ti & 1;
    red[buf][wave][lane] = acc;
    __syncthreads();
    if (wave == 0) {
        float4_t v = red[buf][0][lane];
        for (int q = 1; q < nwaves; q++) {
            const float4_t u = red[buf][q][lane];
#pragma unroll
            for (int r = 0; r < 4; r++) v[r] += u[r];
        }
        out_tiles[ti * 64 + lane] = v;
    }
}

__device__ __forceinline__ void small_add_kept(const float4_t *keep, int n_tiles, int wave, int nwaves, int lane, float4_t *out_tiles) {
    if (!keep) return;
    __syncthreads();
    for (int ti = wave; ti < n_tiles; ti += nwaves) {
        float4_t v = keep[(ti * nwaves) * 64 + lane];
        for (int q = 1; q < nwaves; q++) {
            const float4_t u = keep[(ti * nwaves + q) * 64 + lane];
#pragma unroll
            for (int r = 0; r < 4; r++) v[r] += u[r];
        }
        out_tiles[ti * 64 + lane] = v;
    }
}

// After the last tile: y[m][16 t0 + j] for j over the workgroup's columns (consecutive threads store consecutive columns of
// one row), scaled by the rows' powers of two; or, when a long row is cut into runs over the grid's second dimension,
// the fp32 partial tile of this run, not yet scaled, for k_rw_reduce.
// (mt: 16-row blocks of activations per row tile of weights; the finished tile of block b of row tile ti is slot ti * mt + b)
__device__ __forceinline__ void small_store(const float4_t *out_tiles, int t0, int t1, int M, int Mp, int N,
                                            const float *__restrict__ rowscale, void *__restrict__ yg, int ybf16,
                                            float *__restrict__ partial, const int mt = 1) {
    __syncthreads();
    const int cols = (t1 - t0) * 16;
    for (int idx = (int)threadIdx.x; idx < M * cols; idx += (int)blockDim.x) {
        const int m = idx / cols, j = idx - m * cols;
        const int n = t0 * 16 + j;
        if (n < N) {
            const float sum = out_tiles[((j >> 4) * mt + (m >> 4)) * 64 + ((m & 15) >> 2) * 16 + (j & 15)][m & 3];
            const float o = sum * rowscale[m];
            if (partial) partial[((size_t)blockIdx.y * Mp + m) * N + n] = sum;
            else if (ybf16) reinterpret_cast<uint16_t *>(yg)[(size_t)m * N + n] = (uint16_t)bf16_rne_bits(o);
            else reinterpret_cast<float *>(yg)[(size_t)m * N + n] = o;
        }
    }
}

template <int NSB, int FMT = 0>
struct SmallRun {
    static constexpr int kPerSb = BlockFmt<FMT>::kBytes / 16;  // 16-byte pieces of a super-block: 9 (Q4_K) or 11 (Q5_K)
    static constexpr int kPieces = 16 * kPerSb * NSB;          // ... of a row tile's NSB super-blocks
    static constexpr int kLoads = (kPieces + 63) / 64;         // per lane: 5 or 3 (Q5_K: 6 or 3)
    u32x4 piece[kLoads];  // (a vector type: copies of it are loads and stores that stay in registers)
};

// FMT 1: Q5_K -- eleven pieces per super-block (header, two of qh, eight of quants); a lane takes the qh bytes of its two
// sub-blocks out of its stage as well and ors the fifth bits into the quant dwords as in the large kernel.
// MT: 16-row blocks of activations (1: at most 16 rows, 2: at most 32); a weight operand then feeds MT matrix instructions.
template <int ORDER, int NSB, int FMT = 0, int MT = 1>
__global__ __launch_bounds__(64 * kSmallWaves) void k_qgemm_small(const uint8_t *__restrict__ W, const uint4 *__restrict__ xs,
                                                                   const float *__restrict__ rowscale, void *__restrict__ yg, int M,
                                                                   int Mp, int N, int spr, int tiles, int tiles_per_wg, int ybf16,
                                                                   float *__restrict__ partial) {
    __shared__ float4_t red[2][kSmallWaves][64];
    extern __shared__ float4_t dyn[];  // out_tiles [tiles_per_wg rounded up to whole rounds][64]: lane slots of the finished tiles; then the waves' stages
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nwaves = (int)(blockDim.x >> 6);
    const int nl = lane & 15, kg = lane >> 4;
    const uint32_t low = kg < 2 ? 0xFFFFFFFFu : 0u;
    const int rounds = (tiles_per_wg + kSmallDepth - 1) / kSmallDepth;
    float4_t *out_tiles = dyn;
    float4_t *keep = tiles_per_wg * MT <= kSmallKeepTiles ? dyn + rounds * kSmallDepth * MT * 64 : nullptr;
    u32x4 *stage = reinterpret_cast<u32x4 *>(dyn + rounds * kSmallDepth * MT * 64 * (keep ? 1 + nwaves : 1)) + wave * SmallRun<NSB, FMT>::kPieces;
    int sbi[NSB];
    bool sbv[NSB];  // wave-uniform
#pragma unroll
    for (int i = 0; i < NSB; i++) {
        sbi[i] = (int)blockIdx.y * (NSB * nwaves) + NSB * wave + i;  // adjacent super-blocks: one contiguous piece of every row per wave; workgroup row blockIdx.y of the grid takes the blockIdx.y-th run of NSB * waves super-blocks of a long row
        sbv[i] = sbi[i] < spr;
        sbi[i] = sbv[i] ? sbi[i] : 0;
    }
    // activation operands of this wave's super-blocks: item (2 sb + kg / 2, group 2 t + kg % 2) of rows nl (and 16 + nl), and the sums item
    half8_t af[NSB][MT][8], asum[NSB][MT];
#pragma unroll
    for (int i = 0; i < NSB; i++)
#pragma unroll
        for (int b = 0; b < MT; b++) {
            const uint4 *base = xs + (size_t)((2 * sbi[i] + (kg >> 1)) * kGroups) * Mp + 16 * b + nl;
#pragma unroll
            for (int t = 0; t < 8; t++) af[i][b][t] = __builtin_bit_cast(half8_t, base[(size_t)(2 * t + (kg & 1)) * Mp]);
            asum[i][b] = __builtin_bit_cast(half8_t, base[(size_t)(16 + (kg & 1)) * Mp]);
            if (!sbv[i]) {  // a super-block past the end of the row multiplies zeros (no branch in the streaming loop)
                const half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int t = 0; t < 8; t++) af[i][b][t] = z;
                asum[i][b] = z;
            }
        }
    const int t0 = (int)blockIdx.x * tiles_per_wg;
    const int t1 = t0 + tiles_per_wg < tiles ? t0 + tiles_per_wg : tiles;  // t1 > t0 by the launch geometry
    constexpr int kPerSb = SmallRun<NSB, FMT>::kPerSb, kBlockBytes = BlockFmt<FMT>::kBytes, kQ0 = FMT ? 3 : 1;  // kQ0: first quant piece
    const uint32_t row_bytes = (uint32_t)spr * (uint32_t)kBlockBytes;
    // piece j of this lane: index lane + 64 j of the tile's 16 rows x 9 NSB pieces (a load past the last piece repeats it
    // and is dropped); a super-block past the end of the row is replaced by the row's first
    constexpr int kLoads = SmallRun<NSB, FMT>::kLoads, kPieces = SmallRun<NSB, FMT>::kPieces;
    uint32_t piece_row[kLoads], piece_off[kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; j++) {
        int idx = lane + 64 * j;
        idx = idx < kPieces ? idx : kPieces - 1;
        const int p = idx % (kPerSb * NSB);
        piece_row[j] = (uint32_t)(idx / (kPerSb * NSB));
        piece_off[j] = (uint32_t)(NSB == 2 && p >= kPerSb ? sbi[NSB - 1] : sbi[0]) * (uint32_t)kBlockBytes + 16u * (uint32_t)(p % kPerSb);
    }
    auto issue = [&](int ti, SmallRun<NSB, FMT> &w) __attribute__((always_inline)) {
        int tile = t0 + ti;
        tile = tile < t1 ? tile : t1 - 1;  // past the end: the last tile again (loaded, not used)
#pragma unroll
        for (int j = 0; j < kLoads; j++) {
            int n = tile * 16 + (int)piece_row[j];
            n = n < N ? n : N - 1;
            w.piece[j] = *reinterpret_cast<const u32x4 *>(W + ((uint32_t)n * row_bytes + piece_off[j]));  // the tensor is smaller than 4 GiB (checked by the launcher)
        }
    };
    const u32x4 *mine = stage + nl * (kPerSb * NSB);  // this lane's weight row in the stage
    auto consume = [&](int ti, const SmallRun<NSB, FMT> &w) __attribute__((always_inline)) {
        float4_t acc[MT];
#pragma unroll
        for (int b = 0; b < MT; b++) acc[b] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < kLoads; j++)
            if (lane + 64 * j < kPieces) stage[lane + 64 * j] = w.piece[j];
        // LDS executes a wave's instructions in order: the reads below see the writes above, and the next tile's
        // writes come after these reads
#pragma unroll
        for (int i = 0; i < NSB; i++) {
            const u32x4 hv = mine[kPerSb * i], qav = mine[kPerSb * i + kQ0 + 2 * kg], qbv = mine[kPerSb * i + kQ0 + 1 + 2 * kg];
            const uint4 hdr = make_uint4(hv.x, hv.y, hv.z, hv.w);
            // scales and mins of sub-blocks 2 kg and 2 kg + 1 (6-bit fields, crates/pmetal-gguf/src/quantize.rs:844-855)
            const uint32_t sh = 16u * (uint32_t)(kg & 1);
            const uint32_t yv = hdr.y >> sh, zv = hdr.z >> sh, wv = hdr.w >> sh;
            // sub-blocks 0..3 (kg < 2) and 4..7 store them differently; both forms are computed and one is picked by a
            // per-lane bit mask (a branch here would be taken by half of every wave)
            const uint32_t sc0 = ((yv & 63u) & low) | (((wv & 0xFu) | ((yv >> 2) & 0x30u)) & ~low);
            const uint32_t sc1 = (((yv >> 8) & 63u) & low) | ((((wv >> 8) & 0xFu) | ((yv >> 10) & 0x30u)) & ~low);
            const uint32_t mn0 = ((zv & 63u) & low) | ((((wv >> 4) & 0xFu) | ((zv >> 2) & 0x30u)) & ~low);
            const uint32_t mn1 = (((zv >> 8) & 63u) & low) | ((((wv >> 12) & 0xFu) | ((zv >> 10) & 0x30u)) & ~low);
            const _Float16 s0 = (_Float16)(float)sc0, s1 = (_Float16)(float)sc1;
            const _Float16 o0 = (_Float16)(-1024.0f * (float)sc0), o1 = (_Float16)(-1024.0f * (float)sc1);  // exact: sc <= 63
            const half2_t sc2[2] = {half2_t{s0, s0}, half2_t{s1, s1}}, off2[2] = {half2_t{o0, o0}, half2_t{o1, o1}};
            const uint32_t qd[8] = {qav.x, qav.y, qav.z, qav.w, qbv.x, qbv.y, qbv.z, qbv.w};
            // Q5_K: the fifth bits of k-step t.  GGML order: qh dword t (the same four bytes as quant dword t), bits 2 kg and
            // 2 kg + 1 of every byte.  REF order: byte 4 (2 kg + t / 4) + t % 4 of qh, i.e. of the lane's two qh dwords.
            uint32_t qh[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            if (FMT == 1) {
                if (ORDER == 1) {
                    const u32x4 ha = mine[kPerSb * i + 1], hb = mine[kPerSb * i + 2];
                    const uint32_t h8[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
#pragma unroll
                    for (int t = 0; t < 8; t++) qh[t] = h8[t] >> (2 * kg);
                } else {
                    const uint2 hp = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint8_t *>(mine + kPerSb * i + 1) + 8 * kg);
#pragma unroll
                    for (int t = 0; t < 8; t++) qh[t] = (t < 4 ? hp.x : hp.y) >> (8 * (t & 3));
                }
            }
            float4_t part[MT];
#pragma unroll
            for (int b = 0; b < MT; b++) part[b] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int t = 0; t < 8; t++) {
                Dq d;
#pragma unroll
                for (int c = 0; c < 4; c++) dq_chunk<ORDER, FMT>(c, t, qd[t], sc2, off2, d, qh[t]);
                const half8_t bv = d.value();
#pragma unroll
                for (int b = 0; b < MT; b++) part[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i][b][t], bv, part[b], 0, 0, 0);
            }
            // (of a super-block past the end of the row only zeros may enter the sums, whatever bytes were loaded for it)
            const float dmin = sbv[i] ? f16_bits_to_f32(hdr.x >> 16) : 0.0f, dd = sbv[i] ? f16_bits_to_f32(hdr.x & 0xFFFFu) : 0.0f;
            _Float16 h0, l0, h1, l1;
            neg_min_split(dmin, mn0, h0, l0);
            neg_min_split(dmin, mn1, h1, l1);
            const half8_t br = {h0, h0, l0, l0, h1, h1, l1, l1};
#pragma unroll
            for (int b = 0; b < MT; b++) {
                acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(asum[i][b], br, acc[b], 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; r++) acc[b][r] = __builtin_fmaf(dd, part[b][r], acc[b][r]);
            }
        }
#pragma unroll
        for (int b = 0; b < MT; b++) small_add_waves(red, keep, ti * MT + b, wave, nwaves, lane, acc[b], out_tiles);
    };
    static_assert(kSmallDepth == 2, "the ring is written out as two tiles");
    SmallRun<NSB, FMT> ring0, ring1;
    issue(0, ring0);
    issue(1, ring1);
    // Whole rounds of two tiles, with nothing conditional around the loads, so that the outstanding loads are counted
    // exactly at every wait; the tiles past the workgroup's last one are computed on repeated data and dropped.
    for (int rd = 0; rd < rounds; rd++) {
        consume(2 * rd, ring0);
        issue(2 * rd + 2, ring0);
        consume(2 * rd + 1, ring1);
        issue(2 * rd + 3, ring1);
    }
    small_add_kept(keep, rounds * kSmallDepth * MT, wave, nwaves, lane, out_tiles);
    small_store(out_tiles, t0, t1, M, Mp, N, rowscale, yg, ybf16, partial, MT);
}

// ------------------------------------------------------------------------------------------------
// The same for Q8_0 (34-byte blocks: f16 d, 32 int8).  A k-step of v_mfma_f32_16x16x32_f16 is one block: lane (r, kg)
// holds the eight quants 8 kg .. 8 kg + 7 of the block of weight row r, exact in f16, and the block's d multiplies the
// fp32 product tile of that one k-step.  A wave owns one or two runs of eight blocks (256 elements = 272 bytes) of every
// row, as the Q4_K kernel owns super-blocks.  Nothing in a row of 34-byte blocks is aligned to more than two bytes, and
// loads at such addresses are slow, so the wave copies the 16 x 272 bytes of a row tile's run -- 16-byte aligned at both
// ends -- through registers into its own piece of LDS with whole-wave 16-byte loads (the ring holds these pieces) and
// every lane takes its quants and scales out of LDS: aligned dwords, those of the even blocks shifted by two bytes.  LDS
// executes a wave's instructions in order, so the copy needs no barrier.  Ring, reduction over the waves and epilogue
// as above.
// ------------------------------------------------------------------------------------------------
constexpr int kQ8RunBytes = 272, kQ8TileRunPieces = 16 * kQ8RunBytes / 16;  // 272 pieces of 16 bytes: 4.25 per lane

// (one run's pieces: a tile of two runs is two of these, kept apart so that each stays in registers)
struct SmallRunQ8 {
    u32x4 piece[5];  // (a vector type: copies of it are loads and stores that stay in registers)
};

template <int NSB, int MT = 1>
__global__ __launch_bounds__(64 * kSmallWaves) void k_qgemm_small_q8(const uint8_t *__restrict__ W, const uint4 *__restrict__ xs,
                                                                      const float *__restrict__ rowscale, void *__restrict__ yg, int M,
                                                                      int Mp, int N, int spr, int tiles, int tiles_per_wg, int ybf16,
                                                                   float *__restrict__ partial) {
    __shared__ float4_t red[2][kSmallWaves][64];
    extern __shared__ float4_t dyn[];  // out_tiles [tiles_per_wg rounded up to whole rounds][64], then the waves' stages
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nwaves = (int)(blockDim.x >> 6);
    const int nl = lane & 15, kg = lane >> 4;
    const int rounds = (tiles_per_wg + kSmallDepth - 1) / kSmallDepth;
    float4_t *out_tiles = dyn;
    float4_t *keep = tiles_per_wg * MT <= kSmallKeepTiles ? dyn + rounds * kSmallDepth * MT * 64 : nullptr;
    u32x4 *stage = reinterpret_cast<u32x4 *>(dyn + rounds * kSmallDepth * MT * 64 * (keep ? 1 + nwaves : 1)) + wave * (NSB * kQ8TileRunPieces);
    int sbi[NSB];
    bool sbv[NSB];  // wave-uniform
#pragma unroll
    for (int i = 0; i < NSB; i++) {
        sbi[i] = (int)blockIdx.y * (NSB * nwaves) + NSB * wave + i;
        sbv[i] = sbi[i] < spr;
        sbi[i] = sbv[i] ? sbi[i] : 0;
    }
    // activation operands: block b of run sb holds elements 256 sb + 32 b ..; the item of its k-group kg is item
    // 4 (b % 4) + kg of half 2 sb + b / 4 (the pre-pass writes 16 items of eight consecutive elements per 128)
    half8_t af[NSB][MT][8];  // (MT 16-row blocks of activations: rows nl, 16 + nl)
#pragma unroll
    for (int i = 0; i < NSB; i++)
#pragma unroll
        for (int mb = 0; mb < MT; mb++)
#pragma unroll
            for (int b = 0; b < 8; b++) {
                const uint4 *item = xs + (size_t)((2 * sbi[i] + (b >> 2)) * kGroups + 4 * (b & 3) + kg) * Mp + 16 * mb + nl;
                af[i][mb][b] = __builtin_bit_cast(half8_t, *item);
                if (!sbv[i]) af[i][mb][b] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
            }
    const int t0 = (int)blockIdx.x * tiles_per_wg;
    const int t1 = t0 + tiles_per_wg < tiles ? t0 + tiles_per_wg : tiles;
    const uint32_t row_bytes = (uint32_t)spr * (uint32_t)kQ8RunBytes;
    // piece j of this lane: index lane + 64 j of the tile's 272 (the fifth exists for the first 16 lanes; the others load
    // the last piece again and drop it)
    uint32_t piece_row[5], piece_off[5];
#pragma unroll
    for (int j = 0; j < 5; j++) {
        int idx = lane + 64 * j;
        idx = idx < kQ8TileRunPieces ? idx : kQ8TileRunPieces - 1;
        piece_row[j] = (uint32_t)(idx / 17), piece_off[j] = 16u * (uint32_t)(idx % 17);
    }
    auto issue = [&](int ti, SmallRunQ8 &wa, SmallRunQ8 &wb) __attribute__((always_inline)) {
        int tile = t0 + ti;
        tile = tile < t1 ? tile : t1 - 1;  // past the end: the last tile again (loaded, not used)
#pragma unroll
        for (int j = 0; j < 5; j++) {
            int n = tile * 16 + (int)piece_row[j];
            n = n < N ? n : N - 1;
            const uint8_t *p = W + ((uint32_t)n * row_bytes + piece_off[j]);  // the tensor is smaller than 4 GiB (checked by the launcher)
#pragma unroll
            for (int i = 0; i < NSB; i++) (i == 0 ? wa : wb).piece[j] = *reinterpret_cast<const u32x4 *>(p + (uint32_t)sbi[i] * (uint32_t)kQ8RunBytes);
        }
    };
    const uint32_t *mine = reinterpret_cast<const uint32_t *>(stage) + nl * (kQ8RunBytes / 4);  // this lane's weight row in the stage
    auto consume = [&](int ti, const SmallRunQ8 &wa, const SmallRunQ8 &wb) __attribute__((always_inline)) {
        float4_t acc[MT];
#pragma unroll
        for (int mb = 0; mb < MT; mb++) acc[mb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        const float4_t none = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < NSB; i++) {
            u32x4 *st = stage + i * kQ8TileRunPieces;
            const SmallRunQ8 &w = i == 0 ? wa : wb;
#pragma unroll
            for (int j = 0; j < 4; j++) st[lane + 64 * j] = w.piece[j];
            if (lane < kQ8TileRunPieces - 256) st[lane + 256] = w.piece[4];
            // LDS executes a wave's instructions in order: the reads below see the writes above, and the next tile's
            // writes come after these reads
            const uint32_t *row = mine + i * (kQ8TileRunPieces * 4);
#pragma unroll
            for (int b = 0; b < 8; b++) {
                // block b starts at byte 34 b of the run: on a dword boundary for even b (d in the low half of that dword,
                // the quants from its high half on), two bytes past one for odd b (d in the high half of the dword below)
                uint32_t q0, q1, dbits;
                if ((b & 1) == 0) {
                    const uint32_t *p = row + (34 * b) / 4 + 2 * kg;
                    const uint32_t w0 = p[0], w1 = p[1], w2 = p[2];
                    q0 = __builtin_amdgcn_alignbit(w1, w0, 16), q1 = __builtin_amdgcn_alignbit(w2, w1, 16);
                    dbits = row[(34 * b) / 4] & 0xFFFFu;
                } else {
                    const uint32_t *p = row + (34 * b + 2) / 4 + 2 * kg;
                    q0 = p[0], q1 = p[1];
                    dbits = row[(34 * b - 2) / 4] >> 16;
                }
                // (of a run past the end of the row only zeros may enter the sums, whatever bytes were loaded for it)
                const float d = sbv[i] ? f16_bits_to_f32(dbits) : 0.0f;
                const half8_t bv = q8_operand(q0, q1);
#pragma unroll
                for (int mb = 0; mb < MT; mb++) {
                    const float4_t part = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i][mb][b], bv, none, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[mb][r] = __builtin_fmaf(d, part[r], acc[mb][r]);
                }
            }
        }
#pragma unroll
        for (int mb = 0; mb < MT; mb++) small_add_waves(red, keep, ti * MT + mb, wave, nwaves, lane, acc[mb], out_tiles);
    };
    static_assert(kSmallDepth == 2, "the ring is written out as two tiles");
    SmallRunQ8 ring0a, ring0b, ring1a, ring1b;  // (the b halves are unused with one run per wave)
    issue(0, ring0a, ring0b);
    issue(1, ring1a, ring1b);
    for (int rd = 0; rd < rounds; rd++) {
        consume(2 * rd, ring0a, ring0b);
        issue(2 * rd + 2, ring0a, ring0b);
        consume(2 * rd + 1, ring1a, ring1b);
        issue(2 * rd + 3, ring1a, ring1b);
    }
    small_add_kept(keep, rounds * kSmallDepth * MT, wave, nwaves, lane, out_tiles);
    small_store(out_tiles, t0, t1, M, Mp, N, rowscale, yg, ybf16, partial, MT);
}

// ------------------------------------------------------------------------------------------------
// The same for Q6_K (210-byte super-blocks: ql[128], qh[64], 16 int8 scales, f16 d; value d sc (q - 32),
// crates/pmetal-gguf/src/k_quants.rs:474-496); first for rows of a multiple of eight super-blocks, which start on
// 16-byte boundaries.  A k-step of v_mfma_f32_16x16x16_f16 is one sub-block of 16 elements: lane (r, kg) holds the
// four quants 4 kg .. 4 kg + 3 of the sub-block of weight row r as exact f16 (q - 32), and d sc of the sub-block
// multiplies the fp32 product tile of that step.  Sub-block (hh, g, lh) -- elements 128 hh + 32 g + 16 lh .. of the
// super-block -- takes the low (g < 2) or high nibbles of the ql dword at 64 hh + 32 (g % 2) + 16 lh + 4 kg, bits 2 g of
// the qh dword at 32 hh + 16 lh + 4 kg and scale 8 hh + 2 g + lh; its activation operand is one half of the pre-pass
// item (t = 4 lh + kg, g % 2) of half hh, which holds elements 32 (g % 2) + 4 t .. and those 64 further.
// A wave owns one or two adjacent super-blocks of every row.  Their bytes start (210 NSB wave) % 16 bytes into a
// 16-byte piece: the wave copies the pieces that cover them, row by row, through registers into its own LDS with
// whole-wave 16-byte loads (never past the piece that holds the tensor's last byte), and the lanes read aligned dwords;
// the fields of a super-block sit a wave-uniform 0 or 2 bytes off a dword boundary and are shifted into place.
// ------------------------------------------------------------------------------------------------
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
template <int NSB, bool ANY = false>
struct SmallQ6 {
    // 16-byte pieces that cover 210 NSB bytes from where a wave's super-blocks start in their piece: any even byte for one
    // super-block per wave or rows of any length (ANY), a multiple of four for pairs of super-blocks in rows that start
    // on 16-byte boundaries
    static constexpr int kRowPieces = NSB == 2 ? (ANY ? 28 : 27) : 14;
    static constexpr int kLoads = (16 * kRowPieces + 63) / 64;        // pieces per lane and row tile: 7 or 4
    static constexpr int kStageDwords = 16 * kRowPieces * 4 + 4;      // (+ one piece: the shifted reads look one dword ahead)
};
template <int NSB>
struct SmallRunQ6 {
    u32x4 piece[SmallQ6<NSB>::kLoads];  static_assert(SmallQ6<NSB, true>::kLoads == SmallQ6<NSB, false>::kLoads, "one ring for both forms");  // (a vector type: copies of it are loads and stores that stay in registers)
};

// ANY: rows of any number of super-blocks.  A row then starts at any even address, so where a wave's super-blocks lie in
// their first piece, and whether their fields sit two bytes off a dword boundary, differs from row to row (per lane); the
// last wave with work may own one super-block where the others own two.
template <int NSB, bool ANY>
__global__ __launch_bounds__(64 * kSmallWaves) void k_qgemm_small_q6(const uint8_t *__restrict__ W, const uint4 *__restrict__ xs,
                                                                      const float *__restrict__ rowscale, void *__restrict__ yg, int M,
                                                                      int Mp, int N, int spr, int tiles, int tiles_per_wg, int ybf16,
                                                                      uint32_t w_last, float *__restrict__ partial) {
    constexpr int P = SmallQ6<NSB, ANY>::kRowPieces, kLoads = SmallQ6<NSB, ANY>::kLoads;
    __shared__ float4_t red[2][kSmallWaves][64];
    extern __shared__ float4_t dyn[];  // out_tiles [tiles_per_wg rounded up to whole rounds][64], then the waves' stages
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nwaves = (int)(blockDim.x >> 6);
    const int nl = lane & 15, kg = lane >> 4;
    const int rounds = (tiles_per_wg + kSmallDepth - 1) / kSmallDepth;
    float4_t *out_tiles = dyn;
    float4_t *keep = tiles_per_wg <= kSmallKeepTiles ? dyn + rounds * kSmallDepth * 64 : nullptr;
    uint32_t *stage = reinterpret_cast<uint32_t *>(dyn + rounds * kSmallDepth * 64 * (keep ? 1 + nwaves : 1)) + wave * SmallQ6<NSB, ANY>::kStageDwords;
    // this wave's super-blocks sb0 .. sb0 + NSB - 1 (rows are whole multiples of eight super-blocks, so the NSB of a wave
    // exist together or not at all; a wave past the end of a long row's last run works on the row's first super-blocks
    // with zero activations and zero scales)
    const int sb_here = (int)blockIdx.y * (NSB * nwaves) + NSB * wave;
    bool sbv[NSB];  // wave-uniform; without ANY all of a wave's super-blocks exist or none
#pragma unroll
    for (int i = 0; i < NSB; i++) sbv[i] = sb_here + i < spr;
    const int sb0 = sbv[0] ? sb_here : 0;
    const uint32_t run_start = 210u * (uint32_t)sb0, delta = run_start & 15u;
    // activation operands: item (t = 4 lh + kg, gp) of half 2 sb + hh; index [hh][lh][gp]
    half8_t af[NSB][2][2][2];
#pragma unroll
    for (int i = 0; i < NSB; i++)
#pragma unroll
        for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int lh = 0; lh < 2; lh++)
#pragma unroll
                for (int gp = 0; gp < 2; gp++) {
                    const uint4 *item = xs + (size_t)((2 * (sbv[i] ? sb0 + i : 0) + hh) * kGroups + 2 * (4 * lh + kg) + gp) * Mp + nl;
                    af[i][hh][lh][gp] = __builtin_bit_cast(half8_t, *item);
                    if (!sbv[i]) af[i][hh][lh][gp] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
                }
    const int t0 = (int)blockIdx.x * tiles_per_wg;
    const int t1 = t0 + tiles_per_wg < tiles ? t0 + tiles_per_wg : tiles;
    const uint32_t row_bytes = (uint32_t)spr * 210u;
    uint32_t piece_row[kLoads], piece_off[kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; j++) {
        int idx = lane + 64 * j;
        idx = idx < 16 * P ? idx : 16 * P - 1;  // (the last load of a lane may not exist: it repeats the last piece and is dropped)
        piece_row[j] = (uint32_t)(idx / P), piece_off[j] = (ANY ? 0u : run_start & ~15u) + 16u * (uint32_t)(idx % P);
    }
    auto issue = [&](int ti, SmallRunQ6<NSB> &w) __attribute__((always_inline)) {
        int tile = t0 + ti;
        tile = tile < t1 ? tile : t1 - 1;  // past the end: the last tile again (loaded, not used)
#pragma unroll
        for (int j = 0; j < kLoads; j++) {
            int n = tile * 16 + (int)piece_row[j];
            n = n < N ? n : N - 1;
            uint32_t a = (uint32_t)n * row_bytes + piece_off[j];  // the tensor is smaller than 4 GiB (checked by the launcher)
            if (ANY) a = (((uint32_t)n * row_bytes + run_start) & ~15u) + piece_off[j];  // from the piece that holds the run's first byte in this row
            a = a < w_last ? a : w_last;  // a piece past the one with the tensor's last byte holds nothing of this run
            w.piece[j] = *reinterpret_cast<const u32x4 *>(W + a);
        }
    };
    const uint32_t *mine = stage + nl * (P * 4);  // this lane's weight row in the stage (dwords)
    auto consume = [&](int ti, const SmallRunQ6<NSB> &w) __attribute__((always_inline)) {
        float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
        const float4_t none = {0.0f, 0.0f, 0.0f, 0.0f};
        u32x4 *st = reinterpret_cast<u32x4 *>(stage);
#pragma unroll
        for (int j = 0; j < kLoads; j++)
            if (lane + 64 * j < 16 * P) st[lane + 64 * j] = w.piece[j];
        // LDS executes a wave's instructions in order: the reads below see the writes above, and the next tile's
        // writes come after these reads
        uint32_t delta_row = delta;
        if (ANY) {  // of the row this lane reads, as issue() took it
            int tile = t0 + ti;
            tile = tile < t1 ? tile : t1 - 1;
            int n = tile * 16 + nl;
            n = n < N ? n : N - 1;
            delta_row = ((uint32_t)n * row_bytes + run_start) & 15u;
        }
#pragma unroll
        for (int i = 0; i < NSB; i++) {
            const uint32_t at = delta_row + 210u * (uint32_t)i;  // byte of the super-block in the lane's staged row (wave-uniform without ANY)
            const uint32_t sh = 8u * (at & 2u);
            const uint32_t *blk = mine + (at >> 2);
            auto field = [&](int dword) -> uint32_t {  // the dword at byte 4 * dword of the super-block
                return __builtin_amdgcn_alignbit(blk[dword + 1], blk[dword], sh);
            };
            uint32_t sc[4];
#pragma unroll
            for (int q = 0; q < 4; q++) sc[q] = field(48 + q);
            const float d = sbv[i] ? f16_bits_to_f32(field(52) & 0xFFFFu) : 0.0f;
#pragma unroll
            for (int hh = 0; hh < 2; hh++)
#pragma unroll
                for (int lh = 0; lh < 2; lh++) {
                    const uint32_t qh = field(32 + 8 * hh + 4 * lh + kg);
#pragma unroll
                    for (int gp = 0; gp < 2; gp++) {
                        const uint32_t ql = field(16 * hh + 8 * gp + 4 * lh + kg);
                        const half8_t a8 = af[i][hh][lh][gp];
#pragma unroll
                        for (int up = 0; up < 2; up++) {  // group g = gp + 2 up: the low, then the high nibbles
                            const int g = gp + 2 * up;
                            const uint32_t v = ((ql >> (4 * up)) & 0x0F0F0F0Fu) | (((qh >> (2 * g)) & 0x03030303u) << 4);
                            // 0x6400 | q is the f16 1024 + q; minus 1056 leaves q - 32, exact
                            const half2_t m1056 = {(_Float16)-1056.0f, (_Float16)-1056.0f};
                            const half2_t b01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u)) + m1056;
                            const half2_t b23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u)) + m1056;
                            const half4_t b4 = {b01[0], b01[1], b23[0], b23[1]};
                            const half4_t a4 = up ? half4_t{a8[4], a8[5], a8[6], a8[7]} : half4_t{a8[0], a8[1], a8[2], a8[3]};
                            const float4_t part = __builtin_amdgcn_mfma_f32_16x16x16f16(a4, b4, none, 0, 0, 0);
                            const int si = 8 * hh + 2 * g + lh;  // the sub-block's scale byte
                            const float s = d * (float)((int)(sc[si >> 2] << (24 - 8 * (si & 3))) >> 24);
#pragma unroll
                            for (int r = 0; r < 4; r++) acc[r] = __builtin_fmaf(s, part[r], acc[r]);
                        }
                    }
                }
        }
        small_add_waves(red, keep, ti, wave, nwaves, lane, acc, out_tiles);
    };
    static_assert(kSmallDepth == 2, "the ring is written out as two tiles");
    SmallRunQ6<NSB> ring0, ring1;
    issue(0, ring0);
    issue(1, ring1);
    for (int rd = 0; rd < rounds; rd++) {
        consume(2 * rd, ring0);
        issue(2 * rd + 2, ring0);
        consume(2 * rd + 1, ring1);
        issue(2 * rd + 3, ring1);
    }
    small_add_kept(keep, rounds * kSmallDepth, wave, nwaves, lane, out_tiles);
    small_store(out_tiles, t0, t1, M, Mp, N, rowscale, yg, ybf16, partial);
}

// y[m][n] = rowscale[m] * (partial[0][m][n] + partial[1][m][n] + ...), added in this order
template <bool YBF16>
__global__ __launch_bounds__(256) void k_rw_reduce(const float *__restrict__ partial, int splits, int M, int Mp, int N,
                                                    const float *__restrict__ rowscale, void *__restrict__ yg) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)M * N) return;
    const int m = (int)(idx / N);
    const size_t plane = (size_t)Mp * N;
    float s = partial[idx];
    for (int z = 1; z < splits; z++) s += partial[(size_t)z * plane + idx];
    const float v = s * rowscale[m];
    if (YBF16) {
        uint32_t u = __builtin_bit_cast(uint32_t, v);
        u = ((u & 0x7FFFFFFFu) > 0x7F800000u) ? ((u >> 16) | 0x40u) : ((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
        reinterpret_cast<uint16_t *>(yg)[idx] = (uint16_t)u;
    } else {
        reinterpret_cast<float *>(yg)[idx] = v;
    }
}

// The same over eight consecutive outputs of one row per thread (N a multiple of 8): 16-byte loads and stores.
template <bool YBF16>
__global__ __launch_bounds__(256) void k_rw_reduce8(const float *__restrict__ partial, int splits, int M, int Mp, int N,
                                                     const float *__restrict__ rowscale, void *__restrict__ yg) {
    const size_t idx = ((size_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (idx >= (size_t)M * N) return;
    const int m = (int)(idx / N);
    const size_t plane = (size_t)Mp * N;
    const float4 *p = reinterpret_cast<const float4 *>(partial + idx);
    float4 a = p[0], b = p[1];
    for (int z = 1; z < splits; z++) {
        const float4 *q = reinterpret_cast<const float4 *>(partial + (size_t)z * plane + idx);
        const float4 c = q[0], d = q[1];
        a.x += c.x, a.y += c.y, a.z += c.z, a.w += c.w;
        b.x += d.x, b.y += d.y, b.z += d.z, b.w += d.w;
    }
    const float sc = rowscale[m];
    const float v[8] = {a.x * sc, a.y * sc, a.z * sc, a.w * sc, b.x * sc, b.y * sc, b.z * sc, b.w * sc};
    if (YBF16) {
        *reinterpret_cast<uint4 *>(reinterpret_cast<uint16_t *>(yg) + idx) =
            make_uint4(bf16_rne_bits(v[0]) | (bf16_rne_bits(v[1]) << 16), bf16_rne_bits(v[2]) | (bf16_rne_bits(v[3]) << 16),
                       bf16_rne_bits(v[4]) | (bf16_rne_bits(v[5]) << 16), bf16_rne_bits(v[6]) | (bf16_rne_bits(v[7]) << 16));
    } else {
        float4 *o = reinterpret_cast<float4 *>(reinterpret_cast<float *>(yg) + idx);
        o[0] = make_float4(v[0], v[1], v[2], v[3]);
        o[1] = make_float4(v[4], v[5], v[6], v[7]);
    }
}

template <int MB, int NR, int NW, int FMT = 0>
constexpr size_t rw_lds_bytes() {
    const size_t stages = (size_t)(2 * kGroups * 32 * MB + NW * NR * (3 * 128 + 64 + (FMT ? 64 : 0))) * 16;
    return stages > tile_lds_bytes<MB, NW>() ? stages : tile_lds_bytes<MB, NW>();
}

// ------------------------------------------------------------------------------------------------
// The same for Q3_K and Q2_K (sixteen 16-element sub-blocks).  Lane (r, kg) of v_mfma_f32_16x16x32_f16 stands where lane
// (n, g) of half h stands in the large kernel, with h = kg / 2 and g = kg % 2: the 16 bytes 16 kg .. of the 64 quant bytes
// of weight row r, whose dword t / 2 gives k-step t its eight values, against the pre-pass's item (2 sb + h, 2 t + g); four
// scales per lane; the sub-block sums of the activations (items 16 + g and 18 + g of the half) against the negated min
// coefficients in two further matrix instructions.  Blocks are 84 / 110 bytes and a lane needs few of them, so every lane
// loads its own: Q2_K rows start at multiples of four bytes, the quant piece, the scale bytes of its half and the d / dmin
// dword are plain loads; Q3_K blocks start at any even address, so a lane loads the aligned dwords that cover its pieces
// (quants and hmask: five; scales and d: four -- every one of them holds bytes of the block, none lies wholly past it) and
// shifts them by the block's 0 or 16 bits.  Ring, reduction over the waves and epilogue as above.
// ------------------------------------------------------------------------------------------------
struct __attribute__((packed, aligned(4))) u32x4_a4 {  // sixteen bytes at a 4-byte aligned address
    uint32_t x, y, z, w;
};
struct __attribute__((packed, aligned(4))) u32x2_a4 {
    uint32_t x, y;
};
__device__ __forceinline__ u32x4 load16_a4(const uint8_t *p) {
    const u32x4_a4 v = *reinterpret_cast<const u32x4_a4 *>(p);
    return u32x4{v.x, v.y, v.z, v.w};
}

template <int FMT, int NSB>
struct SmallRun16 {  // what a lane holds of a row tile
    u32x4 q[NSB];          // quant piece (Q3_K: from the dword boundary below it)
    uint32_t qx[NSB];      // Q3_K: the dword behind it
    u32x4 hm[NSB];         // Q3_K: hmask bytes 16 g ..
    uint32_t hmx[NSB];
    u32x4 sc[NSB];         // Q3_K: scales and d; Q2_K: x, y = scale bytes 8 h .., z = d | dmin << 16
};

template <int FMT, int NSB, int MT = 1>
__global__ __launch_bounds__(64 * kSmallWaves) void k_qgemm_small16(const uint8_t *__restrict__ W, const uint4 *__restrict__ xs,
                                                                     const float *__restrict__ rowscale, void *__restrict__ yg, int M,
                                                                     int Mp, int N, int spr, int tiles, int tiles_per_wg, int ybf16,
                                                                     float *__restrict__ partial) {
    using B = Block16<FMT>;
    __shared__ float4_t red[2][kSmallWaves][64];
    extern __shared__ float4_t dyn[];  // out_tiles [tiles_per_wg rounded up to whole rounds][64], then the kept partial tiles
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nwaves = (int)(blockDim.x >> 6);
    const int nl = lane & 15, kg = lane >> 4;
    const uint32_t h = (uint32_t)(kg >> 1), g = (uint32_t)(kg & 1);
    const int rounds = (tiles_per_wg + kSmallDepth - 1) / kSmallDepth;
    float4_t *out_tiles = dyn;
    float4_t *keep = tiles_per_wg * MT <= kSmallKeepTiles ? dyn + rounds * kSmallDepth * MT * 64 : nullptr;
    int sbi[NSB];
    bool sbv[NSB];  // wave-uniform
#pragma unroll
    for (int i = 0; i < NSB; i++) {
        sbi[i] = (int)blockIdx.y * (NSB * nwaves) + NSB * wave + i;
        sbv[i] = sbi[i] < spr;
        sbi[i] = sbv[i] ? sbi[i] : 0;
    }
    half8_t af[NSB][MT][8], asum[NSB][MT][2];  // (MT 16-row blocks of activations: rows nl, 16 + nl)
#pragma unroll
    for (int i = 0; i < NSB; i++)
#pragma unroll
        for (int mb = 0; mb < MT; mb++) {
            const uint4 *base = xs + (size_t)((2 * sbi[i] + (int)h) * kGroups16) * Mp + 16 * mb + nl;
#pragma unroll
            for (int t = 0; t < 8; t++) af[i][mb][t] = __builtin_bit_cast(half8_t, base[(size_t)(2 * t + (int)g) * Mp]);
            asum[i][mb][0] = __builtin_bit_cast(half8_t, base[(size_t)(16 + (int)g) * Mp]);
            asum[i][mb][1] = __builtin_bit_cast(half8_t, base[(size_t)(18 + (int)g) * Mp]);
            if (!sbv[i]) {  // a super-block past the end of the row multiplies zeros (no branch in the streaming loop)
                const half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int t = 0; t < 8; t++) af[i][mb][t] = z;
                asum[i][mb][0] = z, asum[i][mb][1] = z;
            }
        }
    const int t0 = (int)blockIdx.x * tiles_per_wg;
    const int t1 = t0 + tiles_per_wg < tiles ? t0 + tiles_per_wg : tiles;  // t1 > t0 by the launch geometry
    const uint32_t row_bytes = (uint32_t)spr * (uint32_t)B::kBytes;
    auto block_at = [&](int ti, int i) -> uint32_t {  // byte offset of super-block sbi[i] of this lane's row of tile ti (the tensor is smaller than 4 GiB)
        int tile = t0 + ti;
        tile = tile < t1 ? tile : t1 - 1;  // past the end: the last tile again (loaded, not used)
        int n = tile * 16 + nl;
        n = n < N ? n : N - 1;
        return (uint32_t)n * row_bytes + (uint32_t)sbi[i] * (uint32_t)B::kBytes;
    };
    auto issue = [&](int ti, SmallRun16<FMT, NSB> &w) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NSB; i++) {
            const uint32_t blk = block_at(ti, i);
            if (FMT == 3) {
                w.q[i] = load16_a4(W + (blk + 16u + 16u * (uint32_t)kg));
                const u32x2_a4 s2 = *reinterpret_cast<const u32x2_a4 *>(W + (blk + 8u * h));
                const uint32_t dd = *reinterpret_cast<const uint32_t *>(W + (blk + 80u));
                w.sc[i] = u32x4{s2.x, s2.y, dd, 0u};
            } else {
                const uint32_t lo = blk & ~3u;  // (the pieces' offsets inside the block are multiples of four)
                w.q[i] = load16_a4(W + (lo + 32u + 16u * (uint32_t)kg));
                w.qx[i] = *reinterpret_cast<const uint32_t *>(W + (lo + 48u + 16u * (uint32_t)kg));
                w.hm[i] = load16_a4(W + (lo + 16u * g));
                w.hmx[i] = *reinterpret_cast<const uint32_t *>(W + (lo + 16u + 16u * g));
                w.sc[i] = load16_a4(W + (lo + 96u));
            }
        }
    };
    auto consume = [&](int ti, const SmallRun16<FMT, NSB> &w) __attribute__((always_inline)) {
        float4_t acc[MT];
#pragma unroll
        for (int mb = 0; mb < MT; mb++) acc[mb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < NSB; i++) {
            uint32_t qd[4], hm[4] = {0, 0, 0, 0}, s8[3], dbits;
            if (FMT == 3) {
                qd[0] = w.q[i][0], qd[1] = w.q[i][1], qd[2] = w.q[i][2], qd[3] = w.q[i][3];
                s8[0] = w.sc[i][0], s8[1] = w.sc[i][1], s8[2] = 0;
                dbits = w.sc[i][2];  // d | dmin << 16
            } else {
                const uint32_t sh = (block_at(ti, i) & 2u) * 8u;  // the block starts two bytes past a dword boundary, or on one
                qd[0] = __builtin_amdgcn_alignbit(w.q[i][1], w.q[i][0], sh), qd[1] = __builtin_amdgcn_alignbit(w.q[i][2], w.q[i][1], sh);
                qd[2] = __builtin_amdgcn_alignbit(w.q[i][3], w.q[i][2], sh), qd[3] = __builtin_amdgcn_alignbit(w.qx[i], w.q[i][3], sh);
                hm[0] = __builtin_amdgcn_alignbit(w.hm[i][1], w.hm[i][0], sh), hm[1] = __builtin_amdgcn_alignbit(w.hm[i][2], w.hm[i][1], sh);
                hm[2] = __builtin_amdgcn_alignbit(w.hm[i][3], w.hm[i][2], sh), hm[3] = __builtin_amdgcn_alignbit(w.hmx[i], w.hm[i][3], sh);
                s8[0] = __builtin_amdgcn_alignbit(w.sc[i][1], w.sc[i][0], sh), s8[1] = __builtin_amdgcn_alignbit(w.sc[i][2], w.sc[i][1], sh);
                s8[2] = __builtin_amdgcn_alignbit(w.sc[i][3], w.sc[i][2], sh);
                dbits = (w.sc[i][3] >> sh) & 0xFFFFu;
            }
            // (of a super-block past the end of the row only zeros may enter the sums, whatever bytes were loaded for it)
            const float d = sbv[i] ? f16_bits_to_f32(dbits & 0xFFFFu) : 0.0f;
            const float dmin = sbv[i] ? f16_bits_to_f32(dbits >> 16) : 0.0f;
            // scales (and mins) of the lane's four sub-blocks j = 8 h + 4 sp + 2 lh + g, index 2 sp + lh
            half2_t sc2[4], off2[4];
            float nm[4];
#pragma unroll
            for (int sp = 0; sp < 2; sp++)
#pragma unroll
                for (int lh = 0; lh < 2; lh++) {
                    float scf;
                    if (FMT == 3) {  // s8[sp]: bytes 8 h + 4 sp .. of the sixteen; low nibble scale, high nibble min
                        const uint32_t b = (s8[sp] >> (8u * g + 16u * lh)) & 0xFFu;
                        scf = (float)(b & 15u);
                        nm[2 * sp + lh] = -(dmin * (float)(b >> 4));
                    } else {
                        const uint32_t lo4 = (s8[sp] >> (8u * g + 16u * lh + 4u * h)) & 15u;
                        const uint32_t hi2 = (s8[2] >> (8u * g + 16u * lh + 2u * (2u * h + sp))) & 3u;
                        scf = (float)((int)(lo4 | (hi2 << 4)) - 32);
                        nm[2 * sp + lh] = -(d * (4.0f * scf));
                    }
                    const _Float16 s16 = (_Float16)scf, o16 = (_Float16)(-1024.0f * scf);  // exact: |sc| <= 32
                    sc2[2 * sp + lh] = half2_t{s16, s16}, off2[2 * sp + lh] = half2_t{o16, o16};
                }
            float4_t part[MT];
#pragma unroll
            for (int mb = 0; mb < MT; mb++) part[mb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int t = 0; t < 8; t++) {
                const int dw = t >> 1, sp = t & 1;
                uint32_t lo = (qd[dw] >> (4 * sp)) & 0x03030303u, hi = (qd[dw] >> (4 * sp + 2)) & 0x03030303u;
                if (FMT == 2) {
                    const uint32_t m = hm[dw] >> (4u * h + 2u * sp);
                    lo |= (m & 0x01010101u) << 2, hi |= (m & 0x02020202u) << 1;
                }
                const half2_t r0 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, lo, 0x04010400u)), sc2[2 * sp], off2[2 * sp]);
                const half2_t r1 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, lo, 0x04030402u)), sc2[2 * sp], off2[2 * sp]);
                const half2_t r2 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, hi, 0x04010400u)), sc2[2 * sp + 1], off2[2 * sp + 1]);
                const half2_t r3 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, hi, 0x04030402u)), sc2[2 * sp + 1], off2[2 * sp + 1]);
                const half8_t b = half8_t{r0[0], r0[1], r1[0], r1[1], r2[0], r2[1], r3[0], r3[1]};
#pragma unroll
                for (int mb = 0; mb < MT; mb++) part[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i][mb][t], b, part[mb], 0, 0, 0);
            }
#pragma unroll
            for (int sp = 0; sp < 2; sp++) {
                const _Float16 h0 = (_Float16)nm[2 * sp], h1 = (_Float16)nm[2 * sp + 1];
                const _Float16 l0 = (_Float16)(nm[2 * sp] - (float)h0), l1 = (_Float16)(nm[2 * sp + 1] - (float)h1);
                const half8_t br = half8_t{h0, h0, l0, l0, h1, h1, l1, l1};
#pragma unroll
                for (int mb = 0; mb < MT; mb++) acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(asum[i][mb][sp], br, acc[mb], 0, 0, 0);
            }
#pragma unroll
            for (int mb = 0; mb < MT; mb++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[mb][r] = __builtin_fmaf(d, part[mb][r], acc[mb][r]);
        }
#pragma unroll
        for (int mb = 0; mb < MT; mb++) small_add_waves(red, keep, ti * MT + mb, wave, nwaves, lane, acc[mb], out_tiles);
    };
    static_assert(kSmallDepth == 2, "the ring is written out as two tiles");
    SmallRun16<FMT, NSB> ring0, ring1;
    issue(0, ring0);
    issue(1, ring1);
    for (int rd = 0; rd < rounds; rd++) {  // whole rounds of two tiles, nothing conditional around the loads
        consume(2 * rd, ring0);
        issue(2 * rd + 2, ring0);
        consume(2 * rd + 1, ring1);
        issue(2 * rd + 3, ring1);
    }
    small_add_kept(keep, rounds * kSmallDepth * MT, wave, nwaves, lane, out_tiles);
    small_store(out_tiles, t0, t1, M, Mp, N, rowscale, yg, ybf16, partial, MT);
}

}  // namespace

namespace pmh {

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// The fused kernels for at most 16 activation rows.  Rows of more than 16 super-blocks are cut into runs of 16, one
// workgroup row of the grid each, whose partial tiles k_rw_reduce adds (qgemm_plan sets splits and chunk to match).
constexpr int kSmallMaxRuns = 8;  // k <= 32768
// Super-blocks of a row that one short-batch workgroup takes (a longer row goes in runs of that many); 0: no such kernel.
// Up to 16 rows: eight waves of two super-blocks.  17 to 32 rows (two 16-row blocks of activations per weight operand): the
// Q4_K / Q5_K and Q2_K kernels still hold two super-blocks' activations per wave, the Q8_0 kernel one (43.4 -> 27.1 us at 14336 x 4096);
// the Q6_K kernel in that form, with its rows in runs of eight, is no faster than the large kernel (32.2 against 29.9 us).
static int small_run_spr(uint32_t type, int64_t m) {
    const bool any = type == kTypeQ4K || type == kTypeQ5K || type == kTypeQ6K || type == kTypeQ8_0 || type == kTypeQ3K || type == kTypeQ2K;
    if (m <= kSmallMaxM) return any ? kSmallMaxSpr : 0;
    if (m > kSmallMaxM2) return 0;
    if (type == kTypeQ4K || type == kTypeQ5K || type == kTypeQ2K) return kSmallMaxSpr;
    if (type == kTypeQ8_0) return kSmallWaves;
    return 0;
}
static bool qgemm_small_applies(uint32_t type, int64_t m, int64_t n, int64_t k) {
    const int64_t spr = k / 256;
    const int run = small_run_spr(type, m);
    if (run == 0 || spr > (int64_t)run * kSmallMaxRuns) return false;
    if (type == kTypeQ4K) return (uint64_t)n * (uint64_t)spr * 144u < (1ull << 32);
    if (type == kTypeQ5K) return (uint64_t)n * (uint64_t)spr * 176u < (1ull << 32);
    if (type == kTypeQ8_0) return (uint64_t)n * (uint64_t)spr * 272u < (1ull << 32);
    if (type == kTypeQ6K) return (uint64_t)n * (uint64_t)spr * 210u < (1ull << 32);
    if (type == kTypeQ3K) return (uint64_t)n * (uint64_t)spr * 110u < (1ull << 32);
    if (type == kTypeQ2K) return (uint64_t)n * (uint64_t)spr * 84u < (1ull << 32);
    return false;
}

static int compute_units_gemm() {
    static const int n = [] {
        int dev = 0, cu = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 256;
        if (hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cu <= 0) return 256;
        return cu;
    }();
    return n;
}

bool qgemm_fits(uint32_t type, int64_t m, int64_t n, int64_t k) {
    // byte offsets inside a workgroup's rows and item offsets inside the activation copy are 32-bit
    return (type == kTypeQ4K || type == kTypeQ5K || type == kTypeQ6K || type == kTypeQ8_0 || type == kTypeQ3K || type == kTypeQ2K) && m >= 1 && m <= (int64_t)1 << 22 && n >= 1 && k >= 256 && k % 256 == 0 && k <= (int64_t)1 << 22 && n <= 0x7FFFFF00;
}

GemmPlan qgemm_plan(int64_t m, int64_t n, int64_t k, uint32_t type) {
    GemmPlan p;
    // 32, 64 or 128 activation rows per workgroup; up to 192 rows 64-row blocks beat 128-row blocks (fewer K splits
    // for the same number of workgroups: 36.9 against 38.3 us at M = 128, 51.7 against 53.8 at M = 192, 14336x4096;
    // equal at 256, and from 320 rows on the larger block wins)
    p.mb = m <= 32 ? 1 : (m <= 192 ? 2 : 4);
    // few tiles (a narrow weight: k / v projections of 1024 or 2048 rows): 64-row blocks double them and halve the K
    // splits (M = 512: 1024 x 4096 28.7 -> 25.3 us, 2048 x 4096 33.8 -> 30.5; equal from 64 tiles on)
    if (p.mb == 4 && ((n + 255) / 256) * ((m + 127) / 128) <= 32) p.mb = 2;
    p.mp = (m + 32 * p.mb - 1) / (32 * p.mb) * (32 * p.mb);
    p.nw = 8;
    const int64_t spr = k / 256;
    const int64_t rows = 32 * p.nw;
    const int64_t base = (n + rows - 1) / rows * (p.mp / (32 * p.mb));
    // K split: more workgroups fill more of the machine, but every split writes and re-reads an fp32 tile of Y.
    // Estimated time = (time on a full machine) / (fraction of workgroup slots in use) + partial-tile traffic;
    // rates as measured on MI355X (about 700 TFLOP/s of this kernel, 4 TB/s for the weight stream and for the
    // partial tiles, 3 us for the extra launch).
    const double slots = 256.0;  // one workgroup per compute unit keeps the weight stream busy
    const double flops = 2.0 * (double)p.mp * (double)n * (double)k, wbytes = (double)n * (double)k * 0.5625;
    const double t_full = flops / 7.0e14 > wbytes / 4.0e12 ? flops / 7.0e14 : wbytes / 4.0e12;
    double best = 0.0;
    p.splits = 1, p.chunk = (int)spr;
    for (int64_t want = 1; want <= spr; want *= 2) {
        const int64_t chunk = (spr + want - 1) / want, splits = (spr + chunk - 1) / chunk;
        const double groups = (double)(base * splits);
        const double rounds = (double)(int64_t)((groups + slots - 1) / slots);
        const double t = t_full * rounds * slots / groups +
                         (splits > 1 ? (double)splits * (double)m * (double)n * 8.0 / 4.0e12 + 3.0e-6 : 0.0);
        if (want == 1 || t < best) best = t, p.splits = (int)splits, p.chunk = (int)chunk;
    }
    // short batches against long rows: runs of 16 (or 8) super-blocks, the fused kernels' K split (a shape they do not take
    // keeps the split chosen above)
    const int run = small_run_spr(type, m);
    if (run && spr > run && qgemm_small_applies(type, m, n, k)) p.chunk = run, p.splits = (int)((spr + run - 1) / run);
    return p;
}

size_t qgemm_workspace_bytes(uint32_t type, int64_t m, int64_t n, int64_t k) {
    const GemmPlan p = qgemm_plan(m, n, k, type);
    const size_t xs = align256((size_t)(k / 256) * 2 * (type == kTypeQ3K || type == kTypeQ2K ? kGroups16 : kGroups) * p.mp * 16);
    // the short-batch kernels take a row of up to kSmallMaxSpr super-blocks whole: the plan's K split is not used there
    const bool unsplit = qgemm_small_applies(type, m, n, k) && k / 256 <= small_run_spr(type, m);
    const size_t part = p.splits > 1 && !unsplit ? align256((size_t)p.splits * p.mp * n * 4) : 0;
    return xs + align256((size_t)p.mp * 4) + part;
}

template <int ORDER, int MB, int NR, int NW, int FMT = 0>
static hipError_t launch_rw(hipStream_t s, const uint8_t *w, const uint4 *xs, const float *rowscale, void *y, float *partial,
                            int64_t m, int64_t n, int spr, const GemmPlan &p, int mode) {
    auto kern = k_qgemm_rw<ORDER, MB, NR, NW, FMT>;
    constexpr size_t lds = rw_lds_bytes<MB, NR, NW, FMT>();
    constexpr int kRows = 32 * NR * NW;
    if (lds > 64 * 1024) {
        hipError_t a = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (a != hipSuccess) return a;
    }
    const dim3 grid((unsigned)((n + kRows - 1) / kRows), (unsigned)(p.mp / (32 * MB)), (unsigned)p.splits);
    hipLaunchKernelGGL(kern, grid, dim3(64 * NW), lds, s, w, xs, rowscale, y, partial, (int)m, (int)p.mp, (int)n, spr, p.chunk, mode);
    return hipGetLastError();
}

template <int FMT, int MB>
static hipError_t launch_rw16(hipStream_t s, const uint8_t *w, const uint4 *xs, const float *rowscale, void *y, float *partial, int64_t m,
                              int64_t n, int spr, const GemmPlan &p, int mode) {
    auto kern = k_qgemm_rw16<FMT, MB>;
    constexpr size_t lds = rw16_lds_bytes<FMT, MB>();
    if (lds > 64 * 1024) {
        hipError_t a = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (a != hipSuccess) return a;
    }
    const dim3 grid((unsigned)((n + 255) / 256), (unsigned)(p.mp / (32 * MB)), (unsigned)p.splits);
    hipLaunchKernelGGL(kern, grid, dim3(512), lds, s, w, xs, rowscale, y, partial, (int)m, (int)p.mp, (int)n, spr, p.chunk, mode);
    return hipGetLastError();
}

template <int MB>
static hipError_t launch_rw_q6(hipStream_t s, const uint8_t *w, const uint4 *xs, const float *rowscale, void *y, float *partial,
                               int64_t m, int64_t n, int spr, const GemmPlan &p, int mode) {
    auto kern = k_qgemm_rw_q6<MB>;
    constexpr size_t stages = (size_t)(2 * kQ6Groups * 32 * MB + 8 * (3 * kQ6Stage + 64)) * 16;
    constexpr size_t lds = stages > tile_lds_bytes<MB>() ? stages : tile_lds_bytes<MB>();
    hipError_t a = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (a != hipSuccess) return a;
    const dim3 grid((unsigned)((n + 255) / 256), (unsigned)(p.mp / (32 * MB)), (unsigned)p.splits);
    hipLaunchKernelGGL(kern, grid, dim3(512), lds, s, w, xs, rowscale, y, partial, (int)m, (int)p.mp, (int)n, spr, p.chunk, mode);
    return hipGetLastError();
}

template <int MB>
static hipError_t launch_rw_q8(hipStream_t s, const uint8_t *w, const uint4 *xs, const float *rowscale, void *y, float *partial,
                               int64_t m, int64_t n, int spr, const GemmPlan &p, int mode) {
    auto kern = k_qgemm_rw_q8<MB>;
    constexpr size_t stages = (size_t)(2 * kQ6Groups * 32 * MB) * 16;
    constexpr size_t lds = stages > tile_lds_bytes<MB>() ? stages : tile_lds_bytes<MB>();
    if (lds > 64 * 1024) {
        hipError_t a = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (a != hipSuccess) return a;
    }
    const dim3 grid((unsigned)((n + 255) / 256), (unsigned)(p.mp / (32 * MB)), (unsigned)p.splits);
    hipLaunchKernelGGL(kern, grid, dim3(512), lds, s, w, xs, rowscale, y, partial, (int)m, (int)p.mp, (int)n, spr, p.chunk, mode);
    return hipGetLastError();
}

hipError_t launch_qgemm(uint32_t type, const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype,
                                int64_t m, void *y, uint32_t y_dtype, uint32_t order, void *workspace, hipStream_t s, bool reuse_prepass) {
    if (!qgemm_fits(type, m, n, k)) return hipErrorInvalidValue;
    const GemmPlan p = qgemm_plan(m, n, k, type);
    const int spr = (int)(k / 256);
    uint8_t *ws = reinterpret_cast<uint8_t *>(workspace);
    uint4 *xs = reinterpret_cast<uint4 *>(ws);
    const bool q23 = type == kTypeQ3K || type == kTypeQ2K;
    const size_t xs_bytes = align256((size_t)spr * 2 * (q23 ? kGroups16 : kGroups) * p.mp * 16);
    float *rowscale = reinterpret_cast<float *>(ws + xs_bytes);
    float *partial = reinterpret_cast<float *>(ws + xs_bytes + align256((size_t)p.mp * 4));
    const bool xf32 = x_dtype == kDtypeF32, q6 = type == kTypeQ6K, q8 = type == kTypeQ8_0, q5 = type == kTypeQ5K, ref = order == kOrderRef;
    const int xorder = q23 ? 5 : (q8 ? 3 : (q6 ? 2 : (ref ? (q5 ? 4 : 0) : 1)));  // the element order the pre-pass lays the activations out for
#define PMH_PREP(F, O)                                                                                                       \
    do {                                                                                                                     \
        if (p.mp >= 1024)                                                                                                    \
            hipLaunchKernelGGL((k_prep_rw<F, O, 4>), dim3((unsigned)p.mp / 4), dim3(1024), 0, s, x, k, (int)m, (int)p.mp,    \
                               rowscale, xs);                                                                                \
        else                                                                                                                 \
            hipLaunchKernelGGL((k_prep_rw<F, O, 1>), dim3((unsigned)p.mp), dim3(512), 0, s, x, k, (int)m, (int)p.mp,         \
                               rowscale, xs);                                                                                \
    } while (0)
    if (reuse_prepass) {
        // the workspace still holds the converted activations of the previous call (same x, m, k and weight type)
    } else if (xf32) {
        if (xorder == 0) PMH_PREP(true, 0);
        else if (xorder == 1) PMH_PREP(true, 1);
        else if (xorder == 2) PMH_PREP(true, 2);
        else if (xorder == 3) PMH_PREP(true, 3);
        else if (xorder == 4) PMH_PREP(true, 4);
        else PMH_PREP(true, 5);
    } else {
        if (xorder == 0) PMH_PREP(false, 0);
        else if (xorder == 1) PMH_PREP(false, 1);
        else if (xorder == 2) PMH_PREP(false, 2);
        else if (xorder == 3) PMH_PREP(false, 3);
        else if (xorder == 4) PMH_PREP(false, 4);
        else PMH_PREP(false, 5);
    }
#undef PMH_PREP
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const bool ybf = y_dtype == kDtypeBf16;
    if (qgemm_small_applies(type, m, n, k)) {
        const int nwaves = spr < kSmallWaves ? spr : kSmallWaves;
        const int tiles = (int)((n + 15) / 16);
        // one workgroup per compute unit over all runs of a long row: each then walks several row tiles with its activation
        // operands in registers (one tile per workgroup and four times the workgroups: 35 against 27 us at M = 16, 4096 x 14336)
        const int run = small_run_spr(type, m);
        const int runs_of_row = spr > run ? p.splits : 1;
        int64_t slots = (int64_t)compute_units_gemm() * (kSmallWaves / nwaves) / runs_of_row;
        slots = slots < 1 ? 1 : slots;
        const int n_wg = (int)(tiles < slots ? tiles : slots);
        int tiles_per_wg = (tiles + n_wg - 1) / n_wg;
        const int mt = m > kSmallMaxM ? 2 : 1;  // 16-row blocks of activations
        // the finished tiles wait in LDS, 1 KiB each, beside the waves' stages (at most 70 KiB, Q8_0) and the 16 KiB of the
        // reduction buffers: 64 of them keep the workgroup within 160 KiB for every type
        tiles_per_wg = tiles_per_wg < 64 / mt ? tiles_per_wg : 64 / mt;
        // a long row: p.splits runs of 16 super-blocks, one workgroup row of the grid each, partial tiles for k_rw_reduce
        // (for rows of up to 16 super-blocks the plan's split belongs to the large kernel and is not used here)
        const int runs = runs_of_row;
        float *const part_out = runs > 1 ? partial : nullptr;
        const int nsb = run > kSmallWaves && spr > kSmallWaves ? 2 : 1;
        const dim3 grid((unsigned)((tiles + tiles_per_wg - 1) / tiles_per_wg), (unsigned)runs), block((unsigned)(64 * nwaves));
        // (a workgroup of few tiles also keeps every wave's partial tile of each until the end)
        const size_t lds = (size_t)((tiles_per_wg + kSmallDepth - 1) / kSmallDepth * kSmallDepth) * mt * 1024 *
                           (tiles_per_wg * mt <= kSmallKeepTiles ? 1 + nwaves : 1);
#define PMH_SMALL_FM(O, S, F, T)                                                                                                 \
    do {                                                                                                                         \
        const size_t lds4 = lds + (size_t)nwaves * SmallRun<S, F>::kPieces * 16; /* the waves' stages behind the finished tiles */ \
        if (lds4 > 48 * 1024) {                                                                                                   \
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_qgemm_small<O, S, F, T>), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                    (int)lds4);                                                                                   \
            if (e != hipSuccess) return e;                                                                                       \
        }                                                                                                                        \
        hipLaunchKernelGGL((k_qgemm_small<O, S, F, T>), grid, block, lds4, s, w, xs, rowscale, y, (int)m, (int)p.mp, (int)n, spr, tiles, \
                           tiles_per_wg, ybf ? 1 : 0, part_out);                                                                           \
    } while (0)
#define PMH_SMALL_F(O, S, F)               \
    do {                                   \
        if (mt == 2) PMH_SMALL_FM(O, S, F, 2); \
        else PMH_SMALL_FM(O, S, F, 1);         \
    } while (0)
#define PMH_SMALL(O, S)         \
    do {                        \
        if (q5) PMH_SMALL_F(O, S, 1); \
        else PMH_SMALL_F(O, S, 0);    \
    } while (0)
        if (q23) {
#define PMH_SMALL16(F, S, T)                                                                                                     \
    do {                                                                                                                         \
        if (lds > 48 * 1024) {                                                                                                   \
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_qgemm_small16<F, S, T>), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                    (int)lds);                                                                                   \
            if (e != hipSuccess) return e;                                                                                       \
        }                                                                                                                        \
        hipLaunchKernelGGL((k_qgemm_small16<F, S, T>), grid, block, lds, s, w, xs, rowscale, y, (int)m, (int)p.mp, (int)n, spr, tiles, \
                           tiles_per_wg, ybf ? 1 : 0, part_out);                                                                 \
    } while (0)
            if (type == kTypeQ2K) {
                if (mt == 2 && nsb == 2) PMH_SMALL16(3, 2, 2);
                else if (mt == 2) PMH_SMALL16(3, 1, 2);
                else if (nsb == 2) PMH_SMALL16(3, 2, 1);
                else PMH_SMALL16(3, 1, 1);
            } else {
                if (nsb == 2) PMH_SMALL16(2, 2, 1);
                else PMH_SMALL16(2, 1, 1);
            }
#undef PMH_SMALL16
        } else if (q6) {
            const bool any = spr % 8 != 0;  // rows that do not start on 16-byte boundaries
            const size_t stage = (size_t)(nsb == 2 ? SmallQ6<2, true>::kStageDwords : SmallQ6<1>::kStageDwords) * 4;
            const size_t lds6 = lds + (size_t)nwaves * stage;  // the waves' stages behind the finished tiles
            const uint32_t w_last = (uint32_t)(((uint64_t)n * (uint64_t)spr * 210u - 1) & ~(uint64_t)15);
#define PMH_SMALL_Q6(S, A)                                                                                                        \
    do {                                                                                                                         \
        if (lds6 > 48 * 1024) {                                                                                                  \
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_qgemm_small_q6<S, A>), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                    (int)lds6);                                                                                  \
            if (e != hipSuccess) return e;                                                                                       \
        }                                                                                                                        \
        hipLaunchKernelGGL((k_qgemm_small_q6<S, A>), grid, block, lds6, s, w, xs, rowscale, y, (int)m, (int)p.mp, (int)n, spr, tiles, \
                           tiles_per_wg, ybf ? 1 : 0, w_last, part_out);                                                                   \
    } while (0)
            if (nsb == 2 && any) PMH_SMALL_Q6(2, true);
            else if (nsb == 2) PMH_SMALL_Q6(2, false);
            else if (any) PMH_SMALL_Q6(1, true);
            else PMH_SMALL_Q6(1, false);
#undef PMH_SMALL_Q6
        } else if (q8) {
            const size_t lds8 = lds + (size_t)nwaves * nsb * kQ8TileRunPieces * 16;  // the waves' stages behind the finished tiles
#define PMH_SMALL_Q8(S, T)                                                                                                       \
    do {                                                                                                                         \
        if (lds8 > 48 * 1024) {                                                                                                  \
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_qgemm_small_q8<S, T>), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                    (int)lds8);                                                                                  \
            if (e != hipSuccess) return e;                                                                                       \
        }                                                                                                                        \
        hipLaunchKernelGGL((k_qgemm_small_q8<S, T>), grid, block, lds8, s, w, xs, rowscale, y, (int)m, (int)p.mp, (int)n, spr, tiles, \
                           tiles_per_wg, ybf ? 1 : 0, part_out);                                                                           \
    } while (0)
            if (mt == 2) PMH_SMALL_Q8(1, 2);  // (two blocks of activations: one run of eight blocks per wave)
            else if (nsb == 2) PMH_SMALL_Q8(2, 1);
            else PMH_SMALL_Q8(1, 1);
#undef PMH_SMALL_Q8
        } else if (spr > kSmallWaves) {
            static_assert(2 * kSmallWaves >= kSmallMaxSpr, "two super-blocks per wave must cover the longest row");
            if (ref) PMH_SMALL(0, 2);
            else PMH_SMALL(1, 2);
        } else {
            if (ref) PMH_SMALL(0, 1);
            else PMH_SMALL(1, 1);
        }
#undef PMH_SMALL
#undef PMH_SMALL_F
#undef PMH_SMALL_FM
        e = hipGetLastError();
        if (e != hipSuccess || runs == 1) return e;
    } else {
    const int mode = p.splits > 1 ? 2 : (ybf ? 1 : 0);
#define PMH_RW_CASE(O, B, R, NWV) launch_rw<O, B, R, NWV>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode)
    if (q8) {
        e = p.mb == 1   ? launch_rw_q8<1>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode)
            : p.mb == 2 ? launch_rw_q8<2>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode)
                        : launch_rw_q8<4>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode);
    } else if (q6) {
        e = p.mb == 1   ? launch_rw_q6<1>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode)
            : p.mb == 2 ? launch_rw_q6<2>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode)
                        : launch_rw_q6<4>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode);
    } else if (q23) {
        e = type == kTypeQ2K ? (p.mb == 1   ? launch_rw16<3, 1>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode)
                                : p.mb == 2 ? launch_rw16<3, 2>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode)
                                            : launch_rw16<3, 4>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode))
                             : (p.mb == 1   ? launch_rw16<2, 1>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode)
                                : p.mb == 2 ? launch_rw16<2, 2>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode)
                                            : launch_rw16<2, 4>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode));
    } else if (q5) {
#define PMH_RW5_CASE(O, B) launch_rw<O, B, 1, 8, 1>(s, w, xs, rowscale, y, partial, m, n, spr, p, mode)
        e = p.mb == 1   ? (ref ? PMH_RW5_CASE(0, 1) : PMH_RW5_CASE(1, 1))
            : p.mb == 2 ? (ref ? PMH_RW5_CASE(0, 2) : PMH_RW5_CASE(1, 2))
                        : (ref ? PMH_RW5_CASE(0, 4) : PMH_RW5_CASE(1, 4));
#undef PMH_RW5_CASE
    } else if (p.mb == 1) {
        e = ref ? PMH_RW_CASE(0, 1, 1, 8) : PMH_RW_CASE(1, 1, 1, 8);
    } else if (p.mb == 2) {
        e = ref ? PMH_RW_CASE(0, 2, 1, 8) : PMH_RW_CASE(1, 2, 1, 8);
    } else {
        e = ref ? PMH_RW_CASE(0, 4, 1, 8) : PMH_RW_CASE(1, 4, 1, 8);
    }
#undef PMH_RW_CASE
    if (e != hipSuccess || p.splits == 1) return e;
    }
    // the partial tiles of a K split (of the large kernels or of the short-batch kernels' runs), added in split order
    const size_t total = (size_t)m * n;
    if (n % 8 == 0) {
        const dim3 grid8((unsigned)((total / 8 + 255) / 256));
        if (ybf) hipLaunchKernelGGL(k_rw_reduce8<true>, grid8, dim3(256), 0, s, partial, p.splits, (int)m, (int)p.mp, (int)n, rowscale, y);
        else hipLaunchKernelGGL(k_rw_reduce8<false>, grid8, dim3(256), 0, s, partial, p.splits, (int)m, (int)p.mp, (int)n, rowscale, y);
        return hipGetLastError();
    }
    const dim3 rgrid((unsigned)((total + 255) / 256));
    if (ybf) hipLaunchKernelGGL(k_rw_reduce<true>, rgrid, dim3(256), 0, s, partial, p.splits, (int)m, (int)p.mp, (int)n, rowscale, y);
    else hipLaunchKernelGGL(k_rw_reduce<false>, rgrid, dim3(256), 0, s, partial, p.splits, (int)m, (int)p.mp, (int)n, rowscale, y);
    return hipGetLastError();
}

}  // namespace pmh
