// Dequant-fused GEMV for Q2_K and Q3_K matrices on gfx950 (the two low-bit types the KL calibration can choose).
//
// y[n] = sum_k W[n,k] * x[k], W the GGUF block stream, a weight's value what the reference's dequantizer yields:
//   Q2_K (84 bytes per 256 weights: scales[16], qs[64], d, dmin f16; (d (sc & 15)) q - dmin (sc >> 4),
//         crates/pmetal-gguf/src/k_quants.rs:230-266),
//   Q3_K (110 bytes: hmask[32], qs[64], scales[12], d f16; (d (sc6 - 32)) (q2 + 4 hbit - 4), k_quants.rs:281-355).
// Both store the low two bits of element 128 h + 32 p + l in qs[32 h + l] at bit 2 p; Q3_K keeps the third bit at bit
// 4 h + p of hmask[l].  Both have one element order.
//
//  * Lane t of the eight lanes of a super-block owns the qs bytes 8 t .. 8 t + 7 (half h = t / 4, l = 8 (t % 4) + i): 32
//    elements in four groups of eight, group p = the two-bit field p of each byte, lying in sub-block 8 h + 2 p + (t % 4) / 2.
//  * The activations are converted once per workgroup to fixed point: each of those 8-element groups gets a
//    power-of-two scale that puts its largest magnitude below 2^22, and the 23-bit signed integers are written as three
//    balanced base-256 digits in [-128, 127].  sum q x over a group is then 2^e * (65536 dot(q, d2) + 256 dot(q, d1) +
//    dot(q, d0)) with v_dot4_i32_i8 on four assembled values per dword: integer arithmetic, exact up to the fixed-point
//    resolution of x.  The min term (Q2_K) and the offset of 4 (Q3_K) use the group's sum of x, computed with the digits.
//  * One workgroup per compute unit (fewer rows than that: one row per workgroup); a row is ks = ceil(k / 2048) chunks
//    of eight super-blocks.  Wave (g, h) takes chunk h of the rows of row group g, so a lane's digits (24 registers)
//    never change.  Rows start at any multiple of four (Q2_K) or two (Q3_K) bytes: the wave copies the 16-byte pieces
//    that cover its chunk of a row, from the 16-byte boundary below it and never past the piece that holds the tensor's
//    last byte, into its own piece of LDS with one whole-wave load (up to kDepth rows in flight, every load issued
//    unconditionally so that the number of outstanding loads is known at every wait; rows past the end read the first
//    bytes of W), and each lane takes its pieces out of LDS as aligned dwords, which for Q3_K one funnel shift per
//    dword puts into place.  LDS executes a wave's instructions in order, so the copy needs no barrier.  Lane partial
//    sums go to LDS; after a barrier the workgroup adds up each of its rows and stores y.
#include "gemv_chunk.hpp"
#include "internal.hpp"

namespace {

using namespace pmh::gemv;

typedef uint32_t u4v __attribute__((ext_vector_type(4)));  // a 16-byte piece

constexpr int kDepth = 8;  // rows in flight per wave
constexpr int kPre = 2;    // of which this many are requested before x is converted
constexpr int kPlanes = 3;

// Element of group p (0..3), position i (0..7), of lane t of super-block sb.
__device__ __forceinline__ int element_of(int sb, int t, int p, int i) { return 256 * sb + 128 * (t >> 2) + 32 * p + 8 * (t & 3) + i; }

// Activations -> LDS.  A thread converts one group of eight consecutive elements (digit dwords 0 and 1 of the group): the
// group's largest magnitude and the sum of its fixed-point values stay inside the thread.  Groups past the end of a row
// (its last chunk may hold fewer than eight super-blocks) get zero digits, scale and sum.
// xd[(plane * 8 + 2 p + dword) * slots + slot]: four digits; xm[slot * 8 + p] = scale of group p, xm[slot * 8 + 4 + p] = its
// sum of x.
template <bool XF32>
__device__ __forceinline__ void stage_x(const void *__restrict__ xg, int slots, int spr, int nthreads, uint32_t *xd, float *xm) {
    const int total = slots * 4;
    for (int grp = (int)threadIdx.x; grp < total; grp += nthreads) {
        const int p = grp & 3, slot = grp >> 2, sb = slot >> 3, t = slot & 7;
        const int first = element_of(sb, t, p, 0);
        float v[2][4];
        if (sb >= spr) {
#pragma unroll
            for (int c = 0; c < 2; c++) v[c][0] = v[c][1] = v[c][2] = v[c][3] = 0.f;
        } else if (XF32) {
            const float4 *src = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(xg) + first);
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const float4 f = src[c];
                v[c][0] = f.x, v[c][1] = f.y, v[c][2] = f.z, v[c][3] = f.w;
            }
        } else {
            const uint4 a = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(xg) + first);
            const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
            for (int c = 0; c < 2; c++) {
                v[c][0] = __builtin_bit_cast(float, w[2 * c] << 16), v[c][1] = __builtin_bit_cast(float, w[2 * c] & 0xFFFF0000u);
                v[c][2] = __builtin_bit_cast(float, w[2 * c + 1] << 16), v[c][3] = __builtin_bit_cast(float, w[2 * c + 1] & 0xFFFF0000u);
            }
        }
        const uint32_t m0 = max_magnitude_bits(v[0]), m1 = max_magnitude_bits(v[1]);
        const GroupScale gs = group_scale(m0 > m1 ? m0 : m1);
        int sum = 0;
#pragma unroll
        for (int c = 0; c < 2; c++) {
            uint32_t dig[kPlanes];
            sum += to_digits(v[c], gs, dig);
#pragma unroll
            for (int pl = 0; pl < kPlanes; pl++) xd[(pl * 8 + 2 * p + c) * slots + slot] = dig[pl];
        }
        xm[slot * 8 + p] = gs.scale;
        xm[slot * 8 + 4 + p] = (float)sum * gs.scale;
    }
}

// sum over one 8-element group: the two assembled dwords against the group's digits
__device__ __forceinline__ float group_dot(uint32_t v0, uint32_t v1, const uint32_t (&xr)[kPlanes][8], int p) {
    int acc[kPlanes];
#pragma unroll
    for (int pl = 0; pl < kPlanes; pl++) acc[pl] = sdot4(v1, xr[pl][2 * p + 1], sdot4(v0, xr[pl][2 * p], 0));
    float f = (float)acc[kPlanes - 1];
#pragma unroll
    for (int pl = kPlanes - 2; pl >= 0; pl--) f = __builtin_fmaf(f, 256.0f, (float)acc[pl]);
    return f;
}

// N dwords that start `mis` (0 or 2) bytes past the dword p points at
template <int N>
__device__ __forceinline__ void read_shifted(const uint32_t *p, uint32_t sh, uint32_t (&out)[N]) {
    uint32_t w[N + 1];
#pragma unroll
    for (int k = 0; k <= N; k++) w[k] = p[k];
#pragma unroll
    for (int k = 0; k < N; k++) out[k] = __builtin_amdgcn_alignbit(w[k + 1], w[k], sh);
}

struct FormatQ2K {
    static constexpr int kBytes = 84;
    static constexpr int kPieces = 43;  // 8 * 84 = 672 bytes, starting up to 12 bytes into the first piece
    // blk: the dword at which the lane's super-block starts (Q2_K blocks are dword aligned); t: lane of the super-block
    static __device__ __forceinline__ float lane_value(const uint32_t *blk, uint32_t, int t, const uint32_t (&xr)[kPlanes][8],
                                                       const float4 xs, const float4 xsum) {
        const int h = t >> 2, q = (t & 3) >> 1;
        const uint32_t qs0 = blk[4 + 2 * t], qs1 = blk[5 + 2 * t];
        const uint32_t sc0 = blk[2 * h], sc1 = blk[2 * h + 1];  // scales[8 h ..]: byte 2 p + q belongs to group p
        const uint32_t dd = blk[20];
        const float xsv[4] = {xs.x, xs.y, xs.z, xs.w}, xsm[4] = {xsum.x, xsum.y, xsum.z, xsum.w};
        float acc = 0.0f, macc = 0.0f;
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint32_t v0 = (qs0 >> (2 * p)) & 0x03030303u, v1 = (qs1 >> (2 * p)) & 0x03030303u;
            const uint32_t byte = ((p < 2 ? sc0 : sc1) >> (8 * (2 * (p & 1) + q))) & 0xFFu;
            acc = __builtin_fmaf((float)(byte & 0xFu) * xsv[p], group_dot(v0, v1, xr, p), acc);
            macc = __builtin_fmaf((float)(byte >> 4), xsm[p], macc);
        }
        return f16_bits_to_f32(dd & 0xFFFFu) * acc - f16_bits_to_f32(dd >> 16) * macc;
    }
};

struct FormatQ3K {
    static constexpr int kBytes = 110;
    static constexpr int kPieces = 56;  // 8 * 110 = 880 bytes, starting up to 14 bytes into the first piece
    // blk: the dword at or below the start of the lane's super-block, which starts sh / 8 (0 or 2) bytes past it
    static __device__ __forceinline__ float lane_value(const uint32_t *blk, uint32_t sh, int t, const uint32_t (&xr)[kPlanes][8],
                                                       const float4 xs, const float4 xsum) {
        const int h = t >> 2, q = (t & 3) >> 1;
        uint32_t hm[2], qs[2], sc[3];
        read_shifted<2>(blk + 2 * (t & 3), sh, hm);  // hmask[8 (t % 4) ..]
        read_shifted<2>(blk + 8 + 2 * t, sh, qs);    // qs[8 t ..]
        read_shifted<3>(blk + 24, sh, sc);           // scales[12]
        const uint32_t d16 = (blk[27] >> sh) & 0xFFFFu;
        const float xsv[4] = {xs.x, xs.y, xs.z, xs.w}, xsm[4] = {xsum.x, xsum.y, xsum.z, xsum.w};
        float acc = 0.0f;
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const int hb = 4 * h + p;  // the group's bit of the hmask bytes
            const uint32_t v0 = ((qs[0] >> (2 * p)) & 0x03030303u) | (((hm[0] >> hb) & 0x01010101u) << 2);
            const uint32_t v1 = ((qs[1] >> (2 * p)) & 0x03030303u) | (((hm[1] >> hb) & 0x01010101u) << 2);
            // sub-block j = 8 h + 2 p + q: low four bits in a nibble of scales[j % 8], high two bits in scales[8 + j % 4]
            const int j = 8 * h + 2 * p + q, jb = j & 7;
            const uint32_t lo = ((jb < 4 ? sc[0] : sc[1]) >> (8 * (jb & 3) + 4 * h)) & 0xFu;
            const uint32_t hi = (sc[2] >> (8 * (j & 3) + 2 * (j >> 2))) & 3u;
            const float s6 = (float)((int)(lo | (hi << 4)) - 32);
            // the assembled values are q + 4: the offset leaves with the group's sum of x
            acc = __builtin_fmaf(s6, __builtin_fmaf(xsv[p], group_dot(v0, v1, xr, p), -4.0f * xsm[p]), acc);
        }
        return f16_bits_to_f32(d16) * acc;
    }
};

template <class F, bool XF32, bool SINGLE>
__global__ __launch_bounds__(1024) void k_qgemv_q23k_chunk(const uint8_t *__restrict__ W, const void *__restrict__ xg,
                                                            float *__restrict__ y, int n_rows, int spr, int rows_per_wg,
                                                            int rows_per_wave, int n_nominal, int nthreads,
                                                            uint32_t w_last) {
    constexpr int kStageDwords = F::kPieces * 4;
    extern __shared__ uint4 smem[];
    const int ks = (spr + 7) >> 3;
    const int slots = ks * 64;
    const int n_waves = nthreads >> 6;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    uint32_t *stage = reinterpret_cast<uint32_t *>(smem) + wave * kStageDwords;   // this wave's row chunk
    uint32_t *xd = reinterpret_cast<uint32_t *>(smem) + n_waves * kStageDwords;  // [kPlanes * 8][slots]
    float *xm = reinterpret_cast<float *>(xd + kPlanes * 8 * slots);             // [slots][8]
    float *part = xm + 8 * slots;                                                // [group][n_nominal][ks]
    const int lane = threadIdx.x & 63;
    const int t = lane & 7;
    const int h = wave % ks, g = wave / ks;
    const int wg_r0 = blockIdx.x * rows_per_wg;
    const int wg_r1 = wg_r0 + rows_per_wg < n_rows ? wg_r0 + rows_per_wg : n_rows;
    const int wave_r0 = wg_r0 + g * rows_per_wave;
    const int wave_r1 = wave_r0 + rows_per_wave < wg_r1 ? wave_r0 + rows_per_wave : wg_r1;
    const int nt_wave = wave_r1 > wave_r0 ? wave_r1 - wave_r0 : 0;  // real tasks of this wave (wave-uniform)

    const uint32_t rowbytes = (uint32_t)spr * (uint32_t)F::kBytes;
    const uint32_t off = (uint32_t)h * 8u * (uint32_t)F::kBytes + 16u * (uint32_t)(lane < F::kPieces ? lane : F::kPieces - 1);
    auto issue = [&](int i, u4v &a) {
        const bool real = i < nt_wave;  // wave-uniform
        const uint32_t ro = real ? (uint32_t)(wave_r0 + i) * rowbytes : 0u;
        uint32_t pa = (ro + (real ? off : 0u)) & ~15u;  // from the 16-byte boundary below the chunk
        pa = pa < w_last ? pa : w_last;                 // never past the piece that holds the tensor's last byte
        a = *reinterpret_cast<const u4v *>(W + pa);
    };

    u4v ra[kDepth];
#pragma unroll
    for (int i = 0; i < kPre; i++) issue(i, ra[i]);
    stage_x<XF32>(xg, slots, spr, nthreads, xd, xm);
    __syncthreads();

    const int slot = h * 64 + lane;
    uint32_t xr[kPlanes][8];
#pragma unroll
    for (int pl = 0; pl < kPlanes; pl++)
#pragma unroll
        for (int k = 0; k < 8; k++) xr[pl][k] = xd[(pl * 8 + k) * slots + slot];
    const float4 xs = *reinterpret_cast<const float4 *>(xm + 8 * slot), xsum = *reinterpret_cast<const float4 *>(xm + 8 * slot + 4);
    const uint32_t sb_byte = (uint32_t)(lane >> 3) * (uint32_t)F::kBytes;
    const uint32_t chunk_byte = (uint32_t)h * 8u * (uint32_t)F::kBytes;
    const bool lane_valid = h * 8 + (lane >> 3) < spr;  // the last chunk of a row may be short

    float *pp = part + (size_t)(g * n_nominal) * ks + h;
    auto consume = [&](int i, const u4v a) {
        if (i < nt_wave) {  // wave-uniform
            u4v *st4 = reinterpret_cast<u4v *>(stage);
            if (lane < F::kPieces) st4[lane] = a;
            // LDS executes a wave's instructions in order: the reads below see the writes above, and the next row's
            // writes come after these reads
            const uint32_t delta = ((uint32_t)(wave_r0 + i) * rowbytes + chunk_byte) & 15u;  // where the chunk starts in its first piece
            const uint32_t t0 = delta + sb_byte, mis = t0 & 2u;
            const float val = F::lane_value(stage + ((t0 - mis) >> 2), 8u * mis, t, xr, xs, xsum);
            store_chunk_sum(pp + (size_t)i * ks, lane_valid ? val : 0.0f, lane);
        }
    };

    int issued = kPre;
#pragma unroll
    for (int i = 0; i < kDepth; i++) {
        consume(i, ra[i]);
        const int upto = SINGLE ? (kPre + 2 * (i + 1) < kDepth ? kPre + 2 * (i + 1) : kDepth)
                                : (kPre + 2 * (i + 1) < kDepth + i + 1 ? kPre + 2 * (i + 1) : kDepth + i + 1);
#pragma unroll
        for (; issued < upto; issued++) issue(issued, ra[issued % kDepth]);
    }
    if (!SINGLE) {
        int base = kDepth;
        for (; base + kDepth < n_nominal; base += kDepth) {
#pragma unroll
            for (int i = 0; i < kDepth; i++) {
                consume(base + i, ra[i]);
                issue(base + kDepth + i, ra[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < kDepth; i++) consume(base + i, ra[i]);
    }
    __syncthreads();

    reduce_rows(part, ks, wg_r0, wg_r1 - wg_r0, rows_per_wave, n_nominal, nthreads, y);
}

template <class F>
hipError_t launch_format(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y, hipStream_t s) {
    const int spr = (int)(k / 256);
    const int ks = (spr + 7) / 8;
    const uint64_t w_bytes = (uint64_t)n * (uint64_t)spr * (uint64_t)F::kBytes;
    if (ks > 16 || w_bytes >= (1ull << 32)) return hipErrorInvalidValue;
    const size_t slots = (size_t)ks * 64;
    const size_t lds_x = slots * 4 * (kPlanes * 8) + slots * 32;
    const ChunkPlan plan = plan_chunks(n, ks, (size_t)F::kPieces * 16, lds_x);
    const int64_t n_wg = plan.n_wg, rows_per_wg = plan.rows_per_wg, rows_per_wave = plan.rows_per_wave, n_nominal = plan.n_nominal,
                  threads = plan.threads;
    const size_t lds = plan.lds;
    if (lds > kMaxLds) return hipErrorInvalidValue;
    const bool single = n_nominal <= kDepth;
    auto go = [&](auto kern) {
        if (lds > 64 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kern, dim3((unsigned)n_wg), dim3((unsigned)threads), lds, s, w, x, y, (int)n, spr, (int)rows_per_wg,
                           (int)rows_per_wave, (int)n_nominal, (int)threads, (uint32_t)((w_bytes - 1) & ~(uint64_t)15));
        return hipGetLastError();
    };
    if (x_dtype == pmh::kDtypeF32) return single ? go(k_qgemv_q23k_chunk<F, true, true>) : go(k_qgemv_q23k_chunk<F, true, false>);
    return single ? go(k_qgemv_q23k_chunk<F, false, true>) : go(k_qgemv_q23k_chunk<F, false, false>);
}

}  // namespace

namespace pmh {

// Preconditions as for launch_qgemv (k a multiple of 256).  hipErrorInvalidValue when the shape does not fit the kernel:
// rows of more than 16 chunks (k > 32768), tensors of 4 GiB and more, or staged activations that do not fit in LDS.
hipError_t launch_qgemv_q2k(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y, hipStream_t s) {
    return launch_format<FormatQ2K>(w, n, k, x, x_dtype, y, s);
}
hipError_t launch_qgemv_q3k(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y, hipStream_t s) {
    return launch_format<FormatQ3K>(w, n, k, x, x_dtype, y, s);
}

}  // namespace pmh
