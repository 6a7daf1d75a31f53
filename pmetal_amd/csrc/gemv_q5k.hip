// Dequant-fused GEMV for Q5_K matrices on gfx950 (the type the Q4_K_M recipe gives a fused attn_qkv tensor).
//
// y[n] = sum_k W[n,k] * x[k], W the GGUF Q5_K block stream (176 bytes per 256 weights: d, dmin f16, scales[12],
// qh[32], qs[128]; value (d sc) q - dmin m with q = nibble | fifth bit << 4, the 6-bit (sc, m) per 32 elements as in
// Q4_K), in the element order asked for: REF = the order the reference's dequantize_q5k emits
// (crates/pmetal-gguf/src/k_quants.rs:407-462), GGML = the inverse of quantize_q5k's packing (k_quants.rs:1027-1047).
//
//  * Lane t of the eight lanes of a super-block owns the qs bytes 16 t .. 16 t + 15: 32 elements in two groups of 16,
//    A = the low nibbles, B = the high nibbles.
//      REF  order: byte i holds elements 2 i (A) and 2 i + 1 (B) of sub-block t; their fifth bits are bits 2 c and
//                  2 c + 1 of byte i / 4 of the dword qh[4 t ..] (c = i % 4).
//      GGML order: byte i holds element 16 (t % 2) + i of sub-block 2 (t / 2) (A) and of sub-block 2 (t / 2) + 1 (B);
//                  their fifth bits are bits 2 (t / 2) and 2 (t / 2) + 1 of qh[16 (t % 2) + i].
//  * The activations are converted once per workgroup to fixed point: each of those 16-element groups gets a
//    power-of-two scale that puts its largest magnitude below 2^22, and the 23-bit signed integers are written as three
//    balanced base-256 digits in [-128, 127].  sum q x over a group is then 2^e * (65536 dot(q, d2) + 256 dot(q, d1) +
//    dot(q, d0)) with v_dot4_i32_i8 on four assembled 5-bit values per dword: integer arithmetic, exact up to the
//    fixed-point resolution of x.  The min term uses the group's sum of x, computed with the digits.
//  * One workgroup per compute unit (fewer rows than that: one row per workgroup); a row is ks = ceil(k / 2048) chunks
//    of eight super-blocks.  Wave (g, h) takes chunk h of the rows of row group g, so a lane's digits (24 registers)
//    never change.  The wave copies the 1408 contiguous, 16-byte aligned bytes of its chunk of a row into its own
//    piece of LDS with whole-wave 16-byte loads (up to kDepth rows in flight, every load issued unconditionally so
//    that the number of outstanding loads is known at every wait; rows past the end read the first bytes of W), and
//    each lane takes its pieces out of LDS.  LDS executes a wave's instructions in order, so the copy needs no
//    barrier.  Lane partial sums go to LDS; after a barrier the workgroup adds up each of its rows and stores y.
#include "gemv_chunk.hpp"
#include "internal.hpp"

namespace {

using namespace pmh::gemv;

typedef uint32_t u4v __attribute__((ext_vector_type(4)));  // a 16-byte piece

constexpr int kDepth = 6;      // rows in flight per wave
constexpr int kDepthLong = 8;  // ... for the variant that holds all of a wave's seven or eight rows at once (DEEP)
constexpr int kPre = 2;    // of which this many are requested before x is converted
constexpr int kPlanes = 3;
constexpr int kChunkBytes = 8 * 176;  // 1408 = 88 pieces of 16 bytes
constexpr int kStageBytes = kChunkBytes;

// Element of group s (0 = A, 1 = B), position i (0..15), of lane t of super-block sb.
template <int ORDER>
__device__ __forceinline__ int element_of(int sb, int t, int s, int i) {
    if (ORDER == 0) return 256 * sb + 32 * t + 2 * i + s;
    return 256 * sb + 64 * (t >> 1) + 32 * s + 16 * (t & 1) + i;
}

// Activations -> LDS.  A thread converts one 16-element group: the group's largest magnitude and the sum of its
// fixed-point values stay inside the thread.  In REF order the two groups of a lane are the even and the odd elements of
// its 32-element sub-block (the two halves of a dword of bf16 activations); in GGML order a group is 16 consecutive
// elements.  Groups past the end of a row (its last chunk may hold fewer than eight super-blocks) get zero digits, scale
// and sum.
// xd[(plane * 8 + 4 s + dword) * slots + slot]: four digits; xm[slot] = (scale A, scale B, sum of x over A, over B).
template <int ORDER, bool XF32>
__device__ __forceinline__ void stage_x(const void *__restrict__ xg, int slots, int spr, int nthreads, uint32_t *xd, float *xm) {
    const int total = slots * 2;
    for (int grp = (int)threadIdx.x; grp < total; grp += nthreads) {
        const int s = grp & 1, slot = grp >> 1, sb = slot >> 3, t = slot & 7;
        const int first = element_of<ORDER>(sb, t, s, 0);
        float v[4][4];
        if (sb >= spr) {
#pragma unroll
            for (int q = 0; q < 4; q++) v[q][0] = v[q][1] = v[q][2] = v[q][3] = 0.f;
        } else if (ORDER == 0) {
            if (XF32) {
                const float2 *src = reinterpret_cast<const float2 *>(reinterpret_cast<const float *>(xg) + (first - s));
#pragma unroll
                for (int q = 0; q < 4; q++)
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        const float2 f = src[4 * q + c];
                        v[q][c] = s ? f.y : f.x;
                    }
            } else {
                const uint4 *src = reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(xg) + (first - s));
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint4 a = src[q];
                    const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
                    for (int c = 0; c < 4; c++) v[q][c] = __builtin_bit_cast(float, s ? (w[c] & 0xFFFF0000u) : (w[c] << 16));
                }
            }
        } else if (XF32) {
            const float4 *src = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(xg) + first);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 f = src[q];
                v[q][0] = f.x, v[q][1] = f.y, v[q][2] = f.z, v[q][3] = f.w;
            }
        } else {
            const uint4 *src = reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(xg) + first);
            const uint4 a = src[0], b = src[1];
            const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int q = 0; q < 4; q++) {
                v[q][0] = __builtin_bit_cast(float, w[2 * q] << 16), v[q][1] = __builtin_bit_cast(float, w[2 * q] & 0xFFFF0000u);
                v[q][2] = __builtin_bit_cast(float, w[2 * q + 1] << 16), v[q][3] = __builtin_bit_cast(float, w[2 * q + 1] & 0xFFFF0000u);
            }
        }
        uint32_t mb = 0;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t o = max_magnitude_bits(v[q]);
            mb = o > mb ? o : mb;
        }
        const GroupScale gs = group_scale(mb);
        int sum = 0;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            uint32_t dig[kPlanes];
            sum += to_digits(v[q], gs, dig);
#pragma unroll
            for (int p = 0; p < kPlanes; p++) xd[(p * 8 + 4 * s + q) * slots + slot] = dig[p];
        }
        xm[slot * 4 + s] = gs.scale;
        xm[slot * 4 + 2 + s] = (float)sum * gs.scale;
    }
}

// get_scale_min_k4 (crates/pmetal-gguf/src/quantize.rs:844-855) on the 12 scale bytes held as three dwords.
__device__ __forceinline__ void scale_min_k4(int j, uint32_t s0, uint32_t s1, uint32_t s2, float &sc, float &m) {
    const int sh = 8 * (j & 3);
    const uint32_t a = (s0 >> sh) & 0xFFu, b = (s1 >> sh) & 0xFFu, c = (s2 >> sh) & 0xFFu;
    const uint32_t isc = j < 4 ? (a & 63u) : ((c & 0xFu) | ((a >> 6) << 4));
    const uint32_t im = j < 4 ? (b & 63u) : ((c >> 4) | ((b >> 6) << 4));
    sc = (float)isc, m = (float)im;
}

// The even bits of a byte, one per byte of a dword: bit 2 c of b becomes bit 0 of byte c.  The four copies of the masked
// byte that the multiplication adds up overlap in single bit positions whose carries end in unused bits.
__device__ __forceinline__ uint32_t even_bits_to_bytes(uint32_t b) { return ((b & 0x55u) * 0x41041u) & 0x01010101u; }

template <int ORDER, bool XF32, bool SINGLE, bool DEEP = false>
__global__ __launch_bounds__(1024) void k_qgemv_q5k_chunk(const uint8_t *__restrict__ W, const void *__restrict__ xg,
                                                           float *__restrict__ y, int n_rows, int spr, int rows_per_wg,
                                                           int rows_per_wave, int n_nominal, int nthreads,
                                                           uint32_t w_last) {
    constexpr int kDepth = DEEP ? kDepthLong : ::kDepth;
    extern __shared__ uint4 smem[];
    const int ks = (spr + 7) >> 3;
    const int slots = ks * 64;
    const int n_waves = nthreads >> 6;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    uint32_t *stage = reinterpret_cast<uint32_t *>(smem) + wave * (kStageBytes / 4);   // this wave's row chunk
    uint32_t *xd = reinterpret_cast<uint32_t *>(smem) + n_waves * (kStageBytes / 4);  // [kPlanes * 8][slots]
    float *xm = reinterpret_cast<float *>(xd + kPlanes * 8 * slots);                  // [slots][4]
    float *part = xm + 4 * slots;                                                     // [group][n_nominal][ks]
    const int lane = threadIdx.x & 63;
    const int t = lane & 7;
    const int h = wave % ks, g = wave / ks;
    const int wg_r0 = blockIdx.x * rows_per_wg;
    const int wg_r1 = wg_r0 + rows_per_wg < n_rows ? wg_r0 + rows_per_wg : n_rows;
    const int wave_r0 = wg_r0 + g * rows_per_wave;
    const int wave_r1 = wave_r0 + rows_per_wave < wg_r1 ? wave_r0 + rows_per_wave : wg_r1;
    const int nt_wave = wave_r1 > wave_r0 ? wave_r1 - wave_r0 : 0;  // real tasks of this wave (wave-uniform)

    const uint32_t rowbytes = (uint32_t)spr * 176u;
    // a wave's 88 pieces of a row chunk: lane l takes piece l, lanes 0..23 also piece 64 + l; never past the piece that
    // holds the tensor's last byte (the last chunk of a row may be short)
    const uint32_t off_a = (uint32_t)h * kChunkBytes + 16u * (uint32_t)lane;
    const uint32_t off_b = (uint32_t)h * kChunkBytes + 1024u + 16u * (uint32_t)(lane < 24 ? lane : 23);
    auto issue = [&](int i, u4v &a, u4v &b) {
        const bool real = i < nt_wave;  // wave-uniform
        const uint32_t ro = real ? (uint32_t)(wave_r0 + i) * rowbytes : 0u;
        uint32_t pa = ro + (real ? off_a : 0u), pb = ro + (real ? off_b : 0u);
        pa = pa < w_last ? pa : w_last;
        pb = pb < w_last ? pb : w_last;
        a = *reinterpret_cast<const u4v *>(W + pa);
        b = *reinterpret_cast<const u4v *>(W + pb);
    };

    u4v ra[kDepth], rb[kDepth];
#pragma unroll
    for (int i = 0; i < kPre; i++) issue(i, ra[i], rb[i]);
    stage_x<ORDER, XF32>(xg, slots, spr, nthreads, xd, xm);
    __syncthreads();

    const int slot = h * 64 + lane;
    uint32_t xr[kPlanes][8];
#pragma unroll
    for (int p = 0; p < kPlanes; p++)
#pragma unroll
        for (int k = 0; k < 8; k++) xr[p][k] = xd[(p * 8 + k) * slots + slot];
    const float4 xmr = *reinterpret_cast<const float4 *>(xm + 4 * slot);

    const uint32_t *blk = stage + (lane >> 3) * 44;  // 176 bytes per super-block
    const int c2 = 2 * (t >> 1);
    const int sub_a = ORDER == 0 ? t : c2, sub_b = ORDER == 0 ? t : c2 + 1;
    const bool lane_valid = h * 8 + (lane >> 3) < spr;  // the last chunk of a row may be short

    float *pp = part + (size_t)(g * n_nominal) * ks + h;
    auto consume = [&](int i, const u4v a, const u4v b) {
        if (i < nt_wave) {  // wave-uniform
            u4v *st4 = reinterpret_cast<u4v *>(stage);
            st4[lane] = a;
            if (lane < 24) st4[64 + lane] = b;
            // LDS executes a wave's instructions in order: the reads below see the writes above, and the next row's
            // writes come after these reads
            const uint32_t hd = blk[0], s0 = blk[1], s1 = blk[2], s2 = blk[3];
            uint32_t qs[4], bits_a[4], bits_b[4];
#pragma unroll
            for (int k = 0; k < 4; k++) qs[k] = blk[12 + 4 * t + k];
            if (ORDER == 0) {
                const uint32_t qh = blk[4 + t];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t byte = qh >> (8 * k);
                    bits_a[k] = even_bits_to_bytes(byte), bits_b[k] = even_bits_to_bytes(byte >> 1);
                }
            } else {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t qh = blk[4 + 4 * (t & 1) + k];
                    bits_a[k] = (qh >> c2) & 0x01010101u, bits_b[k] = (qh >> (c2 + 1)) & 0x01010101u;
                }
            }
            int acc_a[kPlanes] = {0, 0, 0}, acc_b[kPlanes] = {0, 0, 0};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t va = (qs[k] & 0x0F0F0F0Fu) | (bits_a[k] << 4);
                const uint32_t vb = ((qs[k] >> 4) & 0x0F0F0F0Fu) | (bits_b[k] << 4);
#pragma unroll
                for (int p = 0; p < kPlanes; p++) {
                    acc_a[p] = sdot4(va, xr[p][k], acc_a[p]);
                    acc_b[p] = sdot4(vb, xr[p][4 + k], acc_b[p]);
                }
            }
            float fa = (float)acc_a[kPlanes - 1], fb = (float)acc_b[kPlanes - 1];
#pragma unroll
            for (int p = kPlanes - 2; p >= 0; p--) {
                fa = __builtin_fmaf(fa, 256.0f, (float)acc_a[p]);
                fb = __builtin_fmaf(fb, 256.0f, (float)acc_b[p]);
            }
            float sc_a, m_a, sc_b, m_b;
            scale_min_k4(sub_a, s0, s1, s2, sc_a, m_a);
            scale_min_k4(sub_b, s0, s1, s2, sc_b, m_b);
            const float d = f16_bits_to_f32(hd & 0xFFFFu), dmin = f16_bits_to_f32(hd >> 16);
            const float val = d * __builtin_fmaf(sc_a * xmr.x, fa, (sc_b * xmr.y) * fb) - dmin * __builtin_fmaf(m_a, xmr.z, m_b * xmr.w);
            store_chunk_sum(pp + (size_t)i * ks, lane_valid ? val : 0.0f, lane);
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
    __syncthreads();

    reduce_rows(part, ks, wg_r0, wg_r1 - wg_r0, rows_per_wave, n_nominal, nthreads, y);
}

}  // namespace

namespace pmh {

// Preconditions as for launch_qgemv (k a multiple of 256).  hipErrorInvalidValue when the shape does not fit the kernel:
// rows of more than 16 chunks (k > 32768), tensors of 4 GiB and more, or staged activations that do not fit in LDS.
hipError_t launch_qgemv_q5k(const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y, uint32_t order,
                            hipStream_t s) {
    const int spr = (int)(k / 256);
    const int ks = (spr + 7) / 8;
    const uint64_t w_bytes = (uint64_t)n * (uint64_t)spr * 176u;
    if (ks > 16 || w_bytes >= (1ull << 32)) return hipErrorInvalidValue;
    const size_t slots = (size_t)ks * 64;
    const size_t lds_x = slots * 4 * (kPlanes * 8) + slots * 16;
    const gemv::ChunkPlan plan = gemv::plan_chunks(n, ks, kStageBytes, lds_x);
    const int64_t n_wg = plan.n_wg, rows_per_wg = plan.rows_per_wg, rows_per_wave = plan.rows_per_wave, n_nominal = plan.n_nominal,
                  threads = plan.threads;
    const size_t lds = plan.lds;
    if (lds > gemv::kMaxLds) return hipErrorInvalidValue;
    const bool deep = n_nominal > kDepth && n_nominal <= kDepthLong;  // seven or eight rows per wave: all in flight at once
    const bool single = n_nominal <= kDepth;
    const bool xf32 = x_dtype == kDtypeF32;
    auto go = [&](auto kern) {
        if (lds > 64 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kern, dim3((unsigned)n_wg), dim3((unsigned)threads), lds, s, w, x, y, (int)n, spr, (int)rows_per_wg,
                           (int)rows_per_wave, (int)n_nominal, (int)threads, (uint32_t)((w_bytes - 1) & ~(uint64_t)15));
        return hipGetLastError();
    };
#define PMH_Q5K(O, F) (deep ? go(k_qgemv_q5k_chunk<O, F, true, true>) : single ? go(k_qgemv_q5k_chunk<O, F, true>) : go(k_qgemv_q5k_chunk<O, F, false>))
    if (order == kOrderRef) return xf32 ? PMH_Q5K(0, true) : PMH_Q5K(0, false);
    return xf32 ? PMH_Q5K(1, true) : PMH_Q5K(1, false);
#undef PMH_Q5K
}

}  // namespace pmh
