/*
 * pmetal_oracle.h -- CPU restatement of PMetal's GGUF block-quantized weight path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is the checker the HIP kernels are compared
 * against; nothing in the shipped library links, loads or calls it.  Only the
 * test-suite, the smoke check and the benchmark's CPU-baseline leg use it.
 *
 * Every function follows one function of the reference (Epistates/pmetal,
 * crate pmetal-gguf) and cites it as file:line relative to the reference root.
 * The reference is Rust and cannot be compiled in this environment, so the
 * oracle is pinned without it: by the reference's own known-answer tests, by
 * closed forms, and -- for the order-sensitive scale searches and the bytes of
 * the k-quant quantizers -- by expected values that a second restatement of the
 * same Rust in rational arithmetic produces (tests/exact_ref.py ->
 * tests/golden/exact_cases.json, checked in tests/test_exact_pins.py):
 *   pmo_make_qkx1_quants, pmo_make_qx_quants, pmo_make_q3_quants: inputs whose
 *     sums are exact in any order, so that the result follows from the algorithm's
 *     definition (2 to 5 tries, accepted and refused rescale passes and moves,
 *     every early exit), plus Gaussian inputs with one rounding per operation in
 *     the reference's order;
 *   pmo_quantize_q4k / _q5k / _q6k / _q3k / _q2k: whole super-blocks built from
 *     those inputs, blocks that single out one super-block step each (decoded f16
 *     d / dmin in the requantization, IEEE division, the fold from +0.0, the first
 *     of equal scale magnitudes, the scale code 128, scale code 0, all-zero and
 *     partial blocks), pmo_quantize_q8_0 and the dequantizers likewise;
 *   tests/test_oracle_mutations.py edits pmetal_oracle.c one line at a time and
 *     checks that the fixture alone notices every edit.
 * The oracle is thus pinned by two independent restatements of the Rust, not by
 * the reference itself.  What stays unpinned in the strict sense: nothing was ever compared with output
 * of the Rust itself; a misreading of the Rust shared by the C restatement and
 * the rational one (written separately, from the Rust) would pass.
 */
#ifndef PMETAL_ORACLE_H
#define PMETAL_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GgmlType ids, crates/pmetal-gguf/src/types.rs:16-97 (only the path's types). */
enum {
    PMO_TYPE_F32 = 0,
    PMO_TYPE_F16 = 1,
    PMO_TYPE_Q4_0 = 2, /* the 32-element formats beside Q8_0: quantize / dequantize only */
    PMO_TYPE_Q4_1 = 3,
    PMO_TYPE_Q5_0 = 6,
    PMO_TYPE_Q5_1 = 7,
    PMO_TYPE_Q8_0 = 8,
    PMO_TYPE_Q8_1 = 9,
    PMO_TYPE_Q2K = 10, /* quantize / dequantize only */
    PMO_TYPE_Q3K = 11, /* quantize / dequantize only */
    PMO_TYPE_Q4K = 12,
    PMO_TYPE_Q5K = 13, /* quantize / dequantize only */
    PMO_TYPE_Q6K = 14,
    PMO_TYPE_Q8K = 15, /* quantize / dequantize and the activation side of the integer dot products */
};

/* Error classes mirroring DequantError (dequant.rs:37-70) and
 * PMetalError::Quantization (quantize.rs:82-85). */
enum {
    PMO_OK = 0,
    PMO_ERR_UNSUPPORTED_TYPE = 2,
    PMO_ERR_INVALID_SIZE = 3,
    PMO_ERR_INVALID_SHAPE = 6,
    PMO_ERR_SHAPE_TOO_LARGE = 7,
};

/* Q4_K element order used by dequantize / matvec:
 *   REF  = the order the reference's dequantize_q4k emits (k_quants.rs:365-403);
 *   GGML = the order its own quantizer packs (k_quants.rs:946-951). */
enum { PMO_ORDER_REF = 0, PMO_ORDER_GGML = 1 };

/* half 2.7.1 conversions (Cargo.lock:2429-2432): IEEE binary16 / bfloat16, RNE. */
uint16_t pmo_f32_to_f16(float f);
float pmo_f16_to_f32(uint16_t h);
uint16_t pmo_f32_to_bf16(float f);
float pmo_bf16_to_f32(uint16_t h);

/* quantize.rs:566-570 */
int32_t pmo_nearest_int(float v);
/* quantize.rs:583-644; n <= 256 */
void pmo_make_qkx1_quants(int32_t nmax, int32_t ntry, const float *x, int32_t n,
                          float *scale_out, float *min_out);
/* quantize.rs:738-841; n <= 256; ls receives n values in [0, 2*nmax) */
float pmo_make_qx_quants(int32_t n, int32_t nmax, const float *x, int32_t rmse_type, int8_t *ls);
/* quantize.rs:844-855 */
void pmo_get_scale_min_k4(int32_t j, const uint8_t *q, uint8_t *sc, uint8_t *m);

/* types.rs:102-187 */
size_t pmo_type_size(uint32_t ggml_type);  /* 0 if not one of the path's types */
size_t pmo_block_size(uint32_t ggml_type); /* 0 if not one of the path's types */
size_t pmo_tensor_size(uint32_t ggml_type, size_t n_elements);

/* quantize.rs:268-300, k_quants.rs:876-955, k_quants.rs:1056-1134.
 * dst must hold pmo_tensor_size(type, n) bytes. */
void pmo_quantize_q8_0(const float *x, size_t n, uint8_t *dst);
void pmo_quantize_q4k(const float *x, size_t n, uint8_t *dst);
void pmo_quantize_q6k(const float *x, size_t n, uint8_t *dst);
/* k_quants.rs:960-1051 (176-byte blocks: d, dmin, scales[12], qh[32], qs[128]) */
void pmo_quantize_q5k(const float *x, size_t n, uint8_t *dst);

/* k_quants.rs:1242-1321 (84-byte blocks: scales[16], qs[64], d, dmin) and :1139-1237 (110-byte blocks: hmask[32],
 * qs[64], scales[12], d) */
void pmo_quantize_q2k(const float *x, size_t n, uint8_t *dst);
void pmo_quantize_q3k(const float *x, size_t n, uint8_t *dst);
/* quantize.rs:655-727: returns the scale; ls (may be NULL) receives the n quants, offset by nmax */
float pmo_make_q3_quants(const float *x, int32_t n, int32_t nmax, int32_t do_rmse, int8_t *ls);

/* dequant.rs:466-495, k_quants.rs:358-404 + 515-560, k_quants.rs:474-496 + 614-660.
 * src holds pmo_tensor_size(type, n) bytes; dst receives n floats. */
void pmo_dequantize_q8_0(const uint8_t *src, size_t n, float *dst);
void pmo_dequantize_q4k(const uint8_t *src, size_t n, float *dst, uint32_t order);
void pmo_dequantize_q6k(const uint8_t *src, size_t n, float *dst);
/* k_quants.rs:407-462 + :663-710; order 0 = the reference's emission order, 1 = the inverse of quantize_q5k's packing */
void pmo_dequantize_q5k(const uint8_t *src, size_t n, float *dst, uint32_t order);

/* k_quants.rs:230-266 + :762-810 and :281-355 + :713-760 (both are the inverses of their quantizers' packing) */
void pmo_dequantize_q2k(const uint8_t *src, size_t n, float *dst);
void pmo_dequantize_q3k(const uint8_t *src, size_t n, float *dst);

/* quantize.rs:17-87 (dispatcher) and dequant.rs:92-132 + 184-216 (dispatcher and
 * validation).  Return a PMO_* code. */
void pmo_quantize_q4_0(const float *x, size_t n, uint8_t *dst); /* quantize.rs:93-128 */
void pmo_quantize_q4_1(const float *x, size_t n, uint8_t *dst); /* :130-157 */
void pmo_quantize_q5_0(const float *x, size_t n, uint8_t *dst); /* :159-191 */
void pmo_quantize_q5_1(const float *x, size_t n, uint8_t *dst); /* :193-230 */
void pmo_quantize_q8_1(const float *x, size_t n, uint8_t *dst); /* :302-330 */
void pmo_dequantize_legacy(uint32_t ggml_type, const uint8_t *src, size_t n, float *dst); /* dequant.rs:300-463, :505-528 */
int32_t pmo_quantize(uint32_t ggml_type, const float *x, size_t n, uint8_t *dst, size_t dst_len);
int32_t pmo_dequantize(uint32_t ggml_type, const uint8_t *src, size_t src_len, const int32_t *shape,
                       size_t ndim, float *dst, size_t dst_cap, uint32_t order);

/* crates/pmetal/src/commands/quantize.rs:988-993 */
int32_t pmo_use_more_bits(size_t layer, size_t n_layers);
/* crates/pmetal/src/commands/quantize.rs:955-980 */
int32_t pmo_is_quantizable_gguf_tensor(const char *gguf_name, size_t ndim);
/* crates/pmetal/src/commands/quantize.rs:999-1137 restricted to method q4_k_m:
 * returns the GgmlType id chosen for the tensor. */
uint32_t pmo_q4km_tensor_type(const char *gguf_name, size_t ndim, size_t n_layers);

/* Q8_K activation blocks and the integer dot products over them.
 * k_quants.rs:140-155 BlockQ8K {f32 d; i8 qs[256]; i16 bsums[16]} = 292 bytes; :815-871 quantize_q8k (a trailing
 * partial block stays all-zero); vec_dot.rs:617-656 scalar vec_dot_q4k_q8k, :658-692 scalar vec_dot_q6k_q8k.
 * pmo_qmatvec_q8k: y[r] = vec_dot(row r of W, xq) for W of type Q4K, Q6K, Q5K, Q3K or Q2K, k a multiple of 256. */
size_t pmo_q8k_size(size_t n_elements);
/* k_quants.rs:498-506 + :562-610 */
void pmo_dequantize_q8k(const uint8_t *src, size_t n, float *dst);
/* dynamic.rs:140-180 compute_kl_divergence: normalised RMSE + cosine distance, sequential f64 sums */
double pmo_kl_divergence(const float *original, const float *dequantized, size_t n);
void pmo_quantize_q8k(const float *x, size_t n, uint8_t *dst);
float pmo_vec_dot_q4k_q8k(const uint8_t *xs, const uint8_t *ys, size_t n_blocks);
float pmo_vec_dot_q6k_q8k(const uint8_t *xs, const uint8_t *ys, size_t n_blocks);
/* vec_dot.rs:695-737, :739-777, :779-810: the scalar dot products of the other k-quants, each in the element order that
 * routine itself uses (linear in the element index; not the order the dequantizers of these types use).  Pinned by
 * tests/test_q8k.py: sums derived by hand, single-position blocks against the index arithmetic above. */
float pmo_vec_dot_q5k_q8k(const uint8_t *xs, const uint8_t *ys, size_t n_blocks);
float pmo_vec_dot_q3k_q8k(const uint8_t *xs, const uint8_t *ys, size_t n_blocks);
float pmo_vec_dot_q2k_q8k(const uint8_t *xs, const uint8_t *ys, size_t n_blocks);
int32_t pmo_qmatvec_q8k(uint32_t ggml_type, const uint8_t *w, size_t n_rows, size_t k, const uint8_t *xq, float *y);

/* Not a reference function: "reference dequantize, then matmul", the definition
 * the fused GEMV/GEMM kernels are checked against.  W is [n_rows, k] quantized
 * row-major; x is f32 [k]; y[n] = sum_k W[n,k]*x[k] accumulated in double and
 * rounded once.  The _f32 variant accumulates sequentially in float (what a
 * plain f32 CPU matmul after the reference's dequantize would do) and is the
 * function the CPU baseline times. */
int32_t pmo_qmatvec_f64(uint32_t ggml_type, const uint8_t *w, size_t n_rows, size_t k,
                        const float *x, float *y, uint32_t order);
int32_t pmo_qmatvec_f32(uint32_t ggml_type, const uint8_t *w, size_t n_rows, size_t k,
                        const float *x, float *y, uint32_t order);
/* Y[m, n] = sum_k X[m,k] * W[n,k]; X f32 [m_rows, k] row-major, Y f32 [m_rows, n_rows]. */
int32_t pmo_qmatmul_f64(uint32_t ggml_type, const uint8_t *w, size_t n_rows, size_t k,
                        const float *x, size_t m_rows, float *y, uint32_t order);

/* The functions above over `threads` host threads (ranges of blocks or of rows; bit-identical to the single-threaded
 * results).  Not how the reference runs (it is single-threaded): for whole-tensor tests and the all-cores CPU figure. */
int32_t pmo_quantize_mt(uint32_t ggml_type, const float *x, size_t n, uint8_t *dst, size_t dst_len, int32_t threads);
int32_t pmo_qmatvec_mt(uint32_t ggml_type, const uint8_t *w, size_t n_rows, size_t k, const float *x, float *y,
                       uint32_t order, int32_t f64_acc, int32_t threads);
int32_t pmo_qmatmul_f64_mt(uint32_t ggml_type, const uint8_t *w, size_t n_rows, size_t k, const float *x, size_t m_rows,
                           float *y, uint32_t order, int32_t threads);

#ifdef __cplusplus
}
#endif
#endif
