/*
 * pmetal_hip.h -- C ABI of libpmetal_hip.so: PMetal's GGUF block-quantized weight
 * path (Q8_0, Q4_K and Q6_K first; Q5_K, Q3_K, Q2_K, Q8_K and the other 32-element
 * formats beside them) as hand-written HIP kernels for MI355X (gfx950).
 *
 * This is the surface a Rust `-sys` crate binds (plain pointers and sizes, no
 * C++ or framework types).  Every entry point names the reference interface it
 * stands in for as file:line under the reference tree (Epistates/pmetal).
 *
 * Conventions
 *  - Return value: 0 on success, otherwise one of the PMETAL_HIP_ERR_* classes; the
 *    failing call also stores a message in a thread-local slot (the pattern of
 *    crates/pmetal-bridge/cpp/bridge/common.h:41-58).  Nothing throws or aborts
 *    across the ABI.
 *  - Ownership: the caller owns every buffer it passes and every device allocation
 *    it requested; the library keeps no caller pointer after a call returns.
 *  - Device pointers must be 16-byte aligned (hipMalloc and torch allocations are;
 *    GGUF tensor data is 32-byte aligned in the file).  One exception: the output of
 *    pmetal_hip_qgemv needs 4-byte alignment only, so that it can be a row of an [m, n] matrix.
 *  - `stream` is a hipStream_t passed as void*; NULL is the default stream.  Device
 *    entry points are asynchronous on that stream; host-pointer entry points
 *    synchronise before returning.
 *  - Tensors are flat row-major [rows, k]; blocks run along k.
 *  - There is no CPU fallback: without a usable HIP device every compute entry
 *    point fails with PMETAL_HIP_ERR_NO_DEVICE.
 */
#ifndef PMETAL_HIP_H
#define PMETAL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GgmlType ids: crates/pmetal-gguf/src/types.rs:16-97. */
#define PMETAL_GGML_TYPE_F32 0u
#define PMETAL_GGML_TYPE_F16 1u
/* the 32-element formats beside Q8_0: quantize (quantize.rs:93-230, :302-359) and dequantize (dequant.rs:300-463, :505-528) only */
#define PMETAL_GGML_TYPE_Q4_0 2u
#define PMETAL_GGML_TYPE_Q4_1 3u
#define PMETAL_GGML_TYPE_Q5_0 6u
#define PMETAL_GGML_TYPE_Q5_1 7u
#define PMETAL_GGML_TYPE_Q8_0 8u
#define PMETAL_GGML_TYPE_Q8_1 9u
#define PMETAL_GGML_TYPE_Q2K 10u /* quantize / dequantize (k_quants.rs:1242-1321, :230-266), the fused GEMV and the fused GEMM */
#define PMETAL_GGML_TYPE_Q3K 11u /* quantize / dequantize (k_quants.rs:1139-1237, :281-355), the fused GEMV and the fused GEMM */
#define PMETAL_GGML_TYPE_Q4K 12u
#define PMETAL_GGML_TYPE_Q5K 13u /* quantize / dequantize (k_quants.rs:960-1051, :407-462), the fused GEMV and the fused GEMM */
#define PMETAL_GGML_TYPE_Q6K 14u
#define PMETAL_GGML_TYPE_Q8K 15u /* quantize / dequantize (k_quants.rs:815-871, :498-506) and the activation side of qgemv_q8k */

/* Error classes.  1-3, 6, 7 map onto DequantError (crates/pmetal-gguf/src/dequant.rs:37-70)
 * and PMetalError::Quantization (crates/pmetal-core/src/error.rs:50-52). */
#define PMETAL_HIP_OK 0
#define PMETAL_HIP_ERR_INVALID_ARG 1      /* null pointer, misalignment, bad enum        */
#define PMETAL_HIP_ERR_UNSUPPORTED_TYPE 2 /* DequantError::UnsupportedType / Quantization */
#define PMETAL_HIP_ERR_INVALID_SIZE 3     /* DequantError::InvalidSize                    */
#define PMETAL_HIP_ERR_HIP_RUNTIME 4      /* a HIP call failed; message has hipGetErrorString */
#define PMETAL_HIP_ERR_NO_DEVICE 5
#define PMETAL_HIP_ERR_INVALID_SHAPE 6   /* DequantError::InvalidShape                   */
#define PMETAL_HIP_ERR_SHAPE_TOO_LARGE 7 /* DequantError::ShapeTooLarge                  */
#define PMETAL_HIP_ERR_BUSY 8            /* a shared resource of the library is in use by another call */

/* Q4_K element order for dequantize / GEMV / GEMM.
 *  REF : the order the reference's dequantize_q4k emits (k_quants.rs:365-403); default,
 *        bit-compatible with what `load_gguf` (weight_format.rs:299) hands to the model.
 *  GGML: the inverse of the packing done by the reference's quantize_q4k
 *        (k_quants.rs:946-951), i.e. what llama.cpp/Candle decode.                     */
#define PMETAL_HIP_ORDER_REF 0u
#define PMETAL_HIP_ORDER_GGML 1u

/* Activation / output element types. */
#define PMETAL_HIP_DTYPE_F32 0u
#define PMETAL_HIP_DTYPE_BF16 1u

/* ---- lifecycle and errors (crates/pmetal-bridge/cpp/bridge/common.h:41-58) ---------- */
int32_t pmetal_hip_device_count(void);
/* Selects `device` for the calling thread and loads the kernels. */
int32_t pmetal_hip_init(int32_t device);
int32_t pmetal_hip_last_error_code(void);
/* NUL-terminated, never NULL, valid until the next call on this thread. */
const char *pmetal_hip_last_error_message(void);
void pmetal_hip_clear_error(void);

/* ---- sizes (crates/pmetal-gguf/src/types.rs:102-187) -------------------------------- */
size_t pmetal_hip_type_size(uint32_t ggml_type);  /* bytes per block; 0 if unsupported  */
size_t pmetal_hip_block_size(uint32_t ggml_type); /* elements per block; 0 if unsupported */
size_t pmetal_hip_tensor_size(uint32_t ggml_type, size_t n_elements);
/* dequant.rs:178-206 expected_byte_size_checked: validates `shape`, returns the byte size
 * through *out_bytes and the element count through *out_elements (either may be NULL). */
int32_t pmetal_hip_expected_byte_size(uint32_t ggml_type, const int32_t *shape, size_t ndim,
                                      size_t *out_bytes, size_t *out_elements);
/* dequant.rs:135 is_supported / quantize.rs:17-87 arms, restricted to this path. */
int32_t pmetal_hip_is_supported(uint32_t ggml_type);

/* ---- device memory ------------------------------------------------------------------ */
void *pmetal_hip_alloc(size_t bytes); /* NULL on failure (error slot set) */
int32_t pmetal_hip_free(void *dptr);
int32_t pmetal_hip_h2d(void *dst_dev, const void *src_host, size_t bytes);
int32_t pmetal_hip_d2h(void *dst_host, const void *src_dev, size_t bytes);
int32_t pmetal_hip_memset(void *dst_dev, int value, size_t bytes, void *stream);
int32_t pmetal_hip_sync(void *stream);

/* ---- streams and recorded launch sequences ---------------------------------------------
 * No counterpart in the reference's FFI: there MLX evaluates its lazily built graph and owns the
 * scheduling.  A decode step is some 130 small launches, and issuing them one by one from the host
 * costs more than running them; a recording replays the whole sequence with one submission (a HIP
 * graph).  Between record_begin and record_end every kernel launch issued on `stream` through this
 * library is recorded instead of run.  Record only launch-type calls (qgemv, qgemv_batch,
 * quantize_dev, dequantize_dev, f32_to_bf16_dev, qgemm_noalloc, and qgemm / qlinear once a call of
 * the same or a larger shape has run on that stream: nothing can be allocated while a stream is
 * being recorded, and a qgemm whose scratch does not exist yet fails with INVALID_ARG);
 * pmetal_hip_memset refuses to be recorded.  A recording holds the pointers it was recorded
 * with, the library's scratch buffer of that stream included: that buffer is kept until the
 * stream is destroyed, whatever runs on the stream later.  pmetal_hip_stream_destroy waits for
 * the stream and releases the calling thread's scratch for it; recordings made on a destroyed
 * stream must not be replayed.                                                              */
void *pmetal_hip_stream_create(void); /* NULL on failure (error slot set) */
int32_t pmetal_hip_stream_destroy(void *stream);
int32_t pmetal_hip_record_begin(void *stream); /* `stream` must come from pmetal_hip_stream_create */
void *pmetal_hip_record_end(void *stream);     /* the recording, NULL on failure */
int32_t pmetal_hip_replay(void *recording, void *stream);
int32_t pmetal_hip_recording_destroy(void *recording);

/* ---- events (timing on the stream the kernels run on) -------------------------------- */
void *pmetal_hip_event_create(void);
int32_t pmetal_hip_event_record(void *event, void *stream);
int32_t pmetal_hip_event_elapsed_ms(void *start, void *stop, float *ms); /* syncs on stop */
int32_t pmetal_hip_event_destroy(void *event);

/* ---- quantize: pmetal_gguf::quantize::quantize(data, dtype) -> Vec<u8> ---------------
 * crates/pmetal-gguf/src/quantize.rs:17-87; kernels follow quantize_q8_0 (:268-300),
 * quantize_q4k (k_quants.rs:876-955), quantize_q6k (k_quants.rs:1056-1134).
 * Output bytes are bit-identical to the reference CPU path.  dst_len must equal
 * pmetal_hip_tensor_size(type, n).  A trailing partial 256-super-block is emitted as
 * zero bytes (k_quants.rs:890-892); Q8_0 zero-pads inside its last block.
 * The host variants (here and of dequantize) are synchronous; tensors of 256 Ki elements
 * or more stream through pinned staging buffers that the library keeps (3 x 21 MiB of
 * pinned host and of device memory per device, made on first use), and such calls take
 * turns across threads.                                                                */
int32_t pmetal_hip_quantize(uint32_t ggml_type, const float *src_host, size_t n, uint8_t *dst_host,
                            size_t dst_len);
int32_t pmetal_hip_quantize_dev(uint32_t ggml_type, const float *src_dev, size_t n, uint8_t *dst_dev,
                                size_t dst_len, void *stream);
/* The tensor loop of a model (run_quantization, crates/pmetal/src/commands/quantize.rs:1378-1428: one quantize call
 * per tensor) in one call: the bytes of one pmetal_hip_quantize_dev per descriptor.  The tensors are independent, so the
 * library spreads them over `stream` and a second stream of its own (per calling thread, default priority): one kernel's
 * last workgroups overlap the next kernel's first (a batch of one k-quant tensor of 2^24 elements or more is cut in two for
 * the same reason).  Asynchronous like the single call: the batch starts behind what
 * `stream` holds, and work given to `stream` afterwards runs behind every tensor of the batch.  All descriptors are checked
 * before anything is launched.  A batch issued while `stream` is being recorded runs on `stream` alone.               */
typedef struct pmetal_hip_quantize_desc {
    uint32_t ggml_type;
    uint32_t reserved;
    const float *src_dev;
    size_t n;
    uint8_t *dst_dev;
    size_t dst_len;
} pmetal_hip_quantize_desc;
int32_t pmetal_hip_quantize_batch_dev(const pmetal_hip_quantize_desc *descs, size_t count, void *stream);

/* ---- dequantize: pmetal_gguf::dequant::dequantize(data, dtype, shape) -> Vec<f32> ----
 * crates/pmetal-gguf/src/dequant.rs:92-132 with its validation (:184-216); kernels follow
 * dequantize_q8_0 (:466-495), dequantize_q4k (k_quants.rs:358-404, :515-560),
 * dequantize_q6k (k_quants.rs:474-496, :614-660).  Values are bit-identical to the
 * reference.  dst_len is the capacity of dst in floats and must be >= the element count.
 * The host variant mirrors MlxMetalBridge::dequantize_q4_0 (crates/pmetal-mlx/src/
 * bridge.rs:65-84): host bytes in, synchronous.                                         */
int32_t pmetal_hip_dequantize(uint32_t ggml_type, const uint8_t *src_host, size_t src_len,
                              const int32_t *shape, size_t ndim, float *dst_host, size_t dst_len,
                              uint32_t order);
int32_t pmetal_hip_dequantize_dev(uint32_t ggml_type, const uint8_t *src_dev, size_t src_len, float *dst_dev,
                                  size_t n, uint32_t order, void *stream);

/* ---- quantized linear ------------------------------------------------------------------
 * Stand in for InlineArray::quantized_matmul(x, w, .., transpose = true, ..)
 * (crates/pmetal-bridge/src/inline_array/quantized.rs:55-108, C side
 * crates/pmetal-bridge/cpp/bridge/quantized.h:19-22) and LayerWeight::matmul_from
 * (crates/pmetal-bridge/src/qwen3_native/weights.rs:66-84) for GGUF-typed weights:
 *   y[n]    = sum_k W[n,k] * x[k]                      (qgemv, one token)
 *   Y[m, n] = sum_k X[m,k] * W[n,k]                    (qgemm, m tokens)
 * with W = reference dequantize of the packed blocks (order as given), fp32 accumulation,
 * max relative error <= 1e-3 against dequantize-then-f32-matmul.
 * W: [n, k] packed row-major, k a multiple of the block size.  x/X: f32 or bf16.
 * Types: every type has both kernels (the Q5_K GEMM is the Q4_K kernel with the fifth bit of every quant taken from the
 * block's qh bytes; Q3_K and Q2_K share a kernel for sixteen 16-element sub-blocks).  The GEMV of Q5_K, Q3_K and Q2_K takes
 * k <= 32768 and a tensor below 4 GiB, any number of rows; beyond that qgemv fails with SHAPE_TOO_LARGE and qlinear uses the
 * GEMM.  Every type has a second GEMM kernel for m <= 16 (Q4_K, Q5_K, Q8_0 and Q2_K: m <= 32) that reads the weights once; qlinear runs two activation rows of a
 * Q5_K, Q3_K or Q2_K weight of at most 2^23 elements as two GEMVs, and a larger weight or more rows as one GEMM.
 * y/Y: f32 (qgemv) or f32/bf16 (qgemm), row-major [m, n].
 * qgemm keeps scratch memory (converted activations, partial tiles) inside the library, one
 * buffer per calling thread, device and stream; it grows on demand, which synchronises that
 * stream once.                                                                           */
int32_t pmetal_hip_qgemv(uint32_t ggml_type, const uint8_t *w_dev, int64_t n, int64_t k, const void *x_dev,
                         uint32_t x_dtype, float *y_dev, uint32_t order, void *stream);
int32_t pmetal_hip_qgemm(uint32_t ggml_type, const uint8_t *w_dev, int64_t n, int64_t k, const void *x_dev,
                         uint32_t x_dtype, int64_t m, void *y_dev, uint32_t y_dtype, uint32_t order,
                         void *stream);
/* pmetal_hip_qgemm without any allocation.  No counterpart in the reference (there MLX owns every buffer): it is for
 * callers that cannot call hipMalloc -- code under HIP graph capture, tight serving loops, harnesses that forbid it.
 * Same arguments, kernels and results (bit for bit) as pmetal_hip_qgemm; the scratch memory
 * (converted activations, row scales, partial tiles of a K split) is a fixed array of
 * PMETAL_HIP_NOALLOC_SCRATCH_BYTES inside the library's code object, one copy per device, held until the process ends.
 * A shape that needs more (roughly: m * k * 2.25 bytes plus, for few activation rows, splits * m * n * 4) fails with
 * PMETAL_HIP_ERR_SHAPE_TOO_LARGE before anything is launched.  Calls no hipMalloc / hipFree and nothing else that allocates.
 * pmetal_hip_init(device) looks the array's address up; without it the first call on a device does.  All calls on one
 * device share the array: calls on one stream are ordered and may follow each other without a synchronisation; a call
 * that would overlap another one on the same device -- issued on a different stream before the previous call's kernels
 * have finished, or from a second thread while a call is being issued -- is refused with PMETAL_HIP_ERR_BUSY and launches
 * nothing.  Calls issued while their stream is being recorded cannot be checked this way: keeping replays of such
 * recordings from overlapping each other, and other calls, stays with the caller.                                     */
#define PMETAL_HIP_NOALLOC_SCRATCH_BYTES ((size_t)32 << 20)
int32_t pmetal_hip_qgemm_noalloc(uint32_t ggml_type, const uint8_t *w_dev, int64_t n, int64_t k, const void *x_dev,
                                 uint32_t x_dtype, int64_t m, void *y_dev, uint32_t y_dtype, uint32_t order,
                                 void *stream);
/* Dispatch by m: m == 1 -> qgemv (f32 output only), otherwise qgemm (k must be a multiple of 256).  A Q8_0
 * row that is only a multiple of 32 runs one GEMV per activation row when m > 1 (f32 output only), and so do
 * Q5_K, Q3_K and Q2_K weights of at most 2^23 elements for m = 2, with f32 output. */
int32_t pmetal_hip_qlinear(uint32_t ggml_type, const uint8_t *w_dev, int64_t n, int64_t k, const void *x_dev,
                           uint32_t x_dtype, int64_t m, void *y_dev, uint32_t y_dtype, uint32_t order,
                           void *stream);

/* Several weights against the same [m, k] activations (the gate / up or q / k / v projections of a prefill: what a layer's
 * consecutive LayerWeight::matmul_from calls on one input amount to, weights.rs:66-84): the same results as one
 * pmetal_hip_qgemm per weight, bit for bit, with the activations converted once per element order instead of once per
 * weight.  The weights may differ in type, n, output type and element order (Q4_K and Q5_K weights in the GGML order share
 * one conversion, Q3_K and Q2_K weights another).                                                                       */
typedef struct pmetal_hip_gemm_desc {
    uint32_t ggml_type;
    uint32_t y_dtype;
    uint32_t order;
    uint32_t reserved;
    int64_t n;
    const uint8_t *w_dev;
    void *y_dev;
} pmetal_hip_gemm_desc;
int32_t pmetal_hip_qgemm_batch(const pmetal_hip_gemm_desc *descs, size_t count, int64_t k, const void *x_dev,
                               uint32_t x_dtype, int64_t m, void *stream);

/* Re-blocked weights for the GEMM of Q5_K / Q3_K / Q2_K: the form these types multiplied in before they had matrix kernels of
 * their own, kept for callers that prepared one (pmetal_hip_qgemm on the original blocks is the faster way and needs no copy).
 * The reference brings a weight into the layout its matmul wants once, when the model is loaded (LayerWeight,
 * crates/pmetal-bridge/src/qwen3_native/weights.rs:29-45: dense weights are transposed at load time, quantized ones kept as
 * MLX's quantized_matmul reads them); the counterpart here: the super-blocks convert without loss into one (Q3_K) or two
 * (Q5_K, Q2_K: values and mins) Q6_K tensors.  pmetal_hip_reblock_dev does that conversion once into memory the caller owns
 * (pmetal_hip_reblock_size bytes: 210 bytes per super-block and part, each part rounded up to 16; 0 for a type or shape
 * that is not re-blocked); pmetal_hip_qgemm_reblocked multiplies with it: the same numbers as pmetal_hip_qgemm on the
 * original blocks, to the order of the f32 sums.  `order` applies to Q5_K only.
 * The GEMV of these types reads the original blocks; a caller that wants both keeps both.                              */
size_t pmetal_hip_reblock_size(uint32_t ggml_type, int64_t n, int64_t k);
int32_t pmetal_hip_reblock_dev(uint32_t ggml_type, const uint8_t *w_dev, int64_t n, int64_t k, uint32_t order,
                               uint8_t *dst_dev, size_t dst_len, void *stream);
int32_t pmetal_hip_qgemm_reblocked(uint32_t ggml_type, const uint8_t *reblocked_dev, size_t reblocked_len, int64_t n,
                                   int64_t k, const void *x_dev, uint32_t x_dtype, int64_t m, void *y_dev, uint32_t y_dtype,
                                   void *stream);

/* One decode step's worth of batch-1 projections, launched back to back on one stream
 * (the per-token loop over LayerWeight::matmul_from, weights.rs:66-84). */
typedef struct pmetal_hip_linear_desc {
    uint32_t ggml_type;
    uint32_t x_dtype;
    uint32_t order;
    uint32_t reserved;
    int64_t n;
    int64_t k;
    const uint8_t *w_dev;
    const void *x_dev;
    float *y_dev;
} pmetal_hip_linear_desc;
int32_t pmetal_hip_qgemv_batch(const pmetal_hip_linear_desc *descs, size_t count, void *stream);

/* ---- Q8_K activations and the integer dot products over them ----------------------------
 * quantize_q8k (crates/pmetal-gguf/src/k_quants.rs:815-871) into BlockQ8K (k_quants.rs:140-155:
 * f32 d, i8 qs[256], i16 bsums[16]; 292 bytes per 256 elements, a trailing partial block all-zero),
 * bytes bit-identical to the reference; dst_len must be pmetal_hip_q8k_size(n).
 * qgemv_q8k: y[r] = vec_dot_q4k_q8k / _q6k_ / _q5k_ / _q3k_ / _q2k_q8k (row r of W, xq) as the reference's scalar
 * definitions compute them (crates/pmetal-gguf/src/vec_dot.rs:617-656, :658-692, :695-737, :739-777, :779-810), bit for
 * bit: exact integer sums per super-block, the float sum over the super-blocks in their order.
 * ggml_type Q4K, Q6K, Q5K, Q3K or Q2K; k a multiple of 256, at most 32768; xq_dev holds k / 256 blocks.  For
 * Q4_K the pairing of nibbles and activations is the quantizer's own (GGML) order; for the other types it is the order
 * linear in the element index that each of those dot products uses, which is not the order the dequantizer of the type
 * uses (and vec_dot_q3k_q8k gives the second half of every super-block a zero scale: reproduced as it is).      */
size_t pmetal_hip_q8k_size(size_t n_elements);
int32_t pmetal_hip_quantize_q8k_dev(const float *src_dev, size_t n, uint8_t *dst_dev, size_t dst_len, void *stream);
int32_t pmetal_hip_qgemv_q8k(uint32_t ggml_type, const uint8_t *w_dev, int64_t n, int64_t k, const uint8_t *xq_dev,
                             float *y_dev, void *stream);

/* ---- KL calibration metric -------------------------------------------------------------
 * compute_kl_divergence (crates/pmetal-gguf/src/dynamic.rs:140-180): normalised RMSE plus cosine distance between n
 * original and n dequantized values, both on the device, accumulated in f64 (in a different order than the
 * reference's sequential loop: equal to about 1e-13 relative).  Synchronises the stream; *score is host memory.
 * The quantize -> dequantize -> score loop of calibrate_tensor (dynamic.rs:420-502) is host logic over
 * pmetal_hip_quantize_dev / _dequantize_dev / this (pmetal_gguf::calibrate_tensor, pmetal_amd.gguf.calibrate_tensor). */
int32_t pmetal_hip_kl_divergence_dev(const float *original_dev, const float *dequantized_dev, size_t n, double *score,
                                     void *stream);
/* The dequantize and score steps of that loop (dynamic.rs:462-467) in one pass for the k-quant types (Q2_K .. Q6_K,
 * Q8_K): the first n elements of the blocks are decoded in registers, in the given element order, and compared with
 * original_dev[0..n) without being stored.  Equal to _dequantize_dev followed by _kl_divergence_dev up to the order of
 * the f64 sums.  Any other type: PMETAL_HIP_ERR_UNSUPPORTED_TYPE; n beyond what the blocks hold: ..._INVALID_SIZE. */
int32_t pmetal_hip_kl_divergence_quantized_dev(uint32_t ggml_type, const uint8_t *quantized_dev, size_t quantized_len,
                                               const float *original_dev, size_t n, uint32_t order, double *score,
                                               void *stream);

/* ---- Q4_K_M recipe (crates/pmetal/src/commands/quantize.rs) --------------------------- */
int32_t pmetal_hip_use_more_bits(size_t layer, size_t n_layers);                   /* :988-993  */
int32_t pmetal_hip_is_quantizable_gguf_tensor(const char *gguf_name, size_t ndim); /* :955-980  */
/* llama_style_tensor_type (:999-1137) for method q4_k_m: GgmlType id for the tensor. */
uint32_t pmetal_hip_q4km_tensor_type(const char *gguf_name, size_t ndim, size_t n_layers);

/* ---- synthetic tensors for benchmarks (no reference counterpart) ---------------------- */
/* Fills dst_dev[n] with N(0, std^2) from a counter-based generator keyed by (seed, index);
 * a fraction `outlier_rate` of elements is replaced by +-outlier_mag.                    */
int32_t pmetal_hip_fill_normal_f32(float *dst_dev, size_t n, uint64_t seed, float std, float outlier_rate,
                                   float outlier_mag, void *stream);
/* f32 -> bf16 (round to nearest even), device to device. */
int32_t pmetal_hip_f32_to_bf16_dev(const float *src_dev, uint16_t *dst_dev, size_t n, void *stream);


/* ---- measurement aid (no reference counterpart) ---------------------------------------
 * Launches a register-only loop of `iters` x 4 v_mfma_f32_32x32x16_f16 per wave on `workgroups`
 * workgroups of 8 waves (131072 flops per matrix instruction and wave; no memory traffic), so that a
 * caller can time what the matrix cores of this machine sustain: the published peak assumes the top
 * clock, which a long matrix loop does not hold.  vary = 0: all operands 1.0; vary = 1: operands
 * differ per lane and change over time.  `sink_dev` is a 4-byte device buffer (never written in
 * practice).                                                                                */
int32_t pmetal_hip_mfma_probe_f16(int32_t iters, int32_t vary, int32_t workgroups, float *sink_dev, void *stream);

/* Launches a kernel that does nothing but read `bytes` (rounded down to 16) from src_dev with 16-byte loads, so that a
 * caller can time what a single launch over that many bytes costs on this machine when nothing is computed: the floor the
 * fused GEMV of a tensor of that size is measured against.  `sink_dev` is a 4-byte device buffer (never written in
 * practice).                                                                                                         */
int32_t pmetal_hip_read_probe(const void *src_dev, size_t bytes, uint32_t *sink_dev, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PMETAL_HIP_H */
