/*
 * peregrine_hip.h -- C ABI of libperegrine_hip.so: peregrine's quantized-inference
 * operators served by hand-written HIP kernels for AMD MI355X (gfx950).
 *
 * Every entry point replaces one function of the reference crate
 * (etam103/peregrine v0.32.0); the file:line it replaces is cited beside it.
 * Conventions:
 *   - plain pointers and sizes only; all matrices are dense row-major;
 *   - every function returns pg_status (0 = PG_OK) and never aborts or unwinds
 *     across the ABI; pg_last_error() gives the message of the last failure.
 *     The reference panics on shape mismatch (assert!/assert_eq!); a binding
 *     that wants that contract turns a non-zero status into a panic;
 *   - functions without a `_dev` suffix take HOST pointers, are synchronous, and
 *     the caller allocates every output (sizes are closed-form);
 *   - `_dev` functions take DEVICE pointers, are ordered on the context's HIP
 *     stream, and return without waiting (pg_sync() waits);
 *   - one pg_ctx = one device + one HIP stream; a context is not internally
 *     locked (the reference's callers are single-threaded: Tensor is
 *     Rc<RefCell>, src/tensor.rs:864); distinct contexts may be used from
 *     distinct threads;
 *   - the library keeps no host pointer past the return of a call.
 */
#ifndef PEREGRINE_HIP_H
#define PEREGRINE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int pg_status;
enum {
    PG_OK = 0,
    PG_EINVAL = 1,       /* shape / argument mismatch (the reference's assert!s) */
    PG_EDEVICE = 2,      /* a HIP call failed */
    PG_ENOMEM = 3,       /* device or host allocation failed */
    PG_EUNSUPPORTED = 4  /* valid request this build has no kernel for */
};

/* GGML block types, numbered as src/gguf.rs:14-33 does. */
enum { PG_GGML_Q4_0 = 2, PG_GGML_Q4_1 = 3, PG_GGML_Q8_0 = 8 };
/* Type tag reported by pg_gguf_shape for a tensor made by pg_mxfp4_upload (ggml's own number
 * for MXFP4; the reference's GGUF enum stops before it). */
enum { PG_MXFP4 = 39 };

/* Expert activation of the grouped MoE FFN. */
enum {
    PG_ACT_SILU = 0,      /* Tensor::silu  src/tensor.rs:6120-6135 (deepseek/llama experts) */
    PG_ACT_GELU_TANH = 1  /* Tensor::gelu  src/tensor.rs:3163-3179 (grok1 experts)          */
};

typedef struct pg_ctx pg_ctx;
/* Device-resident quant::QuantizedTensor (src/quant.rs:12-23). */
typedef struct pg_qtensor pg_qtensor;
/* Device-resident GGUF block tensor ([n_out, k_in], blocks of 32 along k_in). */
typedef struct pg_gguf_tensor pg_gguf_tensor;

/* ---- context ------------------------------------------------------------
 * Replaces the thread-local Metal GpuContext singleton
 * (src/metal/context.rs:2472-2510).  `hip_stream` may be NULL (the library
 * creates its own default-priority stream) or an existing hipStream_t the
 * caller owns (for example the stream a host framework launches on). */
pg_status pg_ctx_create(int device, void *hip_stream, pg_ctx **out);
void pg_ctx_destroy(pg_ctx *ctx);
/* GpuContext::sync (used as gpu.sync() in tests/quant_parity.rs:102-107). */
pg_status pg_sync(pg_ctx *ctx);
void *pg_ctx_stream(pg_ctx *ctx);
/* Message of the most recent failure on this thread ("" if none). */
const char *pg_last_error(void);
const char *pg_status_string(pg_status st);

/* Device memory for callers that have no HIP binding of their own
 * (GpuContext::alloc / upload / GpuBuffer::read, src/metal/buffer.rs). */
pg_status pg_dev_alloc(pg_ctx *ctx, size_t bytes, void **dptr);
pg_status pg_dev_free(pg_ctx *ctx, void *dptr);
pg_status pg_memcpy_h2d(pg_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
pg_status pg_memcpy_d2h(pg_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);

/* ---- quant::* (src/quant.rs) ---------------------------------------------- */

/* quant::quantize_weights  src/quant.rs:27-75.
 * w [rows, cols] f32 -> q [rows, cols] i8, q_t [cols, rows] i8 (may be NULL),
 * scales [cols].  scale[n] = absmax(w[:, n]) / 127 (1.0 for a zero column),
 * q = round_half_away(w / scale) clamped to [-127, 127]. */
pg_status pg_quantize_weights(pg_ctx *ctx, const float *w, size_t rows, size_t cols,
                              int8_t *q, int8_t *q_t, float *scales);

/* quant::quantize_activations  src/quant.rs:79-112 (x86 branch :97-109).
 * a [rows, cols] f32 -> q [rows, cols] i8, row_scales [rows]. */
pg_status pg_quantize_activations(pg_ctx *ctx, const float *a, size_t rows, size_t cols,
                                  int8_t *q, float *row_scales);
pg_status pg_quantize_activations_dev(pg_ctx *ctx, const float *a_dev, size_t rows,
                                      size_t cols, int8_t *q_dev, float *row_scales_dev);

/* quant::dequantize  src/quant.rs:115-123.  out[m, n] = (q[m, n] as f32) * scales[n]. */
pg_status pg_dequantize(pg_ctx *ctx, const int8_t *q, const float *scales, size_t rows,
                        size_t cols, float *out);

/* QuantizedTensor::to_gpu  src/quant.rs:174-181: upload data_i8 [rows, cols] and
 * scales [cols].  The device copy is kept K-contiguous ([cols, rows], the
 * reference's data_i8_t, src/quant.rs:57-62) and zero-padded for the kernels. */
pg_status pg_qtensor_upload(pg_ctx *ctx, const int8_t *q, const float *scales, size_t rows,
                            size_t cols, pg_qtensor **out);
/* quantize_weights followed by to_gpu without the round trip through the host:
 * w is a host (`pg_qtensor_from_f32`) or device (`_dev`) [rows, cols] f32 matrix. */
pg_status pg_qtensor_from_f32(pg_ctx *ctx, const float *w, size_t rows, size_t cols,
                              pg_qtensor **out);
pg_status pg_qtensor_from_f32_dev(pg_ctx *ctx, const float *w_dev, size_t rows, size_t cols,
                                  pg_qtensor **out);
/* QuantizedTensor::from_gpu  src/quant.rs:183-190 (q, q_t, scales: any may be NULL). */
pg_status pg_qtensor_download(pg_ctx *ctx, const pg_qtensor *t, int8_t *q, int8_t *q_t,
                              float *scales);
pg_status pg_qtensor_shape(const pg_qtensor *t, size_t *rows, size_t *cols);
void pg_qtensor_free(pg_ctx *ctx, pg_qtensor *t);

/* quant::matmul_quantized  src/quant.rs:129-169 (the W8A8 CPU semantics: per-row
 * dynamic i8 activations, i32 accumulate, out = (acc as f32) * a_scale[m] * w_scale[n])
 * in the slot of quant::matmul_quantized_gpu  src/quant.rs:196-218 /
 * GpuContext::dispatch_matmul_dequant_i8  src/metal/context.rs:2226-2306.
 * a [m, k] f32, k == rows of w; out [m, cols of w]. */
pg_status pg_matmul_quantized(pg_ctx *ctx, const float *a, size_t m, size_t k,
                              const pg_qtensor *w, float *out);
/* Device-pointer form.  acc_dev (may be NULL) receives the raw i32 accumulators [m, n]. */
pg_status pg_matmul_quantized_dev(pg_ctx *ctx, const float *a_dev, size_t m, size_t k,
                                  const pg_qtensor *w, float *out_dev, int32_t *acc_dev);

/* pg_matmul_quantized_dev for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same result, bit for bit; the scratch the product needs (quantised rows, row
 * scales, split-K partial sums) is a fixed 32 MiB array inside the library instead of the
 * context's growable arena, so the call allocates and frees nothing.  A product that needs more
 * than pg_fixed_scratch_bytes() -- about round_up(m, 256) * round_up(k, 128) + 4 * round_up(m, 256)
 * bytes, plus up to 16 * m * n * 4 for 5 .. 256 rows -- is PG_EINVAL (2048 x 14336 rows fit).
 * Every call on one GPU shares that GPU's array: calls that overlap on one GPU (two contexts,
 * two streams) race; calls on one context are stream-ordered and safe. */
pg_status pg_matmul_quantized_fixed_scratch_dev(pg_ctx *ctx, const float *a_dev, size_t m, size_t k,
                                                const pg_qtensor *w, float *out_dev);
size_t pg_fixed_scratch_bytes(void);

/* The fused products of models::llama: `x.matmul(qkv_fused)` / `normed.matmul(gate_up_fused)`
 * over column-concatenated weights (fuse_qkv  src/models/llama/attention.rs:51-71, used :84;
 * fuse_gate_up  src/models/llama/decoder.rs:49-67, used :78), here without a fused copy:
 * `count` (1 .. 4) weights with the same number of rows k, the activation rows quantised once,
 * one launch for more than 256 rows.  out_dev[i] is [m, cols of w[i]] and equals
 * pg_matmul_quantized_dev(a, w[i]) bit for bit (scales are per row and per column). */
pg_status pg_matmul_quantized_multi_dev(pg_ctx *ctx, const float *a_dev, size_t m, size_t k,
                                        const pg_qtensor *const *w, size_t count,
                                        float *const *out_dev);

/* The reference's GPU numerics for the same call (W8A32): f32 activations, weights
 * dequantised to f32, f32 accumulate, no activation quantisation --
 * GpuContext::dispatch_matmul_dequant_i8  src/metal/context.rs:2226-2306, shader
 * matmul_dequant_i8  src/metal/shaders.rs:2329-2375, reached through
 * quant::matmul_quantized_gpu  src/quant.rs:196-218.
 * out[m, n] = sum_k a[m, k] * ((w_i8[k, n] as f32) * scale[n]), within 1e-5 relative. */
pg_status pg_matmul_dequant_i8(pg_ctx *ctx, const float *a, size_t m, size_t k,
                               const pg_qtensor *w, float *out);
pg_status pg_matmul_dequant_i8_dev(pg_ctx *ctx, const float *a_dev, size_t m, size_t k,
                                   const pg_qtensor *w, float *out_dev);

/* ---- gguf::* (src/gguf.rs) -------------------------------------------------- */

/* gguf::f16_to_f32  src/gguf.rs:354-382, applied to n values (bit-exact, NaN payloads
 * included). */
pg_status pg_f16_to_f32(pg_ctx *ctx, const uint16_t *bits, size_t n, float *out);
/* gguf::dequant_q8_0  src/gguf.rs:286-302;  gguf::dequant_q4_0  src/gguf.rs:307-326;
 * gguf::dequant_q4_1  src/gguf.rs:331-351.  num_elements must be a multiple of 32;
 * data holds num_elements/32 blocks of 34 / 18 / 20 bytes. */
pg_status pg_dequant_q8_0(pg_ctx *ctx, const uint8_t *data, size_t num_elements, float *out);
pg_status pg_dequant_q4_0(pg_ctx *ctx, const uint8_t *data, size_t num_elements, float *out);
pg_status pg_dequant_q4_1(pg_ctx *ctx, const uint8_t *data, size_t num_elements, float *out);

/* Keep a GGUF weight quantised on the device instead of materialising f32 as
 * GgufFile::load_tensor_f32 + load_transposed_weight do
 * (src/gguf.rs:485-517, src/models/llama/model.rs:243-257).
 * blocks: the tensor's raw block bytes, [n_out, k_in] with blocks of 32 along k_in; Q4_0,
 * Q4_1 or Q8_0 (18 / 20 / 34 bytes per block, src/gguf.rs:47-55). */
pg_status pg_gguf_upload(pg_ctx *ctx, const void *blocks, int ggml_type, size_t n_out,
                         size_t k_in, pg_gguf_tensor **out);
pg_status pg_gguf_shape(const pg_gguf_tensor *t, size_t *n_out, size_t *k_in, int *ggml_type);
void pg_gguf_free(pg_ctx *ctx, pg_gguf_tensor *t);

/* The dequantise-then-matmul of models::llama, fused:
 * y [m, n_out] = x [m, k_in] . dequant(w)^T, i.e. Tensor::matmul
 * (src/tensor.rs:1342-1353) applied to the transposed dequantised weight.
 * The first call with m > 1 on a Q4_0 / Q8_0 tensor (and an expert's first pg_moe_ffn) adds a
 * second, tile-major copy of the quant payload to the handle (freed by pg_gguf_free): a
 * handle must not see its first such call from two threads at once. */
pg_status pg_gguf_matmul(pg_ctx *ctx, const float *x, size_t m, const pg_gguf_tensor *w,
                         float *y);
pg_status pg_gguf_matmul_dev(pg_ctx *ctx, const float *x_dev, size_t m,
                             const pg_gguf_tensor *w, float *y_dev);

/* Load-time preparation.  The matrix-core block product reads a tile-major copy of a Q4_0 / Q8_0 / Q4_1 tensor's
 * payload plane (as many bytes again as the payload).  Left alone, the first product that needs the copy makes it:
 * a hipMalloc, a launch and a wait inside a call that is otherwise stream-ordered and allocation-free.
 * pg_gguf_prepare makes now whatever products over up to `max_rows` activation rows of this tensor (alone, in a
 * group, inside a Llama block or as an expert of pg_moe_ffn) will need, as the reference rearranges weights at load
 * (load_transposed_weight, src/models/llama/model.rs:243-257); afterwards those calls neither allocate nor wait,
 * which a caller that captures them in a HIP graph requires.  max_rows < 2 makes nothing (one-row products read
 * the planes as uploaded), and neither does an MXFP4 tensor (all of its products do).  pg_gguf_drop_prepared frees
 * the copy again (it waits for the stream); pg_gguf_device_bytes reports what the tensor holds. */
pg_status pg_gguf_prepare(pg_ctx *ctx, const pg_gguf_tensor *w, size_t max_rows);
pg_status pg_gguf_drop_prepared(pg_ctx *ctx, const pg_gguf_tensor *w);
pg_status pg_gguf_device_bytes(const pg_gguf_tensor *w, size_t *uploaded, size_t *derived);

/* ---- MXFP4 (the gpt_oss experts' format) ------------------------------------------ */

/* mxfp4_matmul  examples/gpt_oss/moe.rs:16-53: weight [out_dim, in_dim] as 16-byte blocks of
 * FP4 codes (byte k = elements 2k low nibble, 2k+1 high) in `blocks` [out_dim * in_dim/32 * 16]
 * and one E8M0 scale byte per block in `scales` [out_dim * in_dim/32];
 * output[r] = sum_b ( sum_k LUT[code] * input[32b + k] ) * 2^(scale - 127).
 * in_dim is a multiple of 32, at most 28160 (a row's fixed-point planes live in on-chip memory; larger:
 * PG_EUNSUPPORTED).  Scale byte 0 is the reference's f32::from_bits(0) = 0.0; scale byte 255 (inf there)
 * makes the row's result NaN, as does an inf or NaN anywhere in the input. */
pg_status pg_mxfp4_matmul(pg_ctx *ctx, const float *input, const uint8_t *blocks, const uint8_t *scales,
                          size_t out_dim, size_t in_dim, float *output);
/* The same weight kept on the device: a pg_gguf_tensor (type PG_MXFP4) for pg_gguf_matmul(_dev),
 * each row of x being one mxfp4_matmul. */
pg_status pg_mxfp4_upload(pg_ctx *ctx, const uint8_t *blocks, const uint8_t *scales, size_t out_dim,
                          size_t in_dim, pg_gguf_tensor **out);

/* Mxfp4Expert  examples/gpt_oss/moe.rs:55-117: mlp1 [2*intermediate, hidden] + bias, the
 * gpt-oss SwiGLU over interleaved (gate, linear) pairs (examples/gpt_oss/moe.rs:145-154),
 * mlp2 [hidden, intermediate] + bias. */
typedef struct pg_mxfp4_expert pg_mxfp4_expert;
pg_status pg_mxfp4_expert_create(pg_ctx *ctx, size_t hidden, size_t intermediate, float alpha, float clamp,
                                 const uint8_t *mlp1_blocks, const uint8_t *mlp1_scales,
                                 const uint8_t *mlp2_blocks, const uint8_t *mlp2_scales,
                                 const float *mlp1_bias, const float *mlp2_bias, pg_mxfp4_expert **out);
void pg_mxfp4_expert_free(pg_ctx *ctx, pg_mxfp4_expert *expert);
/* Mxfp4Expert::forward  examples/gpt_oss/moe.rs:84-115 on m rows: x, out [m, hidden]. */
pg_status pg_mxfp4_expert_forward(pg_ctx *ctx, const pg_mxfp4_expert *expert, const float *x, size_t m,
                                  float *out);
/* scratch_dev: m * 3 * intermediate floats, 16-byte aligned. */
pg_status pg_mxfp4_expert_forward_dev(pg_ctx *ctx, const pg_mxfp4_expert *expert, const float *x_dev, size_t m,
                                      float *scratch_dev, float *out_dev);
/* MoELayer::forward after its router, over MXFP4 experts  examples/gpt_oss/moe.rs:286-352 (the router itself:
 * logits = x . gate + bias, top-k, softmax over the k, :289-330, is the caller's): x, out [T, hidden];
 * expert_idx, weight [T, top_k]; out[t] = sum_k weight[t, k] * experts[expert_idx[t, k]].forward(x[t]), the terms
 * added in k order.  All experts of one launch share hidden, intermediate, alpha and clamp.  The reference calls an
 * expert once per (token, k); here the tokens of each expert are gathered and every product is one launch over all
 * experts.  An index outside 0..E-1, or an expert named twice by one token (the reference would panic on the first
 * and never produces the second), is PG_EINVAL from the host-pointer form, which reads the indices; the _dev form
 * cannot look without waiting for the stream, and there such an entry contributes nothing (its weight counts as 0). */
pg_status pg_mxfp4_moe_ffn_routed(pg_ctx *ctx, const float *x, size_t T, const int32_t *expert_idx, const float *weight,
                                  size_t top_k, const pg_mxfp4_expert *const *experts, size_t E, float *out);
pg_status pg_mxfp4_moe_ffn_routed_dev(pg_ctx *ctx, const float *x_dev, size_t T, const int32_t *expert_idx_dev,
                                      const float *weight_dev, size_t top_k, const pg_mxfp4_expert *const *experts,
                                      size_t E, float *out_dev);

/* ---- GGUF container (gguf::GgufFile, src/gguf.rs:403-561) ---------------------
 * Parsing needs no device.  A malformed or truncated file is PG_EINVAL (the reference
 * returns io::Error for a bad magic/version and panics on the rest). */
typedef struct pg_gguf_file pg_gguf_file;
/* GgufFile::parse  src/gguf.rs:411-483.  `data` is borrowed and must outlive the handle. */
pg_status pg_gguf_file_parse(const void *data, size_t len, pg_gguf_file **out);
/* GgufFile::load  src/gguf.rs:405-408 (the file is memory-mapped, not read). */
pg_status pg_gguf_file_open(const char *path, pg_gguf_file **out);
void pg_gguf_file_close(pg_gguf_file *f);
/* metadata.len(), tensors.len(), header version, offset of the data section. */
pg_status pg_gguf_file_counts(const pg_gguf_file *f, size_t *n_tensors, size_t *n_metadata,
                              uint32_t *version, uint64_t *data_start);
/* GgufFile::tensor_names  src/gguf.rs:559-561 (file order). */
pg_status pg_gguf_file_tensor_name(const pg_gguf_file *f, size_t index, const char **name);
/* GgufTensor {dtype, shape, data_offset} + data_size()  src/gguf.rs:143-164.  shape is in
 * GGUF order (innermost first; tensor_shape() reverses it, src/gguf.rs:551-556);
 * data points into the parsed buffer.  Any output may be NULL. */
pg_status pg_gguf_file_tensor_info(const pg_gguf_file *f, const char *name, int *ggml_type,
                                   size_t *n_dims, uint64_t *shape, size_t shape_cap,
                                   uint64_t *data_offset, size_t *data_size, const void **data);
/* GgufFile::get_u32 / get_f32  src/gguf.rs:541-548, MetadataValue::as_str / arrays
 * src/gguf.rs:95-139.  *found = 0 (or *value = NULL, *count = (size_t)-1) when the key is
 * absent or of another type. */
pg_status pg_gguf_file_get_u32(const pg_gguf_file *f, const char *key, uint32_t *value, int *found);
pg_status pg_gguf_file_get_f32(const pg_gguf_file *f, const char *key, float *value, int *found);
pg_status pg_gguf_file_get_str(const pg_gguf_file *f, const char *key, const char **value, size_t *len);
pg_status pg_gguf_file_get_array(const pg_gguf_file *f, const char *key, uint32_t *elem_type, size_t *count);
pg_status pg_gguf_file_get_array_str(const pg_gguf_file *f, const char *key, size_t index, const char **value);
pg_status pg_gguf_file_get_array_f64(const pg_gguf_file *f, const char *key, double *values, size_t cap);
/* GgufFile::load_tensor_f32  src/gguf.rs:485-517 (F32, F16, Q8_0, Q4_0, Q4_1 -> f32). */
pg_status pg_gguf_file_load_tensor_f32(pg_ctx *ctx, const pg_gguf_file *f, const char *name,
                                       float *out, size_t out_cap);
/* The keep-quantised route: a 1-D or 2-D Q4_0 / Q8_0 tensor goes to the device as it is
 * (pg_gguf_upload with n_out = shape[1], k_in = shape[0]) instead of through
 * load_tensor_f32 + transpose  src/models/llama/model.rs:243-257. */
pg_status pg_gguf_file_upload_tensor(pg_ctx *ctx, const pg_gguf_file *f, const char *name,
                                     pg_gguf_tensor **out);

/* ---- int8 wire record (src/serial.rs:124-222) -------------------------------------
 * [name_len u32][name][dtype u8 = 1][ndim u32 = 2][rows u32][cols u32][rows*cols i8][cols f32],
 * little-endian.  Host code, no device needed except for pg_qtensor_from_record. */
pg_status pg_quantized_record_size(size_t name_len, size_t rows, size_t cols, size_t *bytes);
/* serial::write_quantized_tensor  src/serial.rs:126-157 into a caller buffer. */
pg_status pg_write_quantized_tensor(void *buf, size_t cap, const char *name, size_t name_len,
                                    const int8_t *q, const float *scales, size_t rows, size_t cols,
                                    size_t *written);
/* serial::read_quantized_tensor  src/serial.rs:161-222: the outputs point into buf (scales
 * possibly unaligned); a wrong dtype tag or ndim (the reference's assert_eq!s) and a short
 * buffer (its read_exact error) are PG_EINVAL. */
pg_status pg_read_quantized_tensor(const void *buf, size_t len, const char **name, size_t *name_len,
                                   size_t *rows, size_t *cols, const int8_t **q, const void **scales,
                                   size_t *consumed);
/* read_quantized_tensor followed by QuantizedTensor::to_gpu. */
pg_status pg_qtensor_from_record(pg_ctx *ctx, const void *buf, size_t len, pg_qtensor **out,
                                 size_t *consumed);

/* ---- Huffman-coded int8 weights (src/huffman.rs) ------------------------------------
 * Symbols are i8 values, index = value + 128.  The table builder, the encoder and the
 * HuffmanTensor container are host code (no device needed); decoding runs on the device. */
typedef struct pg_huffman_tensor pg_huffman_tensor;
/* HuffmanTable::from_frequencies  src/huffman.rs:35-150: freqs[256] -> bit_lengths[256]
 * (0 = unused, at most 12) and, if codes is not NULL, the canonical codes[256]. */
pg_status pg_huffman_table_from_frequencies(const uint64_t *freqs, uint8_t *bit_lengths, uint32_t *codes);
/* HuffmanTable::canonical_codes  src/huffman.rs:152-186 (what from_bytes, :292-306, rebuilds). */
pg_status pg_huffman_canonical_codes(const uint8_t *bit_lengths, uint32_t *codes);
/* HuffmanTable::encode  src/huffman.rs:216-251: MSB first, last byte zero-padded.  *bytes is
 * the size needed; out may be NULL to ask for it.  A symbol without a code is PG_EINVAL. */
pg_status pg_huffman_encode(const uint8_t *bit_lengths, const int8_t *data, size_t n, uint8_t *out, size_t cap,
                            size_t *bytes);
/* HuffmanTable::decode  src/huffman.rs:254-284 on the device (host pointers in and out).  A
 * stream that ends before num_symbols codes, or an unassigned code (the reference's
 * debug_assert), is PG_EINVAL. */
pg_status pg_huffman_decode(pg_ctx *ctx, const uint8_t *bit_lengths, const uint8_t *bitstream, size_t len,
                            size_t num_symbols, int8_t *out);
/* HuffmanTensor::from_quantized  src/huffman.rs:332-372: q [rows, cols] row-major, scales [cols]. */
pg_status pg_huffman_tensor_from_quantized(const int8_t *q, const float *scales, size_t rows, size_t cols,
                                           size_t num_streams, pg_huffman_tensor **out);
/* The struct literal of serial::read_huffman_tensor  src/serial.rs:367-445: a tensor from
 * its stored parts (everything is copied). */
pg_status pg_huffman_tensor_from_parts(const uint8_t *bit_lengths, const uint8_t *const *streams,
                                       const size_t *stream_bytes, const size_t *stream_lengths, size_t num_streams,
                                       const float *scales, size_t rows, size_t cols, pg_huffman_tensor **out);
void pg_huffman_tensor_free(pg_huffman_tensor *t);
/* rows, cols, num_streams fields and compressed_size()  src/huffman.rs:407-412. */
pg_status pg_huffman_tensor_info(const pg_huffman_tensor *t, size_t *rows, size_t *cols, size_t *num_streams,
                                 size_t *compressed_size);
/* streams[index], its byte length and stream_lengths[index]. */
pg_status pg_huffman_tensor_stream(const pg_huffman_tensor *t, size_t index, const uint8_t **data, size_t *bytes,
                                   size_t *symbols);
/* table.bit_lengths [256] and scales [cols]. */
pg_status pg_huffman_tensor_table(const pg_huffman_tensor *t, const uint8_t **bit_lengths, const float **scales);
/* HuffmanTensor::decode_to_quantized  src/huffman.rs:374-404: q, q_t [rows*cols], scales [cols]. */
pg_status pg_huffman_tensor_decode_to_quantized(pg_ctx *ctx, const pg_huffman_tensor *t, int8_t *q, int8_t *q_t,
                                                float *scales);
/* HuffmanTensor::to_gpu  src/huffman.rs:430-435, decoding on the device. */
pg_status pg_huffman_tensor_to_gpu(pg_ctx *ctx, const pg_huffman_tensor *t, pg_qtensor **out);
/* matmul_huffman  src/huffman.rs:465-474: decode, then pg_matmul_quantized. */
pg_status pg_matmul_huffman(pg_ctx *ctx, const float *a, size_t m, size_t k, const pg_huffman_tensor *t, float *out);

/* ---- Huffman-coded KV cache (src/huffman.rs:476-724) -------------------------------------
 * HuffmanKVCache keeps a window of recent tokens as f32 (a StandardKVCache, on the device)
 * and older tokens as chunks of int8 values, one scale per head, Huffman-coded.  Chunks are
 * built, kept and decoded in device memory; only the 256-entry code table is host work. */
typedef struct pg_kv_cache pg_kv_cache;                   /* attention::StandardKVCache  src/attention.rs:8-15 */
typedef struct pg_huffman_kv_chunk pg_huffman_kv_chunk;   /* CompressedChunk  src/huffman.rs:500-513 */
typedef struct pg_huffman_kv_cache pg_huffman_kv_cache;   /* HuffmanKVCache   src/huffman.rs:484-497 */
/* HuffmanKVCache::compress_chunk  src/huffman.rs:612-658: data [num_heads, num_tokens, head_dim]
 * (host).  Its assert on data.len() is the caller's to keep: the sizes say how much is read. */
pg_status pg_huffman_kv_compress_chunk(pg_ctx *ctx, const float *data, size_t num_tokens, size_t num_heads,
                                       size_t head_dim, pg_huffman_kv_chunk **out);
/* The same on device data; head h starts at data_dev + h * head_stride (floats), as the heads of a
 * StandardKVCache do (src/huffman.rs:579-596 extract_chunk_data without the copy). */
pg_status pg_huffman_kv_compress_chunk_dev(pg_ctx *ctx, const float *data_dev, size_t head_stride, size_t num_tokens,
                                           size_t num_heads, size_t head_dim, pg_huffman_kv_chunk **out);
/* The struct literal CompressedChunk { bitstream, scales, codebook, .. }  src/huffman.rs:649-657
 * from stored parts (copied): scales [num_heads], codebook [256]. */
pg_status pg_huffman_kv_chunk_from_parts(pg_ctx *ctx, const uint8_t *bitstream, size_t bytes, const float *scales,
                                         const uint8_t *codebook, size_t num_tokens, size_t num_heads, size_t head_dim,
                                         pg_huffman_kv_chunk **out);
void pg_huffman_kv_chunk_free(pg_ctx *ctx, pg_huffman_kv_chunk *c);
/* num_tokens, num_heads, head_dim and bitstream.len(); any out pointer may be NULL. */
pg_status pg_huffman_kv_chunk_info(const pg_huffman_kv_chunk *c, size_t *num_tokens, size_t *num_heads, size_t *head_dim,
                                   size_t *bitstream_bytes);
/* Copies of bitstream [bitstream_bytes], scales [num_heads], codebook [256]; any may be NULL. */
pg_status pg_huffman_kv_chunk_parts(pg_ctx *ctx, const pg_huffman_kv_chunk *c, uint8_t *bitstream, float *scales,
                                    uint8_t *codebook);
/* HuffmanKVCache::decompress_chunk  src/huffman.rs:661-680: out [num_heads, num_tokens, head_dim] (host).
 * A codebook that does not decode the stream is PG_EINVAL, as in pg_huffman_decode. */
pg_status pg_huffman_kv_decompress_chunk(pg_ctx *ctx, const pg_huffman_kv_chunk *c, float *out);
/* The same into device memory, head h at out_dev + h * head_stride. */
pg_status pg_huffman_kv_decompress_chunk_dev(pg_ctx *ctx, const pg_huffman_kv_chunk *c, float *out_dev, size_t head_stride);
/* HuffmanKVCache::new  src/huffman.rs:524-540 (compress_threshold = max(compress_threshold, chunk_size)).
 * chunk_size 0, with which the reference's append never returns once the threshold is met, is PG_EINVAL. */
pg_status pg_huffman_kv_cache_create(pg_ctx *ctx, size_t num_kv_heads, size_t head_dim, size_t compress_threshold,
                                     size_t chunk_size, pg_huffman_kv_cache **out);
void pg_huffman_kv_cache_free(pg_ctx *ctx, pg_huffman_kv_cache *c);
/* HuffmanKVCache::append  src/huffman.rs:544-556 (new_k, new_v [num_kv_heads, seq_len, head_dim], host):
 * appends to the hot window, then compresses the oldest chunk_size tokens while the window holds
 * at least compress_threshold (compress_oldest_chunk + remove_oldest_tokens, :559-610). */
pg_status pg_huffman_kv_cache_append(pg_ctx *ctx, pg_huffman_kv_cache *c, const float *new_k, const float *new_v,
                                     size_t seq_len);
pg_status pg_huffman_kv_cache_append_dev(pg_ctx *ctx, pg_huffman_kv_cache *c, const float *new_k_dev, const float *new_v_dev,
                                         size_t seq_len);
/* len()  src/huffman.rs:683-685, the compressed_len and compress_threshold fields, k_chunks.len(). */
size_t pg_huffman_kv_cache_len(const pg_huffman_kv_cache *c);
size_t pg_huffman_kv_cache_compressed_len(const pg_huffman_kv_cache *c);
size_t pg_huffman_kv_cache_compress_threshold(const pg_huffman_kv_cache *c);
size_t pg_huffman_kv_cache_num_chunks(const pg_huffman_kv_cache *c);
/* The `hot` field (owned by the cache; do not free or append to it directly). */
pg_status pg_huffman_kv_cache_hot(pg_huffman_kv_cache *c, pg_kv_cache **out);
/* k_chunks[index] (value_side 0) or v_chunks[index] (1), owned by the cache. */
pg_status pg_huffman_kv_cache_chunk(const pg_huffman_kv_cache *c, int value_side, size_t index,
                                    const pg_huffman_kv_chunk **out);
/* HuffmanKVCache::get_kv  src/huffman.rs:689-724: k, v [num_kv_heads, len(), head_dim] (host), per
 * head the decoded chunks in order, then the hot window.  The hot window of head h is read at
 * h * head_stride(); the reference reads it at h * hot.len * head_dim (:707), which is the same
 * place only for head 0 or a window that fills its capacity. */
pg_status pg_huffman_kv_cache_get_kv(pg_ctx *ctx, const pg_huffman_kv_cache *c, float *k, float *v);
pg_status pg_huffman_kv_cache_get_kv_dev(pg_ctx *ctx, const pg_huffman_kv_cache *c, float *k_dev, float *v_dev);

/* ---- grouped MoE expert FFN ------------------------------------------------- */

/* MoELayer::forward after the router matmul  examples/grok1/moe.rs:70-109
 * (expert body examples/grok1/moe.rs:27-34 or examples/deepseek/moe.rs:55-59):
 *   probs = softmax(router_logits) per token; top_k experts by stable descending
 *   sort; out[t] = sum_k prob_k * ( act(x_t.Wg_e) * (x_t.Wu_e) ) . Wd_e, k order.
 * x [T, d]; router_logits [T, E]; gate[e], up[e]: [ffn, d] block tensors;
 * down[e]: [d, ffn]; out [T, d]. */
pg_status pg_moe_ffn(pg_ctx *ctx, const float *x, size_t T, const float *router_logits,
                     size_t E, size_t top_k, const pg_gguf_tensor *const *gate,
                     const pg_gguf_tensor *const *up, const pg_gguf_tensor *const *down,
                     int act, float *out);
pg_status pg_moe_ffn_dev(pg_ctx *ctx, const float *x_dev, size_t T,
                         const float *router_logits_dev, size_t E, size_t top_k,
                         const pg_gguf_tensor *const *gate, const pg_gguf_tensor *const *up,
                         const pg_gguf_tensor *const *down, int act, float *out_dev);

/* The same expert FFN over a routing the caller's gate made: expert_idx / weight [T, top_k] (a token's experts
 * distinct, each in 0 .. E - 1), out[t] = sum_k weight[t, k] * expert_{idx[t, k]}(x[t]) in k order, multiply then
 * add, then + shared[t] when `shared` ([T, d], the shared experts' output) is not NULL --
 * MoE::forward  examples/deepseek/moe.rs:271-300 after Gate::forward (:111-215: sigmoid or softmax scores, bias and
 * group limits for the selection only, route_scale), and the gpt_oss layer (examples/gpt_oss/moe.rs:286-351: top-k
 * on the logits, softmax over the k).  The host-pointer form rejects an index out of range or named twice
 * (PG_EINVAL; the reference would panic on the first); the device form cannot look, and replaces such an entry by
 * an unused expert with weight 0, so that it stays memory-safe. */
pg_status pg_moe_ffn_routed(pg_ctx *ctx, const float *x, size_t T, const int32_t *expert_idx, const float *weight,
                            size_t E, size_t top_k, const pg_gguf_tensor *const *gate,
                            const pg_gguf_tensor *const *up, const pg_gguf_tensor *const *down, int act,
                            const float *shared, float *out);
pg_status pg_moe_ffn_routed_dev(pg_ctx *ctx, const float *x_dev, size_t T, const int32_t *expert_idx_dev,
                                const float *weight_dev, size_t E, size_t top_k,
                                const pg_gguf_tensor *const *gate, const pg_gguf_tensor *const *up,
                                const pg_gguf_tensor *const *down, int act, const float *shared_dev,
                                float *out_dev);

/* ---- Llama decoder block: the glue around the quantised products -------------- */

typedef struct pg_rope pg_rope;               /* nn::RoPE                  src/nn.rs:1250-1256 */
typedef struct pg_llama_block pg_llama_block; /* LlamaBlock                src/models/llama/decoder.rs:7-16 */

/* attention::AttentionMask  src/attention.rs:102-120 (LocalGlobal is not offered). */
#define PG_MASK_NONE 0
#define PG_MASK_CAUSAL 1                 /* Causal { offset } */
#define PG_MASK_CAUSAL_SLIDING_WINDOW 2  /* CausalSlidingWindow { offset, window, sink_tokens } */
#define PG_MASK_LOCAL_GLOBAL 3           /* LocalGlobal: through pg_gqa_attention_local_global only */

/* nn::RMSNorm::forward, inference path  src/nn.rs:577-652:
 *   out[r, i] = x[r, i] / sqrt(mean_i(x[r]^2) + eps) * w[i];  x, out [rows, dim]; w [dim]. */
pg_status pg_rmsnorm(pg_ctx *ctx, const float *x, size_t rows, size_t dim, const float *w, float eps,
                     float *out);
pg_status pg_rmsnorm_dev(pg_ctx *ctx, const float *x_dev, size_t rows, size_t dim, const float *w_dev,
                         float eps, float *out_dev);

/* nn::RoPE::new  src/nn.rs:1258-1282: cos/sin tables [max_seq_len, head_dim] (f32 libm
 * values computed on the host, then resident on the device).  head_dim must be even. */
pg_status pg_rope_create(pg_ctx *ctx, size_t head_dim, size_t max_seq_len, float base, pg_rope **out);
void pg_rope_free(pg_ctx *ctx, pg_rope *rope);
/* nn::RoPE::apply  src/nn.rs:1286-1338: x, out [seq_len, head_dim], positions
 * offset..offset+seq_len, pairs (i, i + head_dim/2).  A position past max_seq_len (the
 * reference's slice panic) is PG_EINVAL. */
pg_status pg_rope_apply(pg_ctx *ctx, const pg_rope *rope, const float *x, size_t seq_len, size_t offset,
                        float *out);
pg_status pg_rope_apply_dev(pg_ctx *ctx, const pg_rope *rope, const float *x_dev, size_t seq_len,
                            size_t offset, float *out_dev);

/* StandardKVCache::new  src/attention.rs:18-27: empty, capacity 0; head_dim <= 256. */
pg_status pg_kv_cache_create(pg_ctx *ctx, size_t num_kv_heads, size_t head_dim, pg_kv_cache **out);
void pg_kv_cache_free(pg_ctx *ctx, pg_kv_cache *cache);
/* StandardKVCache::append  src/attention.rs:65-83 (growth as ensure_capacity, :31-62:
 * at least double, from 16): new_k, new_v [num_kv_heads, seq_len, head_dim]. */
pg_status pg_kv_cache_append(pg_ctx *ctx, pg_kv_cache *cache, const float *new_k, const float *new_v,
                             size_t seq_len);
pg_status pg_kv_cache_append_dev(pg_ctx *ctx, pg_kv_cache *cache, const float *new_k_dev,
                                 const float *new_v_dev, size_t seq_len);
/* StandardKVCache::rollback_to  src/attention.rs:87-91; new_len > len (its assert!) is PG_EINVAL. */
pg_status pg_kv_cache_rollback_to(pg_kv_cache *cache, size_t new_len);
size_t pg_kv_cache_len(const pg_kv_cache *cache);      /* the `len` field */
size_t pg_kv_cache_capacity(const pg_kv_cache *cache); /* head_stride() / head_dim  src/attention.rs:96-98 */
/* The `k` and `v` fields without the capacity padding: [num_kv_heads, len, head_dim] each. */
pg_status pg_kv_cache_download(pg_ctx *ctx, const pg_kv_cache *cache, float *k, float *v);

/* attention::gqa_attention_cpu  src/attention.rs:141-265 (masks :269-300):
 *   q [num_q_heads, seq_q, head_dim]; keys from k_cache, values from v_cache (same shape
 *   and length); out [seq_q, num_q_heads * head_dim] is ADDED TO, as the reference adds
 *   into `output` (callers pass zeros).  logit_cap > 0 applies cap * tanh(score / cap)
 *   (PostScoreTransform::LogitCap), 0 = PostScoreTransform::None.  offset / window /
 *   sink_tokens are read as the mask kind needs them. */
pg_status pg_gqa_attention(pg_ctx *ctx, const float *q, const pg_kv_cache *k_cache,
                           const pg_kv_cache *v_cache, size_t num_q_heads, size_t seq_q, float scale,
                           int mask_kind, size_t offset, size_t window, size_t sink_tokens,
                           float logit_cap, float *out);
pg_status pg_gqa_attention_dev(pg_ctx *ctx, const float *q_dev, const pg_kv_cache *k_cache,
                               const pg_kv_cache *v_cache, size_t num_q_heads, size_t seq_q, float scale,
                               int mask_kind, size_t offset, size_t window, size_t sink_tokens,
                               float logit_cap, float *out_dev);
/* The same with AttentionMask::LocalGlobal { offset, local_window, global_positions }
 * src/attention.rs:115-119, 287-299: a key is visible when it is not after the query and is
 * either within local_window positions of it or one of the global positions (a host array
 * in both variants; entries past the cache length never match).  The _dev variant waits
 * for the stream once, while the positions are uploaded. */
pg_status pg_gqa_attention_local_global(pg_ctx *ctx, const float *q, const pg_kv_cache *k_cache,
                                        const pg_kv_cache *v_cache, size_t num_q_heads, size_t seq_q,
                                        float scale, size_t offset, size_t local_window,
                                        const size_t *global_positions, size_t num_global,
                                        float logit_cap, float *out);
pg_status pg_gqa_attention_local_global_dev(pg_ctx *ctx, const float *q_dev, const pg_kv_cache *k_cache,
                                            const pg_kv_cache *v_cache, size_t num_q_heads, size_t seq_q,
                                            float scale, size_t offset, size_t local_window,
                                            const size_t *global_positions, size_t num_global,
                                            float logit_cap, float *out_dev);

/* LlamaBlock::new  src/models/llama/decoder.rs:19-47 (with LlamaAttention::new,
 * src/models/llama/attention.rs:25-48). */
pg_status pg_llama_block_create(pg_ctx *ctx, size_t model_dim, size_t num_q_heads, size_t num_kv_heads,
                                size_t head_dim, size_t ffn_dim, size_t max_seq_len, float rope_base,
                                float rms_eps, pg_llama_block **out);
void pg_llama_block_free(pg_ctx *ctx, pg_llama_block *block);
/* The block's seven projections as GGUF block tensors [out, in] (borrowed: they must
 * outlive the block) and its two norm weights [model_dim] (copied).  The reference holds
 * the projections dequantised and transposed (src/models/llama/model.rs:243-257). */
pg_status pg_llama_block_set_weights(pg_ctx *ctx, pg_llama_block *block, const pg_gguf_tensor *q_proj,
                                     const pg_gguf_tensor *k_proj, const pg_gguf_tensor *v_proj,
                                     const pg_gguf_tensor *o_proj, const pg_gguf_tensor *gate_proj,
                                     const pg_gguf_tensor *up_proj, const pg_gguf_tensor *down_proj,
                                     const float *attn_norm_w, const float *ffn_norm_w);
/* LlamaBlock::forward  src/models/llama/decoder.rs:69-155 with LlamaAttention::forward
 * (src/models/llama/attention.rs:73-212), unfused projections: h, out [seq, model_dim];
 * the cache gains seq positions (causal mask at offset = its length on entry). */
pg_status pg_llama_block_forward(pg_ctx *ctx, pg_llama_block *block, const float *h, size_t seq,
                                 pg_kv_cache *cache, float *out);
pg_status pg_llama_block_forward_dev(pg_ctx *ctx, pg_llama_block *block, const float *h_dev, size_t seq,
                                     pg_kv_cache *cache, float *out_dev);

/* ---- diagnostics and measurement: nothing below has a counterpart in the reference ----
 * Timing per kernel, probes of what the part delivers, and the hooks the tests use to name or
 * force the matrix-core product's tile.  None of them is needed to run the path. */

/* Per-kernel timing.  No counterpart in the reference (it times whole calls with
 * Instant::now(), benches/wallclock.rs:28-41): between pg_profile_begin and
 * pg_profile_end every hot-path kernel the library launches on this context carries a
 * start and a stop HIP event stamped with the dispatch's own begin and end times
 * (hipExtLaunchKernel) on the context's stream; pg_profile_end waits for the stream and
 * aggregates elapsed time per kernel name, read back with pg_profile_get. */
pg_status pg_profile_begin(pg_ctx *ctx);
pg_status pg_profile_end(pg_ctx *ctx, size_t *num_kernels);
pg_status pg_profile_get(pg_ctx *ctx, size_t i, const char **name, double *total_ms,
                         size_t *launches);
/* The distinct launch sizes (work-items = grid x workgroup, as a kernel trace lists them) behind
 * entry i and how many launches had each: up to `cap` pairs are written, *count gets their number.
 * Lets a benchmark check that a stored counter summary still describes the launches it makes. */
pg_status pg_profile_get_grids(pg_ctx *ctx, size_t i, size_t *work_items, size_t *launches, size_t cap,
                               size_t *count);

/* Ceilings of the part, measured (no counterpart in the reference; a benchmark reports them
 * beside the published peaks):
 *   pg_probe_mfma_i8    int8 matrix-core rate with every operand in registers, in TOP/s (2 ops
 *                       per multiply-add), one workgroup of 8 wavefronts per CU for `iters` x 8
 *                       MFMAs per wavefront, and the shader clock the loop ran at;
 *   pg_probe_hbm_read   a pure 128-bit read stream: `passes` kernels, each reading
 *                       bytes_per_pass from one of `buffers` distinct buffers in turn (make
 *                       buffers x bytes_per_pass exceed the 256 MB last-level cache), in GB/s;
 *   pg_probe_gemm_clock the shader clock inside the K loop of the W8A8 GEMM's 256x256 tile on an
 *                       [m x k] . [k x n] product, and the mean duration of a workgroup's loop.
 * Each allocates its own buffers and waits for completion. */
pg_status pg_probe_mfma_i8(pg_ctx *ctx, int iters, double *tops, double *clock_ghz);
pg_status pg_probe_hbm_read(pg_ctx *ctx, size_t bytes_per_pass, int buffers, int passes, double *gbs);
/* The same read stream with the launch shape named: `workgroups` of `threads` (256, 512 or 1024) threads, each lane
 * with `loads_in_flight` (4, 8 or 16) 128-bit loads outstanding; pg_probe_hbm_read is 8 x CUs workgroups of 256
 * with 8.  A benchmark sweeps the shape at the size of its own launches and quotes the best as the ceiling. */
pg_status pg_probe_hbm_read_shaped(pg_ctx *ctx, size_t bytes_per_pass, int buffers, int passes, int workgroups,
                                   int threads, int loads_in_flight, double *gbs);
pg_status pg_probe_gemm_clock(pg_ctx *ctx, size_t m, size_t k, size_t n, double *clock_ghz, double *loop_us);

/* Diagnostics of the matrix-core product.  No counterpart in the reference (its Metal
 * dispatcher picks between two shaders by size, src/metal/context.rs:2243, without a query):
 * the output tile (rows x columns) and the number of K splits of the most recent W8A8 GEMM
 * launch on this context, and an override of the dispatcher's tile choice (0 = automatic,
 * 1 = 64x64, 2 = 256x256, 3 = 128x256, 4 = 128x64, 5 = 128x128).  Every tile gives the same
 * bits; tests use the pair to prove each kernel instantiation ran. */
pg_status pg_gemm_w8a8_last_tile(const pg_ctx *ctx, int *bm, int *bn, int *k_splits);
pg_status pg_gemm_w8a8_force_tile(pg_ctx *ctx, int tile);
/* The one-row product that takes the activation row in f32: the workgroup shape (wavefronts per workgroup 4, 8 or
 * 16; weight rows per wavefront 1 or 2, not 16 x 2) instead of the dispatcher's choice by row length; 0, 0 =
 * automatic.  Every shape gives the same bits. */
pg_status pg_gemv_w8a8_force_shape(pg_ctx *ctx, int wavefronts, int rows_per_wavefront);
/* The many-row Q4_0 / Q8_0 product has two matrix-core routes: the int8 block product with 16-bit fixed-point activations
 * per block, and, from about a hundred rows on where the launch fills the part, f16 tiles with the weights unpacked
 * in registers and the activations as two f16 planes per row.  mode 0 = the dispatcher chooses, 1 = the f16 route
 * wherever it can run (Q4_0 or Q8_0, K a multiple of 64, at least two rows), 2 = never.  Both keep the weights exact; they
 * round the activations differently (2^-22 of the row's largest value against 2^-16 of the block's). */
pg_status pg_gguf_hmm_force(pg_ctx *ctx, int mode);

/* Address audit of the streaming kernels, on the host (no device is touched): each function walks every
 * (workgroup, wavefront, lane, step) of one launch of the named kernel shape with the very index functions the
 * kernel uses and returns, per array it streams, the end of the furthest byte a load would touch and the bytes
 * the library allocates for that array.  end <= bytes must hold for every shape the dispatchers can pick; a
 * test without a GPU sweeps them. */
pg_status pg_audit_gemv_w8a8_m1(size_t k, size_t n, int nch, int rows_per_wavefront, int wavefronts, int f32_row,
                                size_t *w_end, size_t *w_bytes, size_t *x_end, size_t *x_bytes);
pg_status pg_audit_gemm_w8a8_skinny(size_t m, size_t k, size_t n, int activation_tiles, int weight_tiles, int wavefronts,
                                    size_t *w_end, size_t *w_bytes, size_t *a_end, size_t *a_bytes);
pg_status pg_audit_gguf_gemv(size_t n_out, size_t k_in, int q8, int blocks_per_lane, int rows_per_wavefront,
                             int wavefronts, size_t *qs_end, size_t *qs_bytes, size_t *d_end, size_t *d_bytes);
pg_status pg_audit_gguf_skinny(size_t n_out, size_t k_in, int q8, int wavefronts, int weight_tiles, size_t *qs_end,
                               size_t *qs_bytes, size_t *d_end, size_t *d_bytes);
pg_status pg_audit_gguf_hmm(size_t m, size_t n_out, size_t k_in, int q8, int wide_tiles, int k_chunks, size_t *plane_end,
                            size_t *plane_bytes, size_t *qs_end, size_t *qs_bytes, size_t *d_end, size_t *d_bytes);
pg_status pg_audit_mxfp4_rows(size_t out_dim, size_t in_dim, int row_groups_per_workgroup, int wavefronts,
                              size_t *qs_end, size_t *qs_bytes, size_t *sc_end, size_t *sc_bytes);
/* The MXFP4 tile kernel and its pre-pass under the plan the launcher makes for m rows on a part of num_cu CUs;
 * rec_* = the token records between the two; ra, tb, ks report the plan (row groups per wavefront, token groups per
 * workgroup, runs of K). */
pg_status pg_audit_mxfp4_tiles(int num_cu, size_t out_dim, size_t in_dim, size_t m, size_t *qs_end, size_t *qs_bytes,
                               size_t *sc_end, size_t *sc_bytes, size_t *rec_end, size_t *rec_bytes, int *ra, int *tb,
                               int *ks);
pg_status pg_audit_probe_read(size_t bytes, int workgroups, int threads, int loads_in_flight, size_t *end,
                              size_t *alloc);

#ifdef __cplusplus
}
#endif
#endif /* PEREGRINE_HIP_H */
