//! `peregrine-hip-sys`: the binding of `libperegrine_hip.so` (include/peregrine_hip.h) for
//! peregrine, in two layers:
//!
//! * the raw `extern "C"` declarations, one per function of the header (the block between the
//!   "generated" markers is written by `gen_bindings.py` and checked against the header by the
//!   repository's tests -- edit the header, not the block);
//! * `quant`, `gguf` and `moe`: the same public signatures as `peregrine::quant`
//!   (src/quant.rs:12-218), `peregrine::gguf::{dequant_q8_0, dequant_q4_0, dequant_q4_1}`
//!   (src/gguf.rs:286-351) and the grok1 MoE layer (examples/grok1/moe.rs:70-109), with bodies
//!   that call the library.  A non-zero status becomes a panic, which is the reference's own
//!   contract for shape errors (`assert!` / `assert_eq!` / `.expect`).
//!
//! No Rust toolchain exists in the image this was written in: the crate is kept honest by
//! mechanical generation and by a test that parses both files, not by `cargo build`.
#![allow(non_camel_case_types)]
#![allow(clippy::missing_safety_doc, clippy::too_many_arguments)]

use std::os::raw::{c_char, c_int, c_void};

/// `pg_status`: 0 = `PG_OK`.
pub type pg_status = c_int;
pub const PG_OK: pg_status = 0;
pub const PG_EINVAL: pg_status = 1;
pub const PG_EDEVICE: pg_status = 2;
pub const PG_ENOMEM: pg_status = 3;
pub const PG_EUNSUPPORTED: pg_status = 4;

/// GGML block types as `src/gguf.rs:14-33` numbers them, and ggml's number for MXFP4.
pub const PG_GGML_Q4_0: c_int = 2;
pub const PG_GGML_Q4_1: c_int = 3;
pub const PG_GGML_Q8_0: c_int = 8;
pub const PG_MXFP4: c_int = 39;
pub const PG_ACT_SILU: c_int = 0;
pub const PG_ACT_GELU_TANH: c_int = 1;
pub const PG_MASK_NONE: c_int = 0;
pub const PG_MASK_CAUSAL: c_int = 1;
pub const PG_MASK_CAUSAL_SLIDING_WINDOW: c_int = 2;
pub const PG_MASK_LOCAL_GLOBAL: c_int = 3;

macro_rules! opaque {
    ($($name:ident),*) => { $( #[repr(C)] pub struct $name { _private: [u8; 0] } )* };
}
opaque!(pg_ctx, pg_qtensor, pg_gguf_tensor, pg_mxfp4_expert, pg_gguf_file, pg_huffman_tensor, pg_huffman_kv_chunk,
        pg_huffman_kv_cache, pg_rope, pg_kv_cache, pg_llama_block);

// ---- generated from include/peregrine_hip.h: begin ----
extern "C" {
    pub fn pg_ctx_create(device: c_int, hip_stream: *mut c_void, out: *mut *mut pg_ctx) -> pg_status;
    pub fn pg_ctx_destroy(ctx: *mut pg_ctx);
    pub fn pg_sync(ctx: *mut pg_ctx) -> pg_status;
    pub fn pg_ctx_stream(ctx: *mut pg_ctx) -> *mut c_void;
    pub fn pg_last_error() -> *const c_char;
    pub fn pg_status_string(st: pg_status) -> *const c_char;
    pub fn pg_dev_alloc(ctx: *mut pg_ctx, bytes: usize, dptr: *mut *mut c_void) -> pg_status;
    pub fn pg_dev_free(ctx: *mut pg_ctx, dptr: *mut c_void) -> pg_status;
    pub fn pg_memcpy_h2d(ctx: *mut pg_ctx, dst_dev: *mut c_void, src_host: *const c_void, bytes: usize) -> pg_status;
    pub fn pg_memcpy_d2h(ctx: *mut pg_ctx, dst_host: *mut c_void, src_dev: *const c_void, bytes: usize) -> pg_status;
    pub fn pg_quantize_weights(ctx: *mut pg_ctx, w: *const f32, rows: usize, cols: usize, q: *mut i8, q_t: *mut i8, scales: *mut f32) -> pg_status;
    pub fn pg_quantize_activations(ctx: *mut pg_ctx, a: *const f32, rows: usize, cols: usize, q: *mut i8, row_scales: *mut f32) -> pg_status;
    pub fn pg_quantize_activations_dev(ctx: *mut pg_ctx, a_dev: *const f32, rows: usize, cols: usize, q_dev: *mut i8, row_scales_dev: *mut f32) -> pg_status;
    pub fn pg_dequantize(ctx: *mut pg_ctx, q: *const i8, scales: *const f32, rows: usize, cols: usize, out: *mut f32) -> pg_status;
    pub fn pg_qtensor_upload(ctx: *mut pg_ctx, q: *const i8, scales: *const f32, rows: usize, cols: usize, out: *mut *mut pg_qtensor) -> pg_status;
    pub fn pg_qtensor_from_f32(ctx: *mut pg_ctx, w: *const f32, rows: usize, cols: usize, out: *mut *mut pg_qtensor) -> pg_status;
    pub fn pg_qtensor_from_f32_dev(ctx: *mut pg_ctx, w_dev: *const f32, rows: usize, cols: usize, out: *mut *mut pg_qtensor) -> pg_status;
    pub fn pg_qtensor_download(ctx: *mut pg_ctx, t: *const pg_qtensor, q: *mut i8, q_t: *mut i8, scales: *mut f32) -> pg_status;
    pub fn pg_qtensor_shape(t: *const pg_qtensor, rows: *mut usize, cols: *mut usize) -> pg_status;
    pub fn pg_qtensor_free(ctx: *mut pg_ctx, t: *mut pg_qtensor);
    pub fn pg_matmul_quantized(ctx: *mut pg_ctx, a: *const f32, m: usize, k: usize, w: *const pg_qtensor, out: *mut f32) -> pg_status;
    pub fn pg_matmul_quantized_dev(ctx: *mut pg_ctx, a_dev: *const f32, m: usize, k: usize, w: *const pg_qtensor, out_dev: *mut f32, acc_dev: *mut i32) -> pg_status;
    pub fn pg_matmul_quantized_fixed_scratch_dev(ctx: *mut pg_ctx, a_dev: *const f32, m: usize, k: usize, w: *const pg_qtensor, out_dev: *mut f32) -> pg_status;
    pub fn pg_fixed_scratch_bytes() -> usize;
    pub fn pg_matmul_quantized_multi_dev(ctx: *mut pg_ctx, a_dev: *const f32, m: usize, k: usize, w: *const *const pg_qtensor, count: usize, out_dev: *const *mut f32) -> pg_status;
    pub fn pg_matmul_dequant_i8(ctx: *mut pg_ctx, a: *const f32, m: usize, k: usize, w: *const pg_qtensor, out: *mut f32) -> pg_status;
    pub fn pg_matmul_dequant_i8_dev(ctx: *mut pg_ctx, a_dev: *const f32, m: usize, k: usize, w: *const pg_qtensor, out_dev: *mut f32) -> pg_status;
    pub fn pg_f16_to_f32(ctx: *mut pg_ctx, bits: *const u16, n: usize, out: *mut f32) -> pg_status;
    pub fn pg_dequant_q8_0(ctx: *mut pg_ctx, data: *const u8, num_elements: usize, out: *mut f32) -> pg_status;
    pub fn pg_dequant_q4_0(ctx: *mut pg_ctx, data: *const u8, num_elements: usize, out: *mut f32) -> pg_status;
    pub fn pg_dequant_q4_1(ctx: *mut pg_ctx, data: *const u8, num_elements: usize, out: *mut f32) -> pg_status;
    pub fn pg_gguf_upload(ctx: *mut pg_ctx, blocks: *const c_void, ggml_type: c_int, n_out: usize, k_in: usize, out: *mut *mut pg_gguf_tensor) -> pg_status;
    pub fn pg_gguf_shape(t: *const pg_gguf_tensor, n_out: *mut usize, k_in: *mut usize, ggml_type: *mut c_int) -> pg_status;
    pub fn pg_gguf_free(ctx: *mut pg_ctx, t: *mut pg_gguf_tensor);
    pub fn pg_gguf_matmul(ctx: *mut pg_ctx, x: *const f32, m: usize, w: *const pg_gguf_tensor, y: *mut f32) -> pg_status;
    pub fn pg_gguf_matmul_dev(ctx: *mut pg_ctx, x_dev: *const f32, m: usize, w: *const pg_gguf_tensor, y_dev: *mut f32) -> pg_status;
    pub fn pg_gguf_prepare(ctx: *mut pg_ctx, w: *const pg_gguf_tensor, max_rows: usize) -> pg_status;
    pub fn pg_gguf_drop_prepared(ctx: *mut pg_ctx, w: *const pg_gguf_tensor) -> pg_status;
    pub fn pg_gguf_device_bytes(w: *const pg_gguf_tensor, uploaded: *mut usize, derived: *mut usize) -> pg_status;
    pub fn pg_mxfp4_matmul(ctx: *mut pg_ctx, input: *const f32, blocks: *const u8, scales: *const u8, out_dim: usize, in_dim: usize, output: *mut f32) -> pg_status;
    pub fn pg_mxfp4_upload(ctx: *mut pg_ctx, blocks: *const u8, scales: *const u8, out_dim: usize, in_dim: usize, out: *mut *mut pg_gguf_tensor) -> pg_status;
    pub fn pg_mxfp4_expert_create(ctx: *mut pg_ctx, hidden: usize, intermediate: usize, alpha: f32, clamp: f32, mlp1_blocks: *const u8, mlp1_scales: *const u8, mlp2_blocks: *const u8, mlp2_scales: *const u8, mlp1_bias: *const f32, mlp2_bias: *const f32, out: *mut *mut pg_mxfp4_expert) -> pg_status;
    pub fn pg_mxfp4_expert_free(ctx: *mut pg_ctx, expert: *mut pg_mxfp4_expert);
    pub fn pg_mxfp4_expert_forward(ctx: *mut pg_ctx, expert: *const pg_mxfp4_expert, x: *const f32, m: usize, out: *mut f32) -> pg_status;
    pub fn pg_mxfp4_expert_forward_dev(ctx: *mut pg_ctx, expert: *const pg_mxfp4_expert, x_dev: *const f32, m: usize, scratch_dev: *mut f32, out_dev: *mut f32) -> pg_status;
    pub fn pg_mxfp4_moe_ffn_routed(ctx: *mut pg_ctx, x: *const f32, T: usize, expert_idx: *const i32, weight: *const f32, top_k: usize, experts: *const *const pg_mxfp4_expert, E: usize, out: *mut f32) -> pg_status;
    pub fn pg_mxfp4_moe_ffn_routed_dev(ctx: *mut pg_ctx, x_dev: *const f32, T: usize, expert_idx_dev: *const i32, weight_dev: *const f32, top_k: usize, experts: *const *const pg_mxfp4_expert, E: usize, out_dev: *mut f32) -> pg_status;
    pub fn pg_gguf_file_parse(data: *const c_void, len: usize, out: *mut *mut pg_gguf_file) -> pg_status;
    pub fn pg_gguf_file_open(path: *const c_char, out: *mut *mut pg_gguf_file) -> pg_status;
    pub fn pg_gguf_file_close(f: *mut pg_gguf_file);
    pub fn pg_gguf_file_counts(f: *const pg_gguf_file, n_tensors: *mut usize, n_metadata: *mut usize, version: *mut u32, data_start: *mut u64) -> pg_status;
    pub fn pg_gguf_file_tensor_name(f: *const pg_gguf_file, index: usize, name: *mut *const c_char) -> pg_status;
    pub fn pg_gguf_file_tensor_info(f: *const pg_gguf_file, name: *const c_char, ggml_type: *mut c_int, n_dims: *mut usize, shape: *mut u64, shape_cap: usize, data_offset: *mut u64, data_size: *mut usize, data: *mut *const c_void) -> pg_status;
    pub fn pg_gguf_file_get_u32(f: *const pg_gguf_file, key: *const c_char, value: *mut u32, found: *mut c_int) -> pg_status;
    pub fn pg_gguf_file_get_f32(f: *const pg_gguf_file, key: *const c_char, value: *mut f32, found: *mut c_int) -> pg_status;
    pub fn pg_gguf_file_get_str(f: *const pg_gguf_file, key: *const c_char, value: *mut *const c_char, len: *mut usize) -> pg_status;
    pub fn pg_gguf_file_get_array(f: *const pg_gguf_file, key: *const c_char, elem_type: *mut u32, count: *mut usize) -> pg_status;
    pub fn pg_gguf_file_get_array_str(f: *const pg_gguf_file, key: *const c_char, index: usize, value: *mut *const c_char) -> pg_status;
    pub fn pg_gguf_file_get_array_f64(f: *const pg_gguf_file, key: *const c_char, values: *mut f64, cap: usize) -> pg_status;
    pub fn pg_gguf_file_load_tensor_f32(ctx: *mut pg_ctx, f: *const pg_gguf_file, name: *const c_char, out: *mut f32, out_cap: usize) -> pg_status;
    pub fn pg_gguf_file_upload_tensor(ctx: *mut pg_ctx, f: *const pg_gguf_file, name: *const c_char, out: *mut *mut pg_gguf_tensor) -> pg_status;
    pub fn pg_quantized_record_size(name_len: usize, rows: usize, cols: usize, bytes: *mut usize) -> pg_status;
    pub fn pg_write_quantized_tensor(buf: *mut c_void, cap: usize, name: *const c_char, name_len: usize, q: *const i8, scales: *const f32, rows: usize, cols: usize, written: *mut usize) -> pg_status;
    pub fn pg_read_quantized_tensor(buf: *const c_void, len: usize, name: *mut *const c_char, name_len: *mut usize, rows: *mut usize, cols: *mut usize, q: *mut *const i8, scales: *mut *const c_void, consumed: *mut usize) -> pg_status;
    pub fn pg_qtensor_from_record(ctx: *mut pg_ctx, buf: *const c_void, len: usize, out: *mut *mut pg_qtensor, consumed: *mut usize) -> pg_status;
    pub fn pg_huffman_table_from_frequencies(freqs: *const u64, bit_lengths: *mut u8, codes: *mut u32) -> pg_status;
    pub fn pg_huffman_canonical_codes(bit_lengths: *const u8, codes: *mut u32) -> pg_status;
    pub fn pg_huffman_encode(bit_lengths: *const u8, data: *const i8, n: usize, out: *mut u8, cap: usize, bytes: *mut usize) -> pg_status;
    pub fn pg_huffman_decode(ctx: *mut pg_ctx, bit_lengths: *const u8, bitstream: *const u8, len: usize, num_symbols: usize, out: *mut i8) -> pg_status;
    pub fn pg_huffman_tensor_from_quantized(q: *const i8, scales: *const f32, rows: usize, cols: usize, num_streams: usize, out: *mut *mut pg_huffman_tensor) -> pg_status;
    pub fn pg_huffman_tensor_from_parts(bit_lengths: *const u8, streams: *const *const u8, stream_bytes: *const usize, stream_lengths: *const usize, num_streams: usize, scales: *const f32, rows: usize, cols: usize, out: *mut *mut pg_huffman_tensor) -> pg_status;
    pub fn pg_huffman_tensor_free(t: *mut pg_huffman_tensor);
    pub fn pg_huffman_tensor_info(t: *const pg_huffman_tensor, rows: *mut usize, cols: *mut usize, num_streams: *mut usize, compressed_size: *mut usize) -> pg_status;
    pub fn pg_huffman_tensor_stream(t: *const pg_huffman_tensor, index: usize, data: *mut *const u8, bytes: *mut usize, symbols: *mut usize) -> pg_status;
    pub fn pg_huffman_tensor_table(t: *const pg_huffman_tensor, bit_lengths: *mut *const u8, scales: *mut *const f32) -> pg_status;
    pub fn pg_huffman_tensor_decode_to_quantized(ctx: *mut pg_ctx, t: *const pg_huffman_tensor, q: *mut i8, q_t: *mut i8, scales: *mut f32) -> pg_status;
    pub fn pg_huffman_tensor_to_gpu(ctx: *mut pg_ctx, t: *const pg_huffman_tensor, out: *mut *mut pg_qtensor) -> pg_status;
    pub fn pg_matmul_huffman(ctx: *mut pg_ctx, a: *const f32, m: usize, k: usize, t: *const pg_huffman_tensor, out: *mut f32) -> pg_status;
    pub fn pg_huffman_kv_compress_chunk(ctx: *mut pg_ctx, data: *const f32, num_tokens: usize, num_heads: usize, head_dim: usize, out: *mut *mut pg_huffman_kv_chunk) -> pg_status;
    pub fn pg_huffman_kv_compress_chunk_dev(ctx: *mut pg_ctx, data_dev: *const f32, head_stride: usize, num_tokens: usize, num_heads: usize, head_dim: usize, out: *mut *mut pg_huffman_kv_chunk) -> pg_status;
    pub fn pg_huffman_kv_chunk_from_parts(ctx: *mut pg_ctx, bitstream: *const u8, bytes: usize, scales: *const f32, codebook: *const u8, num_tokens: usize, num_heads: usize, head_dim: usize, out: *mut *mut pg_huffman_kv_chunk) -> pg_status;
    pub fn pg_huffman_kv_chunk_free(ctx: *mut pg_ctx, c: *mut pg_huffman_kv_chunk);
    pub fn pg_huffman_kv_chunk_info(c: *const pg_huffman_kv_chunk, num_tokens: *mut usize, num_heads: *mut usize, head_dim: *mut usize, bitstream_bytes: *mut usize) -> pg_status;
    pub fn pg_huffman_kv_chunk_parts(ctx: *mut pg_ctx, c: *const pg_huffman_kv_chunk, bitstream: *mut u8, scales: *mut f32, codebook: *mut u8) -> pg_status;
    pub fn pg_huffman_kv_decompress_chunk(ctx: *mut pg_ctx, c: *const pg_huffman_kv_chunk, out: *mut f32) -> pg_status;
    pub fn pg_huffman_kv_decompress_chunk_dev(ctx: *mut pg_ctx, c: *const pg_huffman_kv_chunk, out_dev: *mut f32, head_stride: usize) -> pg_status;
    pub fn pg_huffman_kv_cache_create(ctx: *mut pg_ctx, num_kv_heads: usize, head_dim: usize, compress_threshold: usize, chunk_size: usize, out: *mut *mut pg_huffman_kv_cache) -> pg_status;
    pub fn pg_huffman_kv_cache_free(ctx: *mut pg_ctx, c: *mut pg_huffman_kv_cache);
    pub fn pg_huffman_kv_cache_append(ctx: *mut pg_ctx, c: *mut pg_huffman_kv_cache, new_k: *const f32, new_v: *const f32, seq_len: usize) -> pg_status;
    pub fn pg_huffman_kv_cache_append_dev(ctx: *mut pg_ctx, c: *mut pg_huffman_kv_cache, new_k_dev: *const f32, new_v_dev: *const f32, seq_len: usize) -> pg_status;
    pub fn pg_huffman_kv_cache_len(c: *const pg_huffman_kv_cache) -> usize;
    pub fn pg_huffman_kv_cache_compressed_len(c: *const pg_huffman_kv_cache) -> usize;
    pub fn pg_huffman_kv_cache_compress_threshold(c: *const pg_huffman_kv_cache) -> usize;
    pub fn pg_huffman_kv_cache_num_chunks(c: *const pg_huffman_kv_cache) -> usize;
    pub fn pg_huffman_kv_cache_hot(c: *mut pg_huffman_kv_cache, out: *mut *mut pg_kv_cache) -> pg_status;
    pub fn pg_huffman_kv_cache_chunk(c: *const pg_huffman_kv_cache, value_side: c_int, index: usize, out: *mut *const pg_huffman_kv_chunk) -> pg_status;
    pub fn pg_huffman_kv_cache_get_kv(ctx: *mut pg_ctx, c: *const pg_huffman_kv_cache, k: *mut f32, v: *mut f32) -> pg_status;
    pub fn pg_huffman_kv_cache_get_kv_dev(ctx: *mut pg_ctx, c: *const pg_huffman_kv_cache, k_dev: *mut f32, v_dev: *mut f32) -> pg_status;
    pub fn pg_moe_ffn(ctx: *mut pg_ctx, x: *const f32, T: usize, router_logits: *const f32, E: usize, top_k: usize, gate: *const *const pg_gguf_tensor, up: *const *const pg_gguf_tensor, down: *const *const pg_gguf_tensor, act: c_int, out: *mut f32) -> pg_status;
    pub fn pg_moe_ffn_dev(ctx: *mut pg_ctx, x_dev: *const f32, T: usize, router_logits_dev: *const f32, E: usize, top_k: usize, gate: *const *const pg_gguf_tensor, up: *const *const pg_gguf_tensor, down: *const *const pg_gguf_tensor, act: c_int, out_dev: *mut f32) -> pg_status;
    pub fn pg_moe_ffn_routed(ctx: *mut pg_ctx, x: *const f32, T: usize, expert_idx: *const i32, weight: *const f32, E: usize, top_k: usize, gate: *const *const pg_gguf_tensor, up: *const *const pg_gguf_tensor, down: *const *const pg_gguf_tensor, act: c_int, shared: *const f32, out: *mut f32) -> pg_status;
    pub fn pg_moe_ffn_routed_dev(ctx: *mut pg_ctx, x_dev: *const f32, T: usize, expert_idx_dev: *const i32, weight_dev: *const f32, E: usize, top_k: usize, gate: *const *const pg_gguf_tensor, up: *const *const pg_gguf_tensor, down: *const *const pg_gguf_tensor, act: c_int, shared_dev: *const f32, out_dev: *mut f32) -> pg_status;
    pub fn pg_rmsnorm(ctx: *mut pg_ctx, x: *const f32, rows: usize, dim: usize, w: *const f32, eps: f32, out: *mut f32) -> pg_status;
    pub fn pg_rmsnorm_dev(ctx: *mut pg_ctx, x_dev: *const f32, rows: usize, dim: usize, w_dev: *const f32, eps: f32, out_dev: *mut f32) -> pg_status;
    pub fn pg_rope_create(ctx: *mut pg_ctx, head_dim: usize, max_seq_len: usize, base: f32, out: *mut *mut pg_rope) -> pg_status;
    pub fn pg_rope_free(ctx: *mut pg_ctx, rope: *mut pg_rope);
    pub fn pg_rope_apply(ctx: *mut pg_ctx, rope: *const pg_rope, x: *const f32, seq_len: usize, offset: usize, out: *mut f32) -> pg_status;
    pub fn pg_rope_apply_dev(ctx: *mut pg_ctx, rope: *const pg_rope, x_dev: *const f32, seq_len: usize, offset: usize, out_dev: *mut f32) -> pg_status;
    pub fn pg_kv_cache_create(ctx: *mut pg_ctx, num_kv_heads: usize, head_dim: usize, out: *mut *mut pg_kv_cache) -> pg_status;
    pub fn pg_kv_cache_free(ctx: *mut pg_ctx, cache: *mut pg_kv_cache);
    pub fn pg_kv_cache_append(ctx: *mut pg_ctx, cache: *mut pg_kv_cache, new_k: *const f32, new_v: *const f32, seq_len: usize) -> pg_status;
    pub fn pg_kv_cache_append_dev(ctx: *mut pg_ctx, cache: *mut pg_kv_cache, new_k_dev: *const f32, new_v_dev: *const f32, seq_len: usize) -> pg_status;
    pub fn pg_kv_cache_rollback_to(cache: *mut pg_kv_cache, new_len: usize) -> pg_status;
    pub fn pg_kv_cache_len(cache: *const pg_kv_cache) -> usize;
    pub fn pg_kv_cache_capacity(cache: *const pg_kv_cache) -> usize;
    pub fn pg_kv_cache_download(ctx: *mut pg_ctx, cache: *const pg_kv_cache, k: *mut f32, v: *mut f32) -> pg_status;
    pub fn pg_gqa_attention(ctx: *mut pg_ctx, q: *const f32, k_cache: *const pg_kv_cache, v_cache: *const pg_kv_cache, num_q_heads: usize, seq_q: usize, scale: f32, mask_kind: c_int, offset: usize, window: usize, sink_tokens: usize, logit_cap: f32, out: *mut f32) -> pg_status;
    pub fn pg_gqa_attention_dev(ctx: *mut pg_ctx, q_dev: *const f32, k_cache: *const pg_kv_cache, v_cache: *const pg_kv_cache, num_q_heads: usize, seq_q: usize, scale: f32, mask_kind: c_int, offset: usize, window: usize, sink_tokens: usize, logit_cap: f32, out_dev: *mut f32) -> pg_status;
    pub fn pg_gqa_attention_local_global(ctx: *mut pg_ctx, q: *const f32, k_cache: *const pg_kv_cache, v_cache: *const pg_kv_cache, num_q_heads: usize, seq_q: usize, scale: f32, offset: usize, local_window: usize, global_positions: *const usize, num_global: usize, logit_cap: f32, out: *mut f32) -> pg_status;
    pub fn pg_gqa_attention_local_global_dev(ctx: *mut pg_ctx, q_dev: *const f32, k_cache: *const pg_kv_cache, v_cache: *const pg_kv_cache, num_q_heads: usize, seq_q: usize, scale: f32, offset: usize, local_window: usize, global_positions: *const usize, num_global: usize, logit_cap: f32, out_dev: *mut f32) -> pg_status;
    pub fn pg_llama_block_create(ctx: *mut pg_ctx, model_dim: usize, num_q_heads: usize, num_kv_heads: usize, head_dim: usize, ffn_dim: usize, max_seq_len: usize, rope_base: f32, rms_eps: f32, out: *mut *mut pg_llama_block) -> pg_status;
    pub fn pg_llama_block_free(ctx: *mut pg_ctx, block: *mut pg_llama_block);
    pub fn pg_llama_block_set_weights(ctx: *mut pg_ctx, block: *mut pg_llama_block, q_proj: *const pg_gguf_tensor, k_proj: *const pg_gguf_tensor, v_proj: *const pg_gguf_tensor, o_proj: *const pg_gguf_tensor, gate_proj: *const pg_gguf_tensor, up_proj: *const pg_gguf_tensor, down_proj: *const pg_gguf_tensor, attn_norm_w: *const f32, ffn_norm_w: *const f32) -> pg_status;
    pub fn pg_llama_block_forward(ctx: *mut pg_ctx, block: *mut pg_llama_block, h: *const f32, seq: usize, cache: *mut pg_kv_cache, out: *mut f32) -> pg_status;
    pub fn pg_llama_block_forward_dev(ctx: *mut pg_ctx, block: *mut pg_llama_block, h_dev: *const f32, seq: usize, cache: *mut pg_kv_cache, out_dev: *mut f32) -> pg_status;
    pub fn pg_profile_begin(ctx: *mut pg_ctx) -> pg_status;
    pub fn pg_profile_end(ctx: *mut pg_ctx, num_kernels: *mut usize) -> pg_status;
    pub fn pg_profile_get(ctx: *mut pg_ctx, i: usize, name: *mut *const c_char, total_ms: *mut f64, launches: *mut usize) -> pg_status;
    pub fn pg_profile_get_grids(ctx: *mut pg_ctx, i: usize, work_items: *mut usize, launches: *mut usize, cap: usize, count: *mut usize) -> pg_status;
    pub fn pg_probe_mfma_i8(ctx: *mut pg_ctx, iters: c_int, tops: *mut f64, clock_ghz: *mut f64) -> pg_status;
    pub fn pg_probe_hbm_read(ctx: *mut pg_ctx, bytes_per_pass: usize, buffers: c_int, passes: c_int, gbs: *mut f64) -> pg_status;
    pub fn pg_probe_hbm_read_shaped(ctx: *mut pg_ctx, bytes_per_pass: usize, buffers: c_int, passes: c_int, workgroups: c_int, threads: c_int, loads_in_flight: c_int, gbs: *mut f64) -> pg_status;
    pub fn pg_probe_gemm_clock(ctx: *mut pg_ctx, m: usize, k: usize, n: usize, clock_ghz: *mut f64, loop_us: *mut f64) -> pg_status;
    pub fn pg_gemm_w8a8_last_tile(ctx: *const pg_ctx, bm: *mut c_int, bn: *mut c_int, k_splits: *mut c_int) -> pg_status;
    pub fn pg_gemm_w8a8_force_tile(ctx: *mut pg_ctx, tile: c_int) -> pg_status;
    pub fn pg_gemv_w8a8_force_shape(ctx: *mut pg_ctx, wavefronts: c_int, rows_per_wavefront: c_int) -> pg_status;
    pub fn pg_gguf_hmm_force(ctx: *mut pg_ctx, mode: c_int) -> pg_status;
    pub fn pg_audit_gemv_w8a8_m1(k: usize, n: usize, nch: c_int, rows_per_wavefront: c_int, wavefronts: c_int, f32_row: c_int, w_end: *mut usize, w_bytes: *mut usize, x_end: *mut usize, x_bytes: *mut usize) -> pg_status;
    pub fn pg_audit_gemm_w8a8_skinny(m: usize, k: usize, n: usize, activation_tiles: c_int, weight_tiles: c_int, wavefronts: c_int, w_end: *mut usize, w_bytes: *mut usize, a_end: *mut usize, a_bytes: *mut usize) -> pg_status;
    pub fn pg_audit_gguf_gemv(n_out: usize, k_in: usize, q8: c_int, blocks_per_lane: c_int, rows_per_wavefront: c_int, wavefronts: c_int, qs_end: *mut usize, qs_bytes: *mut usize, d_end: *mut usize, d_bytes: *mut usize) -> pg_status;
    pub fn pg_audit_gguf_skinny(n_out: usize, k_in: usize, q8: c_int, wavefronts: c_int, weight_tiles: c_int, qs_end: *mut usize, qs_bytes: *mut usize, d_end: *mut usize, d_bytes: *mut usize) -> pg_status;
    pub fn pg_audit_gguf_hmm(m: usize, n_out: usize, k_in: usize, q8: c_int, wide_tiles: c_int, k_chunks: c_int, plane_end: *mut usize, plane_bytes: *mut usize, qs_end: *mut usize, qs_bytes: *mut usize, d_end: *mut usize, d_bytes: *mut usize) -> pg_status;
    pub fn pg_audit_mxfp4_rows(out_dim: usize, in_dim: usize, row_groups_per_workgroup: c_int, wavefronts: c_int, qs_end: *mut usize, qs_bytes: *mut usize, sc_end: *mut usize, sc_bytes: *mut usize) -> pg_status;
    pub fn pg_audit_mxfp4_tiles(num_cu: c_int, out_dim: usize, in_dim: usize, m: usize, qs_end: *mut usize, qs_bytes: *mut usize, sc_end: *mut usize, sc_bytes: *mut usize, rec_end: *mut usize, rec_bytes: *mut usize, ra: *mut c_int, tb: *mut c_int, ks: *mut c_int) -> pg_status;
    pub fn pg_audit_probe_read(bytes: usize, workgroups: c_int, threads: c_int, loads_in_flight: c_int, end: *mut usize, alloc: *mut usize) -> pg_status;
}
// ---- generated: end ----

/// Turns a non-zero status into the panic the reference raises in the same place.
pub fn ok(st: pg_status) {
    if st != PG_OK {
        let msg = unsafe { std::ffi::CStr::from_ptr(pg_last_error()) }.to_string_lossy().into_owned();
        panic!("peregrine_hip: {msg}");
    }
}

thread_local! {
    // One context per thread on device 0: the shape of the reference's thread-local Metal
    // singleton (src/metal/context.rs:2472-2510).  Tensor is Rc<RefCell>, so callers are
    // single-threaded per tensor anyway (src/tensor.rs:864).
    static CTX: *mut pg_ctx = unsafe {
        let mut c = std::ptr::null_mut();
        ok(pg_ctx_create(0, std::ptr::null_mut(), &mut c));
        c
    };
}

/// The calling thread's context.
pub fn ctx() -> *mut pg_ctx {
    CTX.with(|c| *c)
}

/// `gpu.sync()` of the reference's GPU path (tests/quant_parity.rs:102-107).
pub fn sync() {
    ok(unsafe { pg_sync(ctx()) });
}

/// Stands where the reference's functions take `&GpuContext` (src/quant.rs:174,183,196-197): the
/// device context itself is the calling thread's (`ctx()`), so the value carries nothing.
pub struct GpuContext;
impl GpuContext {
    /// `gpu.sync()`  tests/quant_parity.rs:104.
    pub fn sync(&self) {
        sync();
    }
}

/// `peregrine::quant` (src/quant.rs) over the library.
pub mod quant {
    use super::*;

    /// Device copy of a `QuantizedTensor`: what `gpu_data_i8` + `gpu_scales` are in the
    /// reference (src/quant.rs:19-22).  Freed on drop.
    pub struct HipQTensor(pub *mut pg_qtensor);
    impl Drop for HipQTensor {
        fn drop(&mut self) {
            unsafe { pg_qtensor_free(ctx(), self.0) }
        }
    }

    /// `quant::QuantizedTensor`  src/quant.rs:12-23.
    pub struct QuantizedTensor {
        pub data_i8: Vec<i8>,
        pub data_i8_t: Vec<i8>,
        pub scales: Vec<f32>,
        pub rows: usize,
        pub cols: usize,
        /// The device copy, made once.  A cell, because `matmul_quantized` takes `&QuantizedTensor`
        /// (src/quant.rs:133) and still has to place the weights on the device on first use; the
        /// reference's callers are single-threaded per tensor (src/tensor.rs:864), so is this.
        pub hip: std::cell::OnceCell<HipQTensor>,
    }

    impl QuantizedTensor {
        fn upload(&self) -> *const pg_qtensor {
            self.hip.get_or_init(|| {
                let mut h = std::ptr::null_mut();
                ok(unsafe { pg_qtensor_upload(ctx(), self.data_i8.as_ptr(), self.scales.as_ptr(), self.rows, self.cols, &mut h) });
                HipQTensor(h)
            }).0
        }

        /// `QuantizedTensor::to_gpu`  src/quant.rs:174-181 (idempotent).
        pub fn to_gpu(&mut self, _gpu: &GpuContext) {
            self.upload();
        }

        /// `QuantizedTensor::from_gpu`  src/quant.rs:183-190.
        pub fn from_gpu(&mut self, _gpu: &GpuContext) {
            if let Some(h) = self.hip.get() {
                ok(unsafe { pg_qtensor_download(ctx(), h.0, self.data_i8.as_mut_ptr(), self.data_i8_t.as_mut_ptr(), self.scales.as_mut_ptr()) });
            }
        }

        fn handle(&self) -> *const pg_qtensor {
            self.hip.get().expect("weights not on GPU").0 // src/quant.rs:208
        }
    }

    /// `quant::quantize_weights`  src/quant.rs:27-75.
    pub fn quantize_weights(data: &[f32], rows: usize, cols: usize) -> QuantizedTensor {
        assert_eq!(data.len(), rows * cols);
        let (mut q, mut q_t, mut s) = (vec![0i8; rows * cols], vec![0i8; rows * cols], vec![0f32; cols]);
        ok(unsafe { pg_quantize_weights(ctx(), data.as_ptr(), rows, cols, q.as_mut_ptr(), q_t.as_mut_ptr(), s.as_mut_ptr()) });
        QuantizedTensor { data_i8: q, data_i8_t: q_t, scales: s, rows, cols, hip: std::cell::OnceCell::new() }
    }

    /// `quant::quantize_activations`  src/quant.rs:79-112.
    pub fn quantize_activations(data: &[f32], rows: usize, cols: usize) -> (Vec<i8>, Vec<f32>) {
        assert_eq!(data.len(), rows * cols);
        let (mut q, mut s) = (vec![0i8; rows * cols], vec![0f32; rows]);
        ok(unsafe { pg_quantize_activations(ctx(), data.as_ptr(), rows, cols, q.as_mut_ptr(), s.as_mut_ptr()) });
        (q, s)
    }

    /// `quant::dequantize`  src/quant.rs:115-123.
    pub fn dequantize(qt: &QuantizedTensor) -> Vec<f32> {
        let mut out = vec![0f32; qt.rows * qt.cols];
        ok(unsafe { pg_dequantize(ctx(), qt.data_i8.as_ptr(), qt.scales.as_ptr(), qt.rows, qt.cols, out.as_mut_ptr()) });
        out
    }

    /// `quant::matmul_quantized`  src/quant.rs:129-169.  The weights go to the device on first
    /// use and stay there (the reference's CPU path has no such state; the result is the same).
    pub fn matmul_quantized(a_data: &[f32], m: usize, k: usize, w: &QuantizedTensor) -> Vec<f32> {
        assert_eq!(w.rows, k);
        assert_eq!(a_data.len(), m * k);
        let h = w.upload();
        let mut out = vec![0f32; m * w.cols];
        ok(unsafe { pg_matmul_quantized(ctx(), a_data.as_ptr(), m, k, h, out.as_mut_ptr()) });
        out
    }

    /// An unsynced device buffer, the `GpuBuffer<T>` that `matmul_quantized_gpu` returns
    /// (src/quant.rs:202; only `GpuBuffer<f32>` is ever made here).
    pub struct GpuBuffer<T> {
        pub ptr: *mut T,
        pub len: usize,
    }
    impl<T: Copy + Default> GpuBuffer<T> {
        /// `GpuBuffer::read` (after `sync()`).
        pub fn read(&self) -> Vec<T> {
            let mut v = vec![T::default(); self.len];
            ok(unsafe { pg_memcpy_d2h(ctx(), v.as_mut_ptr() as *mut c_void, self.ptr as *const c_void, self.len * std::mem::size_of::<T>()) });
            v
        }
    }
    impl<T> Drop for GpuBuffer<T> {
        fn drop(&mut self) {
            unsafe { pg_dev_free(ctx(), self.ptr as *mut c_void) };
        }
    }

    /// `quant::matmul_quantized_gpu`  src/quant.rs:196-218: uploads `a`, enqueues the product,
    /// returns without waiting.  Numerics are the CPU path's W8A8; `matmul_dequant_i8_gpu` gives
    /// the Metal shader's W8A32.
    pub fn matmul_quantized_gpu(_gpu: &GpuContext, a_data: &[f32], m: usize, k: usize, w: &QuantizedTensor) -> GpuBuffer<f32> {
        assert_eq!(w.rows, k);
        assert_eq!(a_data.len(), m * k);
        let h = w.handle();
        let (mut a_dev, mut out_dev) = (std::ptr::null_mut(), std::ptr::null_mut());
        ok(unsafe { pg_dev_alloc(ctx(), m * k * 4, &mut a_dev) });
        ok(unsafe { pg_dev_alloc(ctx(), m * w.cols * 4, &mut out_dev) });
        ok(unsafe { pg_memcpy_h2d(ctx(), a_dev, a_data.as_ptr() as *const c_void, m * k * 4) });
        ok(unsafe { pg_matmul_quantized_dev(ctx(), a_dev as *const f32, m, k, h, out_dev as *mut f32, std::ptr::null_mut()) });
        let out = GpuBuffer { ptr: out_dev as *mut f32, len: m * w.cols };
        drop(GpuBuffer { ptr: a_dev as *mut f32, len: 0 }); // pg_dev_free waits for the stream first
        out
    }

    /// The Metal shader's numerics for the same call (`matmul_dequant_i8`,
    /// src/metal/shaders.rs:2329-2375): f32 activations, dequantised weights, f32 accumulate.
    pub fn matmul_dequant_i8(a_data: &[f32], m: usize, k: usize, w: &QuantizedTensor) -> Vec<f32> {
        assert_eq!(w.rows, k);
        assert_eq!(a_data.len(), m * k);
        let h = w.upload();
        let mut out = vec![0f32; m * w.cols];
        ok(unsafe { pg_matmul_dequant_i8(ctx(), a_data.as_ptr(), m, k, h, out.as_mut_ptr()) });
        out
    }
}

/// `peregrine::gguf` block dequantisation (src/gguf.rs:286-382) and the keep-quantised weight.
pub mod gguf {
    use super::*;

    fn blocks(data: &[u8], num_elements: usize, block_bytes: usize) -> usize {
        assert!(num_elements % 32 == 0); // src/gguf.rs:287,308
        let n = num_elements / 32;
        assert!(data.len() >= n * block_bytes); // src/gguf.rs:290,311
        n
    }

    /// `gguf::dequant_q8_0`  src/gguf.rs:286-302.
    pub fn dequant_q8_0(data: &[u8], num_elements: usize) -> Vec<f32> {
        blocks(data, num_elements, 34);
        let mut out = vec![0f32; num_elements];
        ok(unsafe { pg_dequant_q8_0(ctx(), data.as_ptr(), num_elements, out.as_mut_ptr()) });
        out
    }

    /// `gguf::dequant_q4_0`  src/gguf.rs:307-326.
    pub fn dequant_q4_0(data: &[u8], num_elements: usize) -> Vec<f32> {
        blocks(data, num_elements, 18);
        let mut out = vec![0f32; num_elements];
        ok(unsafe { pg_dequant_q4_0(ctx(), data.as_ptr(), num_elements, out.as_mut_ptr()) });
        out
    }

    /// `gguf::dequant_q4_1`  src/gguf.rs:331-351.
    pub fn dequant_q4_1(data: &[u8], num_elements: usize) -> Vec<f32> {
        blocks(data, num_elements, 20);
        let mut out = vec![0f32; num_elements];
        ok(unsafe { pg_dequant_q4_1(ctx(), data.as_ptr(), num_elements, out.as_mut_ptr()) });
        out
    }

    /// `gguf::f16_to_f32`  src/gguf.rs:354-382 (one value; `f16_to_f32_slice` converts many at once).
    pub fn f16_to_f32(bits: u16) -> f32 {
        f16_to_f32_slice(&[bits])[0]
    }

    /// The same conversion over a slice in one call.
    pub fn f16_to_f32_slice(bits: &[u16]) -> Vec<f32> {
        let mut out = vec![0f32; bits.len()];
        ok(unsafe { pg_f16_to_f32(ctx(), bits.as_ptr(), bits.len(), out.as_mut_ptr()) });
        out
    }

    /// `gguf::load_tensor_q8_as_quantized`  src/gguf.rs:386-401.
    pub fn load_tensor_q8_as_quantized(data: &[u8], rows: usize, cols: usize) -> crate::quant::QuantizedTensor {
        let f32_data = dequant_q8_0(data, rows * cols);
        crate::quant::quantize_weights(&f32_data, rows, cols)
    }

    /// A GGUF weight `[n_out, k_in]` kept quantised on the device: the slot of the
    /// dequantised, transposed `Tensor` that `load_transposed_weight` makes
    /// (src/models/llama/model.rs:243-257).  `matmul` is `x.matmul(&w)` on it.
    pub struct GgufWeight(pub *mut pg_gguf_tensor, pub usize, pub usize);
    impl GgufWeight {
        pub fn new(blocks: &[u8], ggml_type: c_int, n_out: usize, k_in: usize) -> Self {
            let mut h = std::ptr::null_mut();
            ok(unsafe { pg_gguf_upload(ctx(), blocks.as_ptr() as *const c_void, ggml_type, n_out, k_in, &mut h) });
            GgufWeight(h, n_out, k_in)
        }
        /// The load-time step: the derived device copies that products over up to `max_rows` rows need are
        /// made now, so that those products neither allocate nor wait.
        pub fn prepare(&self, max_rows: usize) {
            ok(unsafe { pg_gguf_prepare(ctx(), self.0, max_rows) });
        }
        /// y [m, n_out] = x [m, k_in] . dequant(w)^T  (src/tensor.rs:1342-1353 on the transposed weight).
        pub fn matmul(&self, x: &[f32], m: usize) -> Vec<f32> {
            assert_eq!(x.len(), m * self.2);
            let mut y = vec![0f32; m * self.1];
            ok(unsafe { pg_gguf_matmul(ctx(), x.as_ptr(), m, self.0, y.as_mut_ptr()) });
            y
        }
    }
    impl Drop for GgufWeight {
        fn drop(&mut self) {
            unsafe { pg_gguf_free(ctx(), self.0) }
        }
    }
}

/// The grouped expert FFN behind `MoELayer::forward` (examples/grok1/moe.rs:70-109).
pub mod moe {
    use super::*;

    /// x [t, d], router_logits [t, e]; gate / up [e] of [ffn, d], down [e] of [d, ffn];
    /// returns [t, d].  `act`: `PG_ACT_SILU` or `PG_ACT_GELU_TANH`.
    pub fn moe_ffn(x: &[f32], t: usize, router_logits: &[f32], top_k: usize, gate: &[gguf::GgufWeight],
                   up: &[gguf::GgufWeight], down: &[gguf::GgufWeight], act: c_int) -> Vec<f32> {
        let e = gate.len();
        assert!(e > 0 && up.len() == e && down.len() == e);
        let d = gate[0].2;
        assert_eq!(x.len(), t * d);
        assert_eq!(router_logits.len(), t * e);
        let tab = |w: &[gguf::GgufWeight]| w.iter().map(|g| g.0 as *const pg_gguf_tensor).collect::<Vec<_>>();
        let (g, u, dn) = (tab(gate), tab(up), tab(down));
        let mut out = vec![0f32; t * d];
        ok(unsafe { pg_moe_ffn(ctx(), x.as_ptr(), t, router_logits.as_ptr(), e, top_k, g.as_ptr(), u.as_ptr(), dn.as_ptr(), act, out.as_mut_ptr()) });
        out
    }

    /// The same over a routing another gate made (`Gate::forward`, examples/deepseek/moe.rs:111-215, which returns
    /// `Vec<Vec<(usize, f32)>>`; the gpt_oss router, examples/gpt_oss/moe.rs:298-330): `routing[t]` = the token's
    /// `(expert_idx, weight)` list, every token with the same number of experts; `shared` = the shared experts'
    /// output `[t, d]`, added last (examples/deepseek/moe.rs:298-300).
    pub fn moe_ffn_routed(x: &[f32], routing: &[Vec<(usize, f32)>], gate: &[gguf::GgufWeight], up: &[gguf::GgufWeight],
                          down: &[gguf::GgufWeight], act: c_int, shared: Option<&[f32]>) -> Vec<f32> {
        let (e, t) = (gate.len(), routing.len());
        assert!(e > 0 && up.len() == e && down.len() == e);
        let d = gate[0].2;
        assert_eq!(x.len(), t * d);
        let top_k = routing.first().map_or(0, |r| r.len());
        assert!(routing.iter().all(|r| r.len() == top_k));
        let idx: Vec<i32> = routing.iter().flatten().map(|&(i, _)| i as i32).collect();
        let w: Vec<f32> = routing.iter().flatten().map(|&(_, w)| w).collect();
        if let Some(s) = shared { assert_eq!(s.len(), t * d); }
        let tab = |w: &[gguf::GgufWeight]| w.iter().map(|g| g.0 as *const pg_gguf_tensor).collect::<Vec<_>>();
        let (g, u, dn) = (tab(gate), tab(up), tab(down));
        let mut out = vec![0f32; t * d];
        ok(unsafe { pg_moe_ffn_routed(ctx(), x.as_ptr(), t, idx.as_ptr(), w.as_ptr(), e, top_k, g.as_ptr(), u.as_ptr(), dn.as_ptr(), act,
                                      shared.map_or(std::ptr::null(), |s| s.as_ptr()), out.as_mut_ptr()) });
        out
    }
}
