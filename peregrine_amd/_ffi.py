"""ctypes binding of libperegrine_hip.so (the C ABI declared in include/peregrine_hip.h)."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libperegrine_hip.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
        "or `make -C peregrine_amd/csrc`. peregrine_amd has no CPU fallback."
    )

# A process that also uses PyTorch-ROCm must load torch's bundled HIP runtime first: the library then binds to
# that copy.  Loaded the other way round the process holds two runtimes, and the second to initialise finds no
# device ("no ROCm-capable device is detected" from pg_ctx_create).
try:
    import torch  # noqa: F401
except Exception:  # absent, or present but broken (a failing torch must not take this binding down with it)
    pass

lib = C.CDLL(LIB_PATH)

PG_OK, PG_EINVAL, PG_EDEVICE, PG_ENOMEM, PG_EUNSUPPORTED = 0, 1, 2, 3, 4
GGML_Q4_0, GGML_Q4_1, GGML_Q8_0 = 2, 3, 8
MXFP4 = 39
ACT_SILU, ACT_GELU_TANH = 0, 1
MASK_NONE, MASK_CAUSAL, MASK_CAUSAL_SLIDING_WINDOW, MASK_LOCAL_GLOBAL = 0, 1, 2, 3

_vp, _sz, _int = C.c_void_p, C.c_size_t, C.c_int
_pp = C.POINTER(C.c_void_p)

# name -> argtypes; every function returns pg_status unless listed in _OTHER_RESTYPE.
SIGNATURES = {
    "pg_ctx_create": [_int, _vp, _pp],
    "pg_ctx_destroy": [_vp],
    "pg_sync": [_vp],
    "pg_ctx_stream": [_vp],
    "pg_last_error": [],
    "pg_status_string": [_int],
    "pg_profile_begin": [_vp],
    "pg_profile_end": [_vp, C.POINTER(_sz)],
    "pg_profile_get": [_vp, _sz, C.POINTER(C.c_char_p), C.POINTER(C.c_double), C.POINTER(_sz)],
    "pg_probe_mfma_i8": [_vp, _int, C.POINTER(C.c_double), C.POINTER(C.c_double)],
    "pg_probe_hbm_read": [_vp, _sz, _int, _int, C.POINTER(C.c_double)],
    "pg_probe_hbm_read_shaped": [_vp, _sz, _int, _int, _int, _int, _int, C.POINTER(C.c_double)],
    "pg_probe_gemm_clock": [_vp, _sz, _sz, _sz, C.POINTER(C.c_double), C.POINTER(C.c_double)],
    "pg_profile_get_grids": [_vp, _sz, C.POINTER(_sz), C.POINTER(_sz), _sz, C.POINTER(_sz)],
    "pg_dev_alloc": [_vp, _sz, _pp],
    "pg_dev_free": [_vp, _vp],
    "pg_memcpy_h2d": [_vp, _vp, _vp, _sz],
    "pg_memcpy_d2h": [_vp, _vp, _vp, _sz],
    "pg_quantize_weights": [_vp, _vp, _sz, _sz, _vp, _vp, _vp],
    "pg_quantize_activations": [_vp, _vp, _sz, _sz, _vp, _vp],
    "pg_quantize_activations_dev": [_vp, _vp, _sz, _sz, _vp, _vp],
    "pg_dequantize": [_vp, _vp, _vp, _sz, _sz, _vp],
    "pg_qtensor_upload": [_vp, _vp, _vp, _sz, _sz, _pp],
    "pg_qtensor_from_f32": [_vp, _vp, _sz, _sz, _pp],
    "pg_qtensor_from_f32_dev": [_vp, _vp, _sz, _sz, _pp],
    "pg_qtensor_download": [_vp, _vp, _vp, _vp, _vp],
    "pg_qtensor_shape": [_vp, C.POINTER(_sz), C.POINTER(_sz)],
    "pg_qtensor_free": [_vp, _vp],
    "pg_matmul_quantized": [_vp, _vp, _sz, _sz, _vp, _vp],
    "pg_matmul_quantized_dev": [_vp, _vp, _sz, _sz, _vp, _vp, _vp],
    "pg_matmul_quantized_multi_dev": [_vp, _vp, _sz, _sz, _pp, _sz, _pp],
    "pg_matmul_quantized_fixed_scratch_dev": [_vp, _vp, _sz, _sz, _vp, _vp],
    "pg_fixed_scratch_bytes": [],
    "pg_gemm_w8a8_last_tile": [_vp, C.POINTER(_int), C.POINTER(_int), C.POINTER(_int)],
    "pg_audit_gemv_w8a8_m1": [_sz, _sz, _int, _int, _int, _int, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "pg_audit_gemm_w8a8_skinny": [_sz, _sz, _sz, _int, _int, _int, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "pg_audit_gguf_gemv": [_sz, _sz, _int, _int, _int, _int, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "pg_audit_gguf_hmm": [_sz, _sz, _sz, _int, _int, _int] + [C.POINTER(C.c_size_t)] * 6,
    "pg_audit_gguf_skinny": [_sz, _sz, _int, _int, _int, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "pg_audit_mxfp4_tiles": [_int, _sz, _sz, _sz] + [C.POINTER(C.c_size_t)] * 6 + [C.POINTER(_int)] * 3,
    "pg_audit_mxfp4_rows": [_sz, _sz, _int, _int, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "pg_audit_probe_read": [_sz, _int, _int, _int, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "pg_gemm_w8a8_force_tile": [_vp, _int],
    "pg_gemv_w8a8_force_shape": [_vp, _int, _int],
    "pg_gguf_hmm_force": [_vp, _int],
    "pg_matmul_dequant_i8": [_vp, _vp, _sz, _sz, _vp, _vp],
    "pg_matmul_dequant_i8_dev": [_vp, _vp, _sz, _sz, _vp, _vp],
    "pg_f16_to_f32": [_vp, _vp, _sz, _vp],
    "pg_dequant_q8_0": [_vp, _vp, _sz, _vp],
    "pg_dequant_q4_0": [_vp, _vp, _sz, _vp],
    "pg_dequant_q4_1": [_vp, _vp, _sz, _vp],
    "pg_gguf_upload": [_vp, _vp, _int, _sz, _sz, _pp],
    "pg_gguf_shape": [_vp, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_int)],
    "pg_gguf_free": [_vp, _vp],
    "pg_gguf_matmul": [_vp, _vp, _sz, _vp, _vp],
    "pg_gguf_matmul_dev": [_vp, _vp, _sz, _vp, _vp],
    "pg_gguf_prepare": [_vp, _vp, _sz],
    "pg_gguf_drop_prepared": [_vp, _vp],
    "pg_gguf_device_bytes": [_vp, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "pg_gguf_file_parse": [_vp, _sz, _pp],
    "pg_gguf_file_open": [C.c_char_p, _pp],
    "pg_gguf_file_close": [_vp],
    "pg_gguf_file_counts": [_vp, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(C.c_uint32), C.POINTER(C.c_uint64)],
    "pg_gguf_file_tensor_name": [_vp, _sz, C.POINTER(C.c_char_p)],
    "pg_gguf_file_tensor_info": [_vp, C.c_char_p, C.POINTER(_int), C.POINTER(_sz), C.POINTER(C.c_uint64), _sz,
                                 C.POINTER(C.c_uint64), C.POINTER(_sz), _pp],
    "pg_gguf_file_get_u32": [_vp, C.c_char_p, C.POINTER(C.c_uint32), C.POINTER(_int)],
    "pg_gguf_file_get_f32": [_vp, C.c_char_p, C.POINTER(C.c_float), C.POINTER(_int)],
    "pg_gguf_file_get_str": [_vp, C.c_char_p, C.POINTER(C.c_char_p), C.POINTER(_sz)],
    "pg_gguf_file_get_array": [_vp, C.c_char_p, C.POINTER(C.c_uint32), C.POINTER(_sz)],
    "pg_gguf_file_get_array_str": [_vp, C.c_char_p, _sz, C.POINTER(C.c_char_p)],
    "pg_gguf_file_get_array_f64": [_vp, C.c_char_p, C.POINTER(C.c_double), _sz],
    "pg_gguf_file_load_tensor_f32": [_vp, _vp, C.c_char_p, _vp, _sz],
    "pg_gguf_file_upload_tensor": [_vp, _vp, C.c_char_p, _pp],
    "pg_quantized_record_size": [_sz, _sz, _sz, C.POINTER(_sz)],
    "pg_write_quantized_tensor": [_vp, _sz, C.c_char_p, _sz, _vp, _vp, _sz, _sz, C.POINTER(_sz)],
    "pg_read_quantized_tensor": [_vp, _sz, _pp, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz), _pp, _pp, C.POINTER(_sz)],
    "pg_qtensor_from_record": [_vp, _vp, _sz, _pp, C.POINTER(_sz)],
    "pg_moe_ffn": [_vp, _vp, _sz, _vp, _sz, _sz, _pp, _pp, _pp, _int, _vp],
    "pg_moe_ffn_dev": [_vp, _vp, _sz, _vp, _sz, _sz, _pp, _pp, _pp, _int, _vp],
    "pg_moe_ffn_routed": [_vp, _vp, _sz, _vp, _vp, _sz, _sz, _pp, _pp, _pp, _int, _vp, _vp],
    "pg_moe_ffn_routed_dev": [_vp, _vp, _sz, _vp, _vp, _sz, _sz, _pp, _pp, _pp, _int, _vp, _vp],
    "pg_huffman_table_from_frequencies": [_vp, _vp, _vp],
    "pg_huffman_canonical_codes": [_vp, _vp],
    "pg_huffman_encode": [_vp, _vp, _sz, _vp, _sz, C.POINTER(_sz)],
    "pg_huffman_decode": [_vp, _vp, _vp, _sz, _sz, _vp],
    "pg_huffman_tensor_from_quantized": [_vp, _vp, _sz, _sz, _sz, _pp],
    "pg_huffman_tensor_from_parts": [_vp, _pp, C.POINTER(_sz), C.POINTER(_sz), _sz, _vp, _sz, _sz, _pp],
    "pg_huffman_tensor_free": [_vp],
    "pg_huffman_tensor_info": [_vp, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz)],
    "pg_huffman_tensor_stream": [_vp, _sz, _pp, C.POINTER(_sz), C.POINTER(_sz)],
    "pg_huffman_tensor_table": [_vp, _pp, _pp],
    "pg_huffman_tensor_decode_to_quantized": [_vp, _vp, _vp, _vp, _vp],
    "pg_huffman_tensor_to_gpu": [_vp, _vp, _pp],
    "pg_matmul_huffman": [_vp, _vp, _sz, _sz, _vp, _vp],
    "pg_huffman_kv_compress_chunk": [_vp, _vp, _sz, _sz, _sz, _pp],
    "pg_huffman_kv_compress_chunk_dev": [_vp, _vp, _sz, _sz, _sz, _sz, _pp],
    "pg_huffman_kv_chunk_from_parts": [_vp, _vp, _sz, _vp, _vp, _sz, _sz, _sz, _pp],
    "pg_huffman_kv_chunk_free": [_vp, _vp],
    "pg_huffman_kv_chunk_info": [_vp, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz)],
    "pg_huffman_kv_chunk_parts": [_vp, _vp, _vp, _vp, _vp],
    "pg_huffman_kv_decompress_chunk": [_vp, _vp, _vp],
    "pg_huffman_kv_decompress_chunk_dev": [_vp, _vp, _vp, _sz],
    "pg_huffman_kv_cache_create": [_vp, _sz, _sz, _sz, _sz, _pp],
    "pg_huffman_kv_cache_free": [_vp, _vp],
    "pg_huffman_kv_cache_append": [_vp, _vp, _vp, _vp, _sz],
    "pg_huffman_kv_cache_append_dev": [_vp, _vp, _vp, _vp, _sz],
    "pg_huffman_kv_cache_len": [_vp],
    "pg_huffman_kv_cache_compressed_len": [_vp],
    "pg_huffman_kv_cache_compress_threshold": [_vp],
    "pg_huffman_kv_cache_num_chunks": [_vp],
    "pg_huffman_kv_cache_hot": [_vp, _pp],
    "pg_huffman_kv_cache_chunk": [_vp, _int, _sz, _pp],
    "pg_huffman_kv_cache_get_kv": [_vp, _vp, _vp, _vp],
    "pg_huffman_kv_cache_get_kv_dev": [_vp, _vp, _vp, _vp],
    "pg_mxfp4_matmul": [_vp, _vp, _vp, _vp, _sz, _sz, _vp],
    "pg_mxfp4_upload": [_vp, _vp, _vp, _sz, _sz, _pp],
    "pg_mxfp4_expert_create": [_vp, _sz, _sz, C.c_float, C.c_float, _vp, _vp, _vp, _vp, _vp, _vp, _pp],
    "pg_mxfp4_expert_free": [_vp, _vp],
    "pg_mxfp4_expert_forward": [_vp, _vp, _vp, _sz, _vp],
    "pg_mxfp4_expert_forward_dev": [_vp, _vp, _vp, _sz, _vp, _vp],
    "pg_mxfp4_moe_ffn_routed": [_vp, _vp, _sz, _vp, _vp, _sz, _pp, _sz, _vp],
    "pg_mxfp4_moe_ffn_routed_dev": [_vp, _vp, _sz, _vp, _vp, _sz, _pp, _sz, _vp],
    "pg_rmsnorm": [_vp, _vp, _sz, _sz, _vp, C.c_float, _vp],
    "pg_rmsnorm_dev": [_vp, _vp, _sz, _sz, _vp, C.c_float, _vp],
    "pg_rope_create": [_vp, _sz, _sz, C.c_float, _pp],
    "pg_rope_free": [_vp, _vp],
    "pg_rope_apply": [_vp, _vp, _vp, _sz, _sz, _vp],
    "pg_rope_apply_dev": [_vp, _vp, _vp, _sz, _sz, _vp],
    "pg_kv_cache_create": [_vp, _sz, _sz, _pp],
    "pg_kv_cache_free": [_vp, _vp],
    "pg_kv_cache_append": [_vp, _vp, _vp, _vp, _sz],
    "pg_kv_cache_append_dev": [_vp, _vp, _vp, _vp, _sz],
    "pg_kv_cache_rollback_to": [_vp, _sz],
    "pg_kv_cache_len": [_vp],
    "pg_kv_cache_capacity": [_vp],
    "pg_kv_cache_download": [_vp, _vp, _vp, _vp],
    "pg_gqa_attention": [_vp, _vp, _vp, _vp, _sz, _sz, C.c_float, _int, _sz, _sz, _sz, C.c_float, _vp],
    "pg_gqa_attention_dev": [_vp, _vp, _vp, _vp, _sz, _sz, C.c_float, _int, _sz, _sz, _sz, C.c_float, _vp],
    "pg_gqa_attention_local_global": [_vp, _vp, _vp, _vp, _sz, _sz, C.c_float, _sz, _sz, _vp, _sz, C.c_float, _vp],
    "pg_gqa_attention_local_global_dev": [_vp, _vp, _vp, _vp, _sz, _sz, C.c_float, _sz, _sz, _vp, _sz, C.c_float, _vp],
    "pg_llama_block_create": [_vp, _sz, _sz, _sz, _sz, _sz, _sz, C.c_float, C.c_float, _pp],
    "pg_llama_block_free": [_vp, _vp],
    "pg_llama_block_set_weights": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp],
    "pg_llama_block_forward": [_vp, _vp, _vp, _sz, _vp, _vp],
    "pg_llama_block_forward_dev": [_vp, _vp, _vp, _sz, _vp, _vp],
}
_OTHER_RESTYPE = {
    "pg_ctx_destroy": None,
    "pg_qtensor_free": None,
    "pg_gguf_free": None,
    "pg_gguf_file_close": None,
    "pg_rope_free": None,
    "pg_huffman_tensor_free": None,
    "pg_huffman_kv_chunk_free": None,
    "pg_huffman_kv_cache_free": None,
    "pg_huffman_kv_cache_len": _sz,
    "pg_huffman_kv_cache_compressed_len": _sz,
    "pg_huffman_kv_cache_compress_threshold": _sz,
    "pg_huffman_kv_cache_num_chunks": _sz,
    "pg_mxfp4_expert_free": None,
    "pg_kv_cache_free": None,
    "pg_llama_block_free": None,
    "pg_kv_cache_len": _sz,
    "pg_fixed_scratch_bytes": _sz,
    "pg_kv_cache_capacity": _sz,
    "pg_ctx_stream": _vp,
    "pg_last_error": C.c_char_p,
    "pg_status_string": C.c_char_p,
}

for _name, _args in SIGNATURES.items():
    _fn = getattr(lib, _name)  # AttributeError here = header and library disagree
    _fn.argtypes = _args
    _fn.restype = _OTHER_RESTYPE.get(_name, _int)


class PeregrineError(RuntimeError):
    """A non-zero pg_status.  The reference panics in these places (assert!/expect)."""

    def __init__(self, status, message):
        super().__init__(f"[{lib.pg_status_string(status).decode()}] {message}")
        self.status = status


def check(status):
    if status != PG_OK:
        raise PeregrineError(status, lib.pg_last_error().decode())
