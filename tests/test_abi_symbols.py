"""The C-ABI library loads without a GPU and exports every symbol include/peregrine_hip.h
declares (no compute calls here)."""
import ctypes as C
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "peregrine_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pg_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for must in ("pg_ctx_create", "pg_quantize_weights", "pg_quantize_activations", "pg_dequantize",
                 "pg_matmul_quantized", "pg_matmul_quantized_dev", "pg_qtensor_upload",
                 "pg_dequant_q8_0", "pg_dequant_q4_0", "pg_f16_to_f32", "pg_gguf_upload",
                 "pg_gguf_matmul", "pg_gguf_matmul_dev", "pg_moe_ffn", "pg_moe_ffn_dev"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from peregrine_amd import _ffi

    lib = C.CDLL(_ffi.LIB_PATH)
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, f"declared in the header but not exported: {missing}"
    # and the Python binding table covers the same set
    assert sorted(_ffi.SIGNATURES) == declared_symbols()


def test_status_strings_and_argument_errors_need_no_gpu():
    from peregrine_amd import _ffi

    assert _ffi.lib.pg_status_string(0) == b"ok"
    assert _ffi.lib.pg_status_string(1) == b"invalid argument"
    # shape query on a null handle is an argument error, not a crash
    assert _ffi.lib.pg_qtensor_shape(None, None, None) == _ffi.PG_EINVAL
    assert b"null" in _ffi.lib.pg_last_error()


def test_host_mirror_shape_checks_raise_before_any_device_work():
    import numpy as np
    import pytest
    from peregrine_amd import quant, gguf

    with pytest.raises(ValueError):
        quant._f32(np.zeros(5, np.float32), 6, "x")  # assert_eq!(data.len(), rows*cols)
    with pytest.raises(ValueError):
        gguf._blocks(bytes(18), 31, 18, "dequant_q4_0")  # num_elements % 32
    with pytest.raises(ValueError):
        gguf._blocks(bytes(17), 32, 18, "dequant_q4_0")  # short buffer
