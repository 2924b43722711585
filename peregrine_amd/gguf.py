"""Host-side mirror of the dequantisation half of `peregrine::gguf` (reference:
src/gguf.rs:284-401) and of the dequantise-then-matmul that `models::llama` builds from
it (src/models/llama/model.rs:243-257 + Tensor::matmul src/tensor.rs:1342-1353)."""
import ctypes as C

import numpy as np

from . import _ffi
from .context import default_context
from .quant import _ptr, QuantizedTensor, quantize_weights

Q4_0, Q4_1, Q8_0 = _ffi.GGML_Q4_0, _ffi.GGML_Q4_1, _ffi.GGML_Q8_0
BLOCK_BYTES = {Q4_0: 18, Q4_1: 20, Q8_0: 34}  # GgmlType::block_bytes  src/gguf.rs:47-55


def _blocks(data, num_elements, block_bytes, what):
    if num_elements % 32:  # assert!(num_elements % 32 == 0)  src/gguf.rs:287,308,332
        raise ValueError(f"{what}: num_elements {num_elements} is not a multiple of 32")
    buf = np.frombuffer(bytes(data) if not isinstance(data, np.ndarray) else data.tobytes(), np.uint8)
    need = num_elements // 32 * block_bytes
    if buf.size < need:  # assert!(data.len() >= num_blocks * block_size)
        raise ValueError(f"{what}: need {need} bytes, got {buf.size}")
    return np.ascontiguousarray(buf[:need])


def f16_to_f32(bits, ctx=None):
    """`gguf::f16_to_f32`  src/gguf.rs:354-382, vectorised over an array of u16 patterns."""
    ctx = ctx or default_context()
    b = np.ascontiguousarray(bits, dtype=np.uint16).reshape(-1)
    out = np.empty(b.size, np.float32)
    _ffi.check(_ffi.lib.pg_f16_to_f32(ctx.handle, _ptr(b), b.size, _ptr(out)))
    return out


def _dequant(fn, data, num_elements, bb, what, ctx):
    ctx = ctx or default_context()
    buf = _blocks(data, num_elements, bb, what)
    out = np.empty(num_elements, np.float32)
    _ffi.check(fn(ctx.handle, _ptr(buf), num_elements, _ptr(out)))
    return out


def dequant_q8_0(data, num_elements, ctx=None):
    """`gguf::dequant_q8_0(data, num_elements)`  src/gguf.rs:286-302."""
    return _dequant(_ffi.lib.pg_dequant_q8_0, data, num_elements, 34, "dequant_q8_0", ctx)


def dequant_q4_0(data, num_elements, ctx=None):
    """`gguf::dequant_q4_0(data, num_elements)`  src/gguf.rs:307-326."""
    return _dequant(_ffi.lib.pg_dequant_q4_0, data, num_elements, 18, "dequant_q4_0", ctx)


def dequant_q4_1(data, num_elements, ctx=None):
    """`gguf::dequant_q4_1(data, num_elements)`  src/gguf.rs:331-351."""
    return _dequant(_ffi.lib.pg_dequant_q4_1, data, num_elements, 20, "dequant_q4_1", ctx)


def load_tensor_q8_as_quantized(data, rows, cols, ctx=None):
    """`gguf::load_tensor_q8_as_quantized`  src/gguf.rs:386-401: Q8_0 -> f32 -> per-column
    `quantize_weights` (the reference re-quantises; so does this)."""
    if cols % 32:
        raise ValueError("load_tensor_q8_as_quantized: cols must be a multiple of 32")
    f32 = dequant_q8_0(data, rows * cols, ctx)
    return quantize_weights(f32, rows, cols, ctx)


class GgufWeight:
    """A GGUF block-quantised weight, [n_out, k_in] with blocks of 32 along k_in, kept
    quantised in HBM (what `load_transposed_weight` would have materialised as f32)."""

    def __init__(self, blocks, ggml_type, n_out, k_in, ctx=None):
        self.ctx = ctx or default_context()
        if ggml_type not in BLOCK_BYTES:
            raise ValueError(f"unsupported ggml type {ggml_type}")
        buf = _blocks(blocks, n_out * k_in, BLOCK_BYTES[ggml_type], "GgufWeight")
        self._h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_gguf_upload(self.ctx.handle, _ptr(buf), ggml_type, n_out, k_in, C.byref(self._h)))
        self.ggml_type, self.n_out, self.k_in = ggml_type, n_out, k_in

    def matmul(self, x, m):
        """y[m, n_out] = x[m, k_in] @ dequant(W)^T (x.matmul(&weight) in LlamaBlock::forward)."""
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        if x.size != m * self.k_in:
            raise ValueError(f"GgufWeight.matmul: expected {m * self.k_in} activations, got {x.size}")
        y = np.empty(m * self.n_out, np.float32)
        _ffi.check(_ffi.lib.pg_gguf_matmul(self.ctx.handle, _ptr(x), m, self._h, _ptr(y)))
        return y

    def free(self):
        if self._h:
            _ffi.lib.pg_gguf_free(self.ctx.handle, self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
