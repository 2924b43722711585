"""Host-side mirror of `peregrine::quant` (reference: src/quant.rs) over the HIP library.

Same names, argument meaning and error behaviour as the Rust functions; slices become
1-D/2-D NumPy arrays, `Vec` results are new arrays, and the reference's `assert!`
panics become `PeregrineError` / `ValueError`.
"""
import ctypes as C

import numpy as np

from . import _ffi
from .context import default_context


def _f32(a, n, what):
    a = np.ascontiguousarray(a, dtype=np.float32).reshape(-1)
    if a.size != n:  # assert_eq!(data.len(), rows * cols)  src/quant.rs:28,80,137
        raise ValueError(f"{what}: expected {n} elements, got {a.size}")
    return a


def _ptr(a):
    return C.c_void_p(a.ctypes.data) if a is not None and a.size else C.c_void_p(None)


class QuantizedTensor:
    """`quant::QuantizedTensor` (src/quant.rs:12-23): `data_i8[row*cols+col]`,
    `data_i8_t[col*rows+row]`, `scales[col]`, plus an optional device-resident copy."""

    def __init__(self, data_i8, data_i8_t, scales, rows, cols):
        self.data_i8, self.data_i8_t, self.scales = data_i8, data_i8_t, scales
        self.rows, self.cols = int(rows), int(cols)
        self._gpu = None  # pg_qtensor handle (gpu_data_i8 + gpu_scales of the reference)
        self._ctx = None

    # QuantizedTensor::to_gpu  src/quant.rs:174-181 (idempotent)
    def to_gpu(self, ctx=None):
        if self._gpu is None:
            ctx = ctx or default_context()
            h = C.c_void_p()
            _ffi.check(_ffi.lib.pg_qtensor_upload(ctx.handle, _ptr(self.data_i8), _ptr(self.scales),
                                                  self.rows, self.cols, C.byref(h)))
            self._gpu, self._ctx = h, ctx
        return self

    # QuantizedTensor::from_gpu  src/quant.rs:183-190
    def from_gpu(self, ctx=None):
        if self._gpu is not None:
            q = np.empty(self.rows * self.cols, np.int8)
            qt = np.empty(self.rows * self.cols, np.int8)
            s = np.empty(self.cols, np.float32)
            _ffi.check(_ffi.lib.pg_qtensor_download(self._ctx.handle, self._gpu, _ptr(q), _ptr(qt), _ptr(s)))
            self.data_i8, self.data_i8_t, self.scales = q, qt, s
        return self

    @property
    def on_gpu(self):
        return self._gpu is not None

    def free_gpu(self):
        if self._gpu is not None:
            _ffi.lib.pg_qtensor_free(self._ctx.handle, self._gpu)
            self._gpu = None

    def __del__(self):
        try:
            self.free_gpu()
        except Exception:
            pass


def quantize_weights(data, rows, cols, ctx=None):
    """`quant::quantize_weights(data, rows, cols)`  src/quant.rs:27-75."""
    ctx = ctx or default_context()
    w = _f32(data, rows * cols, "quantize_weights")
    q = np.empty(rows * cols, np.int8)
    qt = np.empty(rows * cols, np.int8)
    s = np.empty(cols, np.float32)
    _ffi.check(_ffi.lib.pg_quantize_weights(ctx.handle, _ptr(w), rows, cols, _ptr(q), _ptr(qt), _ptr(s)))
    return QuantizedTensor(q, qt, s, rows, cols)


def quantize_activations(data, rows, cols, ctx=None):
    """`quant::quantize_activations(data, rows, cols) -> (i8, row_scales)`  src/quant.rs:79-112."""
    ctx = ctx or default_context()
    a = _f32(data, rows * cols, "quantize_activations")
    q = np.empty(rows * cols, np.int8)
    s = np.empty(rows, np.float32)
    _ffi.check(_ffi.lib.pg_quantize_activations(ctx.handle, _ptr(a), rows, cols, _ptr(q), _ptr(s)))
    return q, s


def dequantize(qt, ctx=None):
    """`quant::dequantize(&QuantizedTensor)`  src/quant.rs:115-123."""
    ctx = ctx or default_context()
    out = np.empty(qt.rows * qt.cols, np.float32)
    _ffi.check(_ffi.lib.pg_dequantize(ctx.handle, _ptr(qt.data_i8), _ptr(qt.scales), qt.rows, qt.cols, _ptr(out)))
    return out


def matmul_quantized(a_data, m, k, w, ctx=None):
    """`quant::matmul_quantized(a, m, k, &w)`  src/quant.rs:129-169: W8A8 product
    C[M,N] = A_f32[M,K] @ W_i8[K,N] with per-row dynamic activation quantisation."""
    ctx = ctx or default_context()
    if w.rows != k:  # assert_eq!(w.rows, k)  src/quant.rs:135
        raise ValueError(f"matmul_quantized: w.rows = {w.rows} but k = {k}")
    a = _f32(a_data, m * k, "matmul_quantized")
    w.to_gpu(ctx)
    out = np.empty(m * w.cols, np.float32)
    _ffi.check(_ffi.lib.pg_matmul_quantized(ctx.handle, _ptr(a), m, k, w._gpu, _ptr(out)))
    return out


def matmul_quantized_gpu(ctx, a_data, m, k, w):
    """`quant::matmul_quantized_gpu(gpu, a, m, k, &w)`  src/quant.rs:196-218.  Like the
    reference it requires the weights to be uploaded first (`.expect("weights not on GPU")`)."""
    if not w.on_gpu:
        raise RuntimeError("weights not on GPU")
    return matmul_quantized(a_data, m, k, w, ctx)


def matmul_dequant_i8(a_data, m, k, w, ctx=None):
    """The reference's GPU numerics (W8A32) for `matmul_quantized_gpu`: f32 activations times
    dequantised weights, f32 accumulate (`dispatch_matmul_dequant_i8` src/metal/context.rs:2226-2306,
    shader src/metal/shaders.rs:2329-2375)."""
    ctx = ctx or default_context()
    if w.rows != k:  # assert_eq!(w.rows, k)  src/quant.rs:204
        raise ValueError(f"weight rows ({w.rows}) must equal k ({k})")
    a = _f32(a_data, m * k, "matmul_dequant_i8")
    w.to_gpu(ctx)
    out = np.empty(m * w.cols, np.float32)
    _ffi.check(_ffi.lib.pg_matmul_dequant_i8(ctx.handle, _ptr(a), m, k, w._gpu, _ptr(out)))
    return out
