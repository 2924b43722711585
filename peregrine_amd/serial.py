"""Host-side mirror of the int8 wire record of `peregrine::serial` (reference:
src/serial.rs:124-222): `write_quantized_tensor(file, name, qt)` and
`read_quantized_tensor(file) -> (name, QuantizedTensor)` over binary streams."""
import ctypes as C
import struct

import numpy as np

from . import _ffi
from .quant import QuantizedTensor, _ptr


def write_quantized_tensor(file, name, qt):
    """`serial::write_quantized_tensor`  src/serial.rs:126-157."""
    nm = name.encode()
    q = np.ascontiguousarray(qt.data_i8, np.int8).reshape(-1)
    s = np.ascontiguousarray(qt.scales, np.float32).reshape(-1)
    if q.size != qt.rows * qt.cols or s.size != qt.cols:
        raise ValueError("write_quantized_tensor: data_i8 / scales do not match rows x cols")
    need = C.c_size_t()
    _ffi.check(_ffi.lib.pg_quantized_record_size(len(nm), qt.rows, qt.cols, C.byref(need)))
    buf = np.empty(need.value, np.uint8)
    wrote = C.c_size_t()
    _ffi.check(_ffi.lib.pg_write_quantized_tensor(_ptr(buf), buf.size, nm, len(nm), _ptr(q), _ptr(s), qt.rows, qt.cols,
                                                  C.byref(wrote)))
    file.write(buf[: wrote.value].tobytes())


def read_quantized_tensor(file):
    """`serial::read_quantized_tensor`  src/serial.rs:161-222 (including the transposed copy it
    rebuilds, src/serial.rs:202-208).  A short stream raises EOFError (the reference's
    read_exact error); a wrong dtype tag or ndim raises PeregrineError (its assert_eq!s)."""
    def exact(n):
        b = file.read(n)
        if len(b) != n:
            raise EOFError(f"read_quantized_tensor: wanted {n} bytes, got {len(b)}")
        return b

    head = exact(4)
    name_len = struct.unpack("<I", head)[0]
    head += exact(name_len + 13)
    rows, cols = struct.unpack("<II", head[-8:])
    dtype, ndim = head[4 + name_len], struct.unpack("<I", head[5 + name_len: 9 + name_len])[0]
    body = exact(rows * cols + 4 * cols) if dtype == 1 and ndim == 2 else b""
    rec = np.frombuffer(head + body, np.uint8)
    nm, nl, r, c = C.c_void_p(), C.c_size_t(), C.c_size_t(), C.c_size_t()
    q, sc, used = C.c_void_p(), C.c_void_p(), C.c_size_t()
    _ffi.check(_ffi.lib.pg_read_quantized_tensor(_ptr(rec), rec.size, C.byref(nm), C.byref(nl), C.byref(r), C.byref(c),
                                                 C.byref(q), C.byref(sc), C.byref(used)))
    base = rec.ctypes.data
    name = bytes(rec[nm.value - base: nm.value - base + nl.value]).decode()  # invalid UTF-8 raises, as in the reference
    data_i8 = rec[q.value - base: q.value - base + r.value * c.value].view(np.int8).copy()
    scales = np.frombuffer(bytes(rec[sc.value - base: sc.value - base + 4 * c.value]), np.float32).copy()
    data_i8_t = np.ascontiguousarray(data_i8.reshape(r.value, c.value).T).reshape(-1)
    return name, QuantizedTensor(data_i8, data_i8_t, scales, r.value, c.value)


def quantized_tensor_to_gpu(record, ctx=None):
    """Parse one record from a bytes-like object straight into a device-resident tensor
    (read_quantized_tensor + QuantizedTensor::to_gpu).  Returns (pg_qtensor handle, bytes consumed)."""
    from .context import default_context
    ctx = ctx or default_context()
    rec = np.frombuffer(bytes(record), np.uint8)
    h, used = C.c_void_p(), C.c_size_t()
    _ffi.check(_ffi.lib.pg_qtensor_from_record(ctx.handle, _ptr(rec), rec.size, C.byref(h), C.byref(used)))
    return h, used.value
