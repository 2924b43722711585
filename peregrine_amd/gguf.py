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

    def prepare(self, max_rows):
        """Make now the derived device copies that products over up to `max_rows` rows would otherwise make on
        their first call (the load-time step: afterwards those calls neither allocate nor wait)."""
        _ffi.check(_ffi.lib.pg_gguf_prepare(self.ctx.handle, self._h, max_rows))
        return self

    def drop_prepared(self):
        _ffi.check(_ffi.lib.pg_gguf_drop_prepared(self.ctx.handle, self._h))

    def device_bytes(self):
        """(bytes as uploaded, bytes of derived copies held now)."""
        up, der = C.c_size_t(), C.c_size_t()
        _ffi.check(_ffi.lib.pg_gguf_device_bytes(self._h, C.byref(up), C.byref(der)))
        return up.value, der.value

    def free(self):
        if self._h:
            _ffi.lib.pg_gguf_free(self.ctx.handle, self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    @classmethod
    def _from_handle(cls, handle, ctx):
        self = cls.__new__(cls)
        self.ctx, self._h = ctx, handle
        n_out, k_in, typ = C.c_size_t(), C.c_size_t(), C.c_int()
        _ffi.check(_ffi.lib.pg_gguf_shape(handle, C.byref(n_out), C.byref(k_in), C.byref(typ)))
        self.ggml_type, self.n_out, self.k_in = typ.value, n_out.value, k_in.value
        return self


F32, F16 = 0, 1  # GgmlType  src/gguf.rs:14-21


class GgufTensor:
    """`gguf::GgufTensor`  src/gguf.rs:143-164 (shape in GGUF order, innermost first)."""

    GEOMETRY = {0: (1, 4), 1: (1, 2), 2: (32, 18), 3: (32, 20), 8: (32, 34)}  # block_size, block_bytes  src/gguf.rs:36-56

    def __init__(self, name, dtype, shape, data_offset):
        self.name, self.dtype, self.shape, self.data_offset = name, dtype, shape, data_offset

    def num_elements(self):
        n = 1
        for d in self.shape:
            n *= d
        return n

    def data_size(self):
        n, (bs, bb) = self.num_elements(), self.GEOMETRY[self.dtype]
        if n % bs:  # assert!  src/gguf.rs:160
            raise ValueError(f"tensor elements {n} not divisible by block size {bs}")
        return n // bs * bb


class GgufFile:
    """`gguf::GgufFile`  src/gguf.rs:166-171, 403-561: header, metadata and tensor directory
    of a GGUF v2/v3 file.  `parse` keeps a reference to the buffer it is given; `load` maps
    the file.  A bad magic or version raises (the reference returns io::Error), as do the
    places where the reference panics."""

    def __init__(self, handle, keep=None):
        self._h, self._keep = handle, keep
        nt, nk, ver, ds = C.c_size_t(), C.c_size_t(), C.c_uint32(), C.c_uint64()
        _ffi.check(_ffi.lib.pg_gguf_file_counts(handle, C.byref(nt), C.byref(nk), C.byref(ver), C.byref(ds)))
        self.version, self.data_start, self.n_metadata = ver.value, ds.value, nk.value
        self.tensors = {}
        for i in range(nt.value):
            nm = C.c_char_p()
            _ffi.check(_ffi.lib.pg_gguf_file_tensor_name(handle, i, C.byref(nm)))
            typ, nd, off = C.c_int(), C.c_size_t(), C.c_uint64()
            shape = (C.c_uint64 * 8)()
            _ffi.check(_ffi.lib.pg_gguf_file_tensor_info(handle, nm.value, C.byref(typ), C.byref(nd), shape, 8,
                                                         C.byref(off), None, None))
            name = nm.value.decode()
            self.tensors[name] = GgufTensor(name, typ.value, [int(shape[d]) for d in range(nd.value)], off.value)

    @classmethod
    def parse(cls, data):
        """`GgufFile::parse(data)`  src/gguf.rs:411-483."""
        buf = np.frombuffer(bytes(data), np.uint8) if not isinstance(data, np.ndarray) else np.ascontiguousarray(data, np.uint8)
        h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_gguf_file_parse(_ptr(buf) if buf.size else None, buf.size, C.byref(h)))
        return cls(h, keep=buf)

    @classmethod
    def load(cls, path):
        """`GgufFile::load(path)`  src/gguf.rs:405-408."""
        h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_gguf_file_open(str(path).encode(), C.byref(h)))
        return cls(h)

    def close(self):
        if self._h:
            _ffi.lib.pg_gguf_file_close(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- metadata  src/gguf.rs:536-548
    def get_u32(self, key):
        v, found = C.c_uint32(), C.c_int()
        _ffi.check(_ffi.lib.pg_gguf_file_get_u32(self._h, key.encode(), C.byref(v), C.byref(found)))
        return v.value if found.value else None

    def get_f32(self, key):
        v, found = C.c_float(), C.c_int()
        _ffi.check(_ffi.lib.pg_gguf_file_get_f32(self._h, key.encode(), C.byref(v), C.byref(found)))
        return v.value if found.value else None

    def get_str(self, key):
        v, n = C.c_char_p(), C.c_size_t()
        _ffi.check(_ffi.lib.pg_gguf_file_get_str(self._h, key.encode(), C.byref(v), C.byref(n)))
        return None if v.value is None else C.string_at(v, n.value).decode()

    def get_array(self, key):
        """Array metadata as a Python list (strings or numbers), or None."""
        et, n = C.c_uint32(), C.c_size_t()
        _ffi.check(_ffi.lib.pg_gguf_file_get_array(self._h, key.encode(), C.byref(et), C.byref(n)))
        if n.value == C.c_size_t(-1).value:
            return None
        if et.value == 8:
            out = []
            for i in range(n.value):
                v = C.c_char_p()
                _ffi.check(_ffi.lib.pg_gguf_file_get_array_str(self._h, key.encode(), i, C.byref(v)))
                out.append(v.value.decode())
            return out
        vals = (C.c_double * max(1, n.value))()
        _ffi.check(_ffi.lib.pg_gguf_file_get_array_f64(self._h, key.encode(), vals, n.value))
        return [vals[i] if et.value in (6, 12) else int(vals[i]) for i in range(n.value)]

    # ---- tensors
    def tensor_names(self):
        """`GgufFile::tensor_names`  src/gguf.rs:559-561."""
        return list(self.tensors)

    def tensor_shape(self, name):
        """`GgufFile::tensor_shape`  src/gguf.rs:551-556: Peregrine order (GGUF's reversed)."""
        if name not in self.tensors:
            raise KeyError(f"tensor '{name}' not found")
        return list(reversed(self.tensors[name].shape))

    def load_tensor_f32(self, name, ctx=None):
        """`GgufFile::load_tensor_f32`  src/gguf.rs:485-517."""
        ctx = ctx or default_context()
        n = self.tensors[name].num_elements() if name in self.tensors else 0
        out = np.empty(n, np.float32)
        _ffi.check(_ffi.lib.pg_gguf_file_load_tensor_f32(ctx.handle, self._h, name.encode(), _ptr(out), n))
        return out

    def load_tensor_q8(self, name, ctx=None):
        """`GgufFile::load_tensor_q8`  src/gguf.rs:521-537: dequantise, then per-column
        `quantize_weights` with (rows, cols) = (shape[1], shape[0])."""
        info = self.tensors.get(name)
        if info is None:
            raise KeyError(f"tensor '{name}' not found in GGUF file")
        if len(info.shape) == 1:
            rows, cols = 1, info.shape[0]
        elif len(info.shape) == 2:
            rows, cols = info.shape[1], info.shape[0]
        else:
            raise ValueError(f"expected 1D or 2D tensor for q8 load, got {info.shape}")
        return quantize_weights(self.load_tensor_f32(name, ctx), rows, cols, ctx)

    def upload_tensor(self, name, ctx=None):
        """Keep a Q4_0 / Q8_0 tensor quantised on the device (no counterpart in the reference,
        which materialises f32: src/models/llama/model.rs:243-257)."""
        ctx = ctx or default_context()
        h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_gguf_file_upload_tensor(ctx.handle, self._h, name.encode(), C.byref(h)))
        return GgufWeight._from_handle(h, ctx)
