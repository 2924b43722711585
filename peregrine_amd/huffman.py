"""Host-side mirror of `peregrine::huffman` (src/huffman.rs): canonical Huffman coding of
int8 weights in front of the W8A8 product.  Table building and encoding are host code in
the library; decoding runs on the device."""
import ctypes as C

import numpy as np

from . import _ffi
from .context import default_context
from .quant import QuantizedTensor, _ptr

NUM_SYMBOLS = 256


class HuffmanTable:
    """`HuffmanTable` (src/huffman.rs:19-28): `bit_lengths[256]`, `codes[256]` (index =
    value + 128)."""

    def __init__(self, bit_lengths):
        self.bit_lengths = np.ascontiguousarray(bit_lengths, np.uint8).reshape(-1).copy()
        if self.bit_lengths.size != NUM_SYMBOLS:
            raise ValueError("codebook too short")  # src/huffman.rs:293
        self.codes = np.zeros(NUM_SYMBOLS, np.uint32)
        _ffi.check(_ffi.lib.pg_huffman_canonical_codes(_ptr(self.bit_lengths), _ptr(self.codes)))

    @classmethod
    def from_frequencies(cls, freqs):
        """src/huffman.rs:35-150."""
        f = np.ascontiguousarray(freqs, np.uint64).reshape(-1)
        if f.size != NUM_SYMBOLS:
            raise ValueError("from_frequencies: 256 frequencies expected")
        bl = np.zeros(NUM_SYMBOLS, np.uint8)
        _ffi.check(_ffi.lib.pg_huffman_table_from_frequencies(_ptr(f), _ptr(bl), None))
        return cls(bl)

    def to_bytes(self):
        return self.bit_lengths.tobytes()  # src/huffman.rs:287-289

    @classmethod
    def from_bytes(cls, data):
        if len(data) < NUM_SYMBOLS:
            raise ValueError("codebook too short")
        return cls(np.frombuffer(bytes(data[:NUM_SYMBOLS]), np.uint8))

    def encode(self, data):
        """src/huffman.rs:216-251 -> bytes."""
        d = np.ascontiguousarray(data, np.int8).reshape(-1)
        need = C.c_size_t()
        _ffi.check(_ffi.lib.pg_huffman_encode(_ptr(self.bit_lengths), _ptr(d), d.size, None, 0, C.byref(need)))
        out = np.zeros(need.value, np.uint8)
        _ffi.check(_ffi.lib.pg_huffman_encode(_ptr(self.bit_lengths), _ptr(d), d.size, _ptr(out), out.size, C.byref(need)))
        return out.tobytes()

    def decode(self, bitstream, num_symbols, ctx=None):
        """src/huffman.rs:254-284, on the device."""
        ctx = ctx or default_context()
        b = np.frombuffer(bytes(bitstream), np.uint8)
        out = np.empty(num_symbols, np.int8)
        _ffi.check(_ffi.lib.pg_huffman_decode(ctx.handle, _ptr(self.bit_lengths), _ptr(b), b.size, num_symbols, _ptr(out)))
        return out


class HuffmanTensor:
    """`HuffmanTensor` (src/huffman.rs:311-325)."""

    def __init__(self, handle):
        self._h = handle
        r, c, n, z = C.c_size_t(), C.c_size_t(), C.c_size_t(), C.c_size_t()
        _ffi.check(_ffi.lib.pg_huffman_tensor_info(handle, C.byref(r), C.byref(c), C.byref(n), C.byref(z)))
        self.rows, self.cols, self.num_streams, self._compressed = r.value, c.value, n.value, z.value
        bl, sc = C.c_void_p(), C.c_void_p()
        _ffi.check(_ffi.lib.pg_huffman_tensor_table(handle, C.byref(bl), C.byref(sc)))
        self.table = HuffmanTable(np.ctypeslib.as_array(C.cast(bl, C.POINTER(C.c_uint8)), (NUM_SYMBOLS,)))
        self.scales = np.ctypeslib.as_array(C.cast(sc, C.POINTER(C.c_float)), (self.cols,)).copy() if self.cols else np.zeros(0, np.float32)
        self.streams, self.stream_lengths = [], []
        for s in range(self.num_streams):
            d, nb, ns = C.c_void_p(), C.c_size_t(), C.c_size_t()
            _ffi.check(_ffi.lib.pg_huffman_tensor_stream(handle, s, C.byref(d), C.byref(nb), C.byref(ns)))
            self.streams.append(C.string_at(d, nb.value) if nb.value else b"")
            self.stream_lengths.append(ns.value)

    @classmethod
    def from_quantized(cls, qt, num_streams):
        """src/huffman.rs:332-372."""
        q = np.ascontiguousarray(qt.data_i8, np.int8).reshape(-1)
        s = np.ascontiguousarray(qt.scales, np.float32).reshape(-1)
        if q.size != qt.rows * qt.cols or s.size != qt.cols:
            raise ValueError("HuffmanTensor.from_quantized: tensor fields do not match rows x cols")
        h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_huffman_tensor_from_quantized(_ptr(q), _ptr(s), qt.rows, qt.cols, int(num_streams), C.byref(h)))
        return cls(h)

    @classmethod
    def from_parts(cls, table, streams, stream_lengths, scales, rows, cols):
        """The struct literal that serial::read_huffman_tensor builds (src/serial.rs:433-445)."""
        n = len(streams)
        bufs = [np.frombuffer(bytes(s), np.uint8) for s in streams]
        ptrs = (C.c_void_p * max(n, 1))(*[b.ctypes.data if b.size else None for b in bufs])
        nbytes = (C.c_size_t * max(n, 1))(*[b.size for b in bufs])
        nsyms = (C.c_size_t * max(n, 1))(*[int(v) for v in stream_lengths])
        sc = np.ascontiguousarray(scales, np.float32).reshape(-1)
        if sc.size != cols or len(stream_lengths) != n:
            raise ValueError("HuffmanTensor.from_parts: field lengths")
        h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_huffman_tensor_from_parts(_ptr(table.bit_lengths), C.cast(ptrs, C.POINTER(C.c_void_p)), nbytes, nsyms, n,
                                                         _ptr(sc), rows, cols, C.byref(h)))
        return cls(h)

    def decode_to_quantized(self, ctx=None):
        """src/huffman.rs:374-404, decoding on the device."""
        ctx = ctx or default_context()
        n = self.rows * self.cols
        q, qt, s = np.empty(n, np.int8), np.empty(n, np.int8), np.empty(self.cols, np.float32)
        _ffi.check(_ffi.lib.pg_huffman_tensor_decode_to_quantized(ctx.handle, self._h, _ptr(q), _ptr(qt), _ptr(s)))
        return QuantizedTensor(q, qt, s, self.rows, self.cols)

    def to_gpu(self, ctx=None):
        """src/huffman.rs:430-435: a QuantizedTensor whose device copy is already in place."""
        ctx = ctx or default_context()
        h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_huffman_tensor_to_gpu(ctx.handle, self._h, C.byref(h)))
        qt = QuantizedTensor(None, None, self.scales.copy(), self.rows, self.cols)
        qt._gpu, qt._ctx = h, ctx
        return qt

    def compressed_size(self):
        return self._compressed  # src/huffman.rs:407-412

    def uncompressed_size(self):
        return self.rows * self.cols + self.cols * 4  # src/huffman.rs:415-417

    def compression_ratio(self):
        return self.uncompressed_size() / self.compressed_size()  # src/huffman.rs:420-422

    def free(self):
        if self._h:
            _ffi.lib.pg_huffman_tensor_free(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def matmul_huffman(a_data, m, k, ht, ctx=None):
    """`huffman::matmul_huffman(a, m, k, &ht)`  src/huffman.rs:465-474."""
    ctx = ctx or default_context()
    if ht.rows != k:  # assert_eq!(ht.rows, k)
        raise ValueError(f"matmul_huffman: ht.rows = {ht.rows} but k = {k}")
    a = np.ascontiguousarray(a_data, np.float32).reshape(-1)
    if a.size != m * k:
        raise ValueError("matmul_huffman: a is not [m, k]")
    out = np.empty(m * ht.cols, np.float32)
    _ffi.check(_ffi.lib.pg_matmul_huffman(ctx.handle, _ptr(a), m, k, ht._h, _ptr(out)))
    return out


class CompressedChunk:
    """`CompressedChunk` (src/huffman.rs:500-513).  The bitstream lives in device memory; the
    `bitstream`, `scales` and `codebook` properties copy it out."""

    def __init__(self, handle, ctx, owned=True):
        self._h, self.ctx, self._owned = handle, ctx, owned
        t, h, d, b = C.c_size_t(), C.c_size_t(), C.c_size_t(), C.c_size_t()
        _ffi.check(_ffi.lib.pg_huffman_kv_chunk_info(handle, C.byref(t), C.byref(h), C.byref(d), C.byref(b)))
        self.num_tokens, self.num_heads, self.head_dim, self._bytes = t.value, h.value, d.value, b.value

    @classmethod
    def from_parts(cls, bitstream, scales, codebook, num_tokens, num_heads, head_dim, ctx=None):
        ctx = ctx or default_context()
        b = np.frombuffer(bytes(bitstream), np.uint8)
        s = np.ascontiguousarray(scales, np.float32).reshape(-1)
        cb = np.frombuffer(bytes(codebook), np.uint8)
        if s.size != num_heads or cb.size < NUM_SYMBOLS:
            raise ValueError("CompressedChunk.from_parts: field lengths")
        h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_huffman_kv_chunk_from_parts(ctx.handle, _ptr(b) if b.size else None, b.size, _ptr(s) if s.size else None,
                                                           _ptr(cb), num_tokens, num_heads, head_dim, C.byref(h)))
        return cls(h, ctx)

    def _parts(self):
        b, s, cb = np.zeros(self._bytes, np.uint8), np.zeros(self.num_heads, np.float32), np.zeros(NUM_SYMBOLS, np.uint8)
        _ffi.check(_ffi.lib.pg_huffman_kv_chunk_parts(self.ctx.handle, self._h, _ptr(b) if b.size else None,
                                                      _ptr(s) if s.size else None, _ptr(cb)))
        return b.tobytes(), s, cb.tobytes()

    bitstream = property(lambda self: self._parts()[0])
    scales = property(lambda self: self._parts()[1])
    codebook = property(lambda self: self._parts()[2])

    def free(self):
        if self._h and self._owned:
            _ffi.lib.pg_huffman_kv_chunk_free(self.ctx.handle, self._h)
        self._h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class HuffmanKVCache:
    """`HuffmanKVCache` (src/huffman.rs:484-724): a window of recent tokens as f32 in a device
    StandardKVCache, older tokens as int8 + Huffman chunks in device memory."""

    def __init__(self, num_kv_heads, head_dim, compress_threshold, chunk_size, ctx=None):
        self.ctx = ctx or default_context()
        self.num_kv_heads, self.head_dim, self.chunk_size = int(num_kv_heads), int(head_dim), int(chunk_size)
        self._h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_huffman_kv_cache_create(self.ctx.handle, self.num_kv_heads, self.head_dim, int(compress_threshold),
                                                       self.chunk_size, C.byref(self._h)))

    new = classmethod(lambda cls, *a, **k: cls(*a, **k))

    def append(self, new_k, new_v, seq_len):
        """src/huffman.rs:544-556."""
        k = np.ascontiguousarray(new_k, np.float32).reshape(-1)
        v = np.ascontiguousarray(new_v, np.float32).reshape(-1)
        n = self.num_kv_heads * int(seq_len) * self.head_dim
        if k.size != n or v.size != n:
            raise ValueError("HuffmanKVCache.append: new_k / new_v are not [num_kv_heads, seq_len, head_dim]")
        _ffi.check(_ffi.lib.pg_huffman_kv_cache_append(self.ctx.handle, self._h, _ptr(k) if n else None, _ptr(v) if n else None, int(seq_len)))

    @staticmethod
    def compress_chunk(data, num_tokens, num_heads, head_dim, ctx=None):
        """src/huffman.rs:612-658."""
        ctx = ctx or default_context()
        d = np.ascontiguousarray(data, np.float32).reshape(-1)
        if d.size != num_heads * num_tokens * head_dim:  # assert_eq!(data.len(), total)
            raise ValueError("compress_chunk: data is not [num_heads, num_tokens, head_dim]")
        h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_huffman_kv_compress_chunk(ctx.handle, _ptr(d) if d.size else None, num_tokens, num_heads, head_dim, C.byref(h)))
        return CompressedChunk(h, ctx)

    @staticmethod
    def decompress_chunk(chunk):
        """src/huffman.rs:661-680."""
        out = np.zeros(chunk.num_heads * chunk.num_tokens * chunk.head_dim, np.float32)
        _ffi.check(_ffi.lib.pg_huffman_kv_decompress_chunk(chunk.ctx.handle, chunk._h, _ptr(out) if out.size else None))
        return out

    def len(self):
        return int(_ffi.lib.pg_huffman_kv_cache_len(self._h))  # src/huffman.rs:683-685

    __len__ = len

    @property
    def compressed_len(self):
        return int(_ffi.lib.pg_huffman_kv_cache_compressed_len(self._h))

    @property
    def compress_threshold(self):
        return int(_ffi.lib.pg_huffman_kv_cache_compress_threshold(self._h))

    @property
    def hot_len(self):
        h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_huffman_kv_cache_hot(self._h, C.byref(h)))
        return int(_ffi.lib.pg_kv_cache_len(h))

    def _chunks(self, value_side):
        out = []
        for i in range(int(_ffi.lib.pg_huffman_kv_cache_num_chunks(self._h))):
            h = C.c_void_p()
            _ffi.check(_ffi.lib.pg_huffman_kv_cache_chunk(self._h, value_side, i, C.byref(h)))
            out.append(CompressedChunk(h, self.ctx, owned=False))
        return out

    k_chunks = property(lambda self: self._chunks(0))
    v_chunks = property(lambda self: self._chunks(1))

    def get_kv(self):
        """src/huffman.rs:689-724: (k, v), each [num_kv_heads * len() * head_dim]."""
        n = self.num_kv_heads * self.len() * self.head_dim
        k, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
        _ffi.check(_ffi.lib.pg_huffman_kv_cache_get_kv(self.ctx.handle, self._h, _ptr(k) if n else None, _ptr(v) if n else None))
        return k, v

    def free(self):
        if self._h:
            _ffi.lib.pg_huffman_kv_cache_free(self.ctx.handle, self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
