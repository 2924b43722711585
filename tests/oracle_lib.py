"""ctypes/NumPy front end of the CPU oracle (oracle/peregrine_oracle.c).  Test infrastructure:
only tests, the smoke check and the benchmark's cpu_baseline leg import this."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SO = os.path.join(ROOT, "oracle", "_build", "libperegrine_oracle.so")


def _load():
    if not os.path.exists(SO):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")], stdout=subprocess.DEVNULL)
    return C.CDLL(SO)


lib = _load()
_vp, _sz = C.c_void_p, C.c_size_t
lib.orc_f16_to_f32_bits.restype = C.c_uint32
lib.orc_f16_to_f32_bits.argtypes = [C.c_uint16]
lib.orc_rng_next_u64.restype = C.c_uint64
lib.orc_rng_next_u64.argtypes = [_vp]
lib.orc_rng_seed.argtypes = [_vp, C.c_uint64]
lib.orc_rng_normal.argtypes = [C.c_uint64, _sz, C.c_float, C.c_float, _vp]
lib.orc_philox_4x32_10.argtypes = [_vp, _vp, _vp]
lib.orc_philox_4x32_10.restype = None
lib.orc_random_seed.argtypes = [_vp, C.c_uint64]
lib.orc_random_seed.restype = None
lib.orc_random_normal.argtypes = [_vp, _sz, C.c_float, C.c_float, _vp]
lib.orc_random_normal.restype = None
for _n in ("orc_quantize_weights", "orc_quantize_activations", "orc_dequantize", "orc_gemm_i8",
           "orc_matmul_f32", "orc_softmax_rows", "orc_silu", "orc_gelu_tanh", "orc_swiglu_llama"):
    getattr(lib, _n).restype = None


class _KeptPtr(C.c_void_p):
    """A void pointer that keeps the array it points into alive for as long as it lives."""


def _p(a):
    if a is None:
        return C.c_void_p(None)
    p = _KeptPtr(a.ctypes.data)
    p._keep = a
    return p


def _f32(a):
    return np.ascontiguousarray(a, np.float32)


def quantize_weights(w, rows, cols):
    w = _f32(w).reshape(-1)
    q = np.empty(rows * cols, np.int8)
    qt = np.empty(rows * cols, np.int8)
    s = np.empty(cols, np.float32)
    lib.orc_quantize_weights(_p(w), _sz(rows), _sz(cols), _p(q), _p(qt), _p(s))
    return q, qt, s


def quantize_activations(a, rows, cols):
    a = _f32(a).reshape(-1)
    q = np.empty(rows * cols, np.int8)
    s = np.empty(rows, np.float32)
    lib.orc_quantize_activations(_p(a), _sz(rows), _sz(cols), _p(q), _p(s))
    return q, s


def dequantize(q, scales, rows, cols):
    out = np.empty(rows * cols, np.float32)
    lib.orc_dequantize(_p(np.ascontiguousarray(q, np.int8)), _p(_f32(scales)), _sz(rows), _sz(cols), _p(out))
    return out


def gemm_i8(a_i8, a_scales, b_t, w_scales, m, n, k):
    out = np.empty(m * n, np.float32)
    acc = np.empty(m * n, np.int32)
    lib.orc_gemm_i8(_p(np.ascontiguousarray(a_i8, np.int8)), _p(_f32(a_scales)),
                    _p(np.ascontiguousarray(b_t, np.int8)), _p(_f32(w_scales)),
                    _sz(m), _sz(n), _sz(k), _p(out), _p(acc))
    return out, acc


def matmul_quantized(a, m, k, q_t, w_scales, n):
    a = _f32(a).reshape(-1)
    out = np.empty(m * n, np.float32)
    acc = np.empty(m * n, np.int32)
    rc = lib.orc_matmul_quantized(_p(a), _sz(m), _sz(k), _p(np.ascontiguousarray(q_t, np.int8)),
                                  _p(_f32(w_scales)), _sz(n), _p(out), _p(acc))
    assert rc == 0
    return out, acc


def matmul_dequant_i8(a, m, k, q, w_scales, n):
    out = np.empty(m * n, np.float32)
    lib.orc_matmul_dequant_i8(_p(_f32(a).reshape(-1)), _sz(m), _sz(k), _p(np.ascontiguousarray(q, np.int8)),
                              _p(_f32(w_scales)), _sz(n), _p(out))
    return out


def f16_to_f32_bits(bits):
    return np.array([lib.orc_f16_to_f32_bits(int(b)) for b in np.asarray(bits).reshape(-1)], np.uint32)


def _dequant(fn, data, n):
    buf = np.frombuffer(bytes(data), np.uint8).copy()
    out = np.empty(n, np.float32)
    rc = fn(_p(buf), _sz(n), _p(out))
    if rc != 0:
        raise ValueError("num_elements must be a multiple of 32")
    return out


def dequant_q8_0(data, n):
    return _dequant(lib.orc_dequant_q8_0, data, n)


def dequant_q4_0(data, n):
    return _dequant(lib.orc_dequant_q4_0, data, n)


def dequant_q4_1(data, n):
    return _dequant(lib.orc_dequant_q4_1, data, n)


def matmul_f32(a, b, m, k, n):
    out = np.empty(m * n, np.float32)
    lib.orc_matmul_f32(_p(_f32(a).reshape(-1)), _p(_f32(b).reshape(-1)), _sz(m), _sz(k), _sz(n), _p(out))
    return out


def gguf_matmul(x, m, blocks, ggml_type, n_out, k_in):
    buf = np.frombuffer(bytes(blocks), np.uint8).copy()
    y = np.empty(m * n_out, np.float32)
    rc = lib.orc_gguf_matmul(_p(_f32(x).reshape(-1)), _sz(m), _p(buf), C.c_int(ggml_type), _sz(n_out), _sz(k_in), _p(y))
    assert rc == 0, rc
    return y


def softmax_rows(x, rows, cols):
    out = np.empty(rows * cols, np.float32)
    lib.orc_softmax_rows(_p(_f32(x).reshape(-1)), _sz(rows), _sz(cols), _p(out))
    return out


def unary(name, x):
    x = _f32(x).reshape(-1)
    out = np.empty_like(x)
    getattr(lib, name)(_p(x), _sz(x.size), _p(out))
    return out


def moe_ffn(x, T, d, ffn, E, top_k, logits, gate, up, down, ggml_type, act):
    """gate/up/down: lists of E raw block byte strings."""
    keep = [np.frombuffer(bytes(b), np.uint8).copy() for b in list(gate) + list(up) + list(down)]
    mk = lambda arrs: (C.c_void_p * E)(*[a.ctypes.data for a in arrs])
    g, u, dn = mk(keep[:E]), mk(keep[E:2 * E]), mk(keep[2 * E:])
    out = np.empty(T * d, np.float32)
    idx = np.empty(T * top_k, np.int32)
    prob = np.empty(T * top_k, np.float32)
    rc = lib.orc_moe_ffn(_p(_f32(x).reshape(-1)), _sz(T), _sz(d), _sz(ffn), _sz(E), _sz(top_k),
                         _p(_f32(logits).reshape(-1)), g, u, dn, C.c_int(ggml_type), C.c_int(act),
                         _p(out), _p(idx), _p(prob))
    assert rc == 0, rc
    return out.reshape(T, d), idx.reshape(T, top_k), prob.reshape(T, top_k)


def deepseek_gate(x, T, dim, w, bias, E, topk, n_groups, topk_groups, route_scale, use_sigmoid):
    """Gate::forward (examples/deepseek/moe.rs:111-215): (expert indices [T, topk], weights [T, topk])."""
    idx = np.empty(T * topk, np.int32)
    wt = np.empty(T * topk, np.float32)
    b = None if bias is None else _f32(bias).reshape(-1)
    rc = lib.orc_deepseek_gate(_p(_f32(x).reshape(-1)), _sz(T), _sz(dim), _p(_f32(w).reshape(-1)), _p(b) if b is not None else None,
                               _sz(E), _sz(topk), _sz(n_groups), _sz(topk_groups), C.c_float(route_scale), C.c_int(int(use_sigmoid)),
                               _p(idx), _p(wt))
    assert rc == 0, rc
    return idx.reshape(T, topk), wt.reshape(T, topk)


def gpt_oss_route(logits, gate_bias, T, E, topk):
    """The gpt_oss router (examples/gpt_oss/moe.rs:298-330): top-k on logits + bias, softmax over the k."""
    idx = np.empty(T * topk, np.int32)
    wt = np.empty(T * topk, np.float32)
    rc = lib.orc_gpt_oss_route(_p(_f32(logits).reshape(-1)), _p(_f32(gate_bias).reshape(-1)), _sz(T), _sz(E), _sz(topk), _p(idx), _p(wt))
    assert rc == 0, rc
    return idx.reshape(T, topk), wt.reshape(T, topk)


def moe_ffn_routed(x, T, d, ffn, E, top_k, idx, weight, gate, up, down, ggml_type, act, shared=None):
    """The expert FFN over a given routing, plus the shared experts' output if passed."""
    keep = [np.frombuffer(bytes(b), np.uint8).copy() for b in list(gate) + list(up) + list(down)]
    mk = lambda arrs: (C.c_void_p * E)(*[a.ctypes.data for a in arrs])
    g, u, dn = mk(keep[:E]), mk(keep[E:2 * E]), mk(keep[2 * E:])
    out = np.empty(T * d, np.float32)
    ii = np.ascontiguousarray(idx, np.int32).reshape(-1)
    ww = _f32(weight).reshape(-1)
    sh = None if shared is None else _f32(shared).reshape(-1)
    rc = lib.orc_moe_ffn_routed(_p(_f32(x).reshape(-1)), _sz(T), _sz(d), _sz(ffn), _sz(E), _sz(top_k), _p(ii), _p(ww),
                                g, u, dn, C.c_int(ggml_type), C.c_int(act), _p(sh) if sh is not None else None, _p(out))
    assert rc == 0, rc
    return out.reshape(T, d)


def philox_4x32_10(counter, key):
    """orc_philox_4x32_10 on one (counter[4], key[2]); returns the four u32 outputs."""
    c = (C.c_uint32 * 4)(*counter)
    k = (C.c_uint32 * 2)(*key)
    o = (C.c_uint32 * 4)()
    lib.orc_philox_4x32_10(c, k, o)
    return list(o)


class Random:
    """The oracle's restatement of random::seed / random::normal (both generators)."""

    def __init__(self, seed):
        self._st = (C.c_uint64 * 5)()
        lib.orc_random_seed(self._st, C.c_uint64(seed))

    def normal(self, n, mean=0.0, std=1.0):
        out = np.empty(n, np.float32)
        lib.orc_random_normal(self._st, _sz(n), C.c_float(mean), C.c_float(std), _p(out))
        return out

    def next_u64(self):
        return lib.orc_rng_next_u64(self._st)


def rng_normal(seed, n, mean=0.0, std=1.0):
    out = np.empty(n, np.float32)
    lib.orc_rng_normal(C.c_uint64(seed), _sz(n), C.c_float(mean), C.c_float(std), _p(out))
    return out


# ---- Llama block glue (oracle/peregrine_oracle_llama.c) ----
for _n in ("orc_rmsnorm", "orc_rope_tables", "orc_rope_apply", "orc_gqa_attention", "orc_gqa_attention_local_global"):
    getattr(lib, _n).restype = None


def rmsnorm(x, rows, dim, w, eps):
    out = np.empty(rows * dim, np.float32)
    lib.orc_rmsnorm(_p(_f32(x).reshape(-1)), _sz(rows), _sz(dim), _p(_f32(w)), C.c_float(eps), _p(out))
    return out


def rope_tables(head_dim, max_seq_len, base):
    cos = np.empty((max_seq_len, head_dim), np.float32)
    sin = np.empty((max_seq_len, head_dim), np.float32)
    lib.orc_rope_tables(_sz(head_dim), _sz(max_seq_len), C.c_float(base), _p(cos), _p(sin))
    return cos, sin


def rope_apply(x, seq_len, head_dim, offset, cos, sin):
    out = np.empty(seq_len * head_dim, np.float32)
    lib.orc_rope_apply(_p(_f32(x).reshape(-1)), _sz(seq_len), _sz(head_dim), _sz(offset), _p(cos), _p(sin), _p(out))
    return out


def gqa_attention(q, k, v, length, capacity, nqh, nkvh, seq_q, hd, scale, mask_kind=0, offset=0, window=0, sink=0,
                  logit_cap=0.0):
    """q [nqh, seq_q, hd]; k, v [nkvh, capacity, hd]; returns [seq_q, nqh*hd]."""
    out = np.zeros(seq_q * nqh * hd, np.float32)
    lib.orc_gqa_attention(_p(_f32(q).reshape(-1)), _p(_f32(k).reshape(-1)), _p(_f32(v).reshape(-1)), _sz(length),
                          _sz(capacity), _sz(nqh), _sz(nkvh), _sz(seq_q), _sz(hd), C.c_float(scale), C.c_int(mask_kind),
                          _sz(offset), _sz(window), _sz(sink), C.c_float(logit_cap), _p(out))
    return out


def gqa_attention_local_global(q, k, v, length, capacity, nqh, nkvh, seq_q, hd, scale, offset, local_window,
                               global_positions, logit_cap=0.0):
    """AttentionMask::LocalGlobal; shapes as gqa_attention."""
    out = np.zeros(seq_q * nqh * hd, np.float32)
    gp = np.asarray(list(global_positions), np.uint64)
    lib.orc_gqa_attention_local_global(_p(_f32(q).reshape(-1)), _p(_f32(k).reshape(-1)), _p(_f32(v).reshape(-1)),
                                       _sz(length), _sz(capacity), _sz(nqh), _sz(nkvh), _sz(seq_q), _sz(hd),
                                       C.c_float(scale), _sz(offset), _sz(local_window), _p(gp), _sz(gp.size),
                                       C.c_float(logit_cap), _p(out))
    return out


def llama_block_forward(h, seq, d, nqh, nkvh, hd, ffn, ggml_type, weights, attn_norm_w, ffn_norm_w, eps, cos, sin,
                        k_cache, v_cache, cache_len, capacity):
    """weights: 7 raw block byte strings (q, k, v, o, gate, up, down).  k_cache / v_cache are
    updated in place ([nkvh, capacity, hd] float32 arrays).  Returns out [seq, d]."""
    keep = [np.frombuffer(bytes(b), np.uint8).copy() for b in weights]
    out = np.empty(seq * d, np.float32)
    types = np.asarray([ggml_type] * 7 if np.isscalar(ggml_type) else ggml_type, np.int32)   # one type, or one per projection
    rc = lib.orc_llama_block_forward_types(_p(_f32(h).reshape(-1)), _sz(seq), _sz(d), _sz(nqh), _sz(nkvh), _sz(hd), _sz(ffn),
                                     _p(types), *[_p(a) for a in keep], _p(_f32(attn_norm_w)),
                                     _p(_f32(ffn_norm_w)), C.c_float(eps), _p(cos), _p(sin), _p(k_cache), _p(v_cache),
                                     _sz(cache_len), _sz(capacity), _p(out))
    assert rc == 0, rc
    return out.reshape(seq, d)


# ---- sibling formats (oracle/peregrine_oracle_formats.c) ----
lib.orc_mxfp4_matmul.restype = None


def _u8(b):
    return np.frombuffer(bytes(b), np.uint8).copy() if not isinstance(b, np.ndarray) else np.ascontiguousarray(b, np.uint8).reshape(-1)


def mxfp4_matmul(x, blocks, scales, out_dim, in_dim):
    blocks, scales = _u8(blocks), _u8(scales)
    assert blocks.size == out_dim * in_dim // 2 and scales.size == out_dim * in_dim // 32
    out = np.empty(out_dim, np.float32)
    lib.orc_mxfp4_matmul(_p(_f32(x).reshape(-1)), _p(blocks), _p(scales), _sz(out_dim), _sz(in_dim), _p(out))
    return out


def mxfp4_expert_forward(x, hidden, intermediate, alpha, clamp, b1, s1, b2, s2, bias1, bias2):
    out = np.empty(hidden, np.float32)
    rc = lib.orc_mxfp4_expert_forward(_p(_f32(x).reshape(-1)), _sz(hidden), _sz(intermediate), C.c_float(alpha),
                                      C.c_float(clamp), _p(_u8(b1)), _p(_u8(s1)), _p(_u8(b2)), _p(_u8(s2)),
                                      _p(_f32(bias1)), _p(_f32(bias2)), _p(out))
    assert rc == 0
    return out


def mxfp4_moe_routed(x, T, hidden, intermediate, alpha, clamp, top_k, idx, weight, experts):
    """experts: list of (mlp1_blocks, mlp1_scales, mlp2_blocks, mlp2_scales, mlp1_bias, mlp2_bias)."""
    E = len(experts)
    cols = [[_u8(ex[j]) if j < 4 else _f32(ex[j]) for ex in experts] for j in range(6)]
    tabs = [(C.c_void_p * E)(*[a.ctypes.data for a in col]) for col in cols]
    out = np.empty(T * hidden, np.float32)
    rc = lib.orc_mxfp4_moe_routed(_p(_f32(x).reshape(-1)), _sz(T), _sz(hidden), _sz(intermediate), C.c_float(alpha), C.c_float(clamp),
                                  _sz(E), _sz(top_k), _p(np.ascontiguousarray(idx, np.int32).reshape(-1)), _p(_f32(weight).reshape(-1)),
                                  *tabs, _p(out))
    assert rc == 0, rc
    return out.reshape(T, hidden)


lib.orc_huffman_table.restype = None
lib.orc_huffman_canonical_codes.restype = None
lib.orc_huffman_encode.restype = C.c_size_t


def huffman_table(freqs):
    """(bit_lengths[256] u8, codes[256] u32) from 256 frequencies."""
    f = np.ascontiguousarray(freqs, np.uint64)
    bl, codes = np.zeros(256, np.uint8), np.zeros(256, np.uint32)
    lib.orc_huffman_table(_p(f), _p(bl), _p(codes))
    return bl, codes


def huffman_codes(bl):
    bl = np.ascontiguousarray(bl, np.uint8)
    codes = np.zeros(256, np.uint32)
    lib.orc_huffman_canonical_codes(_p(bl), _p(codes))
    return codes


def huffman_encode(bl, data):
    bl = np.ascontiguousarray(bl, np.uint8)
    codes = huffman_codes(bl)
    d = np.ascontiguousarray(data, np.int8).reshape(-1)
    n = lib.orc_huffman_encode(_p(bl), _p(codes), _p(d), _sz(d.size), None)
    out = np.zeros(n, np.uint8)
    lib.orc_huffman_encode(_p(bl), _p(codes), _p(d), _sz(d.size), _p(out))
    return out.tobytes()


def huffman_decode(bl, stream, num_symbols):
    bl = np.ascontiguousarray(bl, np.uint8)
    b = np.frombuffer(bytes(stream), np.uint8)
    out = np.empty(num_symbols, np.int8)
    rc = lib.orc_huffman_decode(_p(bl), _p(b), _sz(b.size), _sz(num_symbols), _p(out))
    assert rc == 0, "a code does not fit the 12-bit table"
    return out


lib.orc_huffman_kv_compress_chunk.restype = C.c_size_t
lib.orc_huffman_kv_new.restype = _vp
lib.orc_huffman_kv_new.argtypes = [_sz, _sz, _sz, _sz]
lib.orc_huffman_kv_free.restype = None
lib.orc_huffman_kv_free.argtypes = [_vp]
lib.orc_huffman_kv_append.restype = None
lib.orc_huffman_kv_append.argtypes = [_vp, _vp, _vp, _sz]
lib.orc_huffman_kv_stat.restype = C.c_size_t
lib.orc_huffman_kv_stat.argtypes = [_vp, C.c_int]
lib.orc_huffman_kv_chunk.restype = C.c_size_t
lib.orc_huffman_kv_chunk.argtypes = [_vp, C.c_int, _sz, _vp, _vp, _vp, _vp]
lib.orc_huffman_kv_get_kv.restype = None
lib.orc_huffman_kv_get_kv.argtypes = [_vp, C.c_int, _vp, _vp]


def huffman_kv_compress_chunk(data, num_tokens, num_heads, head_dim):
    """-> (bitstream bytes, scales [heads], codebook [256], q [heads * tokens * head_dim])."""
    d = _f32(data).reshape(-1)
    n = num_tokens * num_heads * head_dim
    assert d.size == n
    bits = np.zeros(2 * n + 16, np.uint8)
    scales, codebook, q = np.zeros(num_heads, np.float32), np.zeros(256, np.uint8), np.zeros(n, np.int8)
    nb = lib.orc_huffman_kv_compress_chunk(_p(d), _sz(num_tokens), _sz(num_heads), _sz(head_dim), _p(bits), _p(scales), _p(codebook), _p(q))
    return bits[:nb].tobytes(), scales, codebook, q


def huffman_kv_decompress_chunk(bitstream, scales, codebook, num_tokens, num_heads, head_dim):
    b = np.frombuffer(bytes(bitstream), np.uint8)
    s, cb = _f32(scales), np.ascontiguousarray(codebook, np.uint8)
    out = np.zeros(num_tokens * num_heads * head_dim, np.float32)
    rc = lib.orc_huffman_kv_decompress_chunk(_p(b), _sz(b.size), _p(s), _p(cb), _sz(num_tokens), _sz(num_heads), _sz(head_dim), _p(out))
    assert rc == 0, "a code does not fit the 12-bit table"
    return out


class HuffmanKVCache:
    """The oracle's HuffmanKVCache (state lives in the C library)."""

    def __init__(self, num_kv_heads, head_dim, compress_threshold, chunk_size):
        self.heads, self.head_dim = num_kv_heads, head_dim
        self._h = lib.orc_huffman_kv_new(num_kv_heads, head_dim, compress_threshold, chunk_size)

    def append(self, k, v, seq_len):
        k, v = _f32(k).reshape(-1), _f32(v).reshape(-1)
        assert k.size == v.size == self.heads * seq_len * self.head_dim
        lib.orc_huffman_kv_append(self._h, _p(k), _p(v), seq_len)

    def _stat(self, which):
        return int(lib.orc_huffman_kv_stat(self._h, which))

    len = property(lambda self: self._stat(0))
    compressed_len = property(lambda self: self._stat(1))
    hot_len = property(lambda self: self._stat(2))
    hot_capacity = property(lambda self: self._stat(3))
    num_chunks = property(lambda self: self._stat(4))
    compress_threshold = property(lambda self: self._stat(5))

    def chunk(self, value_side, index):
        """-> (bitstream bytes, scales, codebook, num_tokens)"""
        b, s, cb, t = _vp(), _vp(), _vp(), _sz()
        nb = lib.orc_huffman_kv_chunk(self._h, int(value_side), index, C.byref(b), C.byref(s), C.byref(cb), C.byref(t))
        scales = np.ctypeslib.as_array(C.cast(s, C.POINTER(C.c_float)), (self.heads,)).copy()
        codebook = np.ctypeslib.as_array(C.cast(cb, C.POINTER(C.c_uint8)), (256,)).copy()
        return C.string_at(b, nb), scales, codebook, int(t.value)

    def get_kv(self, literal_hot_offsets=False):
        n = self.heads * self.len * self.head_dim
        k, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
        lib.orc_huffman_kv_get_kv(self._h, int(bool(literal_hot_offsets)), _p(k), _p(v))
        return k, v

    def __del__(self):
        try:
            lib.orc_huffman_kv_free(self._h)
        except Exception:
            pass


def huffman_table_that_decodes(freqs):
    """(bit_lengths, codes, repaired): the reference's table unless its depth clamp over-subscribes the code."""
    f = np.ascontiguousarray(freqs, np.uint64)
    bl, codes = np.zeros(256, np.uint8), np.zeros(256, np.uint32)
    repaired = lib.orc_huffman_table_that_decodes(_p(f), _p(bl), _p(codes))
    return bl, codes, bool(repaired)
