"""Host-side mirror of the glue around the quantised products in peregrine's Llama decoder
block: `nn::RMSNorm` / `nn::RoPE` (src/nn.rs:560-652, 1250-1345), `attention::StandardKVCache`
and `gqa_attention_cpu` (src/attention.rs:8-300), `LlamaBlock` (src/models/llama/decoder.rs)."""
import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import _ffi
from .context import default_context
from .quant import _ptr


def _f32(a):
    return np.ascontiguousarray(a, np.float32).reshape(-1)


class RMSNorm:
    """`nn::RMSNorm` (src/nn.rs:560-575): weight [dim] initialised to ones, `eps`."""

    def __init__(self, dim, eps, ctx=None):
        self.ctx = ctx or default_context()
        self.dim, self.eps = int(dim), float(eps)
        self.weight = np.ones(self.dim, np.float32)

    def forward(self, x):
        """src/nn.rs:577-652: x [..., dim] -> same shape."""
        x = np.ascontiguousarray(x, np.float32)
        if x.size % self.dim or (x.ndim and x.shape[-1] != self.dim):
            raise ValueError(f"RMSNorm.forward: last dimension is not {self.dim}")
        out = np.empty(x.size, np.float32)
        w = _f32(self.weight)
        if w.size != self.dim:
            raise ValueError(f"RMSNorm.forward: weight is not [{self.dim}]")
        _ffi.check(_ffi.lib.pg_rmsnorm(self.ctx.handle, _ptr(x.reshape(-1)), x.size // self.dim, self.dim,
                                       _ptr(w), self.eps, _ptr(out)))
        return out.reshape(x.shape)


class RoPE:
    """`nn::RoPE` (src/nn.rs:1250-1282): cos/sin tables for `max_seq_len` positions."""

    def __init__(self, head_dim, max_seq_len, base, ctx=None):
        self.ctx = ctx or default_context()
        self.head_dim, self.max_seq_len = int(head_dim), int(max_seq_len)
        self._h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_rope_create(self.ctx.handle, self.head_dim, self.max_seq_len, float(base), C.byref(self._h)))

    def apply(self, x, offset):
        """src/nn.rs:1286-1317: x [seq_len, head_dim] at positions offset.. ."""
        x = np.ascontiguousarray(x, np.float32)
        if x.ndim != 2 or x.shape[1] != self.head_dim:
            raise ValueError("RoPE.apply: x is not [seq_len, head_dim]")
        out = np.empty(x.size, np.float32)
        _ffi.check(_ffi.lib.pg_rope_apply(self.ctx.handle, self._h, _ptr(x.reshape(-1)), x.shape[0], int(offset), _ptr(out)))
        return out.reshape(x.shape)

    def free(self):
        if self._h:
            _ffi.lib.pg_rope_free(self.ctx.handle, self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class StandardKVCache:
    """`attention::StandardKVCache` (src/attention.rs:8-100), resident in HBM as
    [num_kv_heads, capacity, head_dim] key and value planes."""

    def __init__(self, num_kv_heads, head_dim, ctx=None):
        self.ctx = ctx or default_context()
        self.num_kv_heads, self.head_dim = int(num_kv_heads), int(head_dim)
        self._h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_kv_cache_create(self.ctx.handle, self.num_kv_heads, self.head_dim, C.byref(self._h)))

    @property
    def len(self):
        return int(_ffi.lib.pg_kv_cache_len(self._h))

    def head_stride(self):
        """src/attention.rs:96-98: capacity * head_dim."""
        return int(_ffi.lib.pg_kv_cache_capacity(self._h)) * self.head_dim

    def append(self, new_k, new_v, seq_len):
        """src/attention.rs:65-83: new_k, new_v [num_kv_heads, seq_len, head_dim]."""
        k, v = _f32(new_k), _f32(new_v)
        n = self.num_kv_heads * int(seq_len) * self.head_dim
        if k.size != n or v.size != n:
            raise ValueError("StandardKVCache.append: new_k / new_v are not [num_kv_heads, seq_len, head_dim]")
        _ffi.check(_ffi.lib.pg_kv_cache_append(self.ctx.handle, self._h, _ptr(k), _ptr(v), int(seq_len)))

    def rollback_to(self, new_len):
        """src/attention.rs:87-91 (its assert! surfaces as PeregrineError)."""
        _ffi.check(_ffi.lib.pg_kv_cache_rollback_to(self._h, int(new_len)))

    def to_host(self):
        """(k, v), each [num_kv_heads, len, head_dim] without the capacity padding."""
        shape = (self.num_kv_heads, self.len, self.head_dim)
        k, v = np.zeros(shape, np.float32), np.zeros(shape, np.float32)
        _ffi.check(_ffi.lib.pg_kv_cache_download(self.ctx.handle, self._h, _ptr(k), _ptr(v)))
        return k, v

    def free(self):
        if self._h:
            _ffi.lib.pg_kv_cache_free(self.ctx.handle, self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


KVCache = StandardKVCache  # src/models/llama/attention.rs:7


@dataclass
class AttentionMask:
    """`attention::AttentionMask` (src/attention.rs:102-120)."""
    kind: int = _ffi.MASK_NONE
    offset: int = 0
    window: int = 0
    sink_tokens: int = 0
    global_positions: tuple = ()

    @classmethod
    def none(cls):
        return cls()

    @classmethod
    def causal(cls, offset):
        return cls(_ffi.MASK_CAUSAL, int(offset))

    @classmethod
    def causal_sliding_window(cls, offset, window, sink_tokens):
        return cls(_ffi.MASK_CAUSAL_SLIDING_WINDOW, int(offset), int(window), int(sink_tokens))

    @classmethod
    def local_global(cls, offset, local_window, global_positions):
        return cls(_ffi.MASK_LOCAL_GLOBAL, int(offset), int(local_window), 0, tuple(int(p) for p in global_positions))


def gqa_attention(q, k_cache, v_cache, num_q_heads, num_kv_heads, seq_q, head_dim, scale, mask, logit_cap, output, ctx=None):
    """`attention::gqa_attention_cpu` (src/attention.rs:141-265): q [num_q_heads, seq_q, head_dim];
    `output` [seq_q, num_q_heads * head_dim] float32 is added to in place.  `logit_cap` None or
    0 is PostScoreTransform::None, a positive value PostScoreTransform::LogitCap."""
    ctx = ctx or default_context()
    if num_kv_heads != k_cache.num_kv_heads or head_dim != k_cache.head_dim:
        raise ValueError("gqa_attention: num_kv_heads / head_dim differ from the cache's")
    q = _f32(q)
    if q.size != num_q_heads * seq_q * head_dim:
        raise ValueError("gqa_attention: q is not [num_q_heads, seq_q, head_dim]")
    if not (isinstance(output, np.ndarray) and output.dtype == np.float32 and output.flags.c_contiguous
            and output.size == q.size):
        raise ValueError("gqa_attention: output must be a contiguous float32 array of seq_q * num_q_heads * head_dim")
    if mask.kind == _ffi.MASK_LOCAL_GLOBAL:
        gp = np.asarray(mask.global_positions, np.uint64)
        _ffi.check(_ffi.lib.pg_gqa_attention_local_global(ctx.handle, _ptr(q), k_cache._h, v_cache._h, num_q_heads, seq_q,
                                                          float(scale), mask.offset, mask.window, _ptr(gp), gp.size,
                                                          float(logit_cap or 0.0), _ptr(output)))
        return output
    _ffi.check(_ffi.lib.pg_gqa_attention(ctx.handle, _ptr(q), k_cache._h, v_cache._h, num_q_heads, seq_q, float(scale),
                                         mask.kind, mask.offset, mask.window, mask.sink_tokens, float(logit_cap or 0.0),
                                         _ptr(output)))
    return output


class LlamaBlock:
    """`LlamaBlock` (src/models/llama/decoder.rs:7-47) over block-quantised projections kept in
    HBM (GgufWeight, [out, in]) instead of dequantised f32 tensors."""

    def __init__(self, model_dim, num_q_heads, num_kv_heads, head_dim, ffn_dim, max_seq_len, rope_base, rms_eps, ctx=None):
        self.ctx = ctx or default_context()
        self.model_dim, self.num_kv_heads, self.head_dim = int(model_dim), int(num_kv_heads), int(head_dim)
        self._h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_llama_block_create(self.ctx.handle, model_dim, num_q_heads, num_kv_heads, head_dim, ffn_dim,
                                                  max_seq_len, float(rope_base), float(rms_eps), C.byref(self._h)))
        self._weights = None

    def set_weights(self, q_proj, k_proj, v_proj, o_proj, gate_proj, up_proj, down_proj, attn_norm_w, ffn_norm_w):
        ws = (q_proj, k_proj, v_proj, o_proj, gate_proj, up_proj, down_proj)
        wa, wf = _f32(attn_norm_w), _f32(ffn_norm_w)
        if wa.size != self.model_dim or wf.size != self.model_dim:
            raise ValueError("LlamaBlock.set_weights: norm weights are not [model_dim]")
        _ffi.check(_ffi.lib.pg_llama_block_set_weights(self.ctx.handle, self._h, *[w._h for w in ws], _ptr(wa), _ptr(wf)))
        self._weights = ws  # the block borrows the handles: keep them alive

    def new_cache(self):
        return StandardKVCache(self.num_kv_heads, self.head_dim, self.ctx)

    def forward(self, h, kv_cache):
        """src/models/llama/decoder.rs:69-155: h [seq, model_dim] -> [seq, model_dim]; the cache
        gains seq positions."""
        h = np.ascontiguousarray(h, np.float32)
        if h.ndim != 2 or h.shape[1] != self.model_dim:
            raise ValueError("LlamaBlock.forward: h is not [seq, model_dim]")
        out = np.empty(h.size, np.float32)
        _ffi.check(_ffi.lib.pg_llama_block_forward(self.ctx.handle, self._h, _ptr(h.reshape(-1)), h.shape[0],
                                                   kv_cache._h, _ptr(out)))
        return out.reshape(h.shape)

    def free(self):
        if self._h:
            _ffi.lib.pg_llama_block_free(self.ctx.handle, self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
