"""Host-side mirror of the gpt_oss example's MXFP4 path (examples/gpt_oss/moe.rs:5-117):
`mxfp4_matmul` and `Mxfp4Expert`, over weights kept on the device."""
import ctypes as C

import numpy as np

from . import _ffi
from .context import default_context
from .gguf import GgufWeight
from .quant import _ptr


def _bytes(b, n, what):
    a = np.frombuffer(bytes(b), np.uint8) if not isinstance(b, np.ndarray) else np.ascontiguousarray(b, np.uint8).reshape(-1)
    if a.size != n:
        raise ValueError(f"{what}: expected {n} bytes, got {a.size}")
    return a


def mxfp4_matmul(input, blocks, scales, out_dim, in_dim, ctx=None):
    """examples/gpt_oss/moe.rs:16-53: input [in_dim] x weight [out_dim, in_dim] -> [out_dim]."""
    ctx = ctx or default_context()
    x = np.ascontiguousarray(input, np.float32).reshape(-1)
    if in_dim % 32 or x.size != in_dim:
        raise ValueError("mxfp4_matmul: input is not [in_dim] with in_dim a multiple of 32")
    b = _bytes(blocks, out_dim * in_dim // 2, "mxfp4_matmul blocks")
    s = _bytes(scales, out_dim * in_dim // 32, "mxfp4_matmul scales")
    out = np.empty(out_dim, np.float32)
    _ffi.check(_ffi.lib.pg_mxfp4_matmul(ctx.handle, _ptr(x), _ptr(b), _ptr(s), out_dim, in_dim, _ptr(out)))
    return out


def upload(blocks, scales, out_dim, in_dim, ctx=None):
    """The weight as a device-resident GgufWeight (type MXFP4): `.matmul(x, m)` runs one
    mxfp4_matmul per row of x."""
    ctx = ctx or default_context()
    if in_dim % 32:
        raise ValueError("mxfp4.upload: in_dim is not a multiple of 32")
    b = _bytes(blocks, out_dim * in_dim // 2, "mxfp4.upload blocks")
    s = _bytes(scales, out_dim * in_dim // 32, "mxfp4.upload scales")
    h = C.c_void_p()
    _ffi.check(_ffi.lib.pg_mxfp4_upload(ctx.handle, _ptr(b), _ptr(s), out_dim, in_dim, C.byref(h)))
    return GgufWeight._from_handle(h, ctx)


class Mxfp4Expert:
    """examples/gpt_oss/moe.rs:55-117."""

    def __init__(self, hidden, intermediate, alpha, clamp, mlp1_blocks, mlp1_scales, mlp2_blocks, mlp2_scales,
                 mlp1_bias=None, mlp2_bias=None, ctx=None):
        self.ctx = ctx or default_context()
        self.hidden, self.intermediate = int(hidden), int(intermediate)
        if self.hidden % 32 or self.intermediate % 32:
            raise ValueError("Mxfp4Expert: hidden and intermediate must be multiples of 32")
        b1 = _bytes(mlp1_blocks, 2 * intermediate * hidden // 2, "mlp1_blocks")
        s1 = _bytes(mlp1_scales, 2 * intermediate * hidden // 32, "mlp1_scales")
        b2 = _bytes(mlp2_blocks, hidden * intermediate // 2, "mlp2_blocks")
        s2 = _bytes(mlp2_scales, hidden * intermediate // 32, "mlp2_scales")
        bias1 = np.zeros(2 * intermediate, np.float32) if mlp1_bias is None else np.ascontiguousarray(mlp1_bias, np.float32).reshape(-1)
        bias2 = np.zeros(hidden, np.float32) if mlp2_bias is None else np.ascontiguousarray(mlp2_bias, np.float32).reshape(-1)
        if bias1.size != 2 * intermediate or bias2.size != hidden:
            raise ValueError("Mxfp4Expert: bias lengths")
        self._h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_mxfp4_expert_create(self.ctx.handle, hidden, intermediate, float(alpha), float(clamp),
                                                   _ptr(b1), _ptr(s1), _ptr(b2), _ptr(s2), _ptr(bias1), _ptr(bias2),
                                                   C.byref(self._h)))

    def forward(self, x):
        """x [hidden] -> [hidden] (the reference's signature), or [m, hidden] -> [m, hidden]."""
        x = np.ascontiguousarray(x, np.float32)
        if x.size % self.hidden:
            raise ValueError("Mxfp4Expert.forward: x is not [.., hidden]")
        out = np.empty(x.size, np.float32)
        _ffi.check(_ffi.lib.pg_mxfp4_expert_forward(self.ctx.handle, self._h, _ptr(x.reshape(-1)), x.size // self.hidden,
                                                    _ptr(out)))
        return out.reshape(x.shape)

    def free(self):
        if self._h:
            _ffi.lib.pg_mxfp4_expert_free(self.ctx.handle, self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def moe_forward_routed(x, expert_idx, weight, experts, ctx=None):
    """`MoELayer::forward` after its router, over `Mxfp4Expert`s (examples/gpt_oss/moe.rs:286-352): x [T, hidden],
    expert_idx / weight [T, top_k] as the router chose them -> [T, hidden]; every product is one launch over all
    experts."""
    ctx = ctx or default_context()
    hidden = experts[0].hidden
    x = np.ascontiguousarray(x, np.float32).reshape(-1, hidden)
    T = x.shape[0]
    idx = np.ascontiguousarray(expert_idx, np.int32).reshape(T, -1)
    w = np.ascontiguousarray(weight, np.float32).reshape(T, -1)
    if idx.shape != w.shape:
        raise ValueError("moe_forward_routed: expert_idx and weight differ in shape")
    tab = (C.c_void_p * len(experts))(*[e._h.value for e in experts])
    out = np.empty((T, hidden), np.float32)
    _ffi.check(_ffi.lib.pg_mxfp4_moe_ffn_routed(ctx.handle, _ptr(x.reshape(-1)), T, _ptr(idx.reshape(-1)), _ptr(w.reshape(-1)), idx.shape[1],
                                                C.cast(tab, C.POINTER(C.c_void_p)), len(experts), _ptr(out.reshape(-1))))
    return out
