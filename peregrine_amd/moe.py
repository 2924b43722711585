"""Host-side mirror of the MoE expert FFN (reference: examples/grok1/moe.rs:27-109,
expert body with SiLU: examples/deepseek/moe.rs:55-59) over block-quantised experts."""
import ctypes as C

import numpy as np

from . import _ffi
from .context import default_context
from .quant import _ptr

SILU, GELU_TANH = _ffi.ACT_SILU, _ffi.ACT_GELU_TANH


class MoEExperts:
    """E experts, each (gate [ffn, d], up [ffn, d], down [d, ffn]) as GgufWeight."""

    def __init__(self, gate, up, down, top_k, act=SILU, ctx=None):
        if not (len(gate) == len(up) == len(down)) or not gate:
            raise ValueError("MoEExperts: gate/up/down must be equally long, non-empty lists")
        self.ctx = ctx or default_context()
        self.gate, self.up, self.down = list(gate), list(up), list(down)
        self.top_k, self.act = int(top_k), int(act)
        self.d, self.ffn = gate[0].k_in, gate[0].n_out

    def _table(self, ws):
        arr = (C.c_void_p * len(ws))(*[w._h for w in ws])
        return C.cast(arr, C.POINTER(C.c_void_p)), arr

    def forward(self, x, router_logits):
        """MoELayer::forward after `logits = x.matmul(&router)` (examples/grok1/moe.rs:76-109):
        x [T, d], router_logits [T, E] -> out [T, d]."""
        E = len(self.gate)
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        T = x.size // self.d
        if x.size != T * self.d:
            raise ValueError("MoEExperts.forward: x is not [T, d]")
        logits = np.ascontiguousarray(router_logits, np.float32).reshape(-1)
        if logits.size != T * E:
            raise ValueError("MoEExperts.forward: router_logits is not [T, E]")
        out = np.empty(T * self.d, np.float32)
        (g, _g), (u, _u), (dn, _d) = self._table(self.gate), self._table(self.up), self._table(self.down)
        _ffi.check(_ffi.lib.pg_moe_ffn(self.ctx.handle, _ptr(x), T, _ptr(logits), E, self.top_k,
                                       g, u, dn, self.act, _ptr(out)))
        return out.reshape(T, self.d)

    def forward_routed(self, x, expert_idx, weight, shared=None):
        """The expert FFN over a routing another gate made (Gate::forward, examples/deepseek/moe.rs:111-215, or the
        gpt_oss top-k-then-softmax, examples/gpt_oss/moe.rs:298-330): expert_idx / weight [T, top_k]; `shared`
        [T, d] is the shared experts' output, added last (examples/deepseek/moe.rs:298-300)."""
        E = len(self.gate)
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        T = x.size // self.d
        if x.size != T * self.d:
            raise ValueError("MoEExperts.forward_routed: x is not [T, d]")
        idx = np.ascontiguousarray(expert_idx, np.int32).reshape(-1)
        w = np.ascontiguousarray(weight, np.float32).reshape(-1)
        if idx.size != T * self.top_k or w.size != T * self.top_k:
            raise ValueError("MoEExperts.forward_routed: expert_idx / weight are not [T, top_k]")
        sh = None
        if shared is not None:
            sh = np.ascontiguousarray(shared, np.float32).reshape(-1)
            if sh.size != T * self.d:
                raise ValueError("MoEExperts.forward_routed: shared is not [T, d]")
        out = np.empty(T * self.d, np.float32)
        (g, _g), (u, _u), (dn, _d) = self._table(self.gate), self._table(self.up), self._table(self.down)
        _ffi.check(_ffi.lib.pg_moe_ffn_routed(self.ctx.handle, _ptr(x), T, _ptr(idx), _ptr(w), E, self.top_k, g, u, dn,
                                              self.act, _ptr(sh) if sh is not None else None, _ptr(out)))
        return out.reshape(T, self.d)
