"""Device buffers for the `_dev` entry points, allocated through the library's own
pg_dev_alloc / pg_memcpy_* (no torch involved)."""
import ctypes as C

import numpy as np

from peregrine_amd import _ffi


class DevBuf:
    def __init__(self, ctx, nbytes=None, host=None):
        self.ctx = ctx
        if host is not None:
            host = np.ascontiguousarray(host)
            nbytes = host.nbytes
        self.nbytes = int(nbytes)
        self.ptr = C.c_void_p()
        _ffi.check(_ffi.lib.pg_dev_alloc(ctx.handle, self.nbytes, C.byref(self.ptr)))
        if host is not None and self.nbytes:
            _ffi.check(_ffi.lib.pg_memcpy_h2d(ctx.handle, self.ptr, C.c_void_p(host.ctypes.data), self.nbytes))

    def to_host(self, dtype, count=None):
        dtype = np.dtype(dtype)
        count = self.nbytes // dtype.itemsize if count is None else count
        out = np.empty(count, dtype)
        if out.nbytes:
            _ffi.check(_ffi.lib.pg_memcpy_d2h(self.ctx.handle, C.c_void_p(out.ctypes.data), self.ptr, out.nbytes))
        return out

    def free(self):
        if self.ptr:
            _ffi.check(_ffi.lib.pg_dev_free(self.ctx.handle, self.ptr))
            self.ptr = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
