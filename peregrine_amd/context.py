"""Device context: one GPU + one HIP stream (the slot of the reference's thread-local
Metal GpuContext, src/metal/context.rs:2472-2510)."""
import ctypes as C

from . import _ffi


class Context:
    def __init__(self, device=0, stream=None):
        """`stream`: an existing hipStream_t handle (int) to launch on, or None for a
        stream owned by the context."""
        self._h = C.c_void_p()
        _ffi.check(_ffi.lib.pg_ctx_create(int(device), C.c_void_p(stream or None), C.byref(self._h)))
        self.device = int(device)

    @property
    def handle(self):
        if not self._h:
            raise RuntimeError("context was closed")
        return self._h

    @property
    def stream(self):
        return _ffi.lib.pg_ctx_stream(self.handle)

    def sync(self):
        _ffi.check(_ffi.lib.pg_sync(self.handle))

    def profile_begin(self):
        """Start stamping every hot-path kernel launch on this context with HIP events."""
        _ffi.check(_ffi.lib.pg_profile_begin(self.handle))

    def profile_end(self):
        """Stop profiling; returns {kernel name: (total_ms, launches)}."""
        n = C.c_size_t()
        _ffi.check(_ffi.lib.pg_profile_end(self.handle, C.byref(n)))
        out = {}
        for i in range(n.value):
            name, ms, cnt = C.c_char_p(), C.c_double(), C.c_size_t()
            _ffi.check(_ffi.lib.pg_profile_get(self.handle, i, C.byref(name), C.byref(ms), C.byref(cnt)))
            out[name.value.decode()] = (ms.value, cnt.value)
        return out

    def profile_grids(self):
        """After profile_end(): {kernel name: {work-items of a launch: launches}}."""
        out = {}
        i = 0
        while True:
            name = C.c_char_p()
            if _ffi.lib.pg_profile_get(self.handle, i, C.byref(name), None, None) != _ffi.PG_OK:
                break
            w, n, cnt = (C.c_size_t * 16)(), (C.c_size_t * 16)(), C.c_size_t()
            _ffi.check(_ffi.lib.pg_profile_get_grids(self.handle, i, w, n, 16, C.byref(cnt)))
            out[name.value.decode()] = {int(w[j]): int(n[j]) for j in range(min(cnt.value, 16))}
            i += 1
        return out

    def close(self):
        if self._h:
            _ffi.lib.pg_ctx_destroy(self._h)
            self._h = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


_default = None


def default_context():
    """Lazily created context on device 0 (the reference's `with_gpu` singleton)."""
    global _default
    if _default is None:
        _default = Context(0)
    return _default
