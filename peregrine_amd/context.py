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
