"""pg_matmul_quantized_fixed_scratch_dev: the W8A8 product for callers that cannot allocate.

Called through the C ABI and compared with pg_matmul_quantized_dev (itself checked against the
oracle in test_gpu_quant.py): every f32 output must be bit-identical.  Calls come in pairs on the
same context, the second with a smaller input, so that whatever the first call left in the
library's fixed scratch (quantised rows, row scales, split-K partial planes) is still there
when the second one runs.
"""
import ctypes as C
import sys

import numpy as np
import pytest

from devbuf import DevBuf

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def both(ctx, orc, seed, m, k, n, check_oracle=False):
    """Run the product through the allocating entry point and the fixed-scratch one; returns
    the two outputs."""
    from peregrine_amd import quant, _ffi
    a = orc.rng_normal(seed, m * k)
    a.reshape(m, k)[:, :: max(1, k // 50)] *= 20
    w = orc.rng_normal(seed + 1, k * n, 0.0, 0.02)
    q, q_t, s = orc.quantize_weights(w, k, n)
    qt = quant.QuantizedTensor(q, q_t, s, k, n).to_gpu(ctx)
    da = DevBuf(ctx, host=a)
    d_ref, d_new = DevBuf(ctx, m * n * 4), DevBuf(ctx, host=np.full(m * n, np.nan, np.float32))
    _ffi.check(_ffi.lib.pg_matmul_quantized_dev(ctx.handle, da.ptr, m, k, qt._gpu, d_ref.ptr, None))
    _ffi.check(_ffi.lib.pg_matmul_quantized_fixed_scratch_dev(ctx.handle, da.ptr, m, k, qt._gpu, d_new.ptr))
    ctx.sync()
    ref, new = d_ref.to_host(np.float32), d_new.to_host(np.float32)
    if check_oracle:
        want, _ = orc.matmul_quantized(a, m, k, q_t, s, n)
        assert (bits(ref) == bits(want)).all()
    qt.free_gpu()
    return ref, new


# (first call, second smaller call): matrix-core tiles, split-K with partial planes, the
# few-row and one-row GEMV routes
PAIRS = [
    ((300, 1024, 520), (130, 512, 300)),
    ((64, 4096, 1000), (40, 1024, 257)),      # both split K: partial planes behind the scales
    ((256, 2048, 1000), (17, 2048, 1000)),
    ((4, 4096, 300), (2, 1000, 77)),          # quantised rows in the scratch, GEMV
    ((1, 4096, 1024), (1, 64, 33)),           # one row: quantised inside the product, no scratch
    ((2048, 4096, 4096), (500, 4096, 1024)),  # a prefill-sized product, then a smaller one
]


@pytest.mark.parametrize("first,second", PAIRS)
def test_fixed_scratch_product_equals_the_allocating_one(ctx, orc, first, second):
    for i, (m, k, n) in enumerate((first, second)):
        say(f"fixed-scratch product m={m} k={k} n={n} (call {i + 1} of the pair)")
        ref, new = both(ctx, orc, 40 + m + n, m, k, n, check_oracle=(m * k * n <= 1 << 28))
        assert (bits(new) == bits(ref)).all(), f"call {i + 1}: m={m} k={k} n={n} differs"


def test_fixed_scratch_limits_and_errors(ctx, orc):
    from peregrine_amd import quant, _ffi
    cap = _ffi.lib.pg_fixed_scratch_bytes()
    assert cap == 32 << 20
    k, n = 14336, 64
    w = orc.rng_normal(5, k * n, 0.0, 0.02)
    q, q_t, s = orc.quantize_weights(w, k, n)
    qt = quant.QuantizedTensor(q, q_t, s, k, n).to_gpu(ctx)
    # 2048 rows of 14336 fit (29.4 MB + scales) ...
    m = 2048
    say(f"fixed-scratch product at the documented maximum m={m} k={k}")
    a = orc.rng_normal(6, m * k)
    da = DevBuf(ctx, host=a)
    d_ref, d_new = DevBuf(ctx, m * n * 4), DevBuf(ctx, m * n * 4)
    _ffi.check(_ffi.lib.pg_matmul_quantized_dev(ctx.handle, da.ptr, m, k, qt._gpu, d_ref.ptr, None))
    _ffi.check(_ffi.lib.pg_matmul_quantized_fixed_scratch_dev(ctx.handle, da.ptr, m, k, qt._gpu, d_new.ptr))
    ctx.sync()
    assert (bits(d_new.to_host(np.float32)) == bits(d_ref.to_host(np.float32))).all()
    # ... 2560 rows do not: a clear error, nothing launched
    st = _ffi.lib.pg_matmul_quantized_fixed_scratch_dev(ctx.handle, da.ptr, 2560, k, qt._gpu, d_new.ptr)
    assert st == _ffi.PG_EINVAL and b"scratch" in _ffi.lib.pg_last_error()
    # the reference's shape assert and the empty product
    assert _ffi.lib.pg_matmul_quantized_fixed_scratch_dev(ctx.handle, da.ptr, 4, k + 1, qt._gpu, d_new.ptr) == _ffi.PG_EINVAL
    assert _ffi.lib.pg_matmul_quantized_fixed_scratch_dev(ctx.handle, None, 0, k, qt._gpu, None) == _ffi.PG_OK
    qt.free_gpu()
