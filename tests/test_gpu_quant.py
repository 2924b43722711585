"""GPU parity of the quant::* path against the CPU oracle, through the C ABI.

Bar: quantised i8 values, f32 scales, i32 accumulators and the f32 outputs of the W8A8
product are all BIT-EXACT (the epilogue keeps the reference's multiplication order, so
even the f32 result has a single correct bit pattern).
"""
import ctypes as C
import sys

import numpy as np
import pytest

import helpers as H
from devbuf import DevBuf

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def edge_rows(cols):
    """Rows the reference's arithmetic treats specially (ties, zero, NaN, inf, subnormal)."""
    r = np.zeros((6, cols), np.float32)
    r[0, :8] = [127, -127, 0.5, -0.5, 1.5, 2.5, -2.5, 0]
    r[2, :] = 4.0
    r[2, 1::2] = -4.0
    r[3, :8] = [np.nan, 1, -2, 0.5, 0, 0, 0, 2]
    r[4, :8] = [np.inf, 1, -1, 0, 0, 0, 0, -np.inf]
    r[5, :8] = [1e-42, -1e-42, 0, 0, 0, 0, 0, 5e-43]
    return r


@pytest.mark.parametrize("rows,cols", [(32, 4096), (1, 4096), (1, 14336), (7, 100), (5, 4100),
                                       (3, 20000), (2, 16384), (9, 33), (4, 1)])
def test_quantize_activations_bit_exact(ctx, orc, rows, cols):
    from peregrine_amd import quant
    say(f"quantize_activations rows={rows} cols={cols}")
    a = orc.rng_normal(1000 + rows * 7 + cols, rows * cols).reshape(rows, cols)
    a[:, :: max(1, cols // 40)] *= 20  # outlier channels
    q, s = quant.quantize_activations(a, rows, cols, ctx)
    qo, so = orc.quantize_activations(a, rows, cols)
    assert (bits(s) == bits(so)).all()
    assert (q == qo).all()


def test_quantize_activations_edge_rows_and_empty(ctx, orc):
    from peregrine_amd import quant
    for cols in (8, 64, 4096):
        say(f"quantize_activations edge rows cols={cols}")
        a = edge_rows(cols)
        q, s = quant.quantize_activations(a, a.shape[0], cols, ctx)
        qo, so = orc.quantize_activations(a, a.shape[0], cols)
        assert (bits(s) == bits(so)).all() and (q == qo).all()
    # constructed near-tie rows that separate x*(1/s) from x/s
    fh = float.fromhex
    tie = np.array([[fh("0x1.13c502p-4"), fh("0x1.e6658ep-10"), fh("-0x1.09ff8ap-4"), fh("-0x1.f9f07ep-5")],
                    [fh("0x1.18d40ep-5"), fh("0x1.1b0a2p-13"), fh("-0x1.1116c6p-5"), fh("-0x1.134cdap-5")]], np.float32)
    q, s = quant.quantize_activations(tie, 2, 4, ctx)
    qo, so = orc.quantize_activations(tie, 2, 4)
    assert (q == qo).all() and (bits(s) == bits(so)).all()
    q, s = quant.quantize_activations(np.zeros(0, np.float32), 0, 16, ctx)  # empty input
    assert q.size == 0 and s.size == 0
    with pytest.raises(ValueError):
        quant.quantize_activations(np.zeros(5, np.float32), 2, 3, ctx)


@pytest.mark.parametrize("rows,cols", [(128, 96), (100, 70), (4096, 64), (64, 1000), (1, 5), (300, 1)])
def test_quantize_weights_bit_exact(ctx, orc, rows, cols):
    from peregrine_amd import quant
    say(f"quantize_weights rows={rows} cols={cols}")
    w = orc.rng_normal(5678 + rows + cols, rows * cols, 0.0, 0.02)
    qt = quant.quantize_weights(w, rows, cols, ctx)
    q, q_t, s = orc.quantize_weights(w, rows, cols)
    assert (bits(qt.scales) == bits(s)).all()
    assert (qt.data_i8 == q).all()
    assert (qt.data_i8_t == q_t).all()
    assert (bits(quant.dequantize(qt, ctx)) == bits(orc.dequantize(q, s, rows, cols))).all()


def test_quantize_weights_edge_columns(ctx, orc):
    from peregrine_amd import quant
    say("quantize_weights edge columns")
    fh = float.fromhex
    w = np.zeros((6, 7), np.float32)
    w[:, 0] = [127, -127, 2.5, -2.5, 0.5, 1.5]
    w[:, 2] = [3, 3, -3, 3, -3, 3]
    w[:, 3] = [np.nan, 1, -2, 0.25, 0, 2]
    w[:, 4] = [np.inf, 1, -1, 0, 5, -np.inf]
    w[:4, 5] = [fh("0x1.13c502p-4"), fh("0x1.e6658ep-10"), fh("-0x1.09ff8ap-4"), fh("-0x1.f9f07ep-5")]
    w[:4, 6] = [fh("0x1.18d40ep-5"), fh("0x1.1b0a2p-13"), fh("-0x1.1116c6p-5"), fh("-0x1.134cdap-5")]
    qt = quant.quantize_weights(w, 6, 7, ctx)
    q, q_t, s = orc.quantize_weights(w, 6, 7)
    assert (bits(qt.scales) == bits(s)).all() and (qt.data_i8 == q).all() and (qt.data_i8_t == q_t).all()


def test_reference_roundtrip_property(ctx):
    # tests/quant_parity.rs:6-32 run against the GPU path
    from peregrine_amd import quant
    rows, cols = 64, 128
    data = H.mod_pattern(rows * cols, 17, 5, 400, 100.0, 2.0)
    qt = quant.quantize_weights(data, rows, cols, ctx)
    rec = quant.dequantize(qt, ctx).reshape(rows, cols)
    d = data.reshape(rows, cols)
    amax = np.abs(d).max(axis=0)
    scale = np.where(amax == 0, 1.0, amax / np.float32(127)).astype(np.float32)
    assert (np.abs(d - rec) <= scale[None, :] + 1e-7).all()


def test_to_gpu_from_gpu_roundtrip(ctx, orc):
    # QuantizedTensor::to_gpu / from_gpu (src/quant.rs:173-191); upload is idempotent
    from peregrine_amd import quant
    rows, cols = 200, 130
    w = orc.rng_normal(77, rows * cols, 0.0, 0.02)
    qt = quant.quantize_weights(w, rows, cols, ctx)
    q0, qt0, s0 = qt.data_i8.copy(), qt.data_i8_t.copy(), qt.scales.copy()
    qt.to_gpu(ctx)
    h = qt._gpu
    qt.to_gpu(ctx)
    assert qt._gpu is h
    qt.data_i8[:] = 0
    qt.from_gpu(ctx)
    assert (qt.data_i8 == q0).all() and (qt.data_i8_t == qt0).all() and (bits(qt.scales) == bits(s0)).all()
    with pytest.raises(RuntimeError):
        quant.matmul_quantized_gpu(ctx, np.zeros(rows, np.float32), 1, rows,
                                   quant.QuantizedTensor(q0, qt0, s0, rows, cols))  # "weights not on GPU"


def run_matmul_dev(ctx, a, m, k, qt):
    """pg_matmul_quantized_dev with the accumulator dump; returns (out, acc)."""
    from peregrine_amd import _ffi
    qt.to_gpu(ctx)
    n = qt.cols
    da = DevBuf(ctx, host=np.ascontiguousarray(a, np.float32))
    dout, dacc = DevBuf(ctx, m * n * 4), DevBuf(ctx, m * n * 4)
    _ffi.check(_ffi.lib.pg_matmul_quantized_dev(ctx.handle, da.ptr, m, k, qt._gpu, dout.ptr, dacc.ptr))
    ctx.sync()
    return dout.to_host(np.float32), dacc.to_host(np.int32)


# (m, k, n): reference test shapes, decode GEMV shapes, every GEMM tile config, ragged edges
MATMUL_SHAPES = [
    (32, 128, 64), (16, 64, 32),                       # tests/quant_parity.rs:35, src/quant.rs:252
    (8, 32, 16), (1, 64, 1), (16, 256, 32),            # tests/huffman_parity.rs:25
    (1, 4096, 14336), (1, 14336, 4096),                # benchmark configuration 2 (decode GEMV)
    (2, 4096, 1024), (3, 1000, 77), (4, 4096, 300),    # GEMV with m = 2..4, ragged k and n
    (32, 4096, 4096),                                  # benchmark configuration 1
    (5, 96, 40), (64, 200, 130), (65, 384, 129),       # 64x64 and 128x128 tiles, ragged
    (196, 768, 3072), (196, 1024, 4096),               # benches/wallclock.rs:758-786
    (300, 512, 1000),                                  # 128x128 tiles, ragged m and n
    (2048, 128, 4096),                                 # 128x256 tiles
    (2050, 192, 4100),                                 # 128x256 tiles, ragged m and n
    (2049, 128, 12300),                                # 256x256 tiles, ragged m and n
    (1030, 256, 4000),                                 # 128x128 tiles unsplit, ragged m and n
    # 2 .. 32 rows: one launch, a workgroup per 16 (or 32) weight rows with its wavefronts on runs of K (ragged everywhere;
    # K of one unit of 128; more than 16 rows on a wide tensor: two weight tiles per workgroup)
    (5, 4096, 1000), (17, 4224, 520), (31, 512, 77), (2, 128, 16), (16, 130, 5), (9, 2000, 33), (20, 1024, 8200),
    (32, 4096, 14336), (17, 384, 8208), (24, 14336, 4096), (3, 14336, 4100),
    # 33 .. 64 rows on products at least as wide as long: the same with four activation tiles a unit
    (33, 1024, 4100), (40, 1024, 14336), (64, 4096, 4096), (50, 384, 8300),
    # 33 .. 64 rows on long, narrow products: K split over workgroups, i32 partial planes, finishing pass
    (64, 14336, 300), (40, 8192, 4096),
    (100, 8192, 300), (130, 4096, 257), (256, 2048, 1000),   # up to 256 rows when K >= 2 N: 128-row tiles
]


@pytest.mark.parametrize("m,k,n", MATMUL_SHAPES)
def test_matmul_quantized_bit_exact(ctx, orc, m, k, n):
    from peregrine_amd import quant
    say(f"matmul_quantized m={m} k={k} n={n}")
    a = orc.rng_normal(1234 + m, m * k)
    if k >= 100:
        a.reshape(m, k)[:, :: k // 50] *= 20  # outlier channels
    w = orc.rng_normal(5678 + n, k * n, 0.0, 0.02)
    qt = quant.quantize_weights(w, k, n, ctx)
    q, q_t, s = orc.quantize_weights(w, k, n)
    assert (qt.data_i8_t == q_t).all()
    want, want_acc = orc.matmul_quantized(a, m, k, q_t, s, n)
    got, got_acc = run_matmul_dev(ctx, a, m, k, qt)
    assert (got_acc == want_acc).all(), "i32 accumulators differ"
    assert (bits(got) == bits(want)).all(), "f32 outputs differ"
    # the host-pointer entry point gives the same answer
    got2 = quant.matmul_quantized(a, m, k, qt, ctx)
    assert (bits(got2) == bits(want)).all()


@pytest.mark.parametrize("k,n", [(8, 5), (64, 33), (4096, 300), (4100, 64), (14336, 128), (16384, 16), (16400, 16)])
def test_matmul_quantized_one_row_quantised_inside_the_product(ctx, orc, k, n):
    """m = 1 with k % 4 == 0 and k <= 16384 runs as ONE launch that quantises the activation row
    itself: the accumulators (hence the row's integers) and the f32 output must be those of the
    two-step path bit for bit, on ordinary rows and on the rows the arithmetic treats specially
    (ties, zero row, NaN, inf, subnormals).  k = 4100 and 16400 are past that route's limits."""
    from peregrine_amd import quant
    say(f"matmul_quantized one row k={k} n={n}")
    w = orc.rng_normal(321 + n, k * n, 0.0, 0.02)
    qt = quant.quantize_weights(w, k, n, ctx)
    q, q_t, s = orc.quantize_weights(w, k, n)
    rows = [orc.rng_normal(77 + k, k)]
    rows[0][:: max(1, k // 40)] *= 20
    rows += list(edge_rows(k))
    for i, a in enumerate(rows):
        want, want_acc = orc.matmul_quantized(a, 1, k, q_t, s, n)
        got, got_acc = run_matmul_dev(ctx, a, 1, k, qt)
        assert (got_acc == want_acc).all(), f"row {i}: i32 accumulators differ"
        finite = np.isfinite(want)
        assert (np.isfinite(got) == finite).all() and (bits(got[finite]) == bits(want[finite])).all(), f"row {i}: f32 outputs differ"
    # a row that does not start on a 16-byte boundary takes the two-launch path: same answer
    from peregrine_amd import _ffi
    a = rows[0]
    want, _ = orc.matmul_quantized(a, 1, k, q_t, s, n)
    shifted = DevBuf(ctx, host=np.concatenate([np.zeros(1, np.float32), a]))
    dout = DevBuf(ctx, n * 4)
    _ffi.check(_ffi.lib.pg_matmul_quantized_dev(ctx.handle, C.c_void_p(shifted.ptr.value + 4), 1, k, qt._gpu, dout.ptr, None))
    ctx.sync()
    assert (bits(dout.to_host(np.float32)) == bits(want)).all()
    qt.free_gpu()


def test_matmul_quantized_extreme_integers(ctx, orc):
    # every product is (-127)*(-127) or 127*(-127): the largest accumulators the path can see
    from peregrine_amd import quant
    m, k, n = 70, 14336, 130
    say(f"matmul_quantized extremes m={m} k={k} n={n}")
    a = np.full((m, k), -3.0, np.float32)
    a[::2] = 3.0
    w = np.full((k, n), -0.5, np.float32)
    qt = quant.quantize_weights(w, k, n, ctx)
    got, acc = run_matmul_dev(ctx, a, m, k, qt)
    want_acc = np.where((np.arange(m) % 2 == 0)[:, None], -127 * 127 * k, 127 * 127 * k) * np.ones((1, n), np.int64)
    assert (acc.reshape(m, n) == want_acc).all()
    q, q_t, s = orc.quantize_weights(w, k, n)
    want, _ = orc.matmul_quantized(a, m, k, q_t, s, n)
    assert (bits(got) == bits(want)).all()


def test_matmul_quantized_shape_mismatch_is_an_error(ctx, orc):
    from peregrine_amd import quant, _ffi
    qt = quant.quantize_weights(np.ones(64 * 8, np.float32), 64, 8, ctx)
    with pytest.raises(ValueError):
        quant.matmul_quantized(np.zeros(2 * 32, np.float32), 2, 32, qt, ctx)  # assert_eq!(w.rows, k)
    qt.to_gpu(ctx)
    out = np.zeros(16, np.float32)
    st = _ffi.lib.pg_matmul_quantized(ctx.handle, C.c_void_p(out.ctypes.data), 2, 32, qt._gpu, C.c_void_p(out.ctypes.data))
    assert st == _ffi.PG_EINVAL and b"rows" in _ffi.lib.pg_last_error()
    assert quant.matmul_quantized(np.zeros(0, np.float32), 0, 64, qt, ctx).size == 0  # m = 0


def last_tile(ctx):
    """(rows, columns, K splits) of the most recent W8A8 matrix-core launch on this context."""
    from peregrine_amd import _ffi
    bm, bn, sp = C.c_int(), C.c_int(), C.c_int()
    _ffi.check(_ffi.lib.pg_gemm_w8a8_last_tile(ctx.handle, C.byref(bm), C.byref(bn), C.byref(sp)))
    return bm.value, bn.value, sp.value


def outlier_acts(orc, seed, m, k):
    """N(0,1) activations with 1 % of the channels scaled x20 (benchmark configuration 3)."""
    a = orc.rng_normal(seed, m * k).reshape(m, k)
    chan = np.random.default_rng(seed).choice(k, max(1, k // 100), replace=False)
    a[:, chan] *= 20
    return a


def np_epilogue(acc, a_s, w_s):
    """((acc as f32) * a_scale[m]) * w_scale[n] in IEEE single, the order of src/quant.rs:163."""
    return (acc.astype(np.float32) * a_s.astype(np.float32)[:, None]) * w_s.astype(np.float32)[None, :]


# benchmark configuration 3: the seven products of one Llama-3-8B layer at M = 2048 are these four shapes;
# the last column is the output tile the dispatcher must pick (so a dispatcher change cannot
# silently leave a tile shape without a test)
PREFILL_SHAPES = [
    ("q/o_proj", 2048, 4096, 4096, (128, 256)),
    ("k/v_proj", 2048, 4096, 1024, (128, 64)),
    ("gate/up_proj", 2048, 4096, 14336, (256, 256)),
    ("down_proj", 2048, 14336, 4096, (128, 256)),
    ("unsplit 128x128", 1024, 256, 4096, (128, 128)),
]


@pytest.mark.parametrize("name,m,k,n,tile", PREFILL_SHAPES, ids=[p[0] for p in PREFILL_SHAPES])
def test_prefill_shape_full_size_properties(ctx, orc, name, m, k, n, tile):
    """Every product shape of benchmark configuration 3 at full size (the oracle would need up to
    1.2e11 scalar MACs for one of them), checked through:
      (a) one row out of every 32-row band of the output (64 rows at M = 2048: every MFMA row tile
          of every workgroup tile, all columns) bit-exactly against the oracle, accumulators and f32;
      (b) 96 sampled columns over ALL rows against an int32 NumPy product of the oracle's
          quantised operands and the IEEE-single epilogue in the reference's order;
      (c) the sum over ALL accumulators against the exact identity
            sum_{m,n} acc[m,n] = sum_k (sum_m a_i8[m,k]) * (sum_n w_t[n,k])   (int64);
      (d) the f32-only call (no accumulator dump: the straight-line, non-temporal epilogue the
          benchmark runs) against the f32 output of the dumping call, every element;
      (e) the tile shape the dispatcher chose."""
    from peregrine_amd import quant, _ffi
    say(f"prefill full size {name}: m={m} k={k} n={n}")
    a = outlier_acts(orc, 4321 + n, m, k)
    w = orc.rng_normal(8765 + k, k * n, 0.0, 0.02)
    q, q_t, s = orc.quantize_weights(w, k, n)
    qt = quant.QuantizedTensor(q, q_t, s, k, n)
    del w
    got, acc = run_matmul_dev(ctx, a, m, k, qt)
    assert last_tile(ctx) == tile + (1,), f"dispatcher picked {last_tile(ctx)}, the test expects {tile}"
    got, acc = got.reshape(m, n), acc.reshape(m, n)
    a_i8, a_s = orc.quantize_activations(a, m, k)
    a_i8 = a_i8.reshape(m, k)
    # (c)
    col = a_i8.astype(np.int64).sum(axis=0)
    wsum = q_t.reshape(n, k).astype(np.int64).sum(axis=0)
    assert int(acc.astype(np.int64).sum()) == int((col * wsum).sum())
    # (a)
    rng = np.random.default_rng(2)
    rows = np.arange(0, m, 32) + rng.integers(0, 32, size=(m + 31) // 32)
    rows = rows[rows < m]
    want, want_acc = orc.matmul_quantized(a[rows], len(rows), k, q_t, s, n)
    assert (acc[rows] == want_acc.reshape(len(rows), n)).all()
    assert (bits(got[rows]) == bits(want.reshape(len(rows), n))).all()
    # (b)
    cols = np.unique(np.concatenate([rng.choice(n, 90, replace=False), [0, 31, 32, n - 33, n - 32, n - 1]]))
    wc = q_t.reshape(n, k)[cols].astype(np.float64)          # [cols, k]
    acc_c = (a_i8.astype(np.float64) @ wc.T).astype(np.int32)  # exact: every partial sum is an integer below 2^53
    assert (acc[:, cols] == acc_c).all()
    assert (bits(got[:, cols]) == bits(np_epilogue(acc_c, a_s, s[cols]))).all()
    # (d)
    da = DevBuf(ctx, host=a)
    dout = DevBuf(ctx, m * n * 4)
    _ffi.check(_ffi.lib.pg_matmul_quantized_dev(ctx.handle, da.ptr, m, k, qt._gpu, dout.ptr, None))
    ctx.sync()
    assert last_tile(ctx) == tile + (1,)
    assert (bits(dout.to_host(np.float32)) == bits(got).reshape(-1)).all(), "f32-only epilogue differs"
    qt.free_gpu()


# pg_gemm_w8a8_force_tile codes -> output tile
TILES = {1: (64, 64), 2: (256, 256), 3: (128, 256), 4: (128, 64), 5: (128, 128)}


@pytest.mark.parametrize("m,k,n", [(300, 512, 1000), (512, 384, 768), (70, 128, 257)])
def test_every_gemm_tile_gives_the_same_bits(ctx, orc, m, k, n):
    """Each instantiation of the matrix-core kernel, forced in turn on ragged and whole-tile
    shapes, with and without the accumulator dump, against the oracle."""
    from peregrine_amd import quant, _ffi
    a = outlier_acts(orc, 99 + m, m, k)
    w = orc.rng_normal(55 + n, k * n, 0.0, 0.02)
    q, q_t, s = orc.quantize_weights(w, k, n)
    qt = quant.QuantizedTensor(q, q_t, s, k, n).to_gpu(ctx)
    want, want_acc = orc.matmul_quantized(a, m, k, q_t, s, n)
    da = DevBuf(ctx, host=a)
    dout, dacc = DevBuf(ctx, m * n * 4), DevBuf(ctx, m * n * 4)
    try:
        for code, tile in TILES.items():
            say(f"gemm tile {tile} on m={m} k={k} n={n}")
            _ffi.check(_ffi.lib.pg_gemm_w8a8_force_tile(ctx.handle, code))
            for acc_ptr in (dacc.ptr, None):
                _ffi.check(_ffi.lib.pg_matmul_quantized_dev(ctx.handle, da.ptr, m, k, qt._gpu, dout.ptr, acc_ptr))
                ctx.sync()
                bm, bn, sp = last_tile(ctx)
                if sp == 1:  # (a split product keeps its own row tile)
                    assert (bm, bn) == tile
                assert (bits(dout.to_host(np.float32)) == bits(want)).all(), f"tile {tile}: f32 outputs differ"
            assert (dacc.to_host(np.int32) == want_acc).all(), f"tile {tile}: accumulators differ"
    finally:
        _ffi.check(_ffi.lib.pg_gemm_w8a8_force_tile(ctx.handle, 0))
    assert _ffi.lib.pg_gemm_w8a8_force_tile(ctx.handle, 9) == _ffi.PG_EINVAL
    qt.free_gpu()


def run_multi(ctx, da, m, k, qts, douts):
    from peregrine_amd import _ffi
    wtab = (C.c_void_p * len(qts))(*[q._gpu.value for q in qts])
    otab = (C.c_void_p * len(qts))(*[d.ptr.value for d in douts])
    _ffi.check(_ffi.lib.pg_matmul_quantized_multi_dev(ctx.handle, da.ptr, m, k, wtab, len(qts), otab))
    ctx.sync()


@pytest.mark.parametrize("m,k,ns", [(300, 512, (1000, 130, 257)), (257, 128, (64, 64, 64, 64)), (40, 1024, (300, 77)),
                                     (1, 4096, (1024, 512)), (1, 14336, (300, 77, 4096)), (3, 200, (33,)), (2048, 4096, (4096, 1024, 1024)),
                                     (2048, 4096, (14336, 14336)), (8, 4096, (4096, 1024, 1030)), (32, 1000, (8200, 520)),
                                     (1, 4096, (14336, 14336))],
                         ids=["ragged3", "four", "few-rows", "one-row", "one-row-long-k", "single", "qkv", "gate-up",
                              "qkv-8-rows-quantised-once", "32-rows-quantised-once", "one-row-gate-up-as-the-decode-benchmark-runs-it"])
def test_matmul_quantized_multi_equals_the_single_products(ctx, orc, m, k, ns):
    """Several weights against one activation matrix (the reference's fused QKV / gate|up
    products): every output equals the single product bit for bit, and sampled rows equal the
    oracle."""
    from peregrine_amd import quant, _ffi
    say(f"matmul_quantized_multi m={m} k={k} ns={ns}")
    a = outlier_acts(orc, 7 + m, m, k)
    da = DevBuf(ctx, host=a)
    qts, parts = [], []
    for i, n in enumerate(ns):
        w = orc.rng_normal(100 + 13 * i + n, k * n, 0.0, 0.02)
        q, q_t, s = orc.quantize_weights(w, k, n)
        parts.append((q_t, s))
        qts.append(quant.QuantizedTensor(q, q_t, s, k, n).to_gpu(ctx))
    douts = [DevBuf(ctx, m * n * 4) for n in ns]
    run_multi(ctx, da, m, k, qts, douts)
    if m == 2048:
        assert last_tile(ctx)[:2] == (256, 256)  # gate, up: a launch each; q|k|v: one launch of 192 tiles
    rows = np.unique(np.random.default_rng(3).choice(m, min(m, 24), replace=False))
    single = DevBuf(ctx, m * max(ns) * 4)
    for i, n in enumerate(ns):
        got = douts[i].to_host(np.float32)
        _ffi.check(_ffi.lib.pg_matmul_quantized_dev(ctx.handle, da.ptr, m, k, qts[i]._gpu, single.ptr, None))
        ctx.sync()
        assert (bits(got) == bits(single.to_host(np.float32, m * n))).all(), f"weight {i}: differs from the single product"
        want, _ = orc.matmul_quantized(a[rows], len(rows), k, parts[i][0], parts[i][1], n)
        assert (bits(got.reshape(m, n)[rows]) == bits(want.reshape(len(rows), n))).all(), f"weight {i}: differs from the oracle"
    # argument errors: too many weights, a weight with another k
    five = (C.c_void_p * 5)(*[qts[0]._gpu.value] * 5)
    outs5 = (C.c_void_p * 5)(*[douts[0].ptr.value] * 5)
    assert _ffi.lib.pg_matmul_quantized_multi_dev(ctx.handle, da.ptr, m, k, five, 5, outs5) == _ffi.PG_EINVAL
    assert _ffi.lib.pg_matmul_quantized_multi_dev(ctx.handle, da.ptr, m, k + 1, five, 1, outs5) == _ffi.PG_EINVAL
    for qt in qts:
        qt.free_gpu()


def test_wire_record_straight_to_device(ctx, orc):
    """read_quantized_tensor + to_gpu in one call (reference src/serial.rs:161-222,
    src/quant.rs:174-181): the device tensor multiplies exactly like the original."""
    import io
    import ctypes as C
    from peregrine_amd import serial, _ffi
    from peregrine_amd.quant import QuantizedTensor
    say("wire record -> device tensor")
    rows, cols, m = 96, 40, 3
    w = orc.rng_normal(31, rows * cols, 0.0, 0.02)
    q, q_t, s = orc.quantize_weights(w, rows, cols)
    buf = io.BytesIO()
    serial.write_quantized_tensor(buf, "odd", QuantizedTensor(q, q_t, s, rows, cols))  # 3-byte name: unaligned payload
    h, used = serial.quantized_tensor_to_gpu(buf.getvalue() + b"trailing", ctx)
    assert used == len(buf.getvalue())
    a = orc.rng_normal(32, m * rows)
    out = np.empty(m * cols, np.float32)
    _ffi.check(_ffi.lib.pg_matmul_quantized(ctx.handle, C.c_void_p(a.ctypes.data), m, rows, h, C.c_void_p(out.ctypes.data)))
    want, _ = orc.matmul_quantized(a, m, rows, q_t, s, cols)
    assert (out.view(np.uint32) == want.view(np.uint32)).all()
    _ffi.lib.pg_qtensor_free(ctx.handle, h)


W8A32_SHAPES = [(32, 128, 64), (1, 4096, 1024), (3, 200, 77), (70, 4096, 300), (191, 256, 130),
                # from 192 rows the three digit planes run as one product over the stacked planes
                (192, 512, 300), (256, 384, 256), (300, 1000, 520), (700, 256, 1000)]


@pytest.mark.parametrize("m,k,n", W8A32_SHAPES)
def test_matmul_dequant_i8_vs_oracle(ctx, orc, m, k, n):
    """W8A32, the reference's GPU numerics (src/metal/shaders.rs:2329-2375).  Two bars: against
    the exact (float64) product of the same f32 activations and dequantised weights, 1e-5 of
    max(|ref|, rms(ref)) -- this implementation's own error (23/24-bit fixed point per row, so a
    row with x20 outlier channels loses ~6 bits on its ordinary elements; exact integer sums);
    against the oracle's K-sequential f32 sum, 2e-5 -- at K = 4096 that sum itself carries up to
    ~1e-5 of rounding error."""
    from peregrine_amd import quant
    say(f"matmul_dequant_i8 m={m} k={k} n={n}")
    a = orc.rng_normal(11 + m, m * k)
    a.reshape(m, k)[:, :: max(1, k // 37)] *= 20
    w = orc.rng_normal(12 + n, k * n, 0.0, 0.02)
    q, q_t, s = orc.quantize_weights(w, k, n)
    qt = quant.QuantizedTensor(q, q_t, s, k, n)
    got = quant.matmul_dequant_i8(a, m, k, qt, ctx).reshape(m, n)
    want = orc.matmul_dequant_i8(a, m, k, q, s, n).reshape(m, n)
    exact = a.reshape(m, k).astype(np.float64) @ orc.dequantize(q, s, k, n).reshape(k, n).astype(np.float64)
    for r in range(m):
        H.assert_close_rel(got[r], exact[r], 1e-5, f"row {r} vs exact")
        H.assert_close_rel(got[r], want[r], 2e-5, f"row {r} vs f32 oracle")
    qt.free_gpu()


def test_matmul_dequant_i8_combining_epilogue_on_every_tile(ctx, orc):
    """From 192 rows the product of the plane of weight 65536 finishes the sum in its epilogue (it reads the other
    two planes' accumulators).  Every tile shape of the matrix-core kernel in turn, on a ragged shape (the
    bounds-checked epilogue at the edges, the straight-line one inside), and two shapes that the dispatcher
    itself gives 256x256 tiles (whole tiles only, and ragged): exact small integers in, exact integers out, and
    the float64 product as the bar for random data."""
    from peregrine_amd import quant, _ffi
    for m, k, n, force in [(300, 256, 520, c) for c in TILES] + [(2048, 128, 5888, 0), (2050, 128, 5900, 0)]:
        say(f"matmul_dequant_i8 m={m} k={k} n={n} tile override {force}")
        a = orc.rng_normal(21 + m, m * k)
        a.reshape(m, k)[:, :: max(1, k // 37)] *= 20
        w = orc.rng_normal(22 + n, k * n, 0.0, 0.02)
        q, q_t, s = orc.quantize_weights(w, k, n)
        qt = quant.QuantizedTensor(q, q_t, s, k, n)
        ai = (np.arange(m * k, dtype=np.float32) % 9 - 4).reshape(m, k)
        qi = (np.arange(k * n).reshape(k, n) % 13 - 6).astype(np.int8)
        qt_int = quant.QuantizedTensor(qi.reshape(-1), np.ascontiguousarray(qi.T).reshape(-1), np.ones(n, np.float32), k, n)
        try:
            _ffi.check(_ffi.lib.pg_gemm_w8a8_force_tile(ctx.handle, force))
            got = quant.matmul_dequant_i8(a, m, k, qt, ctx).reshape(m, n)
            if force:
                assert last_tile(ctx)[:2] == TILES[force]
            else:
                assert last_tile(ctx)[:2] == (256, 256)
            got_int = quant.matmul_dequant_i8(ai, m, k, qt_int, ctx).reshape(m, n)
        finally:
            _ffi.check(_ffi.lib.pg_gemm_w8a8_force_tile(ctx.handle, 0))
        assert (got_int == (ai.astype(np.int64) @ qi.astype(np.int64))).all(), "integer inputs: the product is not exact"
        exact = a.reshape(m, k).astype(np.float64) @ orc.dequantize(q, s, k, n).reshape(k, n).astype(np.float64)
        for r in range(m):
            H.assert_close_rel(got[r], exact[r], 1e-5, f"row {r} vs exact")
        qt.free_gpu()
        qt_int.free_gpu()


def test_matmul_dequant_i8_reference_tolerance_and_closed_form(ctx, orc):
    """tests/quant_parity.rs:79-146 restated: the W8A32 result is within 10 % / 0.02 of the f32
    product of the unquantised weights; plus integer inputs with unit scales give exact integers,
    zero rows give zeros and a NaN poisons exactly its row."""
    from peregrine_amd import quant
    m, k, n = 32, 128, 64
    a = H.mod_pattern(m * k, 7, 3, 200, 200, 0.5)
    w = H.mod_pattern(k * n, 13, 7, 200, 200, 0.5)
    qt = quant.quantize_weights(w, k, n, ctx)
    got = quant.matmul_dequant_i8(a, m, k, qt, ctx)
    ref = orc.matmul_f32(a, w, m, k, n)
    diff = np.abs(got - ref)
    assert ((diff / np.maximum(np.abs(ref), 1e-6) < 0.10) | (diff < 0.02)).all()
    ai = (np.arange(m * k, dtype=np.float32) % 9 - 4).reshape(m, k)
    ai[3] = 0
    qi = (np.arange(k * n).reshape(k, n) % 13 - 6).astype(np.int8)
    qt2 = quant.QuantizedTensor(qi.reshape(-1), np.ascontiguousarray(qi.T).reshape(-1), np.ones(n, np.float32), k, n)
    got = quant.matmul_dequant_i8(ai, m, k, qt2, ctx).reshape(m, n)
    assert (got == ai.astype(np.int64) @ qi.astype(np.int64)).all() and (got[3] == 0).all()
    ai[5, 17] = np.nan
    got = quant.matmul_dequant_i8(ai, m, k, qt2, ctx).reshape(m, n)
    assert np.isnan(got[5]).all() and np.isfinite(np.delete(got, 5, axis=0)).all()
    with pytest.raises(ValueError):
        quant.matmul_dequant_i8(ai, m, k + 1, qt2, ctx)
