"""GPU parity of the gguf::* path against the CPU oracle, through the C ABI.

Bars: f16 conversion and whole-tensor dequantisation are BIT-EXACT; the fused
dequantise-matmul matches the oracle's dequantise -> transpose -> f32 matmul within
1e-3 relative (H.assert_close_rel: relative to max(|ref|, rms(ref))); the tests also
assert the tighter bound the fixed-point kernels actually achieve: 1e-4 for Q4_0
(18-bit activation blocks) and 2e-5 for Q8_0 (22-bit), with x20 outlier channels present.
"""
import sys

import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

RTOL_CONTRACT = 1e-3                 # the stated tolerance for Q4_0/Q8_0 block-dequant paths
RTOL_ACHIEVED = {2: 1e-4, 3: 1e-4, 8: 2e-5}   # what the one-row (GEMV) path is held to, per ggml type
RTOL_ACHIEVED_MM = 4e-4              # several rows: 16-bit fixed-point activations per block


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def test_f16_to_f32_all_patterns_bit_exact(ctx, orc):
    from peregrine_amd import gguf
    b = np.arange(65536, dtype=np.uint16)
    got = gguf.f16_to_f32(b, ctx).view(np.uint32)
    assert (got == orc.f16_to_f32_bits(b)).all()  # includes subnormals and NaN payloads


def _random_blocks(rng, nblocks, bb):
    raw = rng.integers(0, 256, nblocks * bb, dtype=np.uint8).reshape(nblocks, bb)
    raw[:, 1] &= 0x7B  # finite f16 scale (and min for Q4_1 below)
    if bb == 20:
        raw[:, 3] &= 0x7B
    return raw


@pytest.mark.parametrize("name,bb", [("dequant_q8_0", 34), ("dequant_q4_0", 18), ("dequant_q4_1", 20)])
def test_dequant_bit_exact(ctx, orc, name, bb):
    from peregrine_amd import gguf
    say(name)
    rng = np.random.default_rng(bb)
    for nblocks in (1, 257, 4096):
        raw = _random_blocks(rng, nblocks, bb)
        raw[0, 0:2] = [0x01, 0x00]  # a subnormal scale
        got = getattr(gguf, name)(raw.tobytes(), nblocks * 32, ctx)
        want = getattr(orc, name)(raw.tobytes(), nblocks * 32)
        assert (bits(got) == bits(want)).all()
    assert getattr(gguf, name)(b"", 0, ctx).size == 0
    with pytest.raises(ValueError):
        getattr(gguf, name)(bytes(bb), 31, ctx)       # assert!(num_elements % 32 == 0)
    with pytest.raises(ValueError):
        getattr(gguf, name)(bytes(bb - 1), 32, ctx)   # assert!(data.len() >= ...)


def test_dequant_reference_known_answers(ctx):
    from peregrine_amd import gguf
    blk = bytes([0x00, 0x3C]) + bytes(range(32))                       # src/gguf.rs:588-601
    assert (gguf.dequant_q8_0(blk, 32, ctx) == np.arange(32)).all()
    blk = bytes([0x00, 0x3C]) + bytes([0x98] + [0x88] * 15)            # src/gguf.rs:604-615
    out = gguf.dequant_q4_0(blk, 32, ctx)
    assert out[0] == 0.0 and out[1] == 1.0 and (out[2:] == 0).all()
    blk = bytes([0x00, 0x3C, 0x00, 0x49]) + bytes(16)                  # tests/gguf_parity.rs:53-76
    assert (gguf.dequant_q4_1(blk, 32, ctx) == 10.0).all()


def test_load_tensor_q8_as_quantized(ctx, orc):
    # gguf.rs:386-401: Q8_0 -> f32 -> quantize_weights, bit-exact with the oracle's composition
    from peregrine_amd import gguf
    rows, cols = 48, 96
    w = orc.rng_normal(31, rows * cols, 0.0, 0.02)
    raw = H.pack_q8_0(w)
    qt = gguf.load_tensor_q8_as_quantized(raw, rows, cols, ctx)
    q, q_t, s = orc.quantize_weights(orc.dequant_q8_0(raw, rows * cols), rows, cols)
    assert (qt.data_i8 == q).all() and (qt.data_i8_t == q_t).all() and (bits(qt.scales) == bits(s)).all()


# (type, n_out, k_in, m)
GGUF_SHAPES = [
    (2, 256, 4096, 1), (2, 256, 4096, 4), (2, 256, 4096, 16),   # benchmark configuration 4 row counts
    (2, 77, 96, 3), (2, 1000, 2048, 2), (2, 128, 14336, 1),     # ragged n, 1 / 7 blocks per lane
    (2, 64, 32768, 2),                                          # two K segments
    (2, 50, 11008, 1),                                          # partial last lane group
    (8, 256, 4096, 1), (8, 77, 96, 3), (8, 96, 6144, 4), (8, 64, 32768, 2),
    (2, 100, 32768, 1), (2, 40, 64, 1), (2, 9, 32, 1), (2, 8192, 512, 1), (2, 4096, 4096, 1),   # Q4_0 one-launch row product: longest K, spare wavefronts, most rows
    (2, 64, 32800, 1), (2, 8200, 256, 1), (8, 33, 32768, 1), (8, 9, 32, 1),   # past its limits (K, rows) and Q8_0: digits by a launch of their own
    (2, 14336, 4096, 1),                                        # benchmark configuration 4, full size
    (8, 6144, 4096, 1),
    (8, 4096, 14336, 1), (8, 300, 8192, 1), (8, 24, 16384, 1),  # two rows a wavefront under a long row: the digits shared through LDS (ragged last workgroups)
    # more than one row: matrix-core path (token tiles of 32, row tiles of 128, split K)
    (2, 130, 224, 33), (8, 131, 160, 40), (2, 515, 4096, 64), (8, 257, 6144, 35), (2, 14336, 4096, 4), (8, 4096, 14336, 16),
    # Q4_0, two rows over at most 2^24 weights, K up to 8192: one launch, every wavefront's weight rows against both
    # activation rows (the one-row kernel's arithmetic: its tolerance); ragged rows and K segments
    (2, 4096, 4096, 2), (2, 1003, 2080, 2), (2, 33, 96, 2), (2, 520, 8192, 2), (2, 8190, 1024, 2),
    (2, 14336, 4096, 2), (2, 4096, 4096, 3), (2, 1003, 2080, 3), (2, 8190, 1024, 3),
    (2, 4096, 14336, 2), (2, 4096, 14336, 3), (2, 33, 96, 4),   # (more weights, longer K or more rows: matrix cores)
    # Q4_0, 3 .. 16 rows, K a multiple of 256: digits, then ONE matrix-core launch (a workgroup per 16 weight rows, its
    # wavefronts on runs of K with private LDS rings): rings of 4, 8 and 16 token rows, 1 to 8 wavefronts, ragged rows,
    # a K of 4 and of 9 units; 12 rows over a wide tensor keep the product split over K
    (2, 1000, 4096, 7), (2, 333, 1024, 5), (2, 4100, 8192, 16), (2, 96, 2304, 9), (2, 14336, 4096, 12), (2, 4096, 14336, 8),
    (2, 4096, 4096, 5), (2, 40, 36864, 4),
    # up to 8 rows: 4 x 4 x 4 products; from 32 weight rows a CU on two weight tiles a workgroup (ragged last workgroup)
    (2, 14336, 4096, 7), (2, 8200, 1024, 6), (2, 8200, 1024, 3), (8, 8200, 1280, 5), (8, 8200, 1280, 2),
    # the same over Q8_0 (a weight row is two streams of 16-byte half blocks)
    (8, 1000, 4096, 7), (8, 333, 1024, 2), (8, 4100, 8192, 16), (8, 96, 2304, 9), (8, 14336, 4096, 4), (8, 4096, 14336, 8), (8, 14336, 4096, 12),
    # Q4_1 (offset blocks): the streaming kernel with the block-sum term, one item per row
    (3, 256, 4096, 1), (3, 77, 96, 3), (3, 1000, 2048, 2), (3, 50, 11008, 1), (3, 64, 32768, 2), (3, 14336, 4096, 1), (3, 130, 224, 33),
    # Q4_1 from four rows on: the Q4_0 matrix-core product on the same nibbles plus the offsets times the rows' block sums
    (3, 256, 4096, 8), (3, 515, 4096, 64), (3, 14336, 4096, 16), (3, 600, 256, 545), (3, 100, 32768, 9), (3, 40, 32800, 8), (3, 256, 4096, 7),
    # 16 token tiles and more: no split K, XCD-aware super-tiles of 4 row groups x 8 token tiles (ragged on both sides)
    (2, 600, 256, 545), (8, 1100, 128, 700), (2, 128, 512, 512),
]


@pytest.mark.parametrize("typ,n_out,k_in,m", GGUF_SHAPES)
def test_gguf_matmul_vs_oracle(ctx, orc, typ, n_out, k_in, m):
    from peregrine_amd import gguf
    say(f"gguf_matmul type={typ} n_out={n_out} k_in={k_in} m={m}")
    w = orc.rng_normal(900 + n_out + typ, n_out * k_in, 0.0, 0.02)
    if typ == 3:
        w = w + np.float32(0.03)                      # off-centre, so that the block offsets matter
    raw = {2: H.pack_q4_0, 3: H.pack_q4_1, 8: H.pack_q8_0}[typ](w)
    x = orc.rng_normal(17 + m, m * k_in)
    x.reshape(m, k_in)[:, :: max(1, k_in // 40)] *= 20
    gw = gguf.GgufWeight(raw, typ, n_out, k_in, ctx)
    got = gw.matmul(x, m)
    want = orc.gguf_matmul(x, m, raw, typ, n_out, k_in)
    for r in range(m):
        sl = slice(r * n_out, (r + 1) * n_out)
        H.assert_close_rel(got[sl], want[sl], RTOL_CONTRACT, f"row {r} (contract)")
        few_rows = typ == 2 and m == 2 and n_out * k_in <= 1 << 24 and k_in <= 8192
        streaming = m == 1 or few_rows or (typ == 3 and (m < 8 or k_in > 32768)) or k_in < 160
        H.assert_close_rel(got[sl], want[sl], RTOL_ACHIEVED[typ] if streaming else RTOL_ACHIEVED_MM, f"row {r} (achieved)")
    gw.free()


def test_gguf_matmul_full_size_m16_and_linearity(ctx, orc):
    """benchmark configuration 4 at M = 16, full size, plus a size-independent property: the product
    is linear in x, so y(x1 + x2) - y(x1) - y(x2) is zero up to rounding."""
    from peregrine_amd import gguf
    n_out, k_in, m = 14336, 4096, 16
    say(f"gguf_matmul full size n_out={n_out} k_in={k_in} m={m}")
    w = orc.rng_normal(4242, n_out * k_in, 0.0, 0.02)
    raw = H.pack_q4_0(w)
    x = orc.rng_normal(99, m * k_in)
    gw = gguf.GgufWeight(raw, 2, n_out, k_in, ctx)
    got = gw.matmul(x, m).reshape(m, n_out)
    want = orc.gguf_matmul(x, m, raw, 2, n_out, k_in).reshape(m, n_out)
    for r in range(m):
        H.assert_close_rel(got[r], want[r], RTOL_ACHIEVED_MM, f"row {r}")
    xs = x.reshape(m, k_in)
    y12 = gw.matmul(xs[0] + xs[1], 1)
    H.assert_close_rel(y12, got[0].astype(np.float64) + got[1], RTOL_ACHIEVED_MM, "linearity")
    gw.free()


@pytest.mark.parametrize("typ", [2, 8])
def test_prepare_makes_the_derived_copies_up_front(ctx, orc, typ):
    """pg_gguf_prepare: the tile-major copy exists before the first many-row product, the product's bits do not
    depend on who made it, one-row preparation makes nothing, and pg_gguf_drop_prepared gives the memory back."""
    from peregrine_amd import gguf
    n_out, k_in, m = 384, 1024, 40
    say(f"gguf prepare typ={typ}")
    raw = (H.pack_q4_0 if typ == 2 else H.pack_q8_0)(orc.rng_normal(77, n_out * k_in, 0.0, 0.02))
    x = orc.rng_normal(78, m * k_in)
    lazy = gguf.GgufWeight(raw, typ, n_out, k_in, ctx)
    eager = gguf.GgufWeight(raw, typ, n_out, k_in, ctx)
    up, der = eager.device_bytes()
    assert up == n_out * k_in // 32 * (18 if typ == 2 else 34) and der == 0
    eager.prepare(1)
    assert eager.device_bytes()[1] == 0
    eager.prepare(m)
    der = eager.device_bytes()[1]
    assert der >= n_out * k_in // 32 * (16 if typ == 2 else 32)
    y_eager = eager.matmul(x, m)
    assert eager.device_bytes()[1] == der           # the product made nothing more
    y_lazy = lazy.matmul(x, m)                      # makes its own copy on the way
    assert lazy.device_bytes()[1] == der
    assert (y_eager.view(np.uint32) == y_lazy.view(np.uint32)).all()
    H.assert_close_rel(y_eager, orc.gguf_matmul(x, m, raw, typ, n_out, k_in), RTOL_ACHIEVED_MM, "prepared product")
    eager.drop_prepared()
    assert eager.device_bytes()[1] == 0
    assert (eager.matmul(x, m).view(np.uint32) == y_lazy.view(np.uint32)).all()
    lazy.free()
    eager.free()


def test_gguf_matmul_special_inputs(ctx, orc):
    from peregrine_amd import gguf
    n_out, k_in = 40, 128
    w = orc.rng_normal(5, n_out * k_in, 0.0, 0.02)
    raw = H.pack_q4_0(w)
    gw = gguf.GgufWeight(raw, 2, n_out, k_in, ctx)
    assert (gw.matmul(np.zeros(k_in, np.float32), 1) == 0).all()           # zero row
    tiny = np.full(k_in, 1e-30, np.float32)
    H.assert_close_rel(gw.matmul(tiny, 1), orc.gguf_matmul(tiny, 1, raw, 2, n_out, k_in), RTOL_ACHIEVED[2], "tiny")
    big = orc.rng_normal(6, k_in) * np.float32(1e30)
    H.assert_close_rel(gw.matmul(big, 1), orc.gguf_matmul(big, 1, raw, 2, n_out, k_in), RTOL_ACHIEVED[2], "huge")
    bad = np.ones(k_in, np.float32)
    bad[3] = np.nan
    assert np.isnan(gw.matmul(bad, 1)).all() and np.isnan(orc.gguf_matmul(bad, 1, raw, 2, n_out, k_in)).all()
    # a device row that does not start on a 16-byte boundary is an argument error (128-bit loads)
    from devbuf import DevBuf
    from peregrine_amd import _ffi
    import ctypes as C
    shifted = DevBuf(ctx, host=np.zeros(k_in + 1, np.float32))
    dy = DevBuf(ctx, n_out * 4)
    assert _ffi.lib.pg_gguf_matmul_dev(ctx.handle, C.c_void_p(shifted.ptr.value + 4), 1, gw._h, dy.ptr) == _ffi.PG_EINVAL
    assert gw.matmul(np.zeros(0, np.float32), 0).size == 0                  # m = 0
    with pytest.raises(ValueError):
        gw.matmul(np.zeros(k_in + 1, np.float32), 1)
    with pytest.raises(ValueError):
        gguf.GgufWeight(raw, 2, n_out, k_in + 1, ctx)                       # k_in % 32
    gw.free()


# ---- many rows of Q4_0 / Q8_0 on the f16 matrix cores (weights exact, activations as two f16 planes) -----------
RTOL_F16_ROUTE = 2e-5   # what that route is held to: the planes drop less than 2^-22 of a row's largest value

# (n_out, k_in, m): forced onto the f16 route whatever the dispatcher would choose
HMM_SHAPES = [
    (512, 1024, 256),     # two full 256 x 256 tiles, K in two chunks
    (515, 4160, 300),     # ragged rows, weight rows and K chunks (65 stages in 8 chunks)
    (1400, 1088, 1000),   # 24 tiles, 17 stages, no split
    (1100, 2048, 100),    # up to 128 rows: 128 x 512 tiles, ragged
    (77, 256, 2),         # the smallest it takes: two rows, four stages, an odd number of weight rows
    (256, 4096, 129),     # one row past the wide tile
    (4096, 14336, 160),   # a long K in chunks under a half-empty row tile
]


@pytest.mark.parametrize("typ", [2, 8])
@pytest.mark.parametrize("n_out,k_in,m", HMM_SHAPES)
def test_gguf_matmul_f16_route_vs_oracle(ctx, orc, typ, n_out, k_in, m):
    from peregrine_amd import gguf, _ffi
    say(f"gguf_matmul f16 route type={typ} n_out={n_out} k_in={k_in} m={m}")
    w = orc.rng_normal(1900 + n_out, n_out * k_in, 0.0, 0.02)
    raw = (H.pack_q4_0 if typ == 2 else H.pack_q8_0)(w)
    x = orc.rng_normal(117 + m, m * k_in)
    x.reshape(m, k_in)[:, :: max(1, k_in // 40)] *= 20
    gw = gguf.GgufWeight(raw, typ, n_out, k_in, ctx)
    _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 1))
    try:
        ctx.profile_begin()
        got = gw.matmul(x, m)
        prof = ctx.profile_end()
        again = gw.matmul(x, m)
    finally:
        _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 0))
    assert ("gguf_hmm_q4_0" if typ == 2 else "gguf_hmm_q8_0") in prof and "rows_to_f16_planes" in prof, prof
    assert (bits(got) == bits(again)).all()
    rows = range(m) if m * n_out * k_in <= 1 << 31 else sorted({0, 1, m // 2, m - 2, m - 1})
    for r in rows:
        want = orc.gguf_matmul(x.reshape(m, k_in)[r], 1, raw, typ, n_out, k_in)
        H.assert_close_rel(got.reshape(m, n_out)[r], want, RTOL_F16_ROUTE, f"row {r}")
    gw.free()


def test_gguf_matmul_f16_route_prefill_size_is_the_dispatchers_choice(ctx, orc):
    """1024 rows over [4096] -> [14336] (a prefill's gate projection): the dispatcher takes the f16 route by itself;
    rows spot-checked against the oracle, and the int8 block route on the same input agrees within its own bar."""
    from peregrine_amd import gguf, _ffi
    n_out, k_in, m = 14336, 4096, 1024
    say(f"gguf_matmul prefill size n_out={n_out} k_in={k_in} m={m}")
    raw = H.pack_q4_0(orc.rng_normal(4343, n_out * k_in, 0.0, 0.02))
    x = orc.rng_normal(4344, m * k_in)
    gw = gguf.GgufWeight(raw, 2, n_out, k_in, ctx)
    ctx.profile_begin()
    got = gw.matmul(x, m).reshape(m, n_out)
    prof = ctx.profile_end()
    assert "gguf_hmm_q4_0" in prof, prof
    for r in (0, 255, 256, 700, 1023):
        want = orc.gguf_matmul(x.reshape(m, k_in)[r], 1, raw, 2, n_out, k_in)
        H.assert_close_rel(got[r], want, RTOL_F16_ROUTE, f"row {r}")
    _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 2))
    try:
        ctx.profile_begin()
        blockwise = gw.matmul(x, m).reshape(m, n_out)
        prof = ctx.profile_end()
    finally:
        _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 0))
    assert "gguf_hmm_q4_0" not in prof and "gguf_mm_q4_0" in prof, prof
    for r in (0, 511, 1023):
        H.assert_close_rel(blockwise[r], got[r], RTOL_ACHIEVED_MM, f"int8 block route, row {r}")
    gw.free()


def test_gguf_matmul_f16_route_special_rows(ctx, orc):
    """Zero, tiny, huge, denormal, NaN and infinite rows beside ordinary ones: each row has its own exponent."""
    from peregrine_amd import gguf, _ffi
    n_out, k_in, m = 300, 512, 130
    raw = H.pack_q4_0(orc.rng_normal(55, n_out * k_in, 0.0, 0.02))
    x = orc.rng_normal(56, m * k_in).reshape(m, k_in)
    x[1] = 0
    x[2] *= np.float32(1e-30)
    x[3] *= np.float32(1e30)
    x[4] *= np.float32(1e-41)      # denormal floats
    x[5, 7] = np.nan
    x[6, 9] = np.inf
    x[7, :] = 0
    x[7, 100] = 3.0                # one element: the result is 3 * that weight column, exactly representable inputs
    gw = gguf.GgufWeight(raw, 2, n_out, k_in, ctx)
    _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 1))
    try:
        got = gw.matmul(x.reshape(-1), m).reshape(m, n_out)
    finally:
        _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 0))
    assert (got[1] == 0).all()
    assert np.isnan(got[5]).all()
    assert not np.isfinite(got[6]).any()
    for r in (0, 2, 3, 7, 8, 129):
        want = orc.gguf_matmul(x[r], 1, raw, 2, n_out, k_in)
        H.assert_close_rel(got[r], want, RTOL_F16_ROUTE, f"row {r}")
    want = orc.gguf_matmul(x[4], 1, raw, 2, n_out, k_in)
    H.assert_close_rel(got[4], want, 1e-2, "denormal row")   # the inputs themselves carry only a few bits
    w_col = orc.gguf_matmul(x[7], 1, raw, 2, n_out, k_in)
    assert (bits(got[7]) == bits(w_col)).all()                # a single product per output: no rounding anywhere
    gw.free()


@pytest.mark.parametrize("n_out,k_in,m", [(515, 4160, 300), (1100, 2048, 100), (256, 256, 129)])
def test_gguf_matmul_f16_route_q4_1(ctx, orc, n_out, k_in, m):
    """Q4_1 at prefill sizes: the first term as the Q4_0 product on the f16 matrix cores (same nibbles and scales),
    then the launch that adds the blocks' offsets times the rows' block sums."""
    from peregrine_amd import gguf, _ffi
    say(f"gguf_matmul f16 route Q4_1 n_out={n_out} k_in={k_in} m={m}")
    w = orc.rng_normal(2900 + n_out, n_out * k_in, 0.0, 0.02) + np.float32(0.03)
    raw = H.pack_q4_1(w)
    x = orc.rng_normal(217 + m, m * k_in)
    x.reshape(m, k_in)[:, :: max(1, k_in // 40)] *= 20
    gw = gguf.GgufWeight(raw, 3, n_out, k_in, ctx)
    _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 1))
    try:
        ctx.profile_begin()
        got = gw.matmul(x, m).reshape(m, n_out)
        prof = ctx.profile_end()
    finally:
        _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 0))
    assert "gguf_hmm_q4_0" in prof and "gguf_q4_1_offsets" in prof, prof
    for r in sorted({0, 1, m // 2, m - 1}):
        want = orc.gguf_matmul(x.reshape(m, k_in)[r], 1, raw, 3, n_out, k_in)
        H.assert_close_rel(got[r], want, RTOL_ACHIEVED[3], f"row {r}")
    gw.free()


@pytest.mark.parametrize("typ,bb", [(2, 18), (8, 34)])
def test_gguf_matmul_f16_route_every_quant_value(ctx, orc, typ, bb):
    """Blocks of random bytes (every nibble and every int8 value, -128 included) with scales of both signs: the
    unpacking of quants into f16 values is exact for all of them."""
    from peregrine_amd import gguf, _ffi
    n_out, k_in, m = 96, 512, 5
    rng = np.random.default_rng(1234 + typ)
    nblocks = n_out * k_in // 32
    blocks = rng.integers(0, 256, size=(nblocks, bb), dtype=np.uint8)
    scales = (rng.choice([0.5, -0.25, 0.0625, 1.5, -3.0, 0.0], size=nblocks) * 0.01).astype(np.float16)
    blocks[:, :2] = scales.view(np.uint8).reshape(nblocks, 2)
    if typ == 8:
        blocks[0, 2:] = 0x80                       # a block of -128s
    raw = blocks.tobytes()
    x = orc.rng_normal(77, m * k_in)
    gw = gguf.GgufWeight(raw, typ, n_out, k_in, ctx)
    _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 1))
    try:
        got = gw.matmul(x, m).reshape(m, n_out)
    finally:
        _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 0))
    want = orc.gguf_matmul(x, m, raw, typ, n_out, k_in).reshape(m, n_out)
    for r in range(m):
        H.assert_close_rel(got[r], want[r], RTOL_F16_ROUTE, f"row {r}")
    gw.free()
