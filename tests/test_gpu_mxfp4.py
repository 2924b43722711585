"""GPU parity of the MXFP4 path (examples/gpt_oss/moe.rs) against the CPU oracle, through the
C ABI.  Bar: the block-dequant contract, 1e-3 relative (H.assert_close_rel); the fixed-point
kernel is exact up to the final f32 roundings, so the tests also hold it to 2e-5."""
import ctypes as C
import sys

import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu
RTOL_CONTRACT, RTOL_ACHIEVED = 1e-3, 2e-5


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _weights(rng, n, k, lo=118, hi=124):
    return (rng.integers(0, 256, n * k // 2, dtype=np.uint8), rng.integers(lo, hi, n * k // 32, dtype=np.uint8))


def test_mxfp4_codes_scales_and_order_exact(ctx, orc):
    """One-hot inputs read single weights back: every code, both nibbles, a spread of scale bytes."""
    from peregrine_amd import mxfp4
    in_dim, out_dim = 64, 16
    blocks = np.zeros((out_dim, 2, 16), np.uint8)
    for r in range(out_dim):
        blocks[r, 0, 0] = r                    # code r in the low nibble of element 0
        blocks[r, 1, 5] = r << 4               # code r in the high nibble of element 32 + 11
    scales = np.full((out_dim, 2), 127, np.uint8)
    for pos in (0, 1, 43, 42):
        x = np.zeros(in_dim, np.float32)
        x[pos] = 3.0
        got = mxfp4.mxfp4_matmul(x, blocks, scales, out_dim, in_dim, ctx)
        assert (got == orc.mxfp4_matmul(x, blocks, scales, out_dim, in_dim)).all(), pos
    x = np.zeros(in_dim, np.float32)
    x[0] = 1.0
    one = np.zeros((1, 2, 16), np.uint8)
    one[0, 0, 0] = 2
    for e in (0, 1, 2, 60, 126, 127, 128, 200, 253, 254):
        s = np.array([[e, 127]], np.uint8)
        got = mxfp4.mxfp4_matmul(x, one, s, 1, in_dim, ctx)[0]
        want = orc.mxfp4_matmul(x, one, s, 1, in_dim)[0]
        assert got == want, (e, got, want)


@pytest.mark.parametrize("out_dim,in_dim", [(5760, 2880), (2880, 2880), (33, 96), (1, 32), (257, 8192 + 32)])
def test_mxfp4_matmul(ctx, orc, out_dim, in_dim):
    """gpt-oss shapes (hidden 2880, mlp1 rows 2 x 2880) and ragged ones."""
    from peregrine_amd import mxfp4
    say(f"mxfp4 matmul [{in_dim}] -> [{out_dim}]")
    rng = np.random.default_rng(out_dim + in_dim)
    b, s = _weights(rng, out_dim, in_dim)
    x = orc.rng_normal(out_dim, in_dim)
    x[::97] *= 20.0
    got = mxfp4.mxfp4_matmul(x, b, s, out_dim, in_dim, ctx)
    want = orc.mxfp4_matmul(x, b, s, out_dim, in_dim)
    H.assert_close_rel(got, want, RTOL_CONTRACT, "mxfp4 contract")
    H.assert_close_rel(got, want, RTOL_ACHIEVED, "mxfp4 achieved")


def test_mxfp4_resident_weight_rows_and_errors(ctx, orc):
    from peregrine_amd import mxfp4, _ffi
    rng = np.random.default_rng(5)
    out_dim, in_dim, m = 200, 256, 7
    b, s = _weights(rng, out_dim, in_dim, 100, 150)
    w = mxfp4.upload(b, s, out_dim, in_dim, ctx)
    assert (w.n_out, w.k_in, w.ggml_type) == (out_dim, in_dim, _ffi.MXFP4)
    x = orc.rng_normal(3, m * in_dim).reshape(m, in_dim)
    got = w.matmul(x, m).reshape(m, out_dim)
    for i in range(m):
        H.assert_close_rel(got[i], orc.mxfp4_matmul(x[i], b, s, out_dim, in_dim), RTOL_ACHIEVED, f"row {i}")
    with pytest.raises(ValueError):
        mxfp4.mxfp4_matmul(x[0], b, s, out_dim, in_dim + 1, ctx)
    with pytest.raises(ValueError):
        mxfp4.mxfp4_matmul(x[0], b[:-1], s, out_dim, in_dim, ctx)


@pytest.mark.parametrize("m", [1, 3, 40])
def test_mxfp4_expert_forward(ctx, orc, m):
    from peregrine_amd import mxfp4
    hidden, inter, alpha, clamp = 2880, 2880, 1.702, 7.0
    say(f"mxfp4 expert hidden={hidden} intermediate={inter} m={m}")
    rng = np.random.default_rng(21)
    b1, s1 = _weights(rng, 2 * inter, hidden, 116, 120)
    b2, s2 = _weights(rng, hidden, inter, 116, 120)
    bias1 = orc.rng_normal(1, 2 * inter)
    bias2 = orc.rng_normal(2, hidden)
    ex = mxfp4.Mxfp4Expert(hidden, inter, alpha, clamp, b1, s1, b2, s2, bias1, bias2, ctx)
    x = orc.rng_normal(4, m * hidden).reshape(m, hidden)
    got = ex.forward(x if m > 1 else x[0]).reshape(m, hidden)
    for i in range(0, m, 1 if m < 8 else 9):   # (24 rows and more: both products take the matrix-core block product)
        want = orc.mxfp4_expert_forward(x[i], hidden, inter, alpha, clamp, b1, s1, b2, s2, bias1, bias2)
        H.assert_close_rel(got[i], want, RTOL_CONTRACT, f"mxfp4 expert row {i}")
        H.assert_close_rel(got[i], want, 1e-4 if m < 8 else 6e-4, f"mxfp4 expert row {i} (achieved)")


@pytest.mark.parametrize("out_dim,in_dim,m", [(4096, 14336, 1), (14336, 4096, 2), (600, 512, 5), (48, 28160, 1), (8200, 1024, 3)])
def test_mxfp4_workgroup_shapes(ctx, orc, out_dim, in_dim, m):
    """One case per launch shape of the product kernel: 16 wavefronts on one row group (few row groups),
    8 wavefronts on 1, 2 or 4 row groups, one to three activation rows per pass, several passes (m = 5),
    and K at the upper limit of what the digit planes in LDS hold."""
    from peregrine_amd import mxfp4
    say(f"mxfp4 shapes [{m} x {in_dim}] -> [{out_dim}]")
    rng = np.random.default_rng(out_dim * 7 + in_dim + m)
    b, s = _weights(rng, out_dim, in_dim)
    w = mxfp4.upload(b, s, out_dim, in_dim, ctx)
    x = orc.rng_normal(m + 11, m * in_dim).reshape(m, in_dim)
    x[:, ::89] *= 30.0
    got = w.matmul(x, m).reshape(m, out_dim)
    rows = rng.choice(out_dim, size=min(out_dim, 256), replace=False)   # the oracle on a sample of the weight rows
    bb = b.reshape(out_dim, -1)[rows].reshape(-1)
    ss = s.reshape(out_dim, -1)[rows].reshape(-1)
    for i in range(m):
        want = orc.mxfp4_matmul(x[i], bb, ss, len(rows), in_dim)
        H.assert_close_rel(got[i][rows], want, RTOL_ACHIEVED, f"row {i}")
    w.free()


RTOL_TILES = 1e-4   # four planes of base-32 digits per activation block: 20 bits under the block's largest value


@pytest.mark.parametrize("out_dim,in_dim,m,lo,hi,plan", [
    (2880, 2880, 24, 118, 124, (1, 2, 3)), (8192, 4096, 16, 118, 124, (1, 1, 4)), (5760, 2880, 100, 118, 124, (1, 4, 2)),
    (600, 4096, 300, 104, 144, (1, 4, 4)), (520, 512, 40, 100, 150, (1, 4, 1)),          # narrow row tiles, K in runs
    (8192, 256, 512, 100, 150, (2, 4, 1)), (14336, 128, 640, 110, 140, (4, 4, 1)),          # wider row tiles, one run
    (70000, 512, 16, 110, 140, (2, 1, 1)), (70000, 512, 32, 110, 140, (2, 2, 1)),
    (140000, 256, 16, 110, 140, (4, 1, 1)), (140000, 256, 30, 110, 140, (4, 2, 1)),
    (37, 96, 50, 0, 255, (1, 4, 1)),                                                         # every scale byte, ragged everything
])
def test_mxfp4_many_rows(ctx, orc, out_dim, in_dim, m, lo, hi, plan):
    """From 16 activation rows on (24 for a small tensor) the tile kernel on the scaled matrix-core instruction takes the
    product, whatever the block scales: the rows as four planes of base-32 digits (RTOL_TILES with x25 outlier
    channels).  plan = (groups of 16 weight rows per wavefront, groups of 16 tokens per workgroup, runs of K) the
    launcher picks on a 256-CU part.  One row on the same tensor afterwards still takes the decode kernel."""
    from peregrine_amd import mxfp4, _ffi
    say(f"mxfp4 many rows [{m} x {in_dim}] -> [{out_dim}] scales {lo}..{hi - 1}")
    v, got_plan = [C.c_size_t() for _ in range(6)], [C.c_int() for _ in range(3)]
    _ffi.check(_ffi.lib.pg_audit_mxfp4_tiles(256, out_dim, in_dim, m, *[C.byref(x) for x in v], *[C.byref(x) for x in got_plan]))   # an MI355X has 256 CUs
    assert tuple(x.value for x in got_plan) == plan
    rng = np.random.default_rng(out_dim + 3 * in_dim + m)
    b, s = _weights(rng, out_dim, in_dim, lo, hi)
    if hi - lo < 200:
        s[:4] = (lo, hi - 1, 0, lo)            # both ends of the range and a zero block in row 0
    else:
        s[s == 255] = 254                      # (255 is NaN: its own test below)
    w = mxfp4.upload(b, s, out_dim, in_dim, ctx)
    x = orc.rng_normal(m + 5, m * in_dim).reshape(m, in_dim)
    x[:, ::61] *= 25.0
    ctx.profile_begin()
    got = w.matmul(x, m).reshape(m, out_dim)
    prof = ctx.profile_end()
    assert "mxfp4_tiles" in prof and "mxfp4_planes" in prof and ("gguf_mm_sum_parts" in prof) == (got_plan[2].value > 1), prof
    rows = np.concatenate([[0, out_dim - 1], rng.choice(np.arange(1, out_dim), size=min(out_dim - 1, 94), replace=False)])
    bb = b.reshape(out_dim, -1)[rows].reshape(-1)
    ss = s.reshape(out_dim, -1)[rows].reshape(-1)
    wide = hi - lo >= 200                       # scales spread over 2^254: compare where the f32 reference itself is finite
    for i in list(range(0, m, max(1, m // 12))) + [m - 1]:
        want = orc.mxfp4_matmul(x[i], bb, ss, len(rows), in_dim)
        ok = np.isfinite(want) & (np.abs(want) < 1e30) if wide else np.ones(len(rows), bool)
        assert ok.any()
        if wide:                                # each output has its own magnitude: element by element, relative to itself
            rel = np.abs(got[i][rows][ok].astype(np.float64) - want[ok]) / np.maximum(np.abs(want[ok].astype(np.float64)), 1e-300)
            assert np.median(rel) <= RTOL_TILES and (rel <= 5e-2).all(), (i, np.median(rel), rel.max())
        else:
            H.assert_close_rel(got[i][rows], want, RTOL_CONTRACT, f"row {i} (contract)")
            H.assert_close_rel(got[i][rows], want, RTOL_TILES, f"row {i} (achieved)")
    one = w.matmul(x[3], 1)
    if not wide:
        H.assert_close_rel(one[rows], orc.mxfp4_matmul(x[3], bb, ss, len(rows), in_dim), RTOL_ACHIEVED, "one row afterwards")
    xb = x.copy()
    xb[2, 7] = np.nan                           # a NaN poisons its row and no other
    gotb = w.matmul(xb, m).reshape(m, out_dim)
    assert np.isnan(gotb[2]).all() and (gotb[[0, 1, 3, m - 1]] == got[[0, 1, 3, m - 1]]).all()
    w.free()


def test_mxfp4_limits_and_non_finite(ctx, orc):
    from peregrine_amd import mxfp4, _ffi
    rng = np.random.default_rng(9)
    b, s = _weights(rng, 16, 28672)
    with pytest.raises(_ffi.PeregrineError):   # the row's digit planes no longer fit in LDS
        mxfp4.mxfp4_matmul(np.zeros(28672, np.float32), b, s, 16, 28672, ctx)
    out_dim, in_dim = 40, 128
    b, s = _weights(rng, out_dim, in_dim)
    x = orc.rng_normal(1, in_dim)
    base = mxfp4.mxfp4_matmul(x, b, s, out_dim, in_dim, ctx)
    assert np.isfinite(base).all()
    for bad in (np.nan, np.inf, -np.inf):       # the reference's f32 sum turns inf or NaN in every row as well
        xb = x.copy()
        xb[37] = bad
        got = mxfp4.mxfp4_matmul(xb, b, s, out_dim, in_dim, ctx)
        want = orc.mxfp4_matmul(xb, b, s, out_dim, in_dim)
        assert not np.isfinite(got).any() and not np.isfinite(want).any()
    s2 = s.copy().reshape(out_dim, -1)
    s2[3, 1] = 255                              # f32::from_bits(255 << 23) = inf: that row is lost, the others are not
    got = mxfp4.mxfp4_matmul(x, b, s2.reshape(-1), out_dim, in_dim, ctx)
    assert not np.isfinite(got[3]) and not np.isfinite(orc.mxfp4_matmul(x, b, s2.reshape(-1), out_dim, in_dim)[3])
    keep = np.arange(out_dim) != 3
    assert (got[keep] == base[keep]).all()
    s3 = s.copy().reshape(out_dim, -1)
    s3[5, :] = 0                                # f32::from_bits(0) = 0.0: the row is exactly zero
    got = mxfp4.mxfp4_matmul(x, b, s3.reshape(-1), out_dim, in_dim, ctx)
    assert got[5] == 0.0 and orc.mxfp4_matmul(x, b, s3.reshape(-1), out_dim, in_dim)[5] == 0.0


@pytest.mark.parametrize("hidden,inter,E,top_k,T", [
    (64, 96, 4, 2, 1), (128, 64, 32, 4, 8), (2880, 2880, 8, 4, 2),      # few pairs: the decode kernel, a workgroup column per pair
    (64, 96, 5, 3, 7), (256, 160, 8, 2, 64), (512, 512, 8, 4, 300), (128, 64, 32, 4, 40),
    (2880, 2880, 4, 2, 150),        # the gpt-oss expert shape; 75 tokens an expert on average
])
def test_mxfp4_moe_routed_follows_the_oracle(ctx, orc, hidden, inter, E, top_k, T):
    """MoELayer::forward over MXFP4 experts (examples/gpt_oss/moe.rs:286-352), every product one launch over all
    experts, against the reference's per-token walk; experts with no token, with one, and with more than a tile's."""
    from peregrine_amd import mxfp4
    from test_oracle_formats_pins import _mx_expert
    say(f"mxfp4 moe hidden={hidden} inter={inter} E={E} top_k={top_k} T={T}")
    rng = np.random.default_rng(hidden + inter + E + T)
    raw = [_mx_expert(rng, hidden, inter) for _ in range(E)]
    experts = [mxfp4.Mxfp4Expert(hidden, inter, 1.702, 7.0, *r, ctx=ctx) for r in raw]
    x = orc.rng_normal(T + 11, T * hidden).reshape(T, hidden)
    x[:, ::37] *= 10.0
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 0] -= 8.0                                    # expert 0 is (almost) never chosen
    idx, w = orc.gpt_oss_route(logits, np.zeros(E, np.float32), T, E, top_k)
    got = mxfp4.moe_forward_routed(x, idx, w, experts, ctx)
    rows = list(range(0, T, max(1, T // 10))) + [T - 1]
    want = orc.mxfp4_moe_routed(x[rows], len(rows), hidden, inter, 1.702, 7.0, top_k, np.asarray(idx).reshape(T, top_k)[rows],
                                np.asarray(w).reshape(T, top_k)[rows], raw)
    for j, t in enumerate(rows):
        H.assert_close_rel(got[t], want[j], RTOL_CONTRACT, f"token {t} (contract)")
        H.assert_close_rel(got[t], want[j], 2e-4, f"token {t} (achieved)")
    # one expert called alone on the tokens routed to it gives the same rows as the grouped launch did for those pairs
    e = int(np.bincount(np.asarray(idx).reshape(-1), minlength=E).argmax())
    toks = [t for t in range(T) if e in np.asarray(idx).reshape(T, top_k)[t]][:5]
    if top_k == 1 and toks:
        alone = experts[e].forward(x[toks])
        H.assert_close_rel(got[toks] / np.asarray(w).reshape(T, top_k)[toks], alone, 2e-4, "one expert alone")
    with pytest.raises(ValueError):
        mxfp4.moe_forward_routed(x, np.asarray(idx).reshape(T, top_k), np.asarray(w).reshape(T, top_k)[:, :1], experts, ctx)
    from peregrine_amd import _ffi
    bad = np.asarray(idx, np.int32).reshape(T, top_k).copy()
    bad[T - 1, 0] = E                                      # the reference's self.experts[expert_idx] would panic
    with pytest.raises(_ffi.PeregrineError):
        mxfp4.moe_forward_routed(x, bad, w, experts, ctx)
    if top_k > 1:
        bad[T - 1, 0] = bad[T - 1, 1]                      # an expert named twice by one token
        with pytest.raises(_ffi.PeregrineError):
            mxfp4.moe_forward_routed(x, bad, w, experts, ctx)
    for ex in experts:
        ex.free()
