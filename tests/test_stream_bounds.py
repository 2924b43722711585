"""Bounds of the streaming kernels' loads, checked on the host: for every instantiation the dispatchers can pick,
over a grid of ragged shapes, the furthest byte any (workgroup, wavefront, lane, step) would load lies inside the
array the library allocates.  The library's pg_audit_* functions walk the launch with the index functions the
kernels themselves use (peregrine_amd/csrc/pg_stream_addr.h); no device is touched, so the test runs without a GPU.

Why it exists: the first one-row W8A8 kernels fetched chunk `lane` of a weight row for lanes past a row shorter
than 1024 bytes -- up to 896 bytes past the end of the tensor on its last rows.  The device only faults on such a
read when the tensor happens to end a mapping, so no GPU test saw it; K = 32 .. 992 below is that case."""
import ctypes as C
import itertools

import pytest

from peregrine_amd import _ffi

lib, check = _ffi.lib, _ffi.check


def _four():
    return [C.c_size_t() for _ in range(4)]


def _inside(vals, what):
    a_end, a_bytes, b_end, b_bytes = (v.value for v in vals)
    assert a_end <= a_bytes, f"{what}: first array read to byte {a_end} of {a_bytes}"
    assert b_end <= b_bytes, f"{what}: second array read to byte {b_end} of {b_bytes}"
    return a_end, a_bytes, b_end, b_bytes


RAGGED_K = [32, 36, 64, 100, 128, 132, 200, 256, 500, 512, 992, 1000, 1024, 1028, 2048, 4096, 4100, 8192, 14336, 16384]
RAGGED_N = [1, 7, 16, 17, 255, 256, 257, 1000, 4096]


def test_one_row_w8a8_loads_stay_inside_the_weight_plane():
    """gemv_w8a8_m1_kernel (4 wavefronts) and gemv_w8a8_m1_f32x_kernel (4, 8, 16) for NCH in {4, 8, 14, 16} and one or
    two rows per wavefront; K from 32 to 16384 (the row is padded to 128: NCH must cover it)."""
    seen_full = False
    for k, n in itertools.product(RAGGED_K, RAGGED_N):
        k_pad = (k + 127) // 128 * 128
        need = (k_pad // 16 + 63) // 64
        for nch in (4, 8, 14, 16):
            if nch < need:
                continue
            for nw, rpw, f32 in ((4, 1, 0), (4, 2, 0), (4, 1, 1), (4, 2, 1), (8, 1, 1), (8, 2, 1), (16, 1, 1)):
                if f32 and k % 4:
                    continue
                v = _four()
                check(lib.pg_audit_gemv_w8a8_m1(k, n, nch, rpw, nw, f32, *[C.byref(x) for x in v]))
                w_end, w_bytes, _, _ = _inside(v, f"gemv_w8a8_m1 k={k} n={n} NCH={nch} NW={nw} RPW={rpw} f32={f32}")
                seen_full |= w_end == w_bytes
    assert seen_full, "the walk never reached the end of a weight plane: it is not walking the kernel's space"


def test_one_row_w8a8_old_indexing_would_have_been_caught():
    """The audit is only worth something if it fails on the mistake it was written for: with `chunk = lane + 64 j`
    unclamped (what the kernels did), a row of 128 bytes is over-read by lanes 8 .. 63."""
    k_pad, n_pad, nchunk = 128, 256, 8
    worst = max(((n_pad - 1) * k_pad + (lane + 64 * j) * 16 + 16) for lane in range(64) for j in range(4))
    assert worst > n_pad * k_pad
    v = _four()
    check(lib.pg_audit_gemv_w8a8_m1(100, 256, 4, 1, 4, 0, *[C.byref(x) for x in v]))
    assert v[0].value == v[1].value == n_pad * k_pad


def test_few_rows_w8a8_fills_stay_inside_both_planes():
    """gemm_w8a8_skinny_kernel<MB, NB, NW, NST>: every (activation tiles, weight tiles, wavefronts) it is launched with."""
    combos = [(1, 1), (2, 1), (2, 2), (4, 1), (4, 2)]
    for k, n in itertools.product([128, 256, 384, 1000, 4096, 14336], RAGGED_N + [8200]):
        for (mb, nbt), nw in itertools.product(combos, (1, 2, 4, 8)):
            if mb == 4 and nw == 8:
                continue
            for m in {2, 16 * mb - 15, 16 * mb}:
                if m < 2:
                    continue
                v = _four()
                check(lib.pg_audit_gemm_w8a8_skinny(m, k, n, mb, nbt, nw, *[C.byref(x) for x in v]))
                _inside(v, f"gemm_w8a8_skinny m={m} k={k} n={n} MB={mb} NB={nbt} NW={nw}")


def test_block_gemv_loads_stay_inside_payload_and_scale_planes():
    """gguf_gemv_kernel and the few-rows form: blocks per lane 1 .. 4 (longer rows run as K segments), 2 / 4 / 8 rows
    per wavefront, 1 / 4 / 8 / 16 wavefronts per workgroup, Q4_0 and Q8_0 planes."""
    ks = [32, 64, 96, 2048, 2080, 4096, 6144, 8192, 8224, 14336, 32768]
    for k, n in itertools.product(ks, RAGGED_N + [14336]):
        nb = k // 32
        bpl = min(4, (nb + 63) // 64)
        for q8, rw, nw in itertools.product((0, 1), (2, 4, 8), (1, 4, 8, 16)):
            if rw * nw > 64:
                continue
            v = _four()
            check(lib.pg_audit_gguf_gemv(n, k, q8, bpl, rw, nw, *[C.byref(x) for x in v]))
            qs_end, qs_bytes, d_end, d_bytes = _inside(v, f"gguf_gemv n={n} k={k} q8={q8} BPL={bpl} RW={rw} NW={nw}")
            assert qs_end == qs_bytes          # the last row's last block is read by someone


def test_block_few_rows_fills_stay_inside_payload_and_scale_planes():
    """gguf_skinny_kernel: K a multiple of 256, every wavefront count, one or two weight tiles a workgroup."""
    for k, n in itertools.product([1024, 1280, 4096, 14336, 32768], RAGGED_N + [14336]):
        for q8, nw, tiles in itertools.product((0, 1), (1, 2, 4, 8), (1, 2)):
            v = _four()
            check(lib.pg_audit_gguf_skinny(n, k, q8, nw, tiles, *[C.byref(x) for x in v]))
            qs_end, qs_bytes, d_end, d_bytes = _inside(v, f"gguf_skinny n={n} k={k} q8={q8} NW={nw} NB={tiles}")
            assert qs_end == qs_bytes and d_end == d_bytes


def test_f16_matrix_core_fills_stay_inside_planes_payload_and_scales():
    """gguf_hmm_kernel: Q4_0 and Q8_0, both tile shapes, ragged rows on both sides, every K chunk count the dispatcher can pick
    (chunks of whole stages of 64), odd numbers of weight rows (the scale fill takes rows in pairs)."""
    for m, n, k in itertools.product([2, 100, 128, 129, 256, 300, 1000], [2, 77, 256, 515, 1100, 4097], [256, 1088, 4096]):
        for q8, wide in ((0, 1), (1, 1)) if m <= 128 else ((0, 0), (1, 1)):
            for ks in (1, 2, 3, 5, 8):
                if (k // 64) // ks < 1:
                    continue
                v = [C.c_size_t() for _ in range(6)]
                check(lib.pg_audit_gguf_hmm(m, n, k, q8, wide, ks, *[C.byref(x) for x in v]))
                pe, pb, qe, qb, de, db = (x.value for x in v)
                what = f"gguf_hmm m={m} n={n} k={k} q8={q8} wide={wide} ks={ks}"
                assert pe == pb, (what, pe, pb)       # the last row's last chunk is read by someone, and nothing past it
                assert qe == qb, (what, qe, qb)
                assert de <= db, (what, de, db)


def test_mxfp4_rows_loads_stay_inside_the_fragment_planes():
    for k, n in itertools.product([32, 64, 512, 2880, 4096, 28160], [1, 15, 16, 17, 100, 2880]):
        for rg, nw in ((1, 16), (1, 8), (2, 8), (4, 8), (8, 8), (1, 4), (2, 4), (4, 4)):
            v = _four()
            check(lib.pg_audit_mxfp4_rows(n, k, rg, nw, *[C.byref(x) for x in v]))
            _inside(v, f"mxfp4_rows n={n} k={k} RG={rg} NW={nw}")


def test_mxfp4_tiles_stay_inside_the_planes_and_the_token_records():
    """mxfp4_planes_kernel + mxfp4_tiles_kernel under the launcher's own plan, for every row-tile width (1, 2, 4 groups
    of 16 rows per wavefront), token-tile width (1, 2, 4 groups of 16 tokens) and K split it can pick."""
    seen = set()
    for num_cu in (256, 64):
        for k, n, m in itertools.product([32, 96, 512, 2880, 4096, 14336], [1, 15, 16, 17, 100, 2880, 8192, 70000], [16, 17, 32, 33, 100, 640]):
            v = [C.c_size_t() for _ in range(6)]
            plan = [C.c_int() for _ in range(3)]
            check(lib.pg_audit_mxfp4_tiles(num_cu, n, k, m, *[C.byref(x) for x in v], *[C.byref(x) for x in plan]))
            what = f"mxfp4_tiles n={n} k={k} m={m} cus={num_cu} plan={[x.value for x in plan]}"
            _inside(v[:4], what)
            assert v[4].value == v[5].value, f"{what}: the records are used up to byte {v[4].value} of {v[5].value}"
            seen.add((plan[0].value, plan[1].value, min(plan[2].value, 2)))
    assert {(ra, tb) for ra, tb, _ in seen} == {(ra, tb) for ra in (1, 2, 4) for tb in (1, 2, 4)}, seen
    assert {ks for _, _, ks in seen} == {1, 2}


def test_probe_read_covers_its_buffer_exactly_once_in_bounds():
    for nbytes in (1 << 20, 33103872, 58851328, (1 << 20) + 16):
        for wgs, threads, nl in itertools.product((256, 2048, 4096), (256, 1024), (4, 16)):
            end, alloc = C.c_size_t(), C.c_size_t()
            check(lib.pg_audit_probe_read(nbytes, wgs, threads, nl, C.byref(end), C.byref(alloc)))
            assert end.value == alloc.value == nbytes // 16 * 16


def test_audit_argument_errors():
    v = _four()
    with pytest.raises(_ffi.PeregrineError):
        check(lib.pg_audit_gemv_w8a8_m1(4096, 16, 1, 1, 4, 0, *[C.byref(x) for x in v]))   # NCH too small for the row
    with pytest.raises(_ffi.PeregrineError):
        check(lib.pg_audit_gguf_skinny(16, 1000, 0, 4, 1, *[C.byref(x) for x in v]))          # K not a multiple of 256
