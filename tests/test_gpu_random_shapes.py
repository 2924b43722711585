"""Seeded random shapes through the C ABI against the CPU oracle: ragged rows, columns and
block counts around the kernels' tile sizes (32 / 64 / 128 / 256), which the fixed shapes of
the other files only sample.  Same bars as there: the W8A8 product bit-exact, block-dequant
products within 1e-3, attention within 4e-5."""
import sys

import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _pick(rng, *choices):
    return int(rng.choice(choices))


@pytest.mark.parametrize("seed", [11, 12])
def test_w8a8_random_shapes_bit_exact(ctx, orc, seed):
    from peregrine_amd import quant
    rng = np.random.default_rng(seed)
    for case in range(40):
        m = _pick(rng, 1, 2, 3, 17, 31, 33, 63, 64, 65, 100, 129, 255, 257, 300)
        k = _pick(rng, 1, 3, 16, 31, 64, 100, 127, 128, 129, 255, 256, 384, 500, 1000, 1024, 2050)
        n = _pick(rng, 1, 2, 7, 31, 32, 33, 64, 100, 127, 128, 129, 255, 256, 257, 300, 511, 513)
        say(f"w8a8 random case {case}: m={m} k={k} n={n}")
        a = orc.rng_normal(seed * 1000 + case, m * k)
        if rng.random() < 0.3:
            a.reshape(m, k)[rng.integers(m)] = 0.0          # a zero row: scale 1.0
        w = orc.rng_normal(seed * 1000 + 500 + case, k * n, 0.0, 0.02)
        if rng.random() < 0.3:
            w.reshape(k, n)[:, rng.integers(n)] = 0.0       # a zero column: scale 1.0
        qt = quant.quantize_weights(w, k, n, ctx)
        q, q_t, s = orc.quantize_weights(w, k, n)
        assert (qt.data_i8_t == q_t).all() and (bits(qt.scales) == bits(s)).all()
        want, _ = orc.matmul_quantized(a, m, k, q_t, s, n)
        got = quant.matmul_quantized(a, m, k, qt, ctx)
        assert (bits(got) == bits(want)).all()
        qt.free_gpu()


@pytest.mark.parametrize("seed", [21, 22])
def test_gguf_matmul_random_shapes(ctx, orc, seed):
    from peregrine_amd import gguf
    rng = np.random.default_rng(seed)
    for case in range(40):
        typ = _pick(rng, 2, 8, 2, 8, 3)
        m = _pick(rng, 1, 2, 5, 8, 9, 16, 17, 31, 32, 33, 47, 64, 65, 100)
        nb = _pick(rng, 1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 33, 63, 64, 65, 100, 129)
        n_out = _pick(rng, 16, 31, 64, 100, 127, 128, 129, 255, 256, 257, 300, 520)
        k_in = nb * 32
        say(f"gguf random case {case}: type={typ} m={m} n_out={n_out} k_in={k_in}")
        w = orc.rng_normal(seed * 1000 + case, n_out * k_in, 0.0, 0.02)
        if typ == 3:
            w = w + np.float32(0.03)
        raw = {2: H.pack_q4_0, 3: H.pack_q4_1, 8: H.pack_q8_0}[typ](w)
        x = orc.rng_normal(seed * 1000 + 500 + case, m * k_in)
        gw = gguf.GgufWeight(raw, typ, n_out, k_in, ctx)
        got = gw.matmul(x, m)
        want = orc.gguf_matmul(x, m, raw, typ, n_out, k_in)
        for r in range(m):
            sl = slice(r * n_out, (r + 1) * n_out)
            H.assert_close_rel(got[sl], want[sl], 1e-3, f"row {r}")
        gw.free()


@pytest.mark.parametrize("seed", [31, 32])
def test_gguf_few_rows_random_shapes(ctx, orc, seed):
    """2 .. 16 rows over K a multiple of 256: the one-launch matrix-core product (4 x 4 x 4 products up to 8 rows,
    one or two weight tiles a workgroup, 16 x 16 x 32 above), ragged weight rows, outlier channels, a NaN."""
    from peregrine_amd import gguf
    rng = np.random.default_rng(seed)
    for case in range(24):
        typ = _pick(rng, 2, 8)
        m = _pick(rng, 2, 3, 4, 5, 6, 7, 8, 9, 12, 16)
        k_in = 256 * _pick(rng, 4, 5, 8, 9, 16, 17)
        n_out = _pick(rng, 16, 17, 100, 333, 520, 1000, 4100, 8192, 8200, 9001)
        say(f"gguf few rows random case {case}: type={typ} m={m} n_out={n_out} k_in={k_in}")
        w = orc.rng_normal(seed * 1000 + case, n_out * k_in, 0.0, 0.02)
        raw = {2: H.pack_q4_0, 8: H.pack_q8_0}[typ](w)
        x = orc.rng_normal(seed * 1000 + 500 + case, m * k_in)
        x.reshape(m, k_in)[:, :: max(1, k_in // 37)] *= 20
        poisoned = rng.random() < 0.25
        if poisoned:
            x.reshape(m, k_in)[m - 1, int(rng.integers(k_in))] = np.nan      # that row is lost, the others are not
        gw = gguf.GgufWeight(raw, typ, n_out, k_in, ctx)
        got = gw.matmul(x, m).reshape(m, n_out)
        want = orc.gguf_matmul(x, m, raw, typ, n_out, k_in).reshape(m, n_out)
        for r in range(m - 1 if poisoned else m):
            H.assert_close_rel(got[r], want[r], 1e-3, f"row {r}")
        if poisoned:
            assert np.isnan(got[m - 1]).all() and np.isnan(want[m - 1]).all()
        gw.free()


@pytest.mark.parametrize("seed", [41, 42])
def test_gguf_matmul_random_shapes_on_the_f16_matrix_cores(ctx, orc, seed):
    """The many-row route forced for every shape it can take (K a multiple of 64, two rows and more): both tile shapes,
    ragged rows and weight rows, 4 to 130 stages in 1 to 8 K chunks, Q4_0 and Q8_0, outlier channels, a zero row."""
    from peregrine_amd import gguf, _ffi
    rng = np.random.default_rng(seed)
    _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 1))
    try:
        for case in range(30):
            typ = _pick(rng, 2, 8)
            m = _pick(rng, 2, 5, 16, 33, 100, 127, 128, 129, 200, 255, 256, 257, 300, 513)
            k_in = 64 * _pick(rng, 4, 5, 8, 9, 16, 17, 33, 64, 65, 130)
            n_out = _pick(rng, 2, 31, 64, 100, 255, 256, 257, 300, 511, 513, 777, 1025)
            say(f"gguf f16-route random case {case}: type={typ} m={m} n_out={n_out} k_in={k_in}")
            raw = (H.pack_q4_0 if typ == 2 else H.pack_q8_0)(orc.rng_normal(seed * 1000 + case, n_out * k_in, 0.0, 0.02))
            x = orc.rng_normal(seed * 1000 + 500 + case, m * k_in).reshape(m, k_in)
            x[:, :: max(1, k_in // 23)] *= 20
            x[m // 2] = 0
            gw = gguf.GgufWeight(raw, typ, n_out, k_in, ctx)
            ctx.profile_begin()
            got = gw.matmul(x.reshape(-1), m).reshape(m, n_out)
            prof = ctx.profile_end()
            assert any(k.startswith("gguf_hmm") for k in prof), prof
            assert (got[m // 2] == 0).all()
            for r in sorted({0, 1, m // 3, m - 2, m - 1} - {m // 2}):
                H.assert_close_rel(got[r], orc.gguf_matmul(x[r], 1, raw, typ, n_out, k_in), 2e-5, f"row {r}")
            gw.free()
    finally:
        _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 0))


@pytest.mark.parametrize("seed", [31, 32])
def test_attention_random_shapes_and_masks(ctx, orc, seed):
    from peregrine_amd import llama
    rng = np.random.default_rng(seed)
    M = llama.AttentionMask
    for case in range(40):
        nkvh = _pick(rng, 1, 2, 3, 4)
        nqh = nkvh * _pick(rng, 1, 2, 4, 8)
        hd = _pick(rng, 4, 6, 8, 20, 32, 64, 64, 128, 128, 256)
        seq_q = _pick(rng, 1, 1, 2, 5, 31, 32, 33, 70)
        extra = _pick(rng, 0, 1, 7, 63, 64, 65, 200, 700)
        length = seq_q + extra
        kind = _pick(rng, 0, 1, 1, 2, 3)
        offset = extra if kind else 0
        window, sink, cap = _pick(rng, 0, 1, 5, 64, 1000), _pick(rng, 0, 1, 4), _pick(rng, 0, 0, 2)
        glob = [int(v) for v in rng.integers(0, length + 5, size=_pick(rng, 0, 1, 5, 40))]
        say(f"attention random case {case}: heads={nqh}/{nkvh} hd={hd} seq_q={seq_q} len={length} mask={kind} "
            f"window={window} sink={sink} cap={cap}")
        mask = [M.none(), M.causal(offset), M.causal_sliding_window(offset, window, sink),
                M.local_global(offset, window, glob)][kind]
        cache = llama.StandardKVCache(nkvh, hd, ctx)
        k = orc.rng_normal(seed * 1000 + case, nkvh * length * hd).reshape(nkvh, length, hd)
        v = orc.rng_normal(seed * 1000 + 300 + case, nkvh * length * hd).reshape(nkvh, length, hd)
        cache.append(k, v, length)
        q = orc.rng_normal(seed * 1000 + 600 + case, nqh * seq_q * hd).reshape(nqh, seq_q, hd)
        scale = 1 / np.sqrt(hd)
        got = np.zeros(seq_q * nqh * hd, np.float32)
        llama.gqa_attention(q, cache, cache, nqh, nkvh, seq_q, hd, scale, mask, cap, got, ctx)
        if kind == 3:
            want = orc.gqa_attention_local_global(q, k, v, length, length, nqh, nkvh, seq_q, hd, scale, offset, window,
                                                  glob, float(cap))
        else:
            want = orc.gqa_attention(q, k, v, length, length, nqh, nkvh, seq_q, hd, scale, kind, offset, window, sink,
                                     float(cap))
        H.assert_close_rel(got, want, 4e-5, "attention")
