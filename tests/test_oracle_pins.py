"""Pins the CPU oracle (oracle/peregrine_oracle.c) before anything trusts it.

Every oracle function is checked against at least one of:
  (K) a known-answer test the reference's own tests hold (cited file:line),
  (G) a golden fixture file from the reference's tests/fixtures (copied to tests/golden),
  (C) a closed form / invariant the mathematics fixes,
  (B) an independent NumPy restatement (different code path: vectorised float32 / int32
      array arithmetic, libm roundf through ctypes), including constructed tie and
      discriminating cases so that a plausible mistake (half-to-even rounding, divide
      instead of multiply-by-reciprocal, swapped epilogue order, ggml nibble order)
      fails.
Nothing here needs a GPU.
"""
import ctypes as C
import ctypes.util

import numpy as np
import pytest

import helpers as H

libm = C.CDLL(ctypes.util.find_library("m"))
libm.roundf.restype = C.c_float
libm.roundf.argtypes = [C.c_float]


def c_roundf(a):
    return np.array([libm.roundf(float(v)) for v in np.asarray(a, np.float32).reshape(-1)], np.float32)


def sat_i8(v):
    v = np.asarray(v, np.float32)
    out = np.clip(np.nan_to_num(v, nan=0.0), -127, 127)
    return out.astype(np.int8)


# --------------------------------------------------------------------------- f16
def test_f16_known_answers(orc):
    # src/gguf.rs:574-585 and tests/gguf_parity.rs:33,56
    kat = {0x0000: 0.0, 0x3C00: 1.0, 0xBC00: -1.0, 0x3800: 0.5, 0x4000: 2.0, 0x4900: 10.0}
    for bits, want in kat.items():
        got = orc.f16_to_f32_bits([bits]).view(np.float32)[0]
        assert got == np.float32(want), hex(bits)
    neg0 = orc.f16_to_f32_bits([0x8000])[0]
    assert neg0 == 0x80000000  # -0.0 keeps its sign bit


def test_f16_all_patterns_vs_numpy(orc):
    bits = np.arange(65536, dtype=np.uint16)
    got = orc.f16_to_f32_bits(bits)
    want = bits.view(np.float16).astype(np.float32).view(np.uint32)
    finite_or_inf = (bits & 0x7C00) != 0x7C00
    is_inf = (bits & 0x7FFF) == 0x7C00
    sel = finite_or_inf | is_inf
    assert (got[sel] == want[sel]).all()  # includes all 2046 subnormals
    nan = ~sel
    # reference rule for NaN: sign | 0xFF<<23 | mant<<13, payload kept, not quietened
    b = bits[nan].astype(np.uint32)
    rule = ((b >> 15) << 31) | np.uint32(0x7F800000) | ((b & 0x3FF) << 13)
    assert (got[nan] == rule).all()


# ------------------------------------------------------------------ block dequant
def _block(scale_bits, payload):
    return bytes([scale_bits & 0xFF, scale_bits >> 8]) + bytes(payload)


def test_dequant_known_answers(orc):
    # Q8_0: d = 1.0, q = 0..31 -> i            (src/gguf.rs:588-601)
    out = orc.dequant_q8_0(_block(0x3C00, range(32)), 32)
    assert (out == np.arange(32, dtype=np.float32)).all()
    # Q8_0: d = 0.5, q = 1..32 -> (i+1)/2      (tests/gguf_parity.rs:7-28)
    out = orc.dequant_q8_0(_block(0x3800, range(1, 33)), 32)
    assert (out == (np.arange(32, dtype=np.float32) + 1) * 0.5).all()
    # negative i8 bytes are sign-extended
    out = orc.dequant_q8_0(_block(0x3C00, [0xFF, 0x80] + [0] * 30), 32)
    assert out[0] == -1.0 and out[1] == -128.0
    # Q4_0: d = 1.0, byte0 = 0x98 -> out[0] = 0, out[1] = 1: pins the interleaved order
    # (src/gguf.rs:604-615); ggml's own order would put the high nibble at out[16].
    out = orc.dequant_q4_0(_block(0x3C00, [0x98] + [0x88] * 15), 32)
    assert out[0] == 0.0 and out[1] == 1.0 and (out[2:] == 0.0).all()
    # Q4_0: d = 2.0, all 0x88 -> zeros         (tests/gguf_parity.rs:31-50)
    out = orc.dequant_q4_0(_block(0x4000, [0x88] * 16), 32)
    assert (out == 0.0).all()
    # Q4_1: 0x53, d = 1, m = 0 -> 3, 5         (src/gguf.rs:618-631)
    blk = bytes([0x00, 0x3C, 0x00, 0x00]) + bytes([0x53] + [0] * 15)
    out = orc.dequant_q4_1(blk, 32)
    assert out[0] == 3.0 and out[1] == 5.0
    # Q4_1: d = 1, m = 10, nibbles 0 -> 10     (tests/gguf_parity.rs:53-76)
    blk = bytes([0x00, 0x3C, 0x00, 0x49]) + bytes(16)
    assert (orc.dequant_q4_1(blk, 32) == 10.0).all()
    with pytest.raises(ValueError):
        orc.dequant_q4_0(bytes(18), 31)  # assert!(num_elements % 32 == 0)


def test_dequant_vs_numpy_random(orc):
    rng = np.random.default_rng(7)
    n = 32 * 257
    raw8 = rng.integers(0, 256, n // 32 * 34, dtype=np.uint8)
    raw4 = rng.integers(0, 256, n // 32 * 18, dtype=np.uint8)
    for raw, bb in ((raw8, 34), (raw4, 18)):
        v = raw.reshape(-1, bb)
        v[:, 1] &= 0x7B  # keep the random f16 scales finite and non-NaN
    a, b = orc.dequant_q8_0(raw8.tobytes(), n), H.np_dequant_q8_0(raw8.tobytes(), n)
    assert (a.view(np.uint32) == b.view(np.uint32)).all()
    a, b = orc.dequant_q4_0(raw4.tobytes(), n), H.np_dequant_q4_0(raw4.tobytes(), n)
    assert (a.view(np.uint32) == b.view(np.uint32)).all()


# ------------------------------------------------------------------- f32 matmul
@pytest.mark.parametrize("names", [("matmul_a.bin", "matmul_b.bin", "matmul_c.bin"),
                                   ("matmul_rect_a.bin", "matmul_rect_b.bin", "matmul_rect_c.bin")])
def test_matmul_f32_golden(orc, names):
    # tests/pytorch_parity.rs:88-107, tolerance 1e-4 max abs
    a, b, c = (H.load_fixture(n) for n in names)
    got = orc.matmul_f32(a, b, a.shape[0], a.shape[1], b.shape[1]).reshape(c.shape)
    assert np.abs(got - c).max() < 1e-4


def test_matmul_f32_is_k_sequential(orc):
    # closed form: [1, 1e8, -1e8] . [1, 1, 1] summed left to right is 0 in f32
    # (1 + 1e8 rounds to 1e8); a pairwise or reversed sum would give 1.
    a = np.array([[1.0, 1e8, -1e8]], np.float32)
    b = np.ones((3, 1), np.float32)
    assert orc.matmul_f32(a, b, 1, 3, 1)[0] == 0.0
    a = np.array([[1e8, -1e8, 1.0]], np.float32)
    assert orc.matmul_f32(a, b, 1, 3, 1)[0] == 1.0


def test_gguf_matmul_equals_dequant_then_matmul(orc):
    rng = np.random.default_rng(3)
    n_out, k_in, m = 24, 96, 3
    w = rng.normal(0, 0.02, (n_out, k_in)).astype(np.float32)
    x = rng.normal(0, 1, (m, k_in)).astype(np.float32)
    for typ, pack, deq in ((8, H.pack_q8_0, H.np_dequant_q8_0), (2, H.pack_q4_0, H.np_dequant_q4_0)):
        raw = pack(w)
        wf = deq(raw, n_out * k_in).reshape(n_out, k_in)
        want = orc.matmul_f32(x, np.ascontiguousarray(wf.T), m, k_in, n_out)  # [k,n] operand, as the model holds it
        got = orc.gguf_matmul(x, m, raw, typ, n_out, k_in)
        assert (got.view(np.uint32) == want.view(np.uint32)).all()


# ---------------------------------------------------------------------- softmax
@pytest.mark.parametrize("stem", ["softmax", "softmax_large"])
def test_softmax_golden(orc, stem):
    # tests/pytorch_parity.rs:110-127, tolerance 1e-6
    x, y = H.load_fixture(f"{stem}_input.bin"), H.load_fixture(f"{stem}_output.bin")
    got = orc.softmax_rows(x, x.shape[0], x.shape[1]).reshape(y.shape)
    assert np.abs(got - y).max() < 1e-6
    assert np.allclose(got.sum(axis=1), 1.0, atol=1e-6)


def test_activations_vs_float64(orc):
    x = np.linspace(-12, 12, 4001).astype(np.float32)
    xd = x.astype(np.float64)
    silu = xd / (1 + np.exp(-xd))
    gelu = 0.5 * xd * (1 + np.tanh(np.sqrt(2 / np.pi) * (xd + 0.044715 * xd ** 3)))
    assert np.abs(orc.unary("orc_silu", x) - silu).max() < 2e-6
    assert np.abs(orc.unary("orc_gelu_tanh", x) - gelu).max() < 2e-6
    assert orc.unary("orc_silu", [0.0])[0] == 0.0


# ------------------------------------------------------------- quantize_weights
def np_quantize_weights(w, rows, cols, divide=True):
    w = np.asarray(w, np.float32).reshape(rows, cols)
    aw = np.abs(w)
    amax = np.where(np.isnan(aw), np.float32(0), aw).max(axis=0).astype(np.float32)
    scale = np.where(amax == 0, np.float32(1), amax / np.float32(127)).astype(np.float32)
    with np.errstate(all="ignore"):
        v = (w / scale[None, :]) if divide else (w * (np.float32(1) / scale)[None, :])
    q = sat_i8(c_roundf(v.astype(np.float32)).reshape(rows, cols))
    return q, scale


def test_quantize_weights_closed_forms_and_ties(orc):
    rows, cols = 6, 5
    w = np.zeros((rows, cols), np.float32)
    w[:, 0] = [127, -127, 2.5, -2.5, 0.5, 1.5]   # amax 127 -> scale exactly 1 -> exact .5 ties
    w[:, 1] = 0                                   # zero column -> scale 1.0, q 0
    w[:, 2] = [3, 3, -3, 3, -3, 3]                # all |w| equal -> q = +-127
    w[:, 3] = [np.nan, 1, -2, 0.25, 0, 2]         # NaN never wins the max; NaN -> 0
    w[:, 4] = [np.inf, 1, -1, 0, 5, -np.inf]      # inf column: scale inf, finite/inf = 0, inf/inf = NaN -> 0
    q, qt, s = orc.quantize_weights(w, rows, cols)
    q = q.reshape(rows, cols)
    assert s[0] == 1.0 and list(q[:, 0]) == [127, -127, 3, -3, 1, 2]  # half AWAY from zero (half-even: 2,-2,0,2)
    assert s[1] == 1.0 and (q[:, 1] == 0).all()
    assert s[2] == np.float32(3) / np.float32(127) and list(q[:, 2]) == [127, 127, -127, 127, -127, 127]
    assert s[3] == np.float32(2) / np.float32(127) and q[0, 3] == 0 and q[2, 3] == -127 and q[5, 3] == 127
    assert np.isinf(s[4]) and (q[:, 4] == 0).all()
    assert (qt.reshape(cols, rows) == q.T).all()  # data_i8_t[n*rows+k] = data_i8[k*cols+n]


def test_quantize_weights_vs_numpy_and_divide_matters(orc):
    rng = np.random.default_rng(11)
    rows, cols = 96, 80
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    q, qt, s = orc.quantize_weights(w, rows, cols)
    q_div, s_div = np_quantize_weights(w, rows, cols, divide=True)
    assert (s == s_div).all() and (q.reshape(rows, cols) == q_div).all()
    assert np.abs(q).max() == 127 and (s > 0).all()
    # The reference divides (w / scale); multiplying by 1/scale rounds differently on the
    # constructed inputs below (found by search: w sits one rounding away from a .5 tie).
    fh = float.fromhex
    col0 = [fh("0x1.13c502p-4"), fh("0x1.e6658ep-10"), fh("-0x1.09ff8ap-4"), fh("-0x1.f9f07ep-5")]
    col1 = [fh("0x1.18d40ep-5"), fh("0x1.1b0a2p-13"), fh("-0x1.1116c6p-5"), fh("-0x1.134cdap-5")]
    tie = np.array([col0, col1], np.float32).T.copy()
    qd, _ = np_quantize_weights(tie, 4, 2, divide=True)
    qm, _ = np_quantize_weights(tie, 4, 2, divide=False)
    assert (qd != qm).sum() >= 4, "constructed cases no longer separate divide from reciprocal-multiply"
    qo, _, _ = orc.quantize_weights(tie, 4, 2)
    assert (qo.reshape(4, 2) == qd).all()


def test_quantize_weights_reference_property_tests(orc):
    # tests/quant_parity.rs:6-32: err <= scale + 1e-7, 64x128, ((i*17+5)%400)/100 - 2
    for rows, cols, data, slack in (
        (64, 128, H.mod_pattern(64 * 128, 17, 5, 400, 100.0, 2.0), 1e-7),
        # src/quant.rs:225-249: (i - rows*cols/2) * 0.01, 32x64, err <= scale + 1e-6
        (32, 64, ((np.arange(32 * 64, dtype=np.float32) - np.float32(32 * 64 // 2)) * np.float32(0.01)), 1e-6),
    ):
        q, _, s = orc.quantize_weights(data, rows, cols)
        rec = orc.dequantize(q, s, rows, cols).reshape(rows, cols)
        d = data.reshape(rows, cols)
        amax = np.abs(d).max(axis=0)
        scale = np.where(amax == 0, 1.0, amax / np.float32(127)).astype(np.float32)
        assert (s == scale).all()
        assert (np.abs(d - rec) <= scale[None, :] + slack).all()


# --------------------------------------------------------- quantize_activations
def np_quantize_activations(a, rows, cols, reciprocal=True):
    a = np.asarray(a, np.float32).reshape(rows, cols)
    amax = np.nanmax(np.abs(a), axis=1, initial=0.0).astype(np.float32) if cols else np.zeros(rows, np.float32)
    amax = np.where(np.isnan(amax), np.float32(0), amax)
    scale = np.where(amax == 0, np.float32(1), amax / np.float32(127)).astype(np.float32)
    with np.errstate(all="ignore"):
        inv = (np.float32(1) / scale).astype(np.float32)
        v = (a * inv[:, None]) if reciprocal else (a / scale[:, None])
    return sat_i8(c_roundf(v.astype(np.float32)).reshape(rows, cols)), scale


def test_quantize_activations_closed_forms_and_ties(orc):
    a = np.array([
        [127, -127, 0.5, -0.5, 1.5, 2.5, -2.5, 0],     # scale 1: ties go away from zero
        [0, 0, 0, 0, 0, 0, 0, 0],                       # zero row -> scale 1.0
        [4, 4, -4, 4, 4, -4, 4, 4],                     # all equal -> +-127
        [np.nan, 1, -2, 0.5, 0, 0, 0, 2],               # f32::max ignores NaN; NaN -> 0
        [np.inf, 1, -1, 0, 0, 0, 0, -np.inf],           # inv_scale = 0: finite*0 = 0, inf*0 = NaN -> 0
        [1e-42, -1e-42, 0, 0, 0, 0, 0, 5e-43],          # subnormal row: inv_scale = +inf, 0*inf = NaN -> 0
    ], np.float32)
    q, s = orc.quantize_activations(a, a.shape[0], a.shape[1])
    q = q.reshape(a.shape)
    assert s[0] == 1.0 and list(q[0]) == [127, -127, 1, -1, 2, 3, -3, 0]
    assert s[1] == 1.0 and (q[1] == 0).all()
    assert list(q[2]) == [127, 127, -127, 127, 127, -127, 127, 127]
    assert s[3] == np.float32(2) / np.float32(127) and q[3, 0] == 0 and q[3, 2] == -127 and q[3, 7] == 127
    assert np.isinf(s[4]) and (q[4] == 0).all()
    assert s[5] > 0 and list(q[5]) == [127, -127, 0, 0, 0, 0, 0, 127]  # x*inf saturates; 0*inf = NaN -> 0


def test_quantize_activations_vs_numpy_and_reciprocal_matters(orc):
    rng = np.random.default_rng(5)
    rows, cols = 512, 256
    a = rng.normal(0, 1, (rows, cols)).astype(np.float32)
    a[:, ::97] *= 20  # outlier channels
    q, s = orc.quantize_activations(a, rows, cols)
    qr, sr = np_quantize_activations(a, rows, cols, reciprocal=True)
    assert (s == sr).all() and (q.reshape(rows, cols) == qr).all()
    assert np.abs(q).max() == 127
    # The reference multiplies by 1/scale; dividing rounds differently on these
    # constructed rows (row[0] is the absmax, the others sit next to a .5 tie).
    fh = float.fromhex
    tie = np.array([[fh("0x1.13c502p-4"), fh("0x1.e6658ep-10"), fh("-0x1.09ff8ap-4"), fh("-0x1.f9f07ep-5")],
                    [fh("0x1.18d40ep-5"), fh("0x1.1b0a2p-13"), fh("-0x1.1116c6p-5"), fh("-0x1.134cdap-5")]], np.float32)
    qr, _ = np_quantize_activations(tie, 2, 4, reciprocal=True)
    qd, _ = np_quantize_activations(tie, 2, 4, reciprocal=False)
    assert (qr != qd).sum() >= 4, "constructed cases no longer separate x*(1/s) from x/s"
    qo, _ = orc.quantize_activations(tie, 2, 4)
    assert (qo.reshape(2, 4) == qr).all()


# ------------------------------------------------------------------ gemm / matmul
def test_gemm_i8_vs_numpy_int32_and_epilogue_order(orc):
    rng = np.random.default_rng(2)
    m, n, k = 17, 23, 200
    a = rng.integers(-127, 128, (m, k), dtype=np.int8)
    bt = rng.integers(-127, 128, (n, k), dtype=np.int8)
    a_s = rng.uniform(0.001, 0.1, m).astype(np.float32)
    w_s = rng.uniform(0.0001, 0.01, n).astype(np.float32)
    out, acc = orc.gemm_i8(a, a_s, bt, w_s, m, n, k)
    want_acc = a.astype(np.int32) @ bt.astype(np.int32).T
    assert (acc.reshape(m, n) == want_acc).all()
    left = (want_acc.astype(np.float32) * a_s[:, None]) * w_s[None, :]   # reference order
    right = want_acc.astype(np.float32) * (a_s[:, None] * w_s[None, :])  # the plausible mistake
    assert (out.reshape(m, n).view(np.uint32) == left.view(np.uint32)).all()
    assert (left.view(np.uint32) != right.view(np.uint32)).any()
    # extreme values: -127 * -127 * k stays far from i32 overflow and is exact
    a[:] = -127
    bt[:] = -127
    _, acc = orc.gemm_i8(a, a_s, bt, w_s, m, n, k)
    assert (acc == 127 * 127 * k).all()


@pytest.mark.parametrize("m,k,n,mod,rt,at", [(32, 128, 64, 200, 0.15, 0.05),   # tests/quant_parity.rs:35-77
                                             (16, 64, 32, 100, 0.05, 0.01)])  # src/quant.rs:252-291
def test_matmul_quantized_reference_property_tests(orc, m, k, n, mod, rt, at):
    a = H.mod_pattern(m * k, 7, 3, mod, float(mod), 0.5)
    w = H.mod_pattern(k * n, 13, 7, mod, float(mod), 0.5)
    expected = orc.matmul_f32(a, w, m, k, n)
    q, qt, s = orc.quantize_weights(w, k, n)
    got, _ = orc.matmul_quantized(a, m, k, qt, s, n)
    diff = np.abs(got - expected)
    rtol = diff / np.maximum(np.abs(expected), 1e-6)
    assert ((rtol < rt) | (diff < at)).all()


@pytest.mark.parametrize("m,k,n", [(8, 32, 16), (1, 64, 1), (32, 128, 64), (16, 256, 32)])
def test_matmul_quantized_composition_lcg_shapes(orc, m, k, n):
    # shapes and generator of tests/huffman_parity.rs:24-41
    a, w = H.lcg_data(m * k, 42), H.lcg_data(k * n, 123)
    q, qt, s = orc.quantize_weights(w, k, n)
    got, acc = orc.matmul_quantized(a, m, k, qt, s, n)
    qa, sa = np_quantize_activations(a, m, k)
    qw, sw = np_quantize_weights(w, k, n)
    want_acc = qa.astype(np.int32) @ qw.astype(np.int32)
    assert (acc.reshape(m, n) == want_acc).all()
    want = (want_acc.astype(np.float32) * sa[:, None]) * sw[None, :]
    assert (got.reshape(m, n).view(np.uint32) == want.view(np.uint32)).all()


# -------------------------------------------------------------------------- MoE
def test_moe_routing_and_accumulation(orc):
    rng = np.random.default_rng(9)
    T, d, ffn, E, top_k = 5, 64, 96, 4, 2
    x = rng.normal(0, 1, (T, d)).astype(np.float32)
    logits = rng.normal(0, 1, (T, E)).astype(np.float32)
    logits[0] = [0.5, 0.5, 0.5, 0.5]      # full tie: stable sort keeps experts 0, 1
    logits[1] = [0.1, 0.9, 0.9, 0.2]      # tie for first place: 1 before 2
    ws = [[rng.normal(0, 0.05, shp).astype(np.float32) for _ in range(E)]
          for shp in ((ffn, d), (ffn, d), (d, ffn))]
    raw = [[H.pack_q8_0(w) for w in grp] for grp in ws]
    for act in (0, 1):
        out, idx, prob = orc.moe_ffn(x, T, d, ffn, E, top_k, logits, raw[0], raw[1], raw[2], 8, act)
        assert list(idx[0]) == [0, 1] and list(idx[1]) == [1, 2]
        p64 = np.exp(logits.astype(np.float64) - logits.max(axis=1, keepdims=True))
        p64 /= p64.sum(axis=1, keepdims=True)
        for t in range(T):
            order = sorted(range(E), key=lambda e: (-p64[t, e], e))[:top_k]
            if t >= 2:
                assert list(idx[t]) == order
            assert np.allclose(prob[t], p64[t, list(idx[t])], atol=1e-6)  # raw probs, not renormalised
        # float64 restatement of the layer on the dequantised weights
        deq = [[H.np_dequant_q8_0(r, w.size).reshape(w.shape).astype(np.float64) for r, w in zip(rg, wg)]
               for rg, wg in zip(raw, ws)]
        want = np.zeros((T, d))
        for t in range(T):
            for kk in range(top_k):
                e = idx[t, kk]
                g = deq[0][e] @ x[t].astype(np.float64)
                u = deq[1][e] @ x[t].astype(np.float64)
                a = g / (1 + np.exp(-g)) if act == 0 else 0.5 * g * (1 + np.tanh(np.sqrt(2 / np.pi) * (g + 0.044715 * g ** 3)))
                want[t] += p64[t, e] * (deq[2][e] @ (a * u))
        H.assert_close_rel(out, want, 1e-4, f"moe act={act}")


def _logit(p):
    return float(np.log(p / (1 - p)))


def test_deepseek_gate_hand_worked(orc):
    """Gate::forward (examples/deepseek/moe.rs:111-215) on cases worked by hand; dim = 1 and x = 1, so a score is
    sigmoid(w[e]).  Each case is built so that one plausible mistake changes the answer."""
    x = np.ones((1, 1), np.float32)
    w = np.array([0.0, _logit(0.75), _logit(0.25), 0.0], np.float32)          # sigmoid scores .5, .75, .25, .5
    # (a) bias, two groups, one kept.  biased scores .5, .75 | .85, .1: the sum of a group's two largest picks group 0
    #     (1.25 against .95; its maximum would pick group 1), then experts 1 and 0; the weights are the UNbiased
    #     scores .75 and .5, divided by their sum, times route_scale.
    idx, wt = orc.deepseek_gate(x, 1, 1, w, [0, 0, 0.6, -0.4], 4, 2, 2, 1, 2.5, True)
    assert list(idx[0]) == [1, 0]
    assert np.allclose(wt[0], [1.5, 1.0], rtol=1e-6)
    # (b) the same without a bias: the group score is the maximum (.75 against .5): group 0 again
    idx, wt = orc.deepseek_gate(x, 1, 1, w, None, 4, 2, 2, 1, 1.0, True)
    assert list(idx[0]) == [1, 0] and np.allclose(wt[0], [0.6, 0.4], rtol=1e-6)
    # (c) without a bias the maximum decides even when the other group has the larger sum: .6, .6 | .7, .1 -> group 1;
    #     its experts 2 and 3, weights .7 / .8 and .1 / .8
    w2 = np.array([_logit(0.6), _logit(0.6), _logit(0.7), _logit(0.1)], np.float32)
    idx, wt = orc.deepseek_gate(x, 1, 1, w2, None, 4, 2, 2, 1, 1.0, True)
    assert list(idx[0]) == [2, 3] and np.allclose(wt[0], [0.875, 0.125], rtol=1e-5)
    # (d) no group limit (one group): the bias moves expert 3 to the front of the selection, its weight stays .1 / (.1 + .7)
    idx, wt = orc.deepseek_gate(x, 1, 1, w2, [0, 0, 0, 1.0], 4, 2, 1, 1, 1.0, True)
    assert list(idx[0]) == [3, 2] and np.allclose(wt[0], [0.125, 0.875], rtol=1e-5)
    # (e) ties keep the lower expert first; softmax scores are not renormalised over the k, only scaled
    w3 = np.array([1.0, 1.0, 1.0, 0.0], np.float32)
    idx, wt = orc.deepseek_gate(x, 1, 1, w3, None, 4, 2, 1, 1, 2.0, False)
    p = np.exp(w3.astype(np.float64) - 1.0)
    p /= p.sum()
    assert list(idx[0]) == [0, 1] and np.allclose(wt[0], 2.0 * p[:2], rtol=1e-6)
    # (f) a score is the f32 dot product over dim: against float64 on random data, selection recomputed independently
    rng = np.random.default_rng(3)
    T, dim, E = 7, 48, 16
    xs, ws, bs = rng.normal(0, 1, (T, dim)).astype(np.float32), rng.normal(0, 0.3, (E, dim)).astype(np.float32), rng.normal(0, 0.05, E).astype(np.float32)
    idx, wt = orc.deepseek_gate(xs, T, dim, ws, bs, E, 4, 4, 2, 1.7, True)
    sc = 1 / (1 + np.exp(-(xs.astype(np.float64) @ ws.astype(np.float64).T)))
    for t in range(T):
        biased = sc[t] + bs
        gscore = [np.sort(biased[4 * g:4 * g + 4])[::-1][:2].sum() for g in range(4)]
        keep = sorted(range(4), key=lambda g: (-gscore[g], g))[:2]
        masked = np.array([biased[e] if e // 4 in keep else 0.0 for e in range(E)])
        order = sorted(range(E), key=lambda e: (-masked[e], e))[:4]
        assert list(idx[t]) == order
        assert np.allclose(wt[t], 1.7 * sc[t, order] / sc[t, order].sum(), rtol=1e-5)


def test_gpt_oss_route_hand_worked(orc):
    """examples/gpt_oss/moe.rs:298-330: the bias takes part in the selection, ties keep the lower expert, and the
    weights are a softmax over the k selected logits only (they sum to 1)."""
    idx, wt = orc.gpt_oss_route(np.array([[1.0, 3.0, 3.0, 0.5]], np.float32), np.zeros(4, np.float32), 1, 4, 2)
    assert list(idx[0]) == [1, 2] and np.allclose(wt[0], [0.5, 0.5])
    idx, wt = orc.gpt_oss_route(np.array([[np.log(3.0), 0.0, -1.0, -2.0]], np.float32), np.zeros(4, np.float32), 1, 4, 2)
    assert list(idx[0]) == [0, 1] and np.allclose(wt[0], [0.75, 0.25], rtol=1e-6)
    idx, wt = orc.gpt_oss_route(np.zeros((1, 4), np.float32), np.array([0.1, 0.3, 0.2, 0.0], np.float32), 1, 4, 2)
    assert list(idx[0]) == [1, 2]
    e = np.exp(np.array([0.3, 0.2]) - 0.3)
    assert np.allclose(wt[0], e / e.sum(), rtol=1e-6)


def test_moe_ffn_routed_is_the_layer_after_its_gate(orc):
    """orc_moe_ffn_routed fed with the routing orc_moe_ffn reports gives orc_moe_ffn's output bit for bit (pinned
    above), and the shared experts' output is added last, once."""
    rng = np.random.default_rng(11)
    T, d, ffn, E, top_k = 4, 64, 96, 4, 2
    x = rng.normal(0, 1, (T, d)).astype(np.float32)
    logits = rng.normal(0, 1, (T, E)).astype(np.float32)
    raw = [[H.pack_q8_0(rng.normal(0, 0.05, shp).astype(np.float32)) for _ in range(E)] for shp in ((ffn, d), (ffn, d), (d, ffn))]
    want, idx, prob = orc.moe_ffn(x, T, d, ffn, E, top_k, logits, raw[0], raw[1], raw[2], 8, 0)
    got = orc.moe_ffn_routed(x, T, d, ffn, E, top_k, idx, prob, raw[0], raw[1], raw[2], 8, 0)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()
    shared = rng.normal(0, 1, (T, d)).astype(np.float32)
    got2 = orc.moe_ffn_routed(x, T, d, ffn, E, top_k, idx, prob, raw[0], raw[1], raw[2], 8, 0, shared)
    assert ((want + shared).view(np.uint32) == got2.view(np.uint32)).all()
    # the weights are used as given: doubling them doubles the routed part exactly
    got3 = orc.moe_ffn_routed(x, T, d, ffn, E, top_k, idx, 2 * prob, raw[0], raw[1], raw[2], 8, 0)
    assert ((2 * want).view(np.uint32) == got3.view(np.uint32)).all()


# -------------------------------------------------------------------------- RNG
def test_xoshiro_known_answers(orc):
    # Published xoshiro256++ recurrence from state {1,2,3,4}: first outputs derived by hand
    # from result = rotl(s0+s3, 23) + s0: rotl(5,23)+1 = 41943041; next 58720359.
    state = (C.c_uint64 * 4)(1, 2, 3, 4)
    assert orc.lib.orc_rng_next_u64(state) == 41943041
    assert orc.lib.orc_rng_next_u64(state) == 58720359
    # SplitMix64 seeding (src/random.rs:22-33): published outputs for seed 0
    st = (C.c_uint64 * 4)()
    orc.lib.orc_rng_seed(st, 0)
    assert list(st) == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F, 0xF88BB8A8724C81EC]


def test_normal_statistics(orc):
    x = orc.rng_normal(1234, 200001, 0.0, 0.02)
    assert abs(float(x.mean())) < 3e-4 and abs(float(x.std()) - 0.02) < 3e-4
    assert (orc.rng_normal(1234, 10, 0.0, 0.02) == x[:10]).all()  # deterministic, prefix-stable
    y = orc.rng_normal(1234, 7, 1.0, 0.0)
    assert (y == 1.0).all()


def test_matmul_dequant_i8_is_dequantize_then_f32_matmul(orc):
    """The Metal kernel's arithmetic (src/metal/shaders.rs:2329-2375) equals the composition
    of two functions pinned above -- dequantize (one rounding per weight) then the
    K-sequential f32 matmul -- bit for bit, and a closed form: integer activations with
    unit scales give exact integers."""
    m, k, n = 5, 70, 9
    a = H.lcg_data(m * k, 42)
    w = H.lcg_data(k * n, 123)
    q, q_t, s = orc.quantize_weights(w, k, n)
    got = orc.matmul_dequant_i8(a, m, k, q, s, n)
    want = orc.matmul_f32(a, orc.dequantize(q, s, k, n), m, k, n)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()
    ai = np.arange(m * k, dtype=np.float32).reshape(m, k) % 7 - 3
    qi = (np.arange(k * n).reshape(k, n) % 11 - 5).astype(np.int8)
    exact = ai.astype(np.int64) @ qi.astype(np.int64)
    got = orc.matmul_dequant_i8(ai, m, k, qi, np.ones(n, np.float32), n).reshape(m, n)
    assert (got == exact).all()
