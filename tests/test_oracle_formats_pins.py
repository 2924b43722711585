"""Pins for the sibling-format half of the CPU oracle (oracle/peregrine_oracle_formats.c).
The reference holds no test or vector for MXFP4, so the value tables of the OCP Microscaling
formats (E2M1 elements, E8M0 scales), the nibble order and a float64 recomputation stand in."""
import numpy as np

E2M1 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]     # OCP MX v1.0: FP4 E2M1 magnitudes, bit 3 = sign


def mx_dequant(blocks, scales, out_dim, in_dim):
    """float64 weight matrix from packed MXFP4."""
    b = np.frombuffer(bytes(blocks), np.uint8).reshape(out_dim, in_dim // 32, 16)
    lut = np.array(E2M1 + [-v for v in E2M1])
    w = np.empty((out_dim, in_dim // 32, 32))
    w[:, :, 0::2] = lut[b & 15]
    w[:, :, 1::2] = lut[b >> 4]
    s = np.frombuffer(bytes(scales), np.uint8).reshape(out_dim, in_dim // 32).astype(np.int64)
    scale = np.where(s == 0, 0.0, np.ldexp(1.0, s - 127))   # E8M0 (the reference maps byte 0 to +0.0, not 2^-127)
    return (w * scale[:, :, None]).reshape(out_dim, in_dim)


def test_mxfp4_value_tables_and_nibble_order(orc):
    in_dim = 32
    # every code in the low nibble of byte 0 (element 0) and in the high nibble (element 1)
    for code in range(16):
        want = (-1 if code & 8 else 1) * E2M1[code & 7]
        for pos, byte in ((0, code), (1, code << 4)):
            blocks = bytearray(16)
            blocks[0] = byte
            x = np.zeros(in_dim, np.float32)
            x[pos] = 1.0
            assert orc.mxfp4_matmul(x, blocks, bytes([127]), 1, in_dim)[0] == want
            x[:] = 0
            x[1 - pos] = 1.0                       # the other element of the byte reads code 0
            assert orc.mxfp4_matmul(x, blocks, bytes([127]), 1, in_dim)[0] == 0.0
    # byte k holds elements 2k and 2k+1
    blocks = bytes((2 | (4 << 4)) for _ in range(16))        # low = 1.0, high = 2.0
    x = np.arange(32, dtype=np.float32)
    assert orc.mxfp4_matmul(x, blocks, bytes([127]), 1, in_dim)[0] == float(x[0::2].sum() + 2 * x[1::2].sum())
    # every scale byte: 2^(e - 127), byte 0 -> 0.0, byte 255 -> inf
    one = bytes([2]) + bytes(15)                              # element 0 = 1.0
    x = np.zeros(32, np.float32)
    x[0] = 1.0
    for e in range(256):
        got = orc.mxfp4_matmul(x, one, bytes([e]), 1, in_dim)[0]
        if e == 0:
            assert got == 0.0
        elif e == 255:
            assert np.isinf(got)
        else:
            assert got == np.float32(np.ldexp(1.0, e - 127))


def test_mxfp4_matmul_against_float64(orc):
    rng = np.random.default_rng(11)
    out_dim, in_dim = 24, 160
    blocks = rng.integers(0, 256, out_dim * in_dim // 2, dtype=np.uint8).tobytes()
    scales = rng.integers(110, 135, out_dim * in_dim // 32, dtype=np.uint8).tobytes()
    x = rng.standard_normal(in_dim).astype(np.float32)
    want = mx_dequant(blocks, scales, out_dim, in_dim) @ x.astype(np.float64)
    got = orc.mxfp4_matmul(x, blocks, scales, out_dim, in_dim)
    assert np.abs(got - want).max() <= 2e-6 * np.abs(want).max()
    # rows are independent and use their own blocks: permuting rows permutes outputs
    perm = rng.permutation(out_dim)
    b2 = np.frombuffer(blocks, np.uint8).reshape(out_dim, -1)[perm].tobytes()
    s2 = np.frombuffer(scales, np.uint8).reshape(out_dim, -1)[perm].tobytes()
    assert (orc.mxfp4_matmul(x, b2, s2, out_dim, in_dim) == got[perm]).all()


def test_mxfp4_expert_closed_forms_and_float64(orc):
    hidden, inter, alpha, clamp = 32, 32, 1.702, 7.0
    # mlp1 = rows that copy x[0] (code 2 = 1.0 at element 0); mlp2 = identity-like rows
    def unit_rows(n_rows, in_dim, cols):
        b = np.zeros((n_rows, in_dim // 32, 16), np.uint8)
        for r, c in enumerate(cols):
            b[r, c // 32, (c % 32) // 2] = 2 << (4 * (c % 2))
        return b.tobytes(), bytes([127]) * (n_rows * in_dim // 32)
    b1, s1 = unit_rows(2 * inter, hidden, [0] * (2 * inter))           # every mlp1 output = x[0]
    b2, s2 = unit_rows(hidden, inter, list(range(hidden)))             # out[i] = act[i]
    bias1 = np.zeros(2 * inter, np.float32)
    bias1[0], bias1[1] = 100.0, 100.0        # pair 0: gate clamps to 7 from above, linear to 7
    bias1[2], bias1[3] = -100.0, -100.0      # pair 1: gate is NOT clamped from below, linear clamps to -7
    bias1[5] = 0.5                           # pair 2: gate = x0, linear = x0 + 0.5
    bias2 = np.arange(hidden, dtype=np.float32)
    x = np.zeros(hidden, np.float32)
    x[0] = 1.0
    out = orc.mxfp4_expert_forward(x, hidden, inter, alpha, clamp, b1, s1, b2, s2, bias1, bias2) - bias2
    sig = lambda v: 1 / (1 + np.exp(-v))
    assert np.isclose(out[0], 7 * sig(alpha * 7) * (7 + 1), rtol=1e-6)
    assert np.isclose(out[1], -99 * sig(alpha * -99) * (-7 + 1), rtol=1e-5, atol=1e-30)
    assert np.isclose(out[2], 1 * sig(alpha) * (1.5 + 1), rtol=1e-6)
    assert np.isclose(out[3], 1 * sig(alpha) * (1.0 + 1), rtol=1e-6)
    # random case against float64
    rng = np.random.default_rng(12)
    hidden, inter = 64, 96
    mk = lambda n, k: (rng.integers(0, 256, n * k // 2, dtype=np.uint8).tobytes(),
                       rng.integers(118, 124, n * k // 32, dtype=np.uint8).tobytes())
    (b1, s1), (b2, s2) = mk(2 * inter, hidden), mk(hidden, inter)
    bias1 = rng.standard_normal(2 * inter).astype(np.float32)
    bias2 = rng.standard_normal(hidden).astype(np.float32)
    x = rng.standard_normal(hidden).astype(np.float32)
    h = mx_dequant(b1, s1, 2 * inter, hidden) @ x.astype(np.float64) + bias1
    gate, lin = np.minimum(h[0::2], clamp), np.clip(h[1::2], -clamp, clamp)
    act = gate * sig(alpha * gate) * (lin + 1)
    want = mx_dequant(b2, s2, hidden, inter) @ act + bias2
    got = orc.mxfp4_expert_forward(x, hidden, inter, alpha, clamp, b1, s1, b2, s2, bias1, bias2)
    assert np.abs(got - want).max() <= 5e-6 * np.abs(want).max()
