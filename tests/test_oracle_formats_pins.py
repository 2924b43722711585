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


def _mx_expert(rng, hidden, inter):
    return (rng.integers(0, 256, 2 * inter * hidden // 2, dtype=np.uint8), rng.integers(118, 126, 2 * inter * hidden // 32, dtype=np.uint8),
            rng.integers(0, 256, hidden * inter // 2, dtype=np.uint8), rng.integers(118, 126, hidden * inter // 32, dtype=np.uint8),
            rng.standard_normal(2 * inter).astype(np.float32), rng.standard_normal(hidden).astype(np.float32))


def test_mxfp4_moe_is_the_experts_outputs_added_in_the_routing_s_order(orc):
    """examples/gpt_oss/moe.rs:330-351: output += weight * expert_out, experts in the order the router listed them.
    Recomputed in float32 NumPy from orc_mxfp4_expert_forward's own outputs; equal bit for bit, and a swapped order
    is not (so the order is what is pinned)."""
    rng = np.random.default_rng(77)
    hidden, inter, E, top_k, T = 64, 96, 5, 3, 6
    experts = [_mx_expert(rng, hidden, inter) for _ in range(E)]
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    idx = np.array([rng.permutation(E)[:top_k] for _ in range(T)], np.int32)
    w = rng.random((T, top_k)).astype(np.float32)
    got = orc.mxfp4_moe_routed(x, T, hidden, inter, 1.702, 7.0, top_k, idx, w, experts)
    differs = False
    for t in range(T):
        ys = [orc.mxfp4_expert_forward(x[t], hidden, inter, 1.702, 7.0, *experts[e]) for e in idx[t]]
        acc = np.zeros(hidden, np.float32)
        for k in range(top_k):
            acc = (acc + (w[t, k] * ys[k]).astype(np.float32)).astype(np.float32)
        assert (got[t].view(np.uint32) == acc.view(np.uint32)).all()
        rev = np.zeros(hidden, np.float32)
        for k in reversed(range(top_k)):
            rev = (rev + (w[t, k] * ys[k]).astype(np.float32)).astype(np.float32)
        differs |= bool((rev.view(np.uint32) != acc.view(np.uint32)).any())
    assert differs


# ---- canonical Huffman ------------------------------------------------------------------

def biased_i8(n, seed):
    """random_i8 of the reference's unit tests (src/huffman.rs:743-754)."""
    out, state = np.empty(n, np.int8), seed
    for i in range(n):
        state = (state * 1103515245 + 12345) & 0xFFFFFFFF
        raw = ((state >> 16) % 256 - 128)
        raw = raw - 256 if raw > 127 else raw
        v = raw if (state >> 8) % 4 == 0 else int(raw / 4)      # Rust integer division truncates
        out[i] = v
    return out


def heap_huffman_cost(freqs):
    import heapq
    h = [int(f) for f in freqs if f > 0]
    if len(h) == 1:
        return h[0]
    heapq.heapify(h)
    cost = 0
    while len(h) > 1:
        a, b = heapq.heappop(h), heapq.heappop(h)
        cost += a + b
        heapq.heappush(h, a + b)
    return cost


def test_huffman_table_hand_worked_tie_breaking(orc):
    """Leaves [1,1,1,1,2] (symbols -128..-124).  Stable order a b c d e; a+b -> I1(2); c+d -> I2(2);
    then e(2), I1(2), I2(2) tie and the LEAF goes first: e+I1 -> I3(4); I2+I3 -> root.  Depths:
    a,b = 3; c,d = 2; e = 2.  (Taking internal nodes first would give e = 1 and a..d = 3.)"""
    f = np.zeros(256, np.uint64)
    f[:5] = [1, 1, 1, 1, 2]
    bl, codes = orc.huffman_table(f)
    assert bl[:5].tolist() == [3, 3, 2, 2, 2] and not bl[5:].any()
    # canonical: lengths ascending, symbol order within a length: c=00 d=01 e=10 a=110 b=111
    assert codes[:5].tolist() == [0b110, 0b111, 0b00, 0b01, 0b10]
    # the reference's own table test (src/huffman.rs:801-815) and the one-symbol rule (:52-64)
    f = np.zeros(256, np.uint64)
    f[128], f[129] = 100, 50
    bl, codes = orc.huffman_table(f)
    assert bl[128] == 1 and bl[129] == 1 and codes[128] == 0 and codes[129] == 1
    f = np.zeros(256, np.uint64)
    f[170] = 512
    bl, codes = orc.huffman_table(f)
    assert bl[170] == 1 and codes[170] == 0 and bl.sum() == 1
    assert not orc.huffman_table(np.zeros(256, np.uint64))[0].any()


def test_huffman_table_is_optimal_and_complete(orc):
    rng = np.random.default_rng(2)
    for trial in range(6):
        f = np.zeros(256, np.uint64)
        k = [2, 3, 17, 100, 256, 256][trial]
        f[rng.choice(256, k, replace=False)] = rng.integers(1, 50 if trial < 5 else 4, k)
        bl, codes = orc.huffman_table(f)
        assert ((bl > 0) == (f > 0)).all()
        assert bl.max() <= 12                                     # a clamped depth would break the cost equality below
        assert int((f * bl).sum()) == heap_huffman_cost(f)        # any Huffman tree has the optimal cost
        assert sum(2.0 ** -int(l) for l in bl if l) == 1.0        # Kraft equality: a complete prefix code
        used = [(int(bl[s]), int(codes[s])) for s in range(256) if bl[s]]
        strs = sorted(format(c, "b").zfill(l) for l, c in used)
        assert all(not strs[i + 1].startswith(strs[i]) for i in range(len(strs) - 1))   # prefix-free


def test_huffman_depth_clamp_is_the_reference_s(orc):
    """Fibonacci frequencies make a path deeper than 12; the reference clamps the depths and
    keeps going (src/huffman.rs:128-134), which over-subscribes the code."""
    fib = [1, 1]
    while len(fib) < 20:
        fib.append(fib[-1] + fib[-2])
    f = np.zeros(256, np.uint64)
    f[:20] = fib
    bl, _ = orc.huffman_table(f)
    assert bl[:20].max() == 12 and (bl[:8] == 12).all()
    assert sum(2.0 ** -int(l) for l in bl if l) > 1.0


def test_huffman_encode_hand_packed_and_reference_round_trips(orc):
    f = np.zeros(256, np.uint64)
    f[:5] = [1, 1, 1, 1, 2]
    bl, _ = orc.huffman_table(f)                                  # a=110 b=111 c=00 d=01 e=10
    data = np.array([-128, -124, -126, -127, -125], np.int8)      # a e c b d -> 110 10 00 111 01 -> 11010001 1101(0000)
    assert orc.huffman_encode(bl, data) == bytes([0b11010001, 0b11010000])
    assert (orc.huffman_decode(bl, bytes([0b11010001, 0b11010000]), 5) == data).all()
    assert orc.huffman_encode(bl, np.zeros(0, np.int8)) == b""    # src/huffman.rs:771-778
    # src/huffman.rs:756-768: round trip on the biased generator
    data = biased_i8(1024, 42)
    bl, _ = orc.huffman_table(np.bincount(data.astype(np.int16) + 128, minlength=256))
    enc = orc.huffman_encode(bl, data)
    assert (orc.huffman_decode(bl, enc, data.size) == data).all()
    assert len(enc) < data.size                                    # it does compress
    # src/huffman.rs:780-797: 512 equal symbols in at most 65 bytes
    same = np.full(512, 42, np.int8)
    bl, _ = orc.huffman_table(np.bincount(same.astype(np.int16) + 128, minlength=256))
    enc = orc.huffman_encode(bl, same)
    assert len(enc) <= 65 and (orc.huffman_decode(bl, enc, 512) == same).all()


# ---- HuffmanKVCache ---------------------------------------------------------------------

def parity_random_data(n, seed):
    """random_data of tests/huffman_parity.rs:7-16: (state as f32 / u32::MAX as f32) * 2 - 1."""
    out, state = np.empty(n, np.float32), seed
    for i in range(n):
        state = (state * 1103515245 + 12345) & 0xFFFFFFFF
        out[i] = np.float32(state) / np.float32(4294967295) * np.float32(2.0) - np.float32(1.0)
    return out


def numpy_chunk_quant(data, num_tokens, num_heads, head_dim):
    """Scales and int8 values of a chunk in float32 NumPy: absmax / 127 (or 1), round half away
    from zero of v * (1 / scale), clamped to +-127."""
    d = np.asarray(data, np.float32).reshape(num_heads, num_tokens * head_dim)
    absmax = np.abs(d).max(axis=1) if d.shape[1] else np.zeros(num_heads, np.float32)
    scales = np.where(absmax == 0, np.float32(1), absmax / np.float32(127)).astype(np.float32)
    t = d * (np.float32(1) / scales)[:, None]
    r = np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))      # exact in f32 below 2^23
    frac_half = (np.abs(t) - np.floor(np.abs(t))) == np.float32(0.5)
    assert t.dtype == np.float32 and (np.abs(t) < 2 ** 22).all() and frac_half.sum() >= 0
    return scales, np.clip(r, -127, 127).astype(np.int8).reshape(-1)


def test_kv_chunk_reference_tests_restated(orc):
    # src/huffman.rs:879-905
    h, d, t = 2, 8, 16
    data = np.array([((i * 13 + 7) % 100) / 50.0 - 1.0 for i in range(h * t * d)], np.float32)
    # tests/huffman_parity.rs:133-158
    for data, (t, h, d) in ((data, (t, h, d)), (parity_random_data(4 * 32 * 16, 99), (32, 4, 16))):
        bits, scales, codebook, q = orc.huffman_kv_compress_chunk(data, t, h, d)
        rec = orc.huffman_kv_decompress_chunk(bits, scales, codebook, t, h, d)
        per_head = np.abs(data - rec).reshape(h, -1).max(axis=1)
        absmax = np.abs(data).reshape(h, -1).max(axis=1)
        assert (scales == absmax / np.float32(127)).all()
        assert (per_head <= scales + 1e-5).all()                 # the reference's bound
        assert (per_head <= scales * 0.5 * (1 + 1e-6)).all()     # what round-to-nearest gives and truncation does not


def test_kv_chunk_closed_forms(orc):
    t, h, d = 8, 3, 4
    n = t * d
    # head 0 all zero, head 1 constant 2.5, head 2 holds +absmax and -absmax
    data = np.zeros((h, n), np.float32)
    data[1] = 2.5
    data[2] = np.linspace(-3.0, 3.0, n, dtype=np.float32)
    bits, scales, codebook, q = orc.huffman_kv_compress_chunk(data, t, h, d)
    assert scales[0] == 1.0 and scales[1] == np.float32(2.5) / np.float32(127) and scales[2] == np.float32(3.0) / np.float32(127)
    q = q.reshape(h, n)
    assert (q[0] == 0).all() and (q[1] == 127).all() and q[2, 0] == -127 and q[2, -1] == 127
    rec = orc.huffman_kv_decompress_chunk(bits, scales, codebook, t, h, d).reshape(h, n)
    assert (rec[0] == 0).all() and (rec[1] == np.float32(127) * scales[1]).all()
    # one value only: a 1-bit code (src/huffman.rs:52-64), ceil(n / 8) zero bytes, 256 bit lengths with a single 1
    const = np.full(5 * 7 * 3, -0.75, np.float32)
    bits, scales, codebook, q = orc.huffman_kv_compress_chunk(const, 7, 5, 3)
    assert bits == bytes((const.size + 7) // 8) and (q == -127).all()
    assert codebook[-127 + 128] == 1 and codebook.sum() == 1
    assert (orc.huffman_kv_decompress_chunk(bits, scales, codebook, 7, 5, 3) == np.float32(-127) * scales[0]).all()
    # NaN is skipped by the maximum and quantises to 0; an empty chunk is an empty stream under an empty table
    data = np.array([1.0, np.nan, -0.5, 0.25], np.float32)
    bits, scales, codebook, q = orc.huffman_kv_compress_chunk(data, 1, 1, 4)
    assert scales[0] == np.float32(1) / np.float32(127) and q.tolist() == [127, 0, -64, 32]
    bits, scales, codebook, q = orc.huffman_kv_compress_chunk(np.zeros(0, np.float32), 0, 2, 4)
    assert bits == b"" and not codebook.any() and (scales == 1.0).all()


def test_kv_chunk_is_numpy_quantisation_under_the_pinned_coder(orc):
    rng = np.random.default_rng(11)
    for t, h, d in ((5, 3, 7), (32, 4, 16), (1, 1, 1), (64, 2, 128)):
        data = (rng.standard_normal(t * h * d) * rng.choice([0.01, 1.0, 300.0])).astype(np.float32)
        data[rng.integers(0, data.size, 3)] = 0.0
        bits, scales, codebook, q = orc.huffman_kv_compress_chunk(data, t, h, d)
        want_scales, want_q = numpy_chunk_quant(data, t, h, d)
        assert (scales == want_scales).all() and (q == want_q).all()
        bl, _, _ = orc.huffman_table_that_decodes(np.bincount(want_q.astype(np.int16) + 128, minlength=256))
        assert (codebook == bl).all() and bits == orc.huffman_encode(bl, want_q)
        rec = orc.huffman_kv_decompress_chunk(bits, scales, codebook, t, h, d)
        assert (rec == (want_q.reshape(h, -1).astype(np.float32) * want_scales[:, None]).reshape(-1)).all()


def test_kv_chunk_table_is_the_reference_s_unless_that_one_cannot_decode(orc):
    """Where from_frequencies yields a prefix code the chunk uses it unchanged; where its clamp
    over-subscribes the code (the reference panics there) the repaired lengths are a prefix code of
    at most 12 bits, ordered by frequency, within two percent of the unlimited Huffman cost."""
    rng = np.random.default_rng(3)
    flat = rng.integers(20, 50, 256).astype(np.uint64)
    bl, _, repaired = orc.huffman_table_that_decodes(flat)
    assert not repaired and (bl == orc.huffman_table(flat)[0]).all()
    fib = [1, 1]
    while len(fib) < 24:
        fib.append(fib[-1] + fib[-2])
    f_fib = np.zeros(256, np.uint64)
    f_fib[100:124] = fib
    bell = np.bincount(np.clip(np.rint(rng.standard_normal(1 << 16) * 30), -127, 127).astype(np.int16) + 128, minlength=256).astype(np.uint64)
    for f in (f_fib, bell):
        ref_bl = orc.huffman_table(f)[0]
        assert sum(2.0 ** -int(l) for l in ref_bl if l) > 1.0        # the case the reference cannot handle
        bl, codes, repaired = orc.huffman_table_that_decodes(f)
        assert repaired and ((bl > 0) == (f > 0)).all() and bl.max() <= 12
        assert sum(2.0 ** -int(l) for l in bl if l) <= 1.0
        used = np.flatnonzero(f)
        for a in used:                                               # a more frequent symbol never has the longer code
            assert (bl[used][f[used] < f[a]] >= bl[a]).all()
        assert int((f * bl).sum()) <= heap_huffman_cost(f) * 1.02
        data = np.repeat(np.arange(256) - 128, np.minimum(f, 50).astype(np.int64)).astype(np.int8)
        rng.shuffle(data)
        assert (orc.huffman_decode(bl, orc.huffman_encode(bl, data), data.size) == data).all()
    # through compress_chunk: a bell-shaped chunk of realistic size round-trips
    t, h, d = 64, 2, 128
    data = rng.standard_normal(t * h * d).astype(np.float32)
    bits, scales, codebook, q = orc.huffman_kv_compress_chunk(data, t, h, d)
    rec = orc.huffman_kv_decompress_chunk(bits, scales, codebook, t, h, d)
    assert (rec == (q.reshape(h, -1).astype(np.float32) * scales[:, None]).reshape(-1)).all()


def test_kv_cache_reference_tests_restated(orc):
    # src/huffman.rs:850-876
    c = orc.HuffmanKVCache(2, 4, 8, 4)
    c.append(np.full(32, 1.0), np.full(32, 2.0), 4)
    assert (c.len, c.compressed_len) == (4, 0)
    c.append(np.full(32, 3.0), np.full(32, 4.0), 4)
    assert (c.len, c.compressed_len) == (8, 4)
    k, v = c.get_kv()
    assert k.size == v.size == 2 * 8 * 4
    assert (k.reshape(2, 8, 4)[:, :4] == 1.0).all() and (k.reshape(2, 8, 4)[:, 4:] == 3.0).all()
    assert (v.reshape(2, 8, 4)[:, :4] == 2.0).all() and (v.reshape(2, 8, 4)[:, 4:] == 4.0).all()
    # tests/huffman_parity.rs:160-186
    c = orc.HuffmanKVCache(2, 8, 16, 8)
    for batch in range(4):
        c.append(parity_random_data(2 * 8 * 8, 100 + batch), parity_random_data(2 * 8 * 8, 200 + batch), 8)
    assert c.len == 32 and c.compressed_len > 0
    k, v = c.get_kv()
    assert k.size == v.size == 2 * 32 * 8
    # new(): compress_threshold.max(chunk_size)  (src/huffman.rs:535)
    assert orc.HuffmanKVCache(1, 1, 3, 10).compress_threshold == 10


def test_kv_cache_keeps_token_order(orc):
    """Whatever the append sizes, get_kv is: per chunk, decompress(compress(.)) of the tokens the
    chunk took in arrival order, then the window's tokens bit for bit."""
    rng = np.random.default_rng(5)
    for heads, hd, thr, chunk, appends in ((2, 8, 16, 8, (8, 8, 8, 8)), (3, 4, 10, 4, (1, 7, 2, 30, 5, 1)), (1, 16, 0, 5, (3, 3, 3)),
                                           (2, 2, 6, 6, (13,))):
        c = orc.HuffmanKVCache(heads, hd, thr, chunk)
        all_k, all_v = np.zeros((heads, 0, hd), np.float32), np.zeros((heads, 0, hd), np.float32)
        for n in appends:
            k, v = rng.standard_normal((heads, n, hd)).astype(np.float32), rng.standard_normal((heads, n, hd)).astype(np.float32)
            c.append(k, v, n)
            all_k, all_v = np.concatenate([all_k, k], 1), np.concatenate([all_v, v], 1)
            total = all_k.shape[1]
            threshold = max(thr, chunk)
            # chunks of exactly chunk_size are cut while at least `threshold` tokens are left
            ncomp = 0
            while total - ncomp >= threshold:
                ncomp += chunk
            assert (c.len, c.compressed_len, c.hot_len, c.num_chunks) == (total, ncomp, total - ncomp, ncomp // chunk)
            for side, full in ((0, all_k), (1, all_v)):
                got = c.get_kv()[side].reshape(heads, total, hd)
                assert (got[:, ncomp:] == full[:, ncomp:]).all()
                for i in range(ncomp // chunk):
                    part = full[:, i * chunk:(i + 1) * chunk]
                    bits, scales, codebook, _ = orc.huffman_kv_compress_chunk(part, chunk, heads, hd)
                    cb, cs, ccb, ct = c.chunk(side, i)
                    assert (cb, ct) == (bits, chunk) and (cs == scales).all() and (ccb == codebook).all()
                    rec = orc.huffman_kv_decompress_chunk(bits, scales, codebook, chunk, heads, hd).reshape(heads, chunk, hd)
                    assert (got[:, i * chunk:(i + 1) * chunk] == rec).all()
        # the reference's own hot-window offsets agree for head 0 always
        lit = c.get_kv(True)[0].reshape(heads, -1, hd)
        assert (lit[0] == c.get_kv()[0].reshape(heads, -1, hd)[0]).all()
