"""GPU parity of the Huffman decode path against the CPU oracle, through the C ABI.
Bar: decoded symbols bit-exact; matmul_huffman bit-identical to matmul_quantized on the same
tensor (the reference bounds it by 1e-3, tests/huffman_parity.rs:23-42)."""
import sys

import numpy as np
import pytest

import helpers as H
from test_oracle_formats_pins import biased_i8

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _freqs(data):
    return np.bincount(np.asarray(data, np.int8).astype(np.int16) + 128, minlength=256).astype(np.uint64)


def _weights_like(n, seed, sigma=9.0):
    """Bell-shaped integers cut at +-2.7 sigma: the rarest symbol is still frequent enough
    that no code is deeper than 12 bits (the reference clamps deeper ones and then cannot
    decode its own stream, src/huffman.rs:128-134)."""
    lim = int(2.7 * sigma)
    return np.clip(np.rint(np.random.default_rng(seed).standard_normal(n) * sigma), -lim, lim).astype(np.int8)


@pytest.mark.parametrize("n,seed", [(1, 1), (5, 2), (1024, 42), (70001, 3), (3_000_000, 4)])
def test_decode_round_trip_and_oracle(ctx, orc, n, seed):
    """src/huffman.rs:756-768 scaled up: one thread per 256 bits, several workgroups, ragged tail."""
    from peregrine_amd import huffman
    say(f"huffman decode n={n}")
    data = biased_i8(n, seed) if n <= 1024 else _weights_like(n, seed)
    t = huffman.HuffmanTable.from_frequencies(_freqs(data))
    enc = t.encode(data)
    got = t.decode(enc, n, ctx)
    assert (got == data).all()
    if n <= 70001:
        assert (got == orc.huffman_decode(t.bit_lengths, enc, n)).all()
    # fewer symbols than the stream holds: the prefix
    assert (t.decode(enc, max(n // 2, 1), ctx) == data[:max(n // 2, 1)]).all()


def test_decode_hand_packed_and_edge_tables(ctx, orc):
    from peregrine_amd import huffman, _ffi
    f = np.zeros(256, np.uint64)
    f[:5] = [1, 1, 1, 1, 2]                                        # a=110 b=111 c=00 d=01 e=10
    t = huffman.HuffmanTable.from_frequencies(f)
    assert (t.decode(bytes([0b11010001, 0b11010000]), 5, ctx) == np.array([-128, -124, -126, -127, -125], np.int8)).all()
    assert t.decode(b"", 0, ctx).size == 0                          # src/huffman.rs:771-778
    same = np.full(512, 42, np.int8)                                # src/huffman.rs:780-797
    t1 = huffman.HuffmanTable.from_frequencies(_freqs(same))
    enc = t1.encode(same)
    assert len(enc) <= 65 and (t1.decode(enc, 512, ctx) == same).all()
    with pytest.raises(_ffi.PeregrineError):
        t1.decode(bytes([0x80]), 3, ctx)                            # a set bit has no code in a one-symbol table
    with pytest.raises(_ffi.PeregrineError):
        t.decode(bytes([0b11010001]), 40, ctx)                      # the stream ends before 40 symbols


def test_decode_streams_that_never_resynchronise(ctx, orc):
    """128 equally likely symbols all get 7-bit codes: a wrong start stays wrong, so every
    subsequence has to wait for its predecessor (the slow path of the settling loop)."""
    from peregrine_amd import huffman
    rng = np.random.default_rng(8)
    data = rng.integers(-64, 64, 400_000).astype(np.int8)
    f = np.zeros(256, np.uint64)
    f[64:192] = 1000
    t = huffman.HuffmanTable.from_frequencies(f)
    assert set(t.bit_lengths[64:192].tolist()) == {7}
    say("huffman decode, fixed 7-bit codes")
    enc = t.encode(data)
    assert (t.decode(enc, data.size, ctx) == data).all()


def test_decode_arbitrary_bytes_as_a_complete_code(ctx, orc):
    """With a complete code every bit string decodes: random bytes through the device decoder
    equal the oracle's serial walk symbol for symbol."""
    from peregrine_amd import huffman
    t = huffman.HuffmanTable.from_frequencies(_freqs(_weights_like(50000, 6, 3.0)))
    assert sum(2.0 ** -int(l) for l in t.bit_lengths if l) == 1.0
    raw = np.random.default_rng(9).integers(0, 256, 20000, dtype=np.uint8).tobytes()
    n = 160000 // int(t.bit_lengths[t.bit_lengths > 0].max())       # surely inside the stream
    assert (t.decode(raw, n, ctx) == orc.huffman_decode(t.bit_lengths, raw, n)).all()


def test_huffman_tensor_round_trip_and_matmul(ctx, orc):
    """tests/huffman_parity.rs:23-42 and src/huffman.rs:817-833 with the reference's generators."""
    from peregrine_amd import huffman, quant
    for (m, k, n) in ((8, 32, 16), (1, 64, 1), (32, 128, 64), (16, 256, 32), (4, 1024, 777)):
        say(f"matmul_huffman m={m} k={k} n={n}")
        a = H.lcg_data(m * k, 42)
        w = H.lcg_data(k * n, 123)
        qt = quant.quantize_weights(w, k, n, ctx)
        ht = huffman.HuffmanTensor.from_quantized(qt, 4)
        qt2 = ht.decode_to_quantized(ctx)
        assert (qt2.data_i8 == qt.data_i8).all() and (qt2.data_i8_t == qt.data_i8_t).all() and (qt2.scales == qt.scales).all()
        ref = quant.matmul_quantized(a, m, k, qt, ctx)
        got = huffman.matmul_huffman(a, m, k, ht, ctx)
        assert (got.view(np.uint32) == ref.view(np.uint32)).all()
        assert (got.view(np.uint32) == orc.matmul_quantized(a, m, k, qt.data_i8_t, qt.scales, n)[0].view(np.uint32)).all()
        resident = ht.to_gpu(ctx)
        assert (quant.matmul_quantized(a, m, k, resident, ctx).view(np.uint32) == ref.view(np.uint32)).all()
    with pytest.raises(ValueError):
        huffman.matmul_huffman(a, 4, 1023, ht, ctx)                  # assert_eq!(ht.rows, k)


def test_huffman_tensor_compresses_large_weights(ctx, orc):
    """src/huffman.rs:835-851 at a larger size: ratio above 1 and an exact round trip through
    16 streams of unequal length."""
    from peregrine_amd import huffman, quant
    rows, cols = 1024, 1000
    w = (np.arange(rows * cols) * 7 + 3) % 200 / np.float32(200.0) - np.float32(0.5)
    qt = quant.quantize_weights(w.astype(np.float32), rows, cols, ctx)
    ht = huffman.HuffmanTensor.from_quantized(qt, 16)
    assert ht.compression_ratio() > 1.0
    say(f"huffman tensor {rows}x{cols}: ratio {ht.compression_ratio():.3f}")
    assert (ht.decode_to_quantized(ctx).data_i8 == qt.data_i8).all()
