"""The host half of the Huffman path (table builder, canonical codes, encoder, HuffmanTensor
container) through the C ABI against the CPU oracle.  None of these calls touches a device."""
import numpy as np
import pytest

from test_oracle_formats_pins import biased_i8


def _freqs(data):
    return np.bincount(np.asarray(data, np.int8).astype(np.int16) + 128, minlength=256).astype(np.uint64)


def test_table_and_codes_equal_the_oracle(orc):
    from peregrine_amd import huffman
    rng = np.random.default_rng(0)
    cases = [np.zeros(256, np.uint64)]
    f = np.zeros(256, np.uint64); f[:5] = [1, 1, 1, 1, 2]; cases.append(f)          # the tie-breaking case
    f = np.zeros(256, np.uint64); f[170] = 9; cases.append(f)                        # one symbol
    fib = [1, 1]
    while len(fib) < 24:
        fib.append(fib[-1] + fib[-2])
    f = np.zeros(256, np.uint64); f[100:124] = fib; cases.append(f)                  # depth clamp
    for k in (2, 7, 64, 256):
        f = np.zeros(256, np.uint64); f[rng.choice(256, k, replace=False)] = rng.integers(1, 1000, k); cases.append(f)
    cases.append(_freqs(np.clip(np.rint(rng.standard_normal(1 << 16) * 20), -127, 127)))   # weight-like
    for i in range(3000):                                                             # many ties, few to all symbols, wide ranges
        k = int(rng.integers(2, 257))
        f = np.zeros(256, np.uint64)
        hi = (2, 3, 5, 50, 1 << 20, 1 << 40)[i % 6]
        f[rng.choice(256, k, replace=False)] = rng.integers(1, hi, k)
        if i % 7 == 0:
            f[f > 0] = np.sort(f[f > 0])[::-1]                                        # falling with the symbol
        if i % 11 == 0:
            f[f > 0] = 2 ** rng.integers(0, 30, int((f > 0).sum()))                   # powers of two: sums that tie with leaves
        cases.append(f)
    for f in cases:
        t = huffman.HuffmanTable.from_frequencies(f)
        bl, codes = orc.huffman_table(f)
        assert (t.bit_lengths == bl).all() and (t.codes == codes).all()
        assert (huffman.HuffmanTable.from_bytes(t.to_bytes()).codes == codes).all()
    with pytest.raises(ValueError):
        huffman.HuffmanTable.from_bytes(bytes(255))                                   # "codebook too short"


def test_encode_equals_the_oracle_bit_for_bit(orc):
    from peregrine_amd import huffman, _ffi
    for n, seed in ((0, 1), (1, 2), (7, 3), (1024, 42), (100003, 5)):
        data = biased_i8(n, seed) if n <= 1024 else np.clip(np.rint(np.random.default_rng(seed).standard_normal(n) * 9), -24, 24).astype(np.int8)
        t = huffman.HuffmanTable.from_frequencies(_freqs(data))
        assert t.encode(data) == orc.huffman_encode(t.bit_lengths, data)
    t = huffman.HuffmanTable.from_frequencies(_freqs(np.array([1, 2, 2], np.int8)))
    with pytest.raises(_ffi.PeregrineError):
        t.encode(np.array([3], np.int8))                                              # a symbol with no code


def test_huffman_tensor_container(orc):
    """HuffmanTensor::from_quantized (src/huffman.rs:332-372): shared table over all data,
    contiguous chunks of ceil(total / num_streams), empty trailing streams, sizes."""
    from peregrine_amd import huffman
    from peregrine_amd.quant import QuantizedTensor
    rows, cols = 37, 11
    q = np.clip(np.rint(np.random.default_rng(3).standard_normal(rows * cols) * 6), -127, 127).astype(np.int8)
    scales = np.linspace(0.01, 0.02, cols).astype(np.float32)
    qt = QuantizedTensor(q, None, scales, rows, cols)
    for ns in (1, 4, 5, 500):
        ht = huffman.HuffmanTensor.from_quantized(qt, ns)
        bl, _ = orc.huffman_table(_freqs(q))
        assert (ht.table.bit_lengths == bl).all() and ht.num_streams == ns and (ht.scales == scales).all()
        chunk = -(-q.size // ns)
        for s in range(ns):
            part = q[s * chunk:(s + 1) * chunk]
            assert ht.stream_lengths[s] == part.size
            assert ht.streams[s] == orc.huffman_encode(bl, part)
        assert ht.compressed_size() == sum(len(s) for s in ht.streams) + 256 + cols * 4
        assert ht.uncompressed_size() == rows * cols + cols * 4
        ht2 = huffman.HuffmanTensor.from_parts(ht.table, ht.streams, ht.stream_lengths, ht.scales, rows, cols)
        assert ht2.streams == ht.streams and ht2.stream_lengths == ht.stream_lengths
    assert huffman.HuffmanTensor.from_quantized(qt, 0).num_streams == 1               # num_streams.max(1)
