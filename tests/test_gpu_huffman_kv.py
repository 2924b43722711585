"""GPU parity of the Huffman-coded KV cache against the CPU oracle, through the C ABI.
Bar: bit-exact everywhere (scales, code table, bitstream bytes, decoded f32 values, the
cache's lengths and what get_kv returns)."""
import ctypes as C
import sys

import numpy as np
import pytest

from devbuf import DevBuf
from test_oracle_formats_pins import parity_random_data

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _same_chunk(chunk, want):
    bits, scales, codebook = want[:3]
    assert chunk.codebook == codebook.tobytes()
    assert (chunk.scales.view(np.uint32) == scales.view(np.uint32)).all()
    assert chunk.bitstream == bits


def _chunk_data(kind, t, h, d, seed):
    rng = np.random.default_rng(seed)
    n = t * h * d
    if kind == "normal":
        return rng.standard_normal(n).astype(np.float32)
    if kind == "uniform":
        return parity_random_data(n, seed)
    if kind == "scaled_heads":                     # heads of very different magnitude, one of them all zero
        x = rng.standard_normal((h, t * d)).astype(np.float32) * (10.0 ** rng.integers(-6, 6, (h, 1))).astype(np.float32)
        x[rng.integers(0, h)] = 0.0
        return x.reshape(-1)
    if kind == "constant":
        return np.full(n, -0.75, np.float32)
    if kind == "special":                          # NaN is skipped by the maximum and becomes 0; halves round away from zero
        x = rng.standard_normal(n).astype(np.float32)
        x[::7] = np.nan
        x[1::11] = 0.0
        if n > 4:
            x[2], x[3] = 127.0, 63.5
        return x
    raise AssertionError(kind)


@pytest.mark.parametrize("kind,t,h,d", [
    ("uniform", 32, 4, 16),          # tests/huffman_parity.rs:133-158
    ("normal", 5, 3, 7), ("normal", 1, 1, 1), ("normal", 16, 2, 8), ("normal", 256, 2, 8),
    ("normal", 31, 3, 43),           # 3999 symbols: one encoder workgroup with a ragged tail
    ("normal", 64, 2, 128),          # a table whose reference form over-subscribes the code: repaired
    ("normal", 256, 8, 128),         # 262144 symbols, 64 encoder workgroups
    ("scaled_heads", 40, 6, 64), ("constant", 7, 5, 3), ("special", 9, 2, 16), ("special", 300, 3, 64),
])
def test_compress_chunk_is_the_oracle_s(ctx, orc, kind, t, h, d):
    from peregrine_amd import huffman
    say(f"huffman kv compress_chunk {kind} tokens={t} heads={h} head_dim={d}")
    data = _chunk_data(kind, t, h, d, 1000 + t + h + d)
    want = orc.huffman_kv_compress_chunk(data, t, h, d)
    chunk = huffman.HuffmanKVCache.compress_chunk(data, t, h, d, ctx)
    assert (chunk.num_tokens, chunk.num_heads, chunk.head_dim) == (t, h, d)
    _same_chunk(chunk, want)
    got = huffman.HuffmanKVCache.decompress_chunk(chunk)
    ref = orc.huffman_kv_decompress_chunk(*want[:3], t, h, d)
    assert (got.view(np.uint32) == ref.view(np.uint32)).all()
    # a chunk rebuilt from the oracle's parts decodes to the same values
    again = huffman.CompressedChunk.from_parts(want[0], want[1], want[2], t, h, d, ctx)
    assert (huffman.HuffmanKVCache.decompress_chunk(again).view(np.uint32) == ref.view(np.uint32)).all()
    if kind in ("uniform", "normal"):              # the reference's bound, and the half step that rounding to nearest gives
        err = np.abs(got - data).reshape(h, -1).max(axis=1)
        assert (err <= want[1] + 1e-5).all() and (err <= want[1] * 0.5 * (1 + 1e-6)).all()


def test_reference_unit_test_chunk(ctx, orc):
    """src/huffman.rs:879-905."""
    from peregrine_amd import huffman
    h, d, t = 2, 8, 16
    data = np.array([((i * 13 + 7) % 100) / 50.0 - 1.0 for i in range(h * t * d)], np.float32)
    chunk = huffman.HuffmanKVCache.compress_chunk(data, t, h, d, ctx)
    _same_chunk(chunk, orc.huffman_kv_compress_chunk(data, t, h, d))
    rec = huffman.HuffmanKVCache.decompress_chunk(chunk)
    absmax = np.abs(data).reshape(h, -1).max(axis=1)
    assert (np.abs(rec - data).reshape(h, -1).max(axis=1) <= absmax / 127 + 1e-5).all()


def test_empty_chunks_and_errors(ctx, orc):
    from peregrine_amd import huffman, _ffi
    for t, h, d in ((0, 2, 4), (3, 0, 4), (3, 2, 0)):
        chunk = huffman.HuffmanKVCache.compress_chunk(np.zeros(0, np.float32), t, h, d, ctx)
        want = orc.huffman_kv_compress_chunk(np.zeros(0, np.float32), t, h, d)
        _same_chunk(chunk, want)
        assert chunk.bitstream == b"" and huffman.HuffmanKVCache.decompress_chunk(chunk).size == 0
    with pytest.raises(ValueError):
        huffman.HuffmanKVCache.compress_chunk(np.zeros(5, np.float32), 1, 2, 3, ctx)      # assert_eq!(data.len(), total)
    with pytest.raises(_ffi.PeregrineError):
        huffman.HuffmanKVCache(2, 4, 8, 0, ctx)                                           # the reference's append would never return
    # a stream that is too short for its symbol count, and a codebook that cannot produce it
    bits, scales, codebook, _ = orc.huffman_kv_compress_chunk(np.linspace(-1, 1, 64, dtype=np.float32), 8, 2, 4)
    short = huffman.CompressedChunk.from_parts(bits[:len(bits) // 2], scales, codebook, 8, 2, 4, ctx)
    with pytest.raises(_ffi.PeregrineError):
        huffman.HuffmanKVCache.decompress_chunk(short)
    one = np.zeros(256, np.uint8)
    one[128] = 1
    wrong = huffman.CompressedChunk.from_parts(bytes([0xFF] * 8), scales, one, 8, 2, 4, ctx)
    with pytest.raises(_ffi.PeregrineError):
        huffman.HuffmanKVCache.decompress_chunk(wrong)


def test_chunks_from_and_to_strided_device_memory(ctx, orc):
    """The `_dev` entry points: heads `head_stride` floats apart on both sides, as in a StandardKVCache."""
    from peregrine_amd import huffman, _ffi
    t, h, d, stride = 24, 3, 32, 24 * 32 + 160
    rng = np.random.default_rng(8)
    padded = rng.standard_normal((h, stride)).astype(np.float32)
    data = padded[:, :t * d].copy()
    src = DevBuf(ctx, host=padded)
    handle = C.c_void_p()
    _ffi.check(_ffi.lib.pg_huffman_kv_compress_chunk_dev(ctx.handle, src.ptr, stride, t, h, d, C.byref(handle)))
    chunk = huffman.CompressedChunk(handle, ctx)
    want = orc.huffman_kv_compress_chunk(data, t, h, d)
    _same_chunk(chunk, want)
    dst = DevBuf(ctx, host=np.full((h, stride), 7.0, np.float32))
    _ffi.check(_ffi.lib.pg_huffman_kv_decompress_chunk_dev(ctx.handle, chunk._h, dst.ptr, stride))
    ctx.sync()
    got = dst.to_host(np.float32).reshape(h, stride)
    ref = orc.huffman_kv_decompress_chunk(*want[:3], t, h, d).reshape(h, t * d)
    assert (got[:, :t * d].view(np.uint32) == ref.view(np.uint32)).all() and (got[:, t * d:] == 7.0).all()
    with pytest.raises(_ffi.PeregrineError):
        _ffi.check(_ffi.lib.pg_huffman_kv_decompress_chunk_dev(ctx.handle, chunk._h, dst.ptr, t * d - 1))


def test_reference_cache_tests(ctx, orc):
    from peregrine_amd import huffman
    # src/huffman.rs:850-876
    c = huffman.HuffmanKVCache(2, 4, 8, 4, ctx)
    c.append(np.full(32, 1.0, np.float32), np.full(32, 2.0, np.float32), 4)
    assert (c.len(), c.compressed_len) == (4, 0)
    c.append(np.full(32, 3.0, np.float32), np.full(32, 4.0, np.float32), 4)
    assert (c.len(), c.compressed_len) == (8, 4)
    k, v = c.get_kv()
    assert k.size == v.size == 2 * 8 * 4
    assert (k.reshape(2, 8, 4)[:, :4] == 1.0).all() and (k.reshape(2, 8, 4)[:, 4:] == 3.0).all()
    assert (v.reshape(2, 8, 4)[:, :4] == 2.0).all() and (v.reshape(2, 8, 4)[:, 4:] == 4.0).all()
    # tests/huffman_parity.rs:160-186
    c = huffman.HuffmanKVCache(2, 8, 16, 8, ctx)
    o = orc.HuffmanKVCache(2, 8, 16, 8)
    for batch in range(4):
        k, v = parity_random_data(2 * 8 * 8, 100 + batch), parity_random_data(2 * 8 * 8, 200 + batch)
        c.append(k, v, 8)
        o.append(k, v, 8)
    assert c.len() == 32 and c.compressed_len > 0 and c.compressed_len == o.compressed_len
    for got, want in zip(c.get_kv(), o.get_kv()):
        assert got.size == 2 * 32 * 8 and (got.view(np.uint32) == want.view(np.uint32)).all()
    assert huffman.HuffmanKVCache(1, 1, 3, 10, ctx).compress_threshold == 10             # src/huffman.rs:535


@pytest.mark.parametrize("heads,hd,thr,chunk,appends", [
    (2, 8, 16, 8, (8, 8, 8, 8)),
    (3, 4, 10, 4, (1, 7, 2, 30, 5, 1, 0, 3)),      # one append that cuts several chunks, an empty append
    (1, 16, 0, 5, (3, 3, 3, 20)),                  # threshold below the chunk size: raised to it
    (2, 2, 6, 6, (13,)),
    (2, 8, 64, 4, (70, 3, 3, 1)),                  # a window much longer than a chunk: it moves to the front in many slices
    (8, 128, 512, 256, (300, 1, 1, 400, 1)),       # a Llama-sized cache: 262144 symbols per chunk
    (2, 16, 8, 4, (5,) * 60),                      # 74 chunks per side: get_kv decodes 148 streams, each under its own table, in one pass
])
def test_cache_follows_the_oracle(ctx, orc, heads, hd, thr, chunk, appends):
    from peregrine_amd import huffman
    say(f"huffman kv cache heads={heads} head_dim={hd} threshold={thr} chunk={chunk} appends={appends}")
    rng = np.random.default_rng(heads * 1000 + hd)
    c, o = huffman.HuffmanKVCache(heads, hd, thr, chunk, ctx), orc.HuffmanKVCache(heads, hd, thr, chunk)
    assert c.compress_threshold == o.compress_threshold
    for n in appends:
        k = rng.standard_normal((heads, n, hd)).astype(np.float32)
        v = (rng.standard_normal((heads, n, hd)) * 3).astype(np.float32)
        c.append(k, v, n)
        o.append(k, v, n)
        assert (c.len(), c.compressed_len, c.hot_len, len(c.k_chunks)) == (o.len, o.compressed_len, o.hot_len, o.num_chunks)
        for got, want in zip(c.get_kv(), o.get_kv()):
            assert (got.view(np.uint32) == want.view(np.uint32)).all()
    for side, chunks in ((0, c.k_chunks), (1, c.v_chunks)):
        for i, ch in enumerate(chunks):
            bits, scales, codebook, tokens = o.chunk(side, i)
            assert ch.num_tokens == tokens
            _same_chunk(ch, (bits, scales, codebook))


def test_cache_on_device_pointers(ctx, orc):
    """append_dev / get_kv_dev: the caller's tensors never leave the device."""
    from peregrine_amd import huffman, _ffi
    heads, hd = 4, 64
    c, o = huffman.HuffmanKVCache(heads, hd, 48, 32, ctx), orc.HuffmanKVCache(heads, hd, 48, 32)
    rng = np.random.default_rng(21)
    for n in (40, 1, 1, 70, 1):
        k, v = rng.standard_normal((heads, n, hd)).astype(np.float32), rng.standard_normal((heads, n, hd)).astype(np.float32)
        dk, dv = DevBuf(ctx, host=k), DevBuf(ctx, host=v)
        _ffi.check(_ffi.lib.pg_huffman_kv_cache_append_dev(ctx.handle, c._h, dk.ptr, dv.ptr, n))
        o.append(k, v, n)
    assert (c.len(), c.compressed_len) == (o.len, o.compressed_len)
    n = heads * c.len() * hd
    out_k, out_v = DevBuf(ctx, nbytes=4 * n), DevBuf(ctx, nbytes=4 * n)
    _ffi.check(_ffi.lib.pg_huffman_kv_cache_get_kv_dev(ctx.handle, c._h, out_k.ptr, out_v.ptr))
    ctx.sync()
    want_k, want_v = o.get_kv()
    assert (out_k.to_host(np.float32).view(np.uint32) == want_k.view(np.uint32)).all()
    assert (out_v.to_host(np.float32).view(np.uint32) == want_v.view(np.uint32)).all()
