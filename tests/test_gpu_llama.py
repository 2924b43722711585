"""GPU parity of the Llama decoder-block glue against the CPU oracle, through the C ABI.

Bars: RMSNorm, RoPE and attention are f32 ports with a different (tree / sliced) summation
order: 1e-5 relative (H.assert_close_rel).  The KV cache is a byte copy: bit-exact.  The
whole block chains seven block-dequant products, each inside the 1e-3 contract for
Q4_0/Q8_0 paths; the block is held to that same 1e-3 against the oracle's block.
"""
import sys

import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

RTOL_F32 = 1e-5
RTOL_BLOCK = 1e-3


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("rows,dim", [(1, 4096), (5, 96), (3, 257), (64, 4096), (2, 1)])
def test_rmsnorm(ctx, orc, rows, dim):
    from peregrine_amd import llama
    say(f"rmsnorm rows={rows} dim={dim}")
    x = orc.rng_normal(rows * 7 + dim, rows * dim)
    x[:dim] *= 50.0                                   # one loud row
    norm = llama.RMSNorm(dim, 1e-5, ctx)
    norm.weight = (1 + 0.1 * orc.rng_normal(3, dim)).astype(np.float32)
    got = norm.forward(x.reshape(rows, dim))
    H.assert_close_rel(got, orc.rmsnorm(x, rows, dim, norm.weight, 1e-5), RTOL_F32, "rmsnorm")
    assert norm.forward(np.zeros((0, dim), np.float32)).shape == (0, dim)
    with pytest.raises(ValueError):
        norm.forward(np.zeros((2, dim + 1), np.float32))


def test_rmsnorm_closed_form(ctx):
    from peregrine_amd import llama
    norm = llama.RMSNorm(64, 0.0, ctx)
    norm.weight = np.arange(64, dtype=np.float32) / 8
    got = norm.forward(np.full((1, 64), -3.0, np.float32))          # x / rms(x) = -1 for a constant row
    assert np.allclose(got[0], -norm.weight, rtol=0, atol=1e-6 * 8)
    assert (llama.RMSNorm(64, 1e-5, ctx).forward(np.zeros((1, 64), np.float32)) == 0).all()


@pytest.mark.parametrize("hd,seq,offset", [(8, 5, 3), (128, 7, 0), (64, 1, 100), (2, 4, 1), (24, 9, 2), (12, 3, 0), (256, 100, 17)])
def test_rope(ctx, orc, hd, seq, offset):
    from peregrine_amd import llama, _ffi
    say(f"rope hd={hd} seq={seq} offset={offset}")
    n = 128
    rope = llama.RoPE(hd, n, 10000.0, ctx)
    cos, sin = orc.rope_tables(hd, n, 10000.0)
    x = orc.rng_normal(hd + seq, seq * hd).reshape(seq, hd)
    got = rope.apply(x, offset)
    want = orc.rope_apply(x, seq, hd, offset, cos, sin).reshape(seq, hd)
    # same f32 expression per element; only libm's cos/sin/pow may differ in the last bit
    H.assert_close_rel(got, want, 1e-6, "rope")
    assert (rope.apply(x[:1], 0) == x[:1]).all()                    # position 0 is the identity
    with pytest.raises(_ffi.PeregrineError):
        rope.apply(x, n - seq + 1)                                    # past max_seq_len: the reference's slice panic
    with pytest.raises(_ffi.PeregrineError):
        llama.RoPE(7, 16, 10000.0, ctx)


def test_kv_cache_append_growth_rollback(ctx, orc):
    """StandardKVCache semantics (src/attention.rs:18-98): growth keeps old rows, capacity at
    least doubles from 16, rollback truncates logically, appends after rollback overwrite."""
    from peregrine_amd import llama, _ffi
    nkv, hd = 3, 8
    cache = llama.StandardKVCache(nkv, hd, ctx)
    assert cache.len == 0 and cache.head_stride() == 0
    mirror_k = np.zeros((nkv, 0, hd), np.float32)
    mirror_v = np.zeros((nkv, 0, hd), np.float32)
    caps = []
    for step, seq in enumerate((1, 5, 30, 1, 40)):
        k = orc.rng_normal(10 + step, nkv * seq * hd).reshape(nkv, seq, hd)
        v = orc.rng_normal(20 + step, nkv * seq * hd).reshape(nkv, seq, hd)
        cache.append(k, v, seq)
        mirror_k = np.concatenate([mirror_k, k], 1)
        mirror_v = np.concatenate([mirror_v, v], 1)
        gk, gv = cache.to_host()
        assert cache.len == mirror_k.shape[1]
        assert (gk == mirror_k).all() and (gv == mirror_v).all()
        caps.append(cache.head_stride() // hd)
    assert caps == [32, 32, 64, 64, 128]            # needed.max(capacity.max(16) * 2)
    cache.rollback_to(10)
    assert cache.len == 10 and cache.head_stride() == 128 * hd
    with pytest.raises(_ffi.PeregrineError):
        cache.rollback_to(11)
    k = orc.rng_normal(31, nkv * 2 * hd).reshape(nkv, 2, hd)
    cache.append(k, k, 2)
    gk, gv = cache.to_host()
    assert (gk[:, :10] == mirror_k[:, :10]).all() and (gk[:, 10:] == k).all() and (gv[:, 10:] == k).all()
    with pytest.raises(ValueError):
        cache.append(k, k, 3)


def _attention_case(ctx, orc, nqh, nkvh, hd, seq_q, length, mask, logit_cap, seed, appends=None):
    from peregrine_amd import llama
    cache = llama.StandardKVCache(nkvh, hd, ctx)
    k = orc.rng_normal(seed, nkvh * length * hd).reshape(nkvh, length, hd)
    v = orc.rng_normal(seed + 1, nkvh * length * hd).reshape(nkvh, length, hd)
    pos = 0
    for n in appends or (length,):                   # several appends: capacity > len, strides matter
        cache.append(k[:, pos:pos + n], v[:, pos:pos + n], n)
        pos += n
    assert pos == length
    q = orc.rng_normal(seed + 2, nqh * seq_q * hd).reshape(nqh, seq_q, hd)
    scale = 1 / np.sqrt(hd)
    base = orc.rng_normal(seed + 3, seq_q * nqh * hd)            # the output is added to, not overwritten
    got = base.copy()
    llama.gqa_attention(q, cache, cache, nqh, nkvh, seq_q, hd, scale, mask, logit_cap, got, ctx)
    if mask.kind == 3:
        want = orc.gqa_attention_local_global(q, k, v, length, length, nqh, nkvh, seq_q, hd, scale, mask.offset, mask.window,
                                              mask.global_positions, logit_cap or 0.0)
    else:
        want = orc.gqa_attention(q, k, v, length, length, nqh, nkvh, seq_q, hd, scale, mask.kind, mask.offset, mask.window,
                                 mask.sink_tokens, logit_cap or 0.0)
    H.assert_close_rel(got - base, want, RTOL_F32 * 4, "gqa_attention")   # (base + o) - base rounds once more
    return got


@pytest.mark.parametrize("nqh,nkvh,hd,seq_q,length", [
    (2, 2, 4, 2, 3),          # tests/attention.rs MHA shape
    (4, 2, 4, 2, 3),          # GQA ratio 2
    (4, 1, 4, 2, 3),          # MQA
    (32, 8, 128, 1, 1000),    # Llama-3-8B decode step
    (8, 2, 64, 5, 77),
    (6, 3, 20, 3, 40),        # head_dim not a power of two
    (2, 1, 6, 2, 9),          # head_dim not a multiple of 4: the scalar path
    (2, 2, 256, 1, 300),
])
def test_gqa_attention_unmasked(ctx, orc, nqh, nkvh, hd, seq_q, length):
    from peregrine_amd import llama
    say(f"attention nqh={nqh} nkvh={nkvh} hd={hd} seq_q={seq_q} len={length}")
    _attention_case(ctx, orc, nqh, nkvh, hd, seq_q, length, llama.AttentionMask.none(), None, 100 + hd,
                    appends=(1, length - 1) if length > 1 else None)


def test_gqa_attention_masks_and_logit_cap(ctx, orc):
    from peregrine_amd import llama
    M = llama.AttentionMask
    for mask, cap in ((M.causal(0), None), (M.causal(20), None), (M.causal_sliding_window(27, 5, 2), None),
                      (M.causal_sliding_window(27, 0, 0), None), (M.none(), 1.5), (M.causal(27), 30.0)):
        say(f"attention mask={mask} cap={cap}")
        _attention_case(ctx, orc, 8, 2, 32, 4, 31, mask, cap, 7)
    # causal, offset 0, first query row sees only position 0: the output row is v[0] exactly
    cache = llama.StandardKVCache(1, 8, ctx)
    k = orc.rng_normal(1, 5 * 8).reshape(1, 5, 8)
    v = orc.rng_normal(2, 5 * 8).reshape(1, 5, 8)
    cache.append(k, v, 5)
    out = np.zeros(2 * 8, np.float32)
    llama.gqa_attention(orc.rng_normal(3, 2 * 8), cache, cache, 1, 1, 2, 8, 0.35, M.causal(0), None, out, ctx)
    assert (out[:8] == v[0, 0]).all()


def test_gqa_attention_many_rows(ctx, orc):
    """Enough (token, head) rows to fill the chip without key splits: the long-chunk kernel, with
    and without the causal cut of the key range."""
    from peregrine_amd import llama
    say("attention 8 heads x 70 tokens")
    _attention_case(ctx, orc, 8, 2, 64, 70, 90, llama.AttentionMask.none(), None, 61)
    _attention_case(ctx, orc, 8, 2, 64, 70, 90, llama.AttentionMask.causal(20), None, 62)
    _attention_case(ctx, orc, 8, 4, 32, 70, 90, llama.AttentionMask.causal_sliding_window(20, 7, 3), 2.0, 63)
    # head sizes of the tiled kernel (64, 128, 256), key counts that are not multiples of its 64-key blocks,
    # row counts that are not multiples of its 32-row workgroups, several appends (capacity > length)
    say("attention, tiled kernel shapes")
    _attention_case(ctx, orc, 8, 2, 128, 67, 150, llama.AttentionMask.causal(83), None, 64, appends=(100, 50))
    _attention_case(ctx, orc, 8, 2, 128, 67, 150, llama.AttentionMask.none(), 3.0, 65)
    _attention_case(ctx, orc, 4, 4, 256, 131, 131, llama.AttentionMask.causal(0), None, 66)
    _attention_case(ctx, orc, 16, 2, 64, 33, 200, llama.AttentionMask.causal_sliding_window(167, 40, 4), None, 67)


def test_gqa_attention_matrix_core_kernel_pairs_and_masks(ctx, orc):
    """Head sizes 64 and 128 with many rows run on the matrix cores: 32-row items, paired first with last, the
    long item of a pair cut between two wavefronts and joined through LDS.  Shapes with an odd and an even
    number of items, a last item that is not full, every mask kind (tiles that are wholly hidden included),
    a logit cap, and a cache longer than the rows can see."""
    from peregrine_amd import llama
    M = llama.AttentionMask
    say("attention, matrix-core kernel")
    _attention_case(ctx, orc, 8, 2, 128, 150, 150, M.causal(0), None, 81)                       # 19 items: 9 pairs + the middle one
    _attention_case(ctx, orc, 8, 2, 64, 128, 200, M.causal(72), None, 82, appends=(72, 128))    # 16 items, all full
    _attention_case(ctx, orc, 16, 4, 64, 90, 230, M.causal_sliding_window(140, 24, 3), None, 83)  # early tiles wholly hidden
    _attention_case(ctx, orc, 16, 4, 64, 90, 230, M.causal_sliding_window(140, 0, 0), 5.0, 84)
    _attention_case(ctx, orc, 8, 2, 128, 97, 160, M.local_global(63, 9, [0, 5, 31, 32, 64, 65, 159, 1000]), None, 85)
    _attention_case(ctx, orc, 8, 8, 128, 80, 100, M.none(), 2.5, 86)                            # MHA: one head per kv head
    _attention_case(ctx, orc, 12, 2, 64, 75, 75, M.causal(0), None, 87)                         # group of 6: items straddle tokens


def test_gqa_attention_prefill_at_llama_8b_size(ctx, orc):
    """The benchmark's prefill attention at full size (32 query heads over 8 kv heads of 128, 1024 tokens into
    an empty cache, causal): 64 pairs of 32-row items per kv head, up to 32 key tiles per item."""
    from peregrine_amd import llama
    say("attention 32/8 heads x 128, 1024 tokens, causal")
    _attention_case(ctx, orc, 32, 8, 128, 1024, 1024, llama.AttentionMask.causal(0), None, 91)


def test_gqa_attention_local_global(ctx, orc):
    """AttentionMask::LocalGlobal through each of the three kernels (few rows with key splits, the
    generic one, the tiled one), global positions in no order, repeated and past the cache."""
    from peregrine_amd import llama
    M = llama.AttentionMask
    say("attention, local + global mask")
    _attention_case(ctx, orc, 8, 2, 32, 4, 31, M.local_global(27, 3, [0, 9, 9, 17, 400]), None, 71)
    _attention_case(ctx, orc, 8, 2, 32, 4, 31, M.local_global(27, 0, []), 2.0, 72)
    _attention_case(ctx, orc, 32, 8, 128, 1, 1000, M.local_global(999, 64, [0, 1, 2, 500, 731]), None, 73)
    _attention_case(ctx, orc, 6, 3, 20, 90, 120, M.local_global(30, 5, [119, 64, 3]), None, 74)
    _attention_case(ctx, orc, 8, 2, 128, 67, 150, M.local_global(83, 10, [149, 0, 31, 32, 33, 95]), None, 75, appends=(100, 50))
    _attention_case(ctx, orc, 16, 2, 64, 33, 200, M.local_global(167, 1, list(range(0, 200, 7))), 3.0, 76)
    # every position global = the causal mask, bit for bit (same kernels, same order of operations)
    got = _attention_case(ctx, orc, 8, 2, 64, 40, 90, M.local_global(50, 0, range(90)), None, 77)
    assert (got == _attention_case(ctx, orc, 8, 2, 64, 40, 90, M.causal(50), None, 77)).all()


def test_gqa_attention_one_token_heads_of_a_group_together(ctx, orc):
    """One query token with head size 64 or 128: a workgroup serves all query heads of a kv group (in passes of
    four) over one split of the keys, and the last workgroup of a kv head to finish merges the splits.  Lengths
    around the tile sizes (16 / 32 keys a round, up to four rounds a tile), one tile and several per split,
    groups of 1, 2, 4, 5 and 8 heads, every mask kind, a cache longer than the token may see, a logit cap, and
    the same call twice in a row (the arrival counters must be back at zero)."""
    from peregrine_amd import llama
    M = llama.AttentionMask
    seed = 300
    for hd in (128, 64):
        for length in (1, 15, 16, 17, 63, 64, 65, 300):
            say(f"one-token attention hd={hd} len={length}")
            _attention_case(ctx, orc, 8, 2, hd, 1, length, M.none(), None, seed)
            _attention_case(ctx, orc, 8, 2, hd, 1, length, M.causal(length - 1), None, seed + 1,
                            appends=(1, length - 1) if length > 1 else None)
            seed += 2
    for nqh, nkvh in ((4, 4), (4, 2), (10, 2), (16, 2), (5, 1)):
        say(f"one-token attention heads {nqh}/{nkvh}")
        _attention_case(ctx, orc, nqh, nkvh, 128, 1, 200, M.causal(199), None, seed)
        _attention_case(ctx, orc, nqh, nkvh, 64, 1, 333, M.causal(332), 4.0, seed + 1)
        seed += 2
    say("one-token attention, masks")
    _attention_case(ctx, orc, 8, 2, 128, 1, 500, M.causal(250), None, seed)                       # half of the cache is ahead
    _attention_case(ctx, orc, 8, 2, 128, 1, 500, M.causal_sliding_window(499, 100, 4), None, seed + 1)  # whole tiles hidden
    _attention_case(ctx, orc, 8, 2, 64, 1, 500, M.causal_sliding_window(450, 0, 0), None, seed + 2)      # sees itself only
    _attention_case(ctx, orc, 8, 2, 64, 1, 700, M.local_global(699, 37, [0, 5, 64, 65, 300, 698, 5000]), 2.0, seed + 3)
    _attention_case(ctx, orc, 32, 8, 128, 1, 1025, M.causal(1024), None, seed + 4)              # the benchmark's step
    say("one-token attention, several tiles per split")
    _attention_case(ctx, orc, 32, 8, 128, 1, 5000, M.causal(4999), None, seed + 5, appends=(4096, 904))
    _attention_case(ctx, orc, 64, 16, 64, 1, 6001, M.none(), None, seed + 6)
    a = _attention_case(ctx, orc, 8, 1, 128, 1, 9000, M.causal(8999), None, seed + 7)
    assert (a == _attention_case(ctx, orc, 8, 1, 128, 1, 9000, M.causal(8999), None, seed + 7)).all()


def test_gqa_attention_few_rows_under_a_long_cache(ctx, orc):
    """Several query tokens, but too few rows to fill the chip, over a long cache (a chunk of a prefill, draft
    tokens being verified): the matrix-core kernel runs over runs of key tiles and the runs are merged.  Rows
    that fill less than one 32-row item, an odd number of items (a wavefront without work), runs that some rows
    cannot see at all (causal, the chunk at the end of the cache or in its middle), every mask kind, a logit cap."""
    from peregrine_amd import llama
    M = llama.AttentionMask
    say("attention, few rows under a long cache")
    _attention_case(ctx, orc, 32, 8, 128, 2, 1026, M.causal(1024), None, 401)
    _attention_case(ctx, orc, 32, 8, 128, 8, 1032, M.causal(1024), None, 402, appends=(1024, 8))
    _attention_case(ctx, orc, 32, 8, 128, 16, 1040, M.causal(1024), None, 403)
    _attention_case(ctx, orc, 32, 8, 128, 32, 2080, M.none(), None, 404)
    _attention_case(ctx, orc, 6, 2, 64, 30, 700, M.causal(670), 3.0, 405)                        # 90 rows: three items
    _attention_case(ctx, orc, 6, 2, 64, 30, 700, M.causal(200), None, 406)                       # most of the cache is ahead
    _attention_case(ctx, orc, 8, 2, 64, 5, 900, M.causal_sliding_window(895, 100, 4), None, 407)  # whole runs hidden
    _attention_case(ctx, orc, 8, 2, 128, 12, 600, M.local_global(588, 40, [0, 7, 64, 300, 301, 599, 9999]), None, 408)
    _attention_case(ctx, orc, 4, 4, 128, 3, 5000, M.causal(4997), None, 409)                     # one head per kv head
    say("attention, a chunk of a prefill appended to a long cache")
    _attention_case(ctx, orc, 32, 8, 128, 136, 2100, M.causal(1964), None, 411)                  # 17 items per kv head, 66 key tiles
    _attention_case(ctx, orc, 16, 8, 64, 300, 2300, M.causal_sliding_window(2000, 700, 8), None, 412)
    a = _attention_case(ctx, orc, 16, 2, 128, 9, 3000, M.causal(2991), None, 410)
    assert (a == _attention_case(ctx, orc, 16, 2, 128, 9, 3000, M.causal(2991), None, 410)).all()


def test_gqa_attention_long_cache_splits_keys(ctx, orc):
    """A long cache under one query row: the keys are cut into many splits and merged.  Head size 16 takes the
    general kernels; head size 128 at 140 000 keys the one-token kernel with 35 tiles per split (a length at
    which 64-key splits would exceed the merge's limit of 2048)."""
    from peregrine_amd import llama
    say("attention len=40000")
    _attention_case(ctx, orc, 2, 1, 16, 1, 40000, llama.AttentionMask.causal(39999), None, 55)
    say("attention len=140000")
    _attention_case(ctx, orc, 4, 1, 128, 1, 140000, llama.AttentionMask.causal(139999), None, 56)


def test_gqa_attention_edges(ctx, orc):
    from peregrine_amd import llama, _ffi
    cache = llama.StandardKVCache(2, 8, ctx)
    out = np.full(2 * 4 * 8, 3.0, np.float32)
    llama.gqa_attention(np.ones(4 * 2 * 8, np.float32), cache, cache, 4, 2, 2, 8, 1.0, llama.AttentionMask.none(), None, out, ctx)
    assert (out == 3.0).all()                         # empty cache: nothing is added
    with pytest.raises(_ffi.PeregrineError):
        llama.gqa_attention(np.ones(3 * 8, np.float32), cache, cache, 3, 2, 1, 8, 1.0, llama.AttentionMask.none(), None,
                            np.zeros(3 * 8, np.float32), ctx)    # 3 query heads over 2 kv heads
    with pytest.raises(ValueError):
        llama.gqa_attention(np.ones(5, np.float32), cache, cache, 4, 2, 2, 8, 1.0, llama.AttentionMask.none(), None, out, ctx)


def _block_case(ctx, orc, d, nqh, nkvh, hd, ffn, typ, steps, max_seq=64, seed=0, raws=None):
    from peregrine_amd import gguf, llama
    shapes = [(nqh * hd, d), (nkvh * hd, d), (nkvh * hd, d), (d, nqh * hd), (ffn, d), (ffn, d), (d, ffn)]
    types = [typ] * 7 if np.isscalar(typ) else list(typ)
    if raws is None:
        raws = [bytes({2: H.pack_q4_0, 3: H.pack_q4_1, 8: H.pack_q8_0}[t](orc.rng_normal(seed + 40 + i, n * k, 0.0, 1.0 / np.sqrt(k))))
                for i, ((n, k), t) in enumerate(zip(shapes, types))]
    ws = [gguf.GgufWeight(r, t, n, k, ctx) for r, (n, k), t in zip(raws, shapes, types)]
    wa = (1 + 0.1 * orc.rng_normal(seed + 1, d)).astype(np.float32)
    wf = (1 + 0.1 * orc.rng_normal(seed + 2, d)).astype(np.float32)
    eps = 1e-5
    blk = llama.LlamaBlock(d, nqh, nkvh, hd, ffn, max_seq, 10000.0, eps, ctx)
    blk.set_weights(*ws, wa, wf)
    cache = blk.new_cache()
    cos, sin = orc.rope_tables(hd, max_seq, 10000.0)
    kc = np.zeros((nkvh, max_seq, hd), np.float32)
    vc = np.zeros((nkvh, max_seq, hd), np.float32)
    pos = 0
    for i, seq in enumerate(steps):
        say(f"llama block d={d} heads={nqh}/{nkvh} hd={hd} ffn={ffn} type={typ} step {i}: seq={seq} at {pos}")
        h = orc.rng_normal(seed + 90 + i, seq * d).reshape(seq, d)
        got = blk.forward(h, cache)
        want = orc.llama_block_forward(h, seq, d, nqh, nkvh, hd, ffn, typ, raws, wa, wf, eps, cos, sin, kc, vc, pos, max_seq)
        pos += seq
        assert cache.len == pos
        H.assert_close_rel(got, want, RTOL_BLOCK, f"llama block step {i}")
        gk, gv = cache.to_host()
        H.assert_close_rel(gk, kc[:, :pos], RTOL_BLOCK, "k cache")
        H.assert_close_rel(gv, vc[:, :pos], RTOL_BLOCK, "v cache")
    return blk, cache


@pytest.mark.parametrize("typ", [8, 2])
def test_llama_block_prefill_then_decode(ctx, orc, typ):
    """Prefill (matrix-core products), two decode steps (streaming GEMV), another prefill chunk."""
    _block_case(ctx, orc, 256, 8, 2, 32, 512, typ, (5, 1, 1, 33))


def test_llama_block_mixed_block_types(ctx, orc):
    """Q4_0 and Q8_0 projections in one block: their activation digits differ in kind, so the
    one-token step cannot share them and takes the product-by-product route."""
    _block_case(ctx, orc, 128, 4, 2, 32, 256, (8, 2, 8, 2, 2, 8, 8), (3, 1, 1), seed=3)


def test_llama_block_long_prefill_head_128(ctx, orc):
    """A prefill long enough for the tiled attention kernel and the many-token-tile product
    order (140 tokens x 4 heads of 128), then a decode step on top of it."""
    _block_case(ctx, orc, 512, 4, 2, 128, 768, 2, (140, 1), max_seq=160, seed=21)


@pytest.mark.parametrize("typ", [2, 8])
def test_llama_block_decode_steps_head_64_group_of_3(ctx, orc, typ):
    """Several one-token steps in a row with the grouped one-token attention (head size 64, three query heads per
    kv head) and, for Q4_0, the products that leave their output as the next product's digits."""
    _block_case(ctx, orc, 384, 6, 2, 64, 640, typ, (7, 1, 1, 1, 20, 1), seed=31)


@pytest.mark.parametrize("typ", [2, 8])
def test_llama_block_decode_long_ffn_rows(ctx, orc, typ):
    """A down projection with few output rows under a long input row (ffn 8192): its one-token product shares
    one copy of the input digits per workgroup through LDS."""
    _block_case(ctx, orc, 256, 8, 2, 32, 8192, typ, (3, 1, 1), seed=37)


@pytest.mark.parametrize("typ", [2, 8])
def test_llama_block_decode_wide_rows(ctx, orc, typ):
    """One-token steps whose folded products meet long rows: a model dim of 6144 under the norm-folding q|k|v
    product and the gate|up pair (three 64-block groups per lane), and 48 heads of 128 under the o-projection
    that leaves its output as digits."""
    _block_case(ctx, orc, 6144, 8, 2, 64, 256, typ, (2, 1, 1), seed=41)
    _block_case(ctx, orc, 256, 48, 8, 128, 320, typ, (2, 1, 1), seed=43)


def test_llama_block_one_token_steps_at_llama_8b_size(ctx, orc):
    """The benchmark's block at full size (d 4096, 32 / 8 heads of 128, ffn 14336, Q4_0): a three-token prefill and
    two one-token steps against the oracle.  The tensors are written as Q4_0 blocks directly (random nibbles, block
    scales drawn from eight f16 values around 1 / (4 sqrt(K))): packing 218 M normal weights would take minutes."""
    d, nqh, nkvh, hd, ffn = 4096, 32, 8, 128, 14336
    rng = np.random.default_rng(2024)
    raws = []
    for n, k in [(nqh * hd, d), (nkvh * hd, d), (nkvh * hd, d), (d, nqh * hd), (ffn, d), (ffn, d), (d, ffn)]:
        nb = n * k // 32
        raw = np.empty((nb, 18), np.uint8)
        raw[:, 2:] = rng.integers(0, 256, size=(nb, 16), dtype=np.uint8)
        scales = (np.float16(0.25 / np.sqrt(k)) * np.arange(5, 13, dtype=np.float16) / np.float16(8)).astype(np.float16)
        raw[:, :2] = scales.view(np.uint8).reshape(8, 2)[rng.integers(0, 8, size=nb)]
        raws.append(raw.tobytes())
    _block_case(ctx, orc, d, nqh, nkvh, hd, ffn, 2, (3, 1, 1), max_seq=16, seed=51, raws=raws)


@pytest.mark.parametrize("typ", [2, 8])
@pytest.mark.parametrize("heads", [(16, 4, 64), (8, 2, 128)])
def test_llama_block_few_token_steps_through_the_few_row_products(ctx, orc, typ, heads):
    """Steps of 2 to 16 tokens at a model dim where the chained step takes the few-row products (K >= 1024, a
    multiple of 256): 6 and 8 tokens on the eight-row rings with the residual added by the down product, 12 and 16
    on the sixteen-row rings (every tensor group here has fewer than 32 weight rows per CU), a prefill before and a
    one-token step after."""
    nqh, nkvh, hd = heads
    _block_case(ctx, orc, 1024, nqh, nkvh, hd, 2048, typ, (33, 6, 8, 12, 16, 1, 2, 5), max_seq=96, seed=61)


@pytest.mark.parametrize("typ", [2, 8])
def test_llama_block_nine_to_sixteen_tokens_mixed_products(ctx, orc, typ):
    """Nine to sixteen tokens with gate|up too wide for the few-row product (2 x 4096 rows = 32 per CU and more) while
    q|k|v, o and down take it: the planes of the block product and of the few-row products meet in one step; then
    a step of five tokens, where every product is a few-row one."""
    _block_case(ctx, orc, 1024, 8, 2, 128, 4096, typ, (20, 9, 16, 13, 5, 1), max_seq=80, seed=67)


@pytest.mark.parametrize("typ", [2, 8])
@pytest.mark.parametrize("shape", [(1024, 8, 2, 128, 2048, (40, 130, 9, 1)), (512, 8, 4, 64, 1280, (33, 17)),
                                   (5120, 5, 1, 128, 1024, (20,))])
def test_llama_block_many_token_steps_on_the_f16_matrix_cores(ctx, orc, shape, typ):
    """The many-token step with its four product launches forced onto the f16 route (at these sizes the dispatcher
    would keep the int8 block product): RMSNorm and SiLU.up write their rows as f16 planes, the attention output is
    converted, q|k|v and gate|up share a launch each, K chunks are left to the consumers to add up.  Steps of up to
    eight tokens (and up to sixteen on narrow tensors) still take the few-row products; a model dim above 4096 takes
    the RMSNorm kernel's longer-row instance."""
    from peregrine_amd import _ffi
    d, nqh, nkvh, hd, ffn, steps = shape
    _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 1))
    try:
        ctx.profile_begin()
        _block_case(ctx, orc, d, nqh, nkvh, hd, ffn, typ, steps, max_seq=192, seed=71)
        prof = ctx.profile_end()
    finally:
        _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 0))
    for name in ("gguf_hmm_q4_0" if typ == 2 else "gguf_hmm_q8_0", "add_rmsnorm_f16_planes", "swiglu_f16_planes", "rows_to_f16_planes"):
        assert name in prof, (name, sorted(prof))


def test_llama_block_q4_1_weights(ctx, orc):
    """Offset blocks (Q4_1): the streaming kernel, one item per row, up to seven rows; more rows take the Q4_0
    matrix-core product on the same nibbles plus a launch that adds the offsets times the rows' block sums."""
    _block_case(ctx, orc, 128, 4, 2, 32, 256, 3, (3, 1), seed=13)
    _block_case(ctx, orc, 256, 4, 2, 32, 512, 3, (40, 1, 9), seed=14)   # from eight rows: the matrix-core product plus the offsets' launch


def test_llama_block_mha_and_odd_shapes(ctx, orc):
    _block_case(ctx, orc, 96, 3, 3, 32, 160, 8, (1, 2, 1), seed=5)


def test_llama_block_rollback_and_errors(ctx, orc):
    from peregrine_amd import _ffi, llama
    blk, cache = _block_case(ctx, orc, 128, 4, 2, 32, 256, 8, (4,), max_seq=8, seed=9)
    h = orc.rng_normal(1, 2 * 128).reshape(2, 128)
    a = blk.forward(h, cache)
    cache.rollback_to(4)                               # speculative decoding: reject, replay
    b = blk.forward(h, cache)
    assert (a == b).all() and cache.len == 6
    with pytest.raises(_ffi.PeregrineError):
        blk.forward(orc.rng_normal(2, 3 * 128).reshape(3, 128), cache)   # 6 + 3 > max_seq_len 8
    assert cache.len == 6
    with pytest.raises(_ffi.PeregrineError):
        blk.forward(h[:1], llama.StandardKVCache(3, 32, ctx))            # cache of another shape
    with pytest.raises(_ffi.PeregrineError):
        llama.LlamaBlock(128, 4, 2, 32, 256, 8, 10000.0, 1e-5, ctx).forward(h[:1], blk.new_cache())   # weights not set
    with pytest.raises(_ffi.PeregrineError):
        llama.LlamaBlock(128, 4, 3, 32, 256, 8, 10000.0, 1e-5, ctx)      # 4 query heads over 3 kv heads
    assert blk.forward(np.zeros((0, 128), np.float32), cache).shape == (0, 128)
