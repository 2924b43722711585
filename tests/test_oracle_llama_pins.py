"""Pins for the Llama-glue half of the CPU oracle (oracle/peregrine_oracle_llama.c): closed
forms, invariants, NumPy float64 recomputation, and the reference's own attention tests
restated (tests/attention.rs)."""
import numpy as np

import helpers as H


def test_rmsnorm_closed_forms_and_float64(orc):
    dim = 64
    x = np.full(dim, 3.0, np.float32)
    w = np.arange(dim, dtype=np.float32) / 8
    out = orc.rmsnorm(x, 1, dim, w, 0.0)           # x / sqrt(mean x^2) = sign(x) for a constant row
    assert np.allclose(out, w, rtol=0, atol=1e-6 * w.max())
    out = orc.rmsnorm(np.zeros(dim, np.float32), 1, dim, w, 1e-5)
    assert (out == 0).all()                          # eps keeps the zero row finite
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, dim)).astype(np.float32)
    ref = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-5) * w
    got = orc.rmsnorm(x, 5, dim, w, 1e-5).reshape(5, dim)
    assert np.abs(got - ref).max() <= 2e-6 * np.abs(ref).max()
    # a dropped eps or a mean/sum mix-up would show here
    tiny = np.full(dim, 1e-4, np.float32)
    assert np.allclose(orc.rmsnorm(tiny, 1, dim, np.ones(dim, np.float32), 1e-5), 1e-4 / np.sqrt(1e-8 + 1e-5), rtol=1e-6)


def test_rope_tables_and_rotation(orc):
    hd, n, base = 8, 33, 10000.0
    cos, sin = orc.rope_tables(hd, n, base)
    assert (cos[0] == 1).all() and (sin[0] == 0).all()                    # position 0 is the identity
    assert (cos[:, :4] == cos[:, 4:]).all() and (sin[:, :4] == sin[:, 4:]).all()
    i = np.arange(4)
    theta = 7 / base ** (2 * i / hd)
    assert np.allclose(cos[7, :4], np.cos(theta), atol=1e-6) and np.allclose(sin[7, :4], np.sin(theta), atol=1e-6)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, hd)).astype(np.float32)
    y = orc.rope_apply(x, 5, hd, 3, cos, sin).reshape(5, hd)
    # pairs (i, i + hd/2) rotate by theta: norms are preserved, position 0 leaves x unchanged
    assert np.allclose((y ** 2).sum(1), (x ** 2).sum(1), rtol=1e-5)
    assert (orc.rope_apply(x[:1], 1, hd, 0, cos, sin) == x[0]).all()
    for t in range(5):
        th = (3 + t) / base ** (2 * i / hd)
        assert np.allclose(y[t, :4], x[t, :4] * np.cos(th) - x[t, 4:] * np.sin(th), atol=2e-6)
        assert np.allclose(y[t, 4:], x[t, :4] * np.sin(th) + x[t, 4:] * np.cos(th), atol=2e-6)


def naive_attention(q, k, v, seq_q, seq_kv, hd, scale, causal, offset):
    """tests/attention.rs:5-56 in float64."""
    out = np.zeros((seq_q, hd))
    for qt in range(seq_q):
        s = (k[:seq_kv] @ q[qt]) * scale
        if causal:
            s[np.arange(seq_kv) > offset + qt] = -np.inf
        p = np.exp(s - s.max())
        out[qt] = (p / p.sum()) @ v[:seq_kv]
    return out


def _qkv(nqh, nkvh, seq_q, seq_kv, hd, cap):
    q = np.sin(np.arange(nqh * seq_q * hd) * 0.1).astype(np.float32).reshape(nqh, seq_q, hd)   # tests/attention.rs:137-147
    k = np.zeros((nkvh, cap, hd), np.float32)
    v = np.zeros((nkvh, cap, hd), np.float32)
    k[:, :seq_kv] = np.cos(np.arange(nkvh * seq_kv * hd) * 0.2).astype(np.float32).reshape(nkvh, seq_kv, hd)
    v[:, :seq_kv] = np.sin(np.arange(nkvh * seq_kv * hd) * 0.15).astype(np.float32).reshape(nkvh, seq_kv, hd)
    return q, k, v


def test_gqa_matches_naive_attention_with_grouping_mqa_and_capacity(orc):
    """tests/attention.rs:59-262: MHA, GQA (ratio 2) and MQA against the per-head naive form,
    with a cache whose capacity exceeds its length (head stride = capacity * head_dim)."""
    hd, seq_q, seq_kv, cap = 4, 2, 3, 16
    scale = 1 / np.sqrt(hd)
    for nqh, nkvh in ((2, 2), (4, 2), (4, 1)):
        q, k, v = _qkv(nqh, nkvh, seq_q, seq_kv, hd, cap)
        out = orc.gqa_attention(q, k, v, seq_kv, cap, nqh, nkvh, seq_q, hd, scale).reshape(seq_q, nqh, hd)
        for qh in range(nqh):
            want = naive_attention(q[qh].astype(np.float64), k[qh // (nqh // nkvh)].astype(np.float64),
                                   v[qh // (nqh // nkvh)].astype(np.float64), seq_q, seq_kv, hd, scale, False, 0)
            assert np.abs(out[:, qh] - want).max() < 1e-5


def test_causal_masks_and_window_and_cap(orc):
    """tests/attention.rs:265-510: causal, causal with offset, sliding window with sinks, logit cap."""
    hd, nqh, nkvh, cap = 4, 2, 1, 8
    scale = 0.5
    q, k, v = _qkv(nqh, nkvh, 3, 5, hd, cap)
    for offset in (0, 2):
        out = orc.gqa_attention(q, k, v, 5, cap, nqh, nkvh, 3, hd, scale, mask_kind=1, offset=offset).reshape(3, nqh, hd)
        for qh in range(nqh):
            want = naive_attention(q[qh].astype(np.float64), k[0].astype(np.float64), v[0].astype(np.float64), 3, 5, hd, scale, True, offset)
            assert np.abs(out[:, qh] - want).max() < 1e-5
    # the first query row with offset 0 sees only position 0: its output is v[0] exactly
    out = orc.gqa_attention(q, k, v, 5, cap, nqh, nkvh, 3, hd, scale, mask_kind=1, offset=0).reshape(3, nqh, hd)
    assert (out[0, 0] == v[0, 0]).all()
    # sliding window 1 with 1 sink token, query position 4: visible = {0 (sink), 3, 4}
    q1 = q[:, :1]
    out = orc.gqa_attention(q1, k, v, 5, cap, nqh, nkvh, 1, hd, scale, mask_kind=2, offset=4, window=1, sink=1).reshape(nqh, hd)
    for qh in range(nqh):
        s = (k[0, :5].astype(np.float64) @ q1[qh, 0]) * scale
        s[[1, 2]] = -np.inf
        p = np.exp(s - s.max())
        assert np.abs(out[qh] - (p / p.sum()) @ v[0, :5]).max() < 1e-5
    # logit cap: cap * tanh(score / cap) before the softmax
    out = orc.gqa_attention(q1, k, v, 5, cap, nqh, nkvh, 1, hd, 4.0, logit_cap=1.5).reshape(nqh, hd)
    for qh in range(nqh):
        s = 1.5 * np.tanh((k[0, :5].astype(np.float64) @ q1[qh, 0]) * 4.0 / 1.5)
        p = np.exp(s - s.max())
        assert np.abs(out[qh] - (p / p.sum()) @ v[0, :5]).max() < 1e-5


def test_local_global_mask(orc):
    """AttentionMask::LocalGlobal (src/attention.rs:287-299) against an explicit visibility set
    in float64, and its reductions: every position global, or a window as long as the cache,
    is the causal mask; no global positions is the sliding window without sinks."""
    hd, nqh, nkvh, cap, n = 4, 2, 1, 16, 9
    scale = 0.5
    q, k, v = _qkv(nqh, nkvh, 3, n, hd, cap)
    offset, window, glob = 6, 1, [0, 3, 12]            # position 12 is past the cache: never a key
    out = orc.gqa_attention_local_global(q, k, v, n, cap, nqh, nkvh, 3, hd, scale, offset, window, glob).reshape(3, nqh, hd)
    for qt in range(3):
        pos = offset + qt
        visible = [kt for kt in range(n) if kt <= pos and (pos - kt <= window or kt in glob)]
        assert visible == [0, 3, pos - 1, pos]
        for qh in range(nqh):
            s = (k[0, :n].astype(np.float64) @ q[qh, qt]) * scale
            hidden = np.ones(n, bool)
            hidden[visible] = False
            s[hidden] = -np.inf
            p = np.exp(s - s.max())
            assert np.abs(out[qt, qh] - (p / p.sum()) @ v[0, :n]).max() < 1e-5
    causal = orc.gqa_attention(q, k, v, n, cap, nqh, nkvh, 3, hd, scale, mask_kind=1, offset=offset)
    assert (orc.gqa_attention_local_global(q, k, v, n, cap, nqh, nkvh, 3, hd, scale, offset, 0, range(n)) == causal).all()
    assert (orc.gqa_attention_local_global(q, k, v, n, cap, nqh, nkvh, 3, hd, scale, offset, n, []) == causal).all()
    window_only = orc.gqa_attention(q, k, v, n, cap, nqh, nkvh, 3, hd, scale, mask_kind=2, offset=offset, window=2, sink=0)
    assert (orc.gqa_attention_local_global(q, k, v, n, cap, nqh, nkvh, 3, hd, scale, offset, 2, []) == window_only).all()


def test_llama_block_against_float64_numpy(orc):
    """The block composition (decoder.rs:69-155 + attention.rs:74-212) recomputed in float64
    from the same dequantised weights: residuals, norms, RoPE positions, cache append and
    causal offset all have to line up.  Prefill of 3 tokens then a decode step."""
    d, nqh, nkvh, hd, ffn, cap, eps = 64, 4, 2, 16, 96, 8, 1e-5
    rng = np.random.default_rng(3)
    shapes = [(nqh * hd, d), (nkvh * hd, d), (nkvh * hd, d), (d, nqh * hd), (ffn, d), (ffn, d), (d, ffn)]
    raws = [H.pack_q8_0(orc.rng_normal(40 + i, n * k, 0.0, 0.1)) for i, (n, k) in enumerate(shapes)]
    W = [orc.dequant_q8_0(r, n * k).reshape(n, k).astype(np.float64) for r, (n, k) in zip(raws, shapes)]
    wa = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    wf = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    cos, sin = orc.rope_tables(hd, cap, 10000.0)
    kc = np.zeros((nkvh, cap, hd), np.float32)
    vc = np.zeros((nkvh, cap, hd), np.float32)
    K64 = np.zeros((nkvh, cap, hd))
    V64 = np.zeros((nkvh, cap, hd))

    def rms(x, w):
        return x / np.sqrt((x ** 2).mean(-1, keepdims=True) + eps) * w

    def rope(x, pos):
        c, s = cos[pos].astype(np.float64), sin[pos].astype(np.float64)
        return np.concatenate([x[..., : hd // 2] * c[: hd // 2] - x[..., hd // 2:] * s[: hd // 2],
                               x[..., : hd // 2] * s[: hd // 2] + x[..., hd // 2:] * c[: hd // 2]], -1)

    def block64(h, cache_len):
        seq = h.shape[0]
        n = rms(h, wa)
        q = (n @ W[0].T).reshape(seq, nqh, hd)
        k = (n @ W[1].T).reshape(seq, nkvh, hd)
        v = (n @ W[2].T).reshape(seq, nkvh, hd)
        att = np.zeros((seq, nqh, hd))
        for t in range(seq):
            K64[:, cache_len + t] = rope(k[t], cache_len + t)
            V64[:, cache_len + t] = v[t]
        for t in range(seq):
            for qh in range(nqh):
                kv = qh // (nqh // nkvh)
                L = cache_len + t + 1
                s = K64[kv, :L] @ rope(q[t, qh], cache_len + t) / np.sqrt(hd)
                p = np.exp(s - s.max())
                att[t, qh] = (p / p.sum()) @ V64[kv, :L]
        h1 = h + att.reshape(seq, nqh * hd) @ W[3].T
        n2 = rms(h1, wf)
        g, u = n2 @ W[4].T, n2 @ W[5].T
        return h1 + (g / (1 + np.exp(-g)) * u) @ W[6].T

    h = rng.standard_normal((3, d)).astype(np.float32)
    got = orc.llama_block_forward(h, 3, d, nqh, nkvh, hd, ffn, 8, raws, wa, wf, eps, cos, sin, kc, vc, 0, cap)
    want = block64(h.astype(np.float64), 0)
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()
    assert np.abs(kc - K64).max() < 1e-5 and np.abs(vc - V64).max() < 1e-5
    h2 = rng.standard_normal((1, d)).astype(np.float32)
    got = orc.llama_block_forward(h2, 1, d, nqh, nkvh, hd, ffn, 8, raws, wa, wf, eps, cos, sin, kc, vc, 3, cap)
    want = block64(h2.astype(np.float64), 3)
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()
