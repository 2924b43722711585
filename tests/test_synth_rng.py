"""The benchmark's input generators (peregrine_amd/synth.py: Xoshiro256++, Philox 4x32-10,
Box-Muller, restated from the reference's src/random.rs) against published vectors and
against the oracle's C restatement of the same source.  CPU only."""
import numpy as np

from peregrine_amd import synth


def test_philox_published_vectors(orc):
    """Known-answer vectors of Philox4x32-10 (Random123's kat_vectors): the oracle on all three,
    the array code on the one whose counter has the (lo, hi, 0, 0) shape the reference uses."""
    kats = [((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
            ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
            ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
             (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1))]
    for ctr, key, want in kats:
        assert tuple(orc.philox_4x32_10(ctr, key)) == want
    out = synth.philox_4x32_10(np.array([0], np.int64), np.array([0], np.int64), (0, 0))
    assert tuple(int(v[0]) for v in out) == kats[0][2]


def test_philox_array_code_equals_the_oracle():
    import oracle_lib as orc
    rng = np.random.default_rng(0)
    lo = rng.integers(0, 1 << 32, 200, dtype=np.int64)
    hi = rng.integers(0, 1 << 32, 200, dtype=np.int64)
    lo[:3], hi[:3] = (0xFFFFFFFF, 0, 0xFFFFFFFE), (0, 0xFFFFFFFF, 7)
    for key in (synth.Random.KEY_U1, synth.Random.KEY_U2, (0x12345678, 0x9ABCDEF0)):
        out = synth.philox_4x32_10(lo, hi, key)
        for i in range(len(lo)):
            assert [int(o[i]) for o in out] == orc.philox_4x32_10((int(lo[i]), int(hi[i]), 0, 0), key)


def test_xoshiro_stream_equals_the_oracle(orc):
    for seed in (0, 42, 1234, (1 << 64) - 1):
        a, b = synth.Xoshiro256pp(seed), orc.Random(seed)
        assert [a.next_u64() for _ in range(64)] == [b.next_u64() for _ in range(64)]
    # SplitMix64's published first outputs for seed 0 are the generator's initial state
    assert synth.Xoshiro256pp(0).s[:2] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4]


def close_ulps(a, b, what):
    """Same integers underneath, libm calls from different libraries on top: a few ulp of the
    value, with an absolute floor where cos/sin cross zero."""
    tol = 8 * np.spacing(np.maximum(np.abs(b), np.float32(1.0)).astype(np.float32))
    bad = np.abs(a.astype(np.float64) - b.astype(np.float64)) > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} of {a.size} differ, first at {int(np.argmax(bad))}"


def test_normal_both_paths_equal_the_oracle(orc):
    # below the threshold: the sequential stream; odd and even counts; the state carries over
    a, b = synth.Random(1234), orc.Random(1234)
    for n in (1, 2, 7, 4096, 14336):
        close_ulps(a.normal(n), b.normal(n), f"xoshiro path n={n}")
    # at and above it: the counter-based path; the counter advances by 2 * ceil(pairs / 4) per call
    for n, mean, std in ((200_000, 0.0, 1.0), (200_003, 0.5, 0.02), (262_144, 0.0, 0.02)):
        close_ulps(a.normal(n, mean, std), b.normal(n, mean, std), f"philox path n={n}")
    assert a.philox_counter == 1234 + 2 * (25_000 + 25_001 + 32_768)
    # moments of a large draw
    z = synth.Random(7).normal(1 << 20)
    assert abs(float(z.mean())) < 5e-3 and abs(float(z.std()) - 1.0) < 5e-3
    # the counter carry from the low into the high word
    c, d = synth.Random(0), orc.Random(0)
    c.philox_counter = (1 << 32) - 100
    d._st[4] = (1 << 32) - 100
    close_ulps(c.normal(200_000), d.normal(200_000), "counter carry")


def test_normal_torch_path_equals_numpy():
    import torch
    a, b = synth.Random(99), synth.Random(99)
    x = a.normal(300_000, 0.0, 0.02)
    y = b.normal(300_000, 0.0, 0.02, device=torch.device("cpu")).numpy()
    close_ulps(y, x, "torch path")
    assert synth.Random(5).distinct_below(40, 4096) == synth.Random(5).distinct_below(40, 4096)
    ch = synth.Random(5).distinct_below(40, 4096)
    assert len(set(ch)) == 40 and max(ch) < 4096 and ch == sorted(ch)
