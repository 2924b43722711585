"""Shared test helpers: fixture loading, deterministic generators the reference's own
tests use, and block packers for synthetic GGUF tensors."""
import os
import struct

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_fixture(name):
    """[ndim u32][shape u32...][f32 data]  (reference: tests/pytorch_parity.rs:16-39)."""
    buf = open(os.path.join(GOLDEN, name), "rb").read()
    ndim = struct.unpack_from("<I", buf, 0)[0]
    shape = struct.unpack_from(f"<{ndim}I", buf, 4)
    data = np.frombuffer(buf, np.float32, int(np.prod(shape)), 4 + 4 * ndim)
    return data.reshape(shape).copy()


def lcg_data(n, seed):
    """tests/huffman_parity.rs:7-16: s = s*1103515245 + 12345 (u32); f = s/u32::MAX*2 - 1."""
    out = np.empty(n, np.float32)
    s = seed & 0xFFFFFFFF
    umax = np.float32(4294967295.0)
    for i in range(n):
        s = (s * 1103515245 + 12345) & 0xFFFFFFFF
        out[i] = np.float32(s) / umax * np.float32(2.0) - np.float32(1.0)
    return out


def mod_pattern(n, mul, add, mod, div, sub):
    """((i*mul + add) % mod) as f32 / div - sub  (tests/quant_parity.rs:10-12,40-45)."""
    i = np.arange(n, dtype=np.int64)
    return (((i * mul + add) % mod).astype(np.float32) / np.float32(div) - np.float32(sub)).astype(np.float32)


from peregrine_amd.synth import pack_q4_0, pack_q8_0  # noqa: E402,F401


def np_dequant_q4_0(raw, n):
    """Independent NumPy statement of the Q4_0 format (value = (q - 8) * d, interleaved)."""
    b = np.frombuffer(raw, np.uint8)[: n // 32 * 18].reshape(-1, 18)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32)
    lo = (b[:, 2:] & 15).astype(np.int32) - 8
    hi = (b[:, 2:] >> 4).astype(np.int32) - 8
    out = np.empty((b.shape[0], 32), np.float32)
    out[:, 0::2] = lo.astype(np.float32) * d
    out[:, 1::2] = hi.astype(np.float32) * d
    return out.reshape(-1)


def np_dequant_q8_0(raw, n):
    b = np.frombuffer(raw, np.uint8)[: n // 32 * 34].reshape(-1, 34)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32)
    q = b[:, 2:].copy().view(np.int8).astype(np.float32)
    return (q * d).reshape(-1)


def assert_close_rel(got, ref, rtol, what=""):
    """|got - ref| <= rtol * max(|ref|, rms(ref)): relative to each element, with the
    vector's RMS as the floor for entries that cancel to near zero."""
    got = np.asarray(got, np.float64).reshape(-1)
    ref = np.asarray(ref, np.float64).reshape(-1)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    floor = np.sqrt(np.mean(ref * ref)) if ref.size else 0.0
    bound = rtol * np.maximum(np.abs(ref), floor)
    err = np.abs(got - ref)
    worst = int(np.argmax(err - bound)) if ref.size else 0
    assert (err <= bound).all(), (
        f"{what}: element {worst}: got {got[worst]!r}, want {ref[worst]!r}, err {err[worst]:.3e} > {bound[worst]:.3e}")
