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


def pack_q8_0(w):
    """Quantise f32 [n_out, k_in] into GGUF Q8_0 blocks (d = f16(absmax/127)).  Any packer
    will do: parity is always against the dequantisation of these same bytes."""
    w = np.ascontiguousarray(w, np.float32).reshape(-1, 32)
    d = (np.abs(w).max(axis=1) / 127.0).astype(np.float16)
    df = d.astype(np.float32)
    q = np.where(df[:, None] > 0, np.rint(w / np.where(df[:, None] > 0, df[:, None], 1)), 0)
    q = np.clip(q, -127, 127).astype(np.int8)
    out = np.empty((w.shape[0], 34), np.uint8)
    out[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q.view(np.uint8)
    return out.tobytes()


def pack_q4_0(w):
    """Quantise f32 into GGUF Q4_0 blocks in the reference's element order
    (byte i holds element 2i in its low nibble, 2i+1 in its high nibble; src/gguf.rs:317-323)."""
    w = np.ascontiguousarray(w, np.float32).reshape(-1, 32)
    idx = np.abs(w).argmax(axis=1)
    mx = w[np.arange(w.shape[0]), idx]
    d = (mx / -8.0).astype(np.float16)
    df = d.astype(np.float32)
    inv = np.where(df != 0, 1.0 / np.where(df != 0, df, 1), 0).astype(np.float32)
    q = np.clip(np.floor(w * inv[:, None] + 8.5), 0, 15).astype(np.uint8)
    out = np.empty((w.shape[0], 18), np.uint8)
    out[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q[:, 0::2] | (q[:, 1::2] << 4)
    return out.tobytes()


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
