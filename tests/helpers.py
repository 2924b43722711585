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


from peregrine_amd.synth import pack_q4_0, pack_q4_1, pack_q8_0  # noqa: E402,F401


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


# ---- a GGUF writer for the container tests (format: reference src/gguf.rs:411-483) ----
GGUF_TYPE_CODES = {"u8": 0, "i8": 1, "u16": 2, "i16": 3, "u32": 4, "i32": 5, "f32": 6, "bool": 7, "str": 8,
                   "arr": 9, "u64": 10, "i64": 11, "f64": 12}
_GGUF_FMT = {"u8": "<B", "i8": "<b", "u16": "<H", "i16": "<h", "u32": "<I", "i32": "<i", "f32": "<f", "bool": "<B",
             "u64": "<Q", "i64": "<q", "f64": "<d"}


def _gguf_str(s):
    import struct
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _gguf_value(kind, v):
    import struct
    if kind == "str":
        return _gguf_str(v)
    if kind == "arr":  # v = (element kind, [elements])
        ek, items = v
        return struct.pack("<IQ", GGUF_TYPE_CODES[ek], len(items)) + b"".join(_gguf_value(ek, x) for x in items)
    return struct.pack(_GGUF_FMT[kind], v)


def build_gguf(metadata, tensors, version=3, magic=0x46554747):
    """metadata: list of (key, kind, value); tensors: list of (name, ggml_type, shape_gguf_order, raw_bytes).
    Returns (file bytes, data_start, {name: offset in data section})."""
    import struct
    align = 32
    for key, kind, v in metadata:
        if key == "general.alignment":
            align = int(v)
    head = struct.pack("<IIQQ", magic, version, len(tensors), len(metadata))
    for key, kind, v in metadata:
        head += _gguf_str(key) + struct.pack("<I", GGUF_TYPE_CODES[kind]) + _gguf_value(kind, v)
    offsets, off = {}, 0
    for name, typ, shape, raw in tensors:
        offsets[name] = off
        head += _gguf_str(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape)
        head += struct.pack("<IQ", typ, off)
        off = (off + len(raw) + align - 1) // align * align
    data_start = (len(head) + align - 1) // align * align
    body = bytearray(off)
    for name, typ, shape, raw in tensors:
        body[offsets[name]: offsets[name] + len(raw)] = raw
    return head + b"\0" * (data_start - len(head)) + bytes(body), data_start, offsets
