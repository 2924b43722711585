"""Synthetic GGUF block data: quantise f32 matrices into Q8_0 / Q4_0 / Q4_1 blocks on the host.

Input synthesis for tests and the benchmark (there are no real .gguf files offline); any
packer will do, because parity is always judged against the dequantisation of the same bytes.
Importing this module needs NumPy only.
"""
import numpy as np


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


def pack_q4_1(w):
    """Quantise f32 into GGUF Q4_1 blocks (d = f16((max - min) / 15), m = f16(min), q = 0..15,
    value = q * d + m; same nibble order as Q4_0, src/gguf.rs:331-351)."""
    w = np.ascontiguousarray(w, np.float32).reshape(-1, 32)
    lo, hi = w.min(axis=1), w.max(axis=1)
    d = ((hi - lo) / 15.0).astype(np.float16)
    m = lo.astype(np.float16)
    df, mf = d.astype(np.float32), m.astype(np.float32)
    inv = np.where(df != 0, 1.0 / np.where(df != 0, df, 1), 0).astype(np.float32)
    q = np.clip(np.rint((w - mf[:, None]) * inv[:, None]), 0, 15).astype(np.uint8)
    out = np.empty((w.shape[0], 20), np.uint8)
    out[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
    out[:, 2:4] = m.view(np.uint8).reshape(-1, 2)
    out[:, 4:] = q[:, 0::2] | (q[:, 1::2] << 4)
    return out.tobytes()
