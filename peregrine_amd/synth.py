"""Synthetic inputs for tests and the benchmark (there are no real weights offline).

* `Random`: the reference's generators restated (src/random.rs): SplitMix64-seeded
  Xoshiro256++ for tensors below 200 000 elements, the counter-based Philox 4x32-10 path above
  (what `random::normal` runs for every benchmark-sized tensor), Box-Muller normals.  The
  Philox path is array code over NumPy or, given a torch device, over torch on that device.
* Block packers: quantise f32 matrices into GGUF Q8_0 / Q4_0 / Q4_1 blocks on the host; any
  packer will do, because parity is always judged against the dequantisation of the same bytes.
Importing this module needs NumPy only.
"""
import numpy as np

_M64 = (1 << 64) - 1
PHILOX_THRESHOLD = 200_000  # src/random.rs:79


class Xoshiro256pp:
    """Xoshiro256PlusPlus  src/random.rs:16-53 (scalar; Python integers)."""

    def __init__(self, seed):
        sm, self.s = seed & _M64, []
        for _ in range(4):  # SplitMix64
            sm = (sm + 0x9E3779B97F4A7C15) & _M64
            z = sm
            z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
            z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
            self.s.append(z ^ (z >> 31))

    @staticmethod
    def _rotl(x, k):
        return ((x << k) | (x >> (64 - k))) & _M64

    def next_u64(self):
        s = self.s
        result = (self._rotl((s[0] + s[3]) & _M64, 23) + s[0]) & _M64
        t = (s[1] << 17) & _M64
        s[2] ^= s[0]
        s[3] ^= s[1]
        s[1] ^= s[2]
        s[0] ^= s[3]
        s[2] ^= t
        s[3] = self._rotl(s[3], 45)
        return result

    def next_f32(self):
        """Uniform in [0, 1): the top 24 bits (exact in f32)."""
        return np.float32(self.next_u64() >> 40) / np.float32(1 << 24)


def philox_4x32_10(ctr_lo, ctr_hi, key, xp=np):
    """philox_4x32_10  src/random.rs:88-103 on arrays: counters (ctr_lo, ctr_hi, 0, 0) with one
    key for all.  Inputs and the four outputs are int64 arrays holding u32 values (64-bit
    products wrap, which leaves their low 64 bits intact)."""
    c = [ctr_lo, ctr_hi, ctr_lo * 0, ctr_lo * 0]
    k0, k1 = key
    mask = 0xFFFFFFFF
    for _ in range(10):
        p0, p1 = c[0] * 0xD2511F53, c[2] * 0xCD9E8D57
        lo0, hi0 = p0 & mask, (p0 >> 32) & mask
        lo1, hi1 = p1 & mask, (p1 >> 32) & mask
        c = [hi1 ^ c[1] ^ k0, lo1, hi0 ^ c[3] ^ k1, lo0]
        k0, k1 = (k0 + 0x9E3779B9) & mask, (k1 + 0xBB67AE85) & mask
    return c


class Random:
    """The reference's global generator state (`random::seed`, src/random.rs:273-278) and
    `random::normal` (src/random.rs:311-380): below 200 000 elements the sequential Xoshiro
    stream, at or above it two Philox streams (u1, u2) indexed by a counter that every call
    advances; both feed the same Box-Muller transform
        out[2i] = mean + std * sqrt(-2 ln u1) * cos(2 pi u2),  out[2i+1] = ... sin(...),
    u1 clamped to >= 1e-10.  The libm calls are NumPy's (or torch's): values agree with a C
    libm to a few ulp, the underlying integers exactly."""

    KEY_U1, KEY_U2 = (0xDEADBEEF, 0xCAFEBABE), (0xFEEDFACE, 0xBAADF00D)

    def __init__(self, seed=42):
        self.seed(seed)

    def seed(self, s):
        self.xo = Xoshiro256pp(s)
        self.philox_counter = s & _M64

    def _philox_uniform(self, first_call, calls, count, key, device):
        """`count` u32 draws (as int64): outputs 0..3 of the calls first_call .. first_call+calls-1."""
        if device is None:
            idx = np.arange(calls, dtype=np.int64)
            xp = np
        else:
            import torch
            idx = torch.arange(calls, dtype=torch.int64, device=device)
            xp = torch
        lo = (idx + (first_call & 0xFFFFFFFF))
        carry = lo >> 32
        hi = (carry + ((first_call >> 32) & 0xFFFFFFFF)) & 0xFFFFFFFF
        out = philox_4x32_10(lo & 0xFFFFFFFF, hi, key, xp)
        return xp.stack(out, 1).reshape(-1)[:count]

    def normal(self, n, mean=0.0, std=1.0, device=None):
        """`n` normals as f32: a NumPy array, or a torch tensor on `device`."""
        n = int(n)
        if n < PHILOX_THRESHOLD:
            pairs = (n + 1) // 2
            u1 = np.empty(pairs, np.float32)
            u2 = np.empty(pairs, np.float32)
            for i in range(pairs):
                u1[i] = self.xo.next_f32()
                u2[i] = self.xo.next_f32()
            out = _box_muller(np, np.maximum(u1, np.float32(1e-10)), u2, mean, std)[:n]
            if device is not None:
                import torch
                return torch.from_numpy(out).to(device)
            return out
        pairs = (n + (n & 1)) // 2
        calls = (pairs + 3) // 4
        base = self.philox_counter
        self.philox_counter = (base + 2 * calls) & _M64
        r1 = self._philox_uniform(base, calls, pairs, self.KEY_U1, device)
        r2 = self._philox_uniform((base + calls) & _M64, calls, pairs, self.KEY_U2, device)
        if device is None:
            scale = np.float32(1.0) / np.float32(1 << 32)
            u1 = np.maximum(r1.astype(np.float32) * scale, np.float32(1e-10))
            u2 = r2.astype(np.float32) * scale
            return _box_muller(np, u1, u2, mean, std)[:n]
        import torch
        scale = 1.0 / float(1 << 32)
        u1 = torch.clamp_min(r1.to(torch.float32) * scale, 1e-10)
        u2 = r2.to(torch.float32) * scale
        return _box_muller(torch, u1, u2, mean, std)[:n]

    def distinct_below(self, count, bound):
        """`count` distinct integers in [0, bound) from the sequential stream (next_u64 % bound,
        repeats skipped), sorted: the benchmark's outlier channels."""
        seen = []
        while len(seen) < count:
            v = self.xo.next_u64() % bound
            if v not in seen:
                seen.append(v)
        return sorted(seen)


def _box_muller(xp, u1, u2, mean, std):
    f = np.float32 if xp is np else (lambda v: v)
    two_pi = np.float32(2.0) * np.float32(np.pi) if xp is np else float(np.float32(2.0) * np.float32(np.pi))
    r = xp.sqrt(f(-2.0) * xp.log(u1))
    theta = two_pi * u2
    sr = f(std) * r
    z0, z1 = f(mean) + sr * xp.cos(theta), f(mean) + sr * xp.sin(theta)
    return xp.stack([z0, z1], 1).reshape(-1)


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
