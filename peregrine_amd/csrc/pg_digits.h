// Activation blocks -> fixed-point digits for the streaming (one-row) block-dequant product:
// the step every producer of a GEMV input ends with, so that the f32 row need not be written
// and read back by a separate kernel.
#pragma once
#include "pg_internal.h"

// Eight consecutive lanes hold one block of 32 activations, four each (`sub` = lane within the
// group, f = its elements 4*sub .. 4*sub+3 of block b of activation row `row`); all eight
// must call together.  Writes the block's digit planes and its power-of-two scale:
//   xs[row][b]          the scale s (NaN if the block holds a NaN or inf)
//   digits[row][j][b]   16 bytes per (plane j, block b)
//     NIB (Q4_0):  |X| < 2^18, X = sum_j 16^j n_j with five signed 4-bit digits; plane j holds
//                  n_j of the block's 32 elements, element e in nibble e.
//     bytes (Q8_0): |X| < 2^22, X = 65536 a0 + 256 a1 + a2 with signed byte digits;
//                  plane 2j+h holds a_j of elements 16h..16h+15.
// With `xsum` (Q4_1, whose blocks carry an offset m: sum_k (q d + m) x = d sum q x + m sum x) the
// block's sum of fixed-point values, sum_k X[k], is stored too: xsum[row][b] (exact: < 2^23).
// A DPP move within groups of 8 lanes: 0xB1 = quad_perm [1,0,3,2], 0x4E = quad_perm [2,3,0,1],
// 0x141 = row_half_mirror (lane i of the 8 takes lane 7 - i).
template <int CTRL>
__device__ __forceinline__ int pg_dpp8(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}

template <bool NIB>
__device__ __forceinline__ void pg_emit_digits(const float (&f)[4], size_t row, int b, int sub, int nb,
                                               int8_t *__restrict__ digits, float *__restrict__ xs,
                                               float *__restrict__ xsum = nullptr) {
    float amax = fmaxf(fmaxf(fabsf(f[0]), fabsf(f[1])), fmaxf(fabsf(f[2]), fabsf(f[3])));
    int bad = (f[0] != f[0]) | (f[1] != f[1]) | (f[2] != f[2]) | (f[3] != f[3]);
    // over the 8 lanes of the group with DPP moves (no LDS round trips): neighbour, other pair, then the
    // mirror image within the 8 lanes, which pairs the two quads (max, or and + are symmetric)
    amax = fmaxf(amax, __builtin_bit_cast(float, pg_dpp8<0xB1>(__builtin_bit_cast(int, amax))));
    bad |= pg_dpp8<0xB1>(bad);
    amax = fmaxf(amax, __builtin_bit_cast(float, pg_dpp8<0x4E>(__builtin_bit_cast(int, amax))));
    bad |= pg_dpp8<0x4E>(bad);
    amax = fmaxf(amax, __builtin_bit_cast(float, pg_dpp8<0x141>(__builtin_bit_cast(int, amax))));
    bad |= pg_dpp8<0x141>(bad);
    constexpr int BITS = NIB ? 18 : 22;
    float s = 1.0f, inv = 1.0f;
    if (bad || !(amax <= 3.4028234663852886e38f)) {
        s = __uint_as_float(0x7FC00000u);
        inv = 0.0f;
    } else if (amax > 0.0f) {
        int ex;
        (void)frexpf(amax, &ex);  // amax = f * 2^ex, f in [0.5, 1)
        int se = ex - BITS;       // |x| / 2^se < 2^BITS
        if (se < -126) se = -126;
        s = ldexpf(1.0f, se);
        inv = ldexpf(1.0f, -se);
    }
    int X[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float t = f[e] * inv;
        X[e] = (t != t) ? 0 : (int)rintf(t);
    }
    if (xsum) {  // the same for all lanes
        int part = X[0] + X[1] + X[2] + X[3];
        part += pg_dpp8<0xB1>(part);
        part += pg_dpp8<0x4E>(part);
        part += pg_dpp8<0x141>(part);
        if (sub == 0) xsum[row * (size_t)nb + b] = (float)part;
    }
    int8_t *drow = digits + row * (size_t)nb * 96;
    if (NIB) {
        // Balanced base-16 digits n_j in [-8, 7] without a carry loop: X + 0x88888 = sum_j 16^j (n_j + 8),
        // and n_j + 8 with its top bit flipped is n_j in 4-bit two's complement, so nibble j of
        // (X + 0x88888) ^ 0x88888 is digit j as stored (|X| < 2^18 lies well inside the range).
        unsigned W[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) W[e] = (unsigned)(X[e] + 0x88888) ^ 0x88888u;
#pragma unroll
        for (int j = 0; j < 5; ++j) {
            const unsigned packed = __builtin_amdgcn_ubfe(W[0], 4 * j, 4) | (__builtin_amdgcn_ubfe(W[1], 4 * j, 4) << 4) |
                                    (__builtin_amdgcn_ubfe(W[2], 4 * j, 4) << 8) | (__builtin_amdgcn_ubfe(W[3], 4 * j, 4) << 12);
            // this thread's elements 4*sub .. 4*sub+3 are nibbles 4*sub.. of the block: bytes 2*sub, 2*sub+1
            *reinterpret_cast<uint16_t *>(drow + ((size_t)j * nb + b) * 16 + 2 * sub) = (uint16_t)packed;
        }
    } else {
        // The same in base 256: byte k of (X + 0x808080) ^ 0x808080 is the signed byte digit of weight 256^k.
        unsigned W[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) W[e] = (unsigned)(X[e] + 0x808080) ^ 0x808080u;
        const int e0 = sub * 4, h = e0 >> 4;
#pragma unroll
        for (int j = 0; j < 3; ++j) {  // plane pair j holds the digit of weight 256^(2-j)
            const int k = 2 - j;
            const unsigned packed = ((W[0] >> (8 * k)) & 255u) | (((W[1] >> (8 * k)) & 255u) << 8) |
                                    (((W[2] >> (8 * k)) & 255u) << 16) | (((W[3] >> (8 * k)) & 255u) << 24);
            *reinterpret_cast<unsigned *>(drow + ((size_t)(2 * j + h) * nb + b) * 16 + (e0 & 15)) = packed;
        }
    }
    if (sub == 0) xs[row * (size_t)nb + b] = s;
}

// ---- activation blocks -> two byte-digit planes for the matrix-core block product (gguf_mm_kernel) ----
// digits[row][plane][b][half][16]: plane 0 = high digit, 1 = low digit of X[k] = round(x[k] / xs[b]).
// The 16 bytes of (b, half) follow the order in which the weight operand presents its k:
//   Q8_0: half h holds elements 16h .. 16h+15;
//   Q4_0: half h holds elements 2i + h (i = 0..15): the low (h = 0) or high (h = 1) nibbles
//         of the block's 16 bytes (byte i = elements 2i, 2i+1, src/gguf.rs:316-323).
// xs[row][nbp]: block scales absmax / 32639 (NaN for a block holding NaN or inf), nbp = nb
// rounded up to 4.
// Bytes from one activation row's digits to the next: the two planes (nb * 64 bytes) padded to
// an odd number of 256-byte lines.  The 32 token rows of a tile are fetched at the same K
// offset at the same time; an even (worst: power-of-two, 64 KiB at K = 32768) stride sends
// all of them to the same memory channels.
__host__ __device__ static inline size_t pg_mm_row_bytes(size_t nb) {
    const size_t lines = (nb * 64 + 255) / 256;
    return (lines | 1) * 256;
}

// Eight consecutive lanes hold block b of activation row `row`, four elements each (as for pg_emit_digits);
// all eight must call together.
// With `xsum` (Q4_1: sum_k (q d + m) x = d sum q x + m sum x) the block's plain f32 sum of x is stored too, in
// xsum[row][nbp] (lanes' partial sums added pairwise, fixed order).
template <bool NIB>
__device__ __forceinline__ void pg_emit_mm_digits(const float (&f)[4], size_t row, int b, int sub, int nb, int nbp,
                                                  int8_t *__restrict__ digits, float *__restrict__ xs,
                                                  float *__restrict__ xsum = nullptr) {
    if (xsum) {  // the same for all lanes
        float t = (f[0] + f[1]) + (f[2] + f[3]);
        t += __builtin_bit_cast(float, pg_dpp8<0xB1>(__builtin_bit_cast(int, t)));
        t += __builtin_bit_cast(float, pg_dpp8<0x4E>(__builtin_bit_cast(int, t)));
        t += __builtin_bit_cast(float, pg_dpp8<0x141>(__builtin_bit_cast(int, t)));
        if (sub == 0) xsum[row * (size_t)nbp + b] = t;
    }
    float amax = fmaxf(fmaxf(fabsf(f[0]), fabsf(f[1])), fmaxf(fabsf(f[2]), fabsf(f[3])));
    int bad = (f[0] != f[0]) | (f[1] != f[1]) | (f[2] != f[2]) | (f[3] != f[3]);
    amax = fmaxf(amax, __builtin_bit_cast(float, pg_dpp8<0xB1>(__builtin_bit_cast(int, amax))));
    bad |= pg_dpp8<0xB1>(bad);
    amax = fmaxf(amax, __builtin_bit_cast(float, pg_dpp8<0x4E>(__builtin_bit_cast(int, amax))));
    bad |= pg_dpp8<0x4E>(bad);
    amax = fmaxf(amax, __builtin_bit_cast(float, pg_dpp8<0x141>(__builtin_bit_cast(int, amax))));
    bad |= pg_dpp8<0x141>(bad);
    float s = 1.0f, inv = 1.0f;
    if (bad || !(amax <= 3.4028234663852886e38f)) {
        s = __uint_as_float(0x7FC00000u);
        inv = 0.0f;
    } else if (amax > 0.0f) {
        // the two signed byte digits reach 127 * 256 + 127: map the block's absmax onto that
        s = fmaxf(amax / 32639.0f, 1.17549435e-38f);
        inv = 1.0f / s;
    }
    int hi[4], lo[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float t = f[e] * inv;
        const int X = (t != t) ? 0 : (int)rintf(t);
        lo[e] = ((X + 128) & 255) - 128;
        hi[e] = (X - lo[e]) >> 8;
    }
    int8_t *d0 = digits + row * pg_mm_row_bytes(nb) + (size_t)b * 32;  // plane 0, block b: [half][16]
    int8_t *d1 = d0 + (size_t)nb * 32;
    if (NIB) {
        // elements 4*sub + {0, 2} -> half 0 positions 2*sub, 2*sub+1;  {1, 3} -> half 1, same positions
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            *reinterpret_cast<uint16_t *>(d0 + h * 16 + 2 * sub) = (uint16_t)((hi[h] & 255) | ((hi[h + 2] & 255) << 8));
            *reinterpret_cast<uint16_t *>(d1 + h * 16 + 2 * sub) = (uint16_t)((lo[h] & 255) | ((lo[h + 2] & 255) << 8));
        }
    } else {
        const int h = sub >> 2, pos = (sub & 3) * 4;
        *reinterpret_cast<unsigned *>(d0 + h * 16 + pos) = (unsigned)(hi[0] & 255) | ((unsigned)(hi[1] & 255) << 8) |
                                                          ((unsigned)(hi[2] & 255) << 16) | ((unsigned)(hi[3] & 255) << 24);
        *reinterpret_cast<unsigned *>(d1 + h * 16 + pos) = (unsigned)(lo[0] & 255) | ((unsigned)(lo[1] & 255) << 8) |
                                                          ((unsigned)(lo[2] & 255) << 16) | ((unsigned)(lo[3] & 255) << 24);
    }
    if (sub == 0) xs[row * (size_t)nbp + b] = s;
}
