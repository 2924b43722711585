// Activation rows as two f16 planes for the f16 matrix-core block product (pg_gguf_hmm.hip):
// x * 2^e = hi + lo with one exponent e per row, chosen so that the row's largest magnitude
// lands in [2^14, 2^15).  hi is x * 2^e rounded to f16 (11 significant bits), lo the rounded
// remainder (the next 11): what the pair drops is below 2^-22 of the row's largest value.
// Shared by every kernel that writes such rows (the plain converter, RMSNorm, SiLU.up).
#pragma once
#include <hip/hip_runtime.h>

// The row's two scale factors and their inverses from its largest magnitude (`amax` must be
// INFINITY if the row holds a NaN or an infinity: the row then keeps e = 0).  2^e is carried
// as two factors because |e| passes 127 for rows of denormals.
struct pg_f16_row_scale {
    float s1, s2, i1, i2;
};
__device__ __forceinline__ pg_f16_row_scale pg_f16_row_scale_of(float amax) {
    int e = 0;
    if (amax > 0.0f && amax < INFINITY) {
        int ex;
        (void)frexpf(amax, &ex);  // amax = f * 2^ex, f in [0.5, 1)
        e = 15 - ex;
    }
    const int e1 = e / 2, e2 = e - e1;
    return {ldexpf(1.0f, e1), ldexpf(1.0f, e2), ldexpf(1.0f, -e1), ldexpf(1.0f, -e2)};
}

// |v| as it enters the row's maximum: INFINITY for a NaN too.
__device__ __forceinline__ float pg_f16_mag(float v) {
    const float a = fabsf(v);
    return a < INFINITY ? a : INFINITY;
}

// Four consecutive elements -> four hi and four lo halves (8 bytes each).  A non-finite
// remainder (the element itself was not finite, or overflowed f16 in an e = 0 row) gives lo = 0.
__device__ __forceinline__ void pg_f16_split4(const float f[4], const pg_f16_row_scale &sc, uint2 *hi, uint2 *lo) {
    _Float16 h[4], l[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float v = f[j] * sc.s1 * sc.s2;
        h[j] = (_Float16)v;
        const float r = v - (float)h[j];
        l[j] = fabsf(r) < INFINITY ? (_Float16)r : (_Float16)0.0f;
    }
    __builtin_memcpy(hi, h, 8);
    __builtin_memcpy(lo, l, 8);
}
