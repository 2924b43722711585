// gguf::* entry points: f16 conversion, block dequantisation, and the fused
// dequantise-matmul over GGUF Q4_0 / Q8_0 weights kept quantised in HBM.
//
// Fused product, y[m, n] = sum_k x[m, k] * (q[n, k] * d[n, k/32]):
//  * each activation row is first rewritten as 24-bit fixed point,
//    x[k] = s * X[k] with s a power of two and |X| < 2^22 (absolute error
//    <= 2^-23 * max|x| per element, the rounding an f32 accumulation of the row
//    would commit anyway), and X split into three signed byte digits
//    X = 65536*a0 + 256*a1 + a2;
//  * the inner sums over one block of 32, sum_k q*a_j, are then exact integer
//    dot products (v_dot4_i32_i8 on the packed bytes, no per-element int->float
//    conversion), recombined and scaled by d in f32 once per block.
// The result differs from the reference's dequantise-then-f32-matmul only by
// f32 rounding noise (relative tolerance 1e-3 is the contract; observed ~1e-6).
#include <new>
#include "pg_internal.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

inline unsigned grid_for(size_t n, unsigned block) { return (unsigned)((n + block - 1) / block); }

// ---- f16 -> f32, bit-exact with gguf::f16_to_f32 (src/gguf.rs:354-382) ----------
__device__ __forceinline__ uint32_t f16_bits_to_f32_bits(uint32_t h) {
    const uint32_t sign = (h >> 15) & 1u, exp = (h >> 10) & 0x1Fu, mant = h & 0x3FFu;
    if (exp == 0) {
        if (mant == 0) return sign << 31;
        const int shift = __clz(mant) - 21;  // moves the leading 1 to bit 10
        const uint32_t m = (mant << shift) & 0x3FFu;
        return (sign << 31) | ((uint32_t)(113 - shift) << 23) | (m << 13);
    }
    if (exp == 31) return (sign << 31) | 0x7F800000u | (mant << 13);
    return (sign << 31) | ((exp + 112u) << 23) | (mant << 13);
}

__device__ __forceinline__ float f16_to_f32_dev(uint16_t h) {
    return __uint_as_float(f16_bits_to_f32_bits(h));
}

__global__ void f16_to_f32_kernel(const uint16_t *__restrict__ in, size_t n, uint32_t *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = f16_bits_to_f32_bits(in[i]);
}

// ---- whole-tensor dequantisation (one thread per block of 32) -------------------
__device__ __forceinline__ uint16_t ld_u16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

__global__ void dequant_q8_0_kernel(const uint8_t *__restrict__ data, size_t nblocks, float *__restrict__ out) {
    const size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const uint8_t *blk = data + b * 34;
    const float d = f16_to_f32_dev(ld_u16(blk));
    float *o = out + b * 32;
#pragma unroll
    for (int i = 0; i < 32; ++i) o[i] = (float)(int8_t)blk[2 + i] * d;
}

__global__ void dequant_q4_0_kernel(const uint8_t *__restrict__ data, size_t nblocks, float *__restrict__ out) {
    const size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const uint8_t *blk = data + b * 18;
    const float d = f16_to_f32_dev(ld_u16(blk));
    float *o = out + b * 32;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int byte = blk[2 + i];
        o[2 * i] = (float)((byte & 0x0F) - 8) * d;
        o[2 * i + 1] = (float)((byte >> 4) - 8) * d;
    }
}

__global__ void dequant_q4_1_kernel(const uint8_t *__restrict__ data, size_t nblocks, float *__restrict__ out) {
    const size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const uint8_t *blk = data + b * 20;
    const float d = f16_to_f32_dev(ld_u16(blk));
    const float mn = f16_to_f32_dev(ld_u16(blk + 2));
    float *o = out + b * 32;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int byte = blk[4 + i];
        o[2 * i] = (float)(byte & 0x0F) * d + mn;       // mul then add, not fused
        o[2 * i + 1] = (float)(byte >> 4) * d + mn;
    }
}

// ---- upload: split raw blocks into planes ---------------------------------------
// Q4_0: qs[(n*nb + b)*16 .. +16] = the block's 16 nibble bytes.
// Q8_0: qs[((n*2 + h)*nb + b)*16 .. +16] = bytes 16h..16h+15 of the block's 32 i8.
// d[n*nb + b] = the block's f16 scale.
__global__ void split_blocks_kernel(const uint8_t *__restrict__ raw, size_t n_out, size_t nb,
                                    int ggml_type, uint8_t *__restrict__ qs,
                                    uint16_t *__restrict__ d) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_out * nb) return;
    const size_t n = i / nb, b = i - n * nb;
    if (ggml_type == PG_GGML_Q4_0) {
        const uint8_t *blk = raw + i * 18;
        d[i] = ld_u16(blk);
        for (int j = 0; j < 16; ++j) qs[i * 16 + j] = blk[2 + j];
    } else {
        const uint8_t *blk = raw + i * 34;
        d[i] = ld_u16(blk);
        for (int h = 0; h < 2; ++h)
            for (int j = 0; j < 16; ++j) qs[((n * 2 + h) * nb + b) * 16 + j] = blk[2 + 16 * h + j];
    }
}

// ---- activation rows -> 24-bit fixed point, three byte digits -------------------
// Output for row m (all of it in the scratch arena):
//   digits[j][m][k']  j = 0..2, k' = k for Q8_0; for Q4_0 each block of 32 is stored
//                     as its 16 even-indexed elements followed by its 16 odd-indexed
//                     ones, matching (byte & 15) / (byte >> 4) unpacked as dwords;
//   xs[m]             the power-of-two scale (NaN if the row holds a NaN or inf);
//   bsum[j][m][b]     sum of digit j over block b (Q4_0's -8 offset needs it).
__device__ __forceinline__ void split_digits(int X, int &a0, int &a1, int &a2) {
    a2 = ((X + 128) & 255) - 128;
    const int X1 = (X - a2) >> 8;
    a1 = ((X1 + 128) & 255) - 128;
    a0 = (X1 - a1) >> 8;
}

__global__ __launch_bounds__(256) void x_to_digits_kernel(const float *__restrict__ x, size_t k,
                                                          int deinterleave, size_t rows,
                                                          int8_t *__restrict__ digits,
                                                          float *__restrict__ xs,
                                                          int *__restrict__ bsum) {
    __shared__ float red[4];
    __shared__ int bad[4];
    const size_t row = blockIdx.x;
    const float *xr = x + row * k;
    float amax = 0.0f;
    int nan_seen = 0;
    for (size_t i = threadIdx.x; i < k; i += 256) {
        const float v = xr[i];
        nan_seen |= (v != v);
        amax = fmaxf(amax, fabsf(v));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        amax = fmaxf(amax, __shfl_xor(amax, off, 64));
        nan_seen |= __shfl_xor(nan_seen, off, 64);
    }
    if ((threadIdx.x & 63) == 0) { red[threadIdx.x >> 6] = amax; bad[threadIdx.x >> 6] = nan_seen; }
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    nan_seen = bad[0] | bad[1] | bad[2] | bad[3];
    float s = 1.0f, inv = 1.0f;
    if (nan_seen || !(amax <= 3.4028234663852886e38f)) {
        s = __uint_as_float(0x7FC00000u);
        inv = 0.0f;
    } else if (amax > 0.0f) {
        int ex;
        (void)frexpf(amax, &ex);  // amax = f * 2^ex, f in [0.5, 1)
        int se = ex - 22;         // |x| / 2^se < 2^22
        if (se < -126) se = -126;
        s = ldexpf(1.0f, se);
        inv = ldexpf(1.0f, -se);
    }
    if (threadIdx.x == 0) xs[row] = s;
    const size_t nb = k / 32;
    // 8 consecutive threads cover one block of 32 (4 elements each).
    for (size_t g = threadIdx.x; g < k / 4; g += 256) {
        const float4 v = reinterpret_cast<const float4 *>(xr)[g];
        const float f[4] = {v.x, v.y, v.z, v.w};
        int a[3][4];
        int sum[3] = {0, 0, 0};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float t = f[e] * inv;
            const int X = (t != t) ? 0 : (int)rintf(t);
            split_digits(X, a[0][e], a[1][e], a[2][e]);
#pragma unroll
            for (int j = 0; j < 3; ++j) sum[j] += a[j][e];
        }
        const size_t b = g / 8;
        const int e0 = (int)(g & 7) * 4;  // first element of this thread within the block
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            int8_t *dst = digits + ((size_t)j * rows + row) * k + b * 32;
            if (deinterleave) {
                dst[e0 / 2] = (int8_t)a[j][0];
                dst[e0 / 2 + 1] = (int8_t)a[j][2];
                dst[16 + e0 / 2] = (int8_t)a[j][1];
                dst[16 + e0 / 2 + 1] = (int8_t)a[j][3];
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) dst[e0 + e] = (int8_t)a[j][e];
            }
            int t = sum[j];
            t += __shfl_xor(t, 1, 64);
            t += __shfl_xor(t, 2, 64);
            t += __shfl_xor(t, 4, 64);
            if ((g & 7) == 0) bsum[((size_t)j * rows + row) * nb + b] = t;
        }
    }
}

// ---- M = 1 fused dequant-GEMV ------------------------------------------------------
// Workgroup = 4 wavefronts; wavefront w owns R consecutive weight rows.  Lane l
// owns blocks l, l+64, ... (BPL of them per K segment of 64*BPL blocks): its
// activation digits for those blocks sit in registers for all R rows, and one
// wavefront load of weights covers 64 consecutive blocks (1 KiB) of one row.
// The workgroup first stages the row's digits in LDS as [digit][16B-half][block]
// so the per-lane 128-bit LDS reads are conflict-free.
template <int QT>  // 4 = Q4_0, 8 = Q8_0
struct BlockDot;

template <>
struct BlockDot<4> {
    // w: 16 nibble bytes; xe/xo: even/odd element digits (4 dwords each).
    static __device__ __forceinline__ int dot(const v4i w, const v4i xe, const v4i xo, int acc) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int lo = w[t] & 0x0F0F0F0F;
            const int hi = (w[t] >> 4) & 0x0F0F0F0F;
            acc = __builtin_amdgcn_sdot4(lo, xe[t], acc, false);
            acc = __builtin_amdgcn_sdot4(hi, xo[t], acc, false);
        }
        return acc;
    }
};

template <>
struct BlockDot<8> {
    static __device__ __forceinline__ int dot(const v4i w0, const v4i w1, const v4i x0, const v4i x1, int acc) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            acc = __builtin_amdgcn_sdot4(w0[t], x0[t], acc, false);
            acc = __builtin_amdgcn_sdot4(w1[t], x1[t], acc, false);
        }
        return acc;
    }
};

// Hardware f16 -> f32 (exact for every non-NaN input).
__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// blockIdx.x = batch item (activation row / MoE pair), blockIdx.y = group of 4*R
// weight rows.  With a table, item i multiplies by expert table[expert_of[i]] and
// reads activation row i / x_row_div; without one, every item uses (qs0, d0).
template <int QT, int BPL, int R>
__global__ __launch_bounds__(256) void gguf_gemv_kernel(
    const uint8_t *__restrict__ qs0, const uint16_t *__restrict__ d0, pg_gemv_batch batch,
    int n_out, int nb, const int8_t *__restrict__ digits_base, size_t digit_plane_stride,
    const int *__restrict__ bsum_base, size_t bsum_plane_stride, const float *__restrict__ xs_base,
    float *__restrict__ y_base) {
    extern __shared__ v4i xl[];  // [3][2][seg_blocks] 16-byte halves
    constexpr int SEG = 64 * BPL;  // blocks per K segment
    const int item = blockIdx.x;
    const uint8_t *__restrict__ qs = qs0;
    const uint16_t *__restrict__ dsc = d0;
    if (batch.qs_table) {
        const int e = batch.expert_of[item];
        qs = batch.qs_table[e];
        dsc = batch.d_table[e];
    }
    const size_t xrow = (size_t)(item / batch.x_row_div);
    const int8_t *__restrict__ digits = digits_base + xrow * (size_t)nb * 32;
    const int *__restrict__ bsum = bsum_base + xrow * (size_t)nb;
    const float *__restrict__ xs = xs_base + xrow;
    float *__restrict__ y = y_base + (size_t)item * n_out;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int row0 = (blockIdx.y * 4 + wave) * R;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;

    for (int seg0 = 0; seg0 < nb; seg0 += SEG) {
        const int seg_n = (nb - seg0 < SEG) ? nb - seg0 : SEG;
        __syncthreads();  // previous segment fully consumed
        for (int i = threadIdx.x; i < 3 * 2 * seg_n; i += 256) {
            const int j = i / (2 * seg_n), rem = i - j * 2 * seg_n;
            const int b = rem >> 1, h = rem & 1;
            const v4i v = *reinterpret_cast<const v4i *>(digits + (size_t)j * digit_plane_stride +
                                                         (size_t)(seg0 + b) * 32 + h * 16);
            xl[(j * 2 + h) * SEG + b] = v;
        }
        __syncthreads();
        // this lane's digits and block sums for the segment
        v4i xd[BPL][3][2];
        int off8[BPL][3];
#pragma unroll
        for (int p = 0; p < BPL; ++p) {
            const int bl = lane + 64 * p;
            const bool live = bl < seg_n;
#pragma unroll
            for (int j = 0; j < 3; ++j) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    v4i v = xl[(j * 2 + h) * SEG + (live ? bl : 0)];
                    if (!live) v = (v4i){0, 0, 0, 0};
                    xd[p][j][h] = v;
                }
                off8[p][j] = (QT == 4 && live) ? -8 * bsum[(size_t)j * bsum_plane_stride + seg0 + bl] : 0;
            }
        }
        if (row0 < n_out) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int row = (row0 + r < n_out) ? row0 + r : n_out - 1;  // clamp, masked at the store
#pragma unroll
                for (int p = 0; p < BPL; ++p) {
                    const int bl = lane + 64 * p;
                    const int b = seg0 + ((bl < seg_n) ? bl : 0);
                    int i0 = off8[p][0], i1 = off8[p][1], i2 = off8[p][2];
                    if (QT == 4) {
                        const v4i w = __builtin_nontemporal_load(
                            reinterpret_cast<const v4i *>(qs + ((size_t)row * nb + b) * 16));
                        i0 = BlockDot<4>::dot(w, xd[p][0][0], xd[p][0][1], i0);
                        i1 = BlockDot<4>::dot(w, xd[p][1][0], xd[p][1][1], i1);
                        i2 = BlockDot<4>::dot(w, xd[p][2][0], xd[p][2][1], i2);
                    } else {
                        const v4i w0 = __builtin_nontemporal_load(
                            reinterpret_cast<const v4i *>(qs + (((size_t)row * 2 + 0) * nb + b) * 16));
                        const v4i w1 = __builtin_nontemporal_load(
                            reinterpret_cast<const v4i *>(qs + (((size_t)row * 2 + 1) * nb + b) * 16));
                        i0 = BlockDot<8>::dot(w0, w1, xd[p][0][0], xd[p][0][1], i0);
                        i1 = BlockDot<8>::dot(w0, w1, xd[p][1][0], xd[p][1][1], i1);
                        i2 = BlockDot<8>::dot(w0, w1, xd[p][2][0], xd[p][2][1], i2);
                    }
                    const float d = half_bits_to_float(dsc[(size_t)row * nb + b]);
                    // X-weighted block sum: 65536*i0 + 256*i1 + i2 (each term exact in f32)
                    const float f = fmaf((float)i0, 65536.0f, (float)(i1 * 256 + i2));
                    acc[r] = fmaf(d, f, acc[r]);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = wave_sum_f32(acc[r]);
    if (lane == 0) {
        const float s = xs[0];
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (row0 + r < n_out) y[row0 + r] = acc[r] * s;
    }
}

template <int QT, int BPL>
pg_status launch_gemv_bpl(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d,
                          const pg_gemv_batch &batch, const pg_xdigits &xd, float *y) {
    const int nb = (int)(k_in / 32);
    const size_t lds = (size_t)3 * 2 * 64 * BPL * 16;
    const size_t want_waves = (size_t)ctx->num_cu * 8;
    const size_t dps = xd.rows * xd.k, bps = xd.rows * (size_t)nb;
#define PG_GGUF_GEMV_LAUNCH(RR)                                                                    \
    do {                                                                                           \
        const dim3 grid((unsigned)batch.count, grid_for(n_out, 4 * RR));                           \
        pg_prof_scope ps(ctx, QT == 4 ? "gguf_gemv_q4_0" : "gguf_gemv_q8_0");                      \
        gguf_gemv_kernel<QT, BPL, RR><<<grid, 256, lds, ctx->stream>>>(                            \
            qs, d, batch, (int)n_out, nb, xd.digits, dps, xd.bsum, bps, xd.xs, y);                 \
    } while (0)
    if (n_out / 4 * batch.count >= want_waves) PG_GGUF_GEMV_LAUNCH(4);
    else if (n_out / 2 * batch.count >= want_waves) PG_GGUF_GEMV_LAUNCH(2);
    else PG_GGUF_GEMV_LAUNCH(1);
#undef PG_GGUF_GEMV_LAUNCH
    return pg_launch_check("gguf_gemv");
}

template <int QT>
pg_status launch_gemv(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d,
                      const pg_gemv_batch &batch, const pg_xdigits &xd, float *y) {
    const size_t nb = k_in / 32;
    size_t bpl = (nb + 63) / 64;
    if (bpl > 8) bpl = 8;  // longer rows run as several K segments
    switch (bpl) {
        case 1: return launch_gemv_bpl<QT, 1>(ctx, n_out, k_in, qs, d, batch, xd, y);
        case 2: return launch_gemv_bpl<QT, 2>(ctx, n_out, k_in, qs, d, batch, xd, y);
        case 3: return launch_gemv_bpl<QT, 3>(ctx, n_out, k_in, qs, d, batch, xd, y);
        case 4: return launch_gemv_bpl<QT, 4>(ctx, n_out, k_in, qs, d, batch, xd, y);
        case 5: return launch_gemv_bpl<QT, 5>(ctx, n_out, k_in, qs, d, batch, xd, y);
        case 6: return launch_gemv_bpl<QT, 6>(ctx, n_out, k_in, qs, d, batch, xd, y);
        case 7: return launch_gemv_bpl<QT, 7>(ctx, n_out, k_in, qs, d, batch, xd, y);
        default: return launch_gemv_bpl<QT, 8>(ctx, n_out, k_in, qs, d, batch, xd, y);
    }
}

}  // namespace

size_t pg_xdigits_bytes(size_t rows, size_t k) {
    const size_t nb = k / 32;
    return pg_round_up(3 * rows * k, 256) + pg_round_up(3 * rows * nb * sizeof(int), 256) +
           pg_round_up(rows * sizeof(float), 256);
}

pg_xdigits pg_xdigits_carve(void *base, size_t rows, size_t k) {
    const size_t nb = k / 32;
    pg_xdigits xd;
    char *p = static_cast<char *>(base);
    xd.digits = reinterpret_cast<int8_t *>(p);
    p += pg_round_up(3 * rows * k, 256);
    xd.bsum = reinterpret_cast<int *>(p);
    p += pg_round_up(3 * rows * nb * sizeof(int), 256);
    xd.xs = reinterpret_cast<float *>(p);
    xd.rows = rows;
    xd.k = k;
    return xd;
}

pg_status pg_launch_x_to_digits(pg_ctx *ctx, const float *x_dev, size_t rows, size_t k,
                                int ggml_type, const pg_xdigits &xd) {
    if (rows == 0) return PG_OK;
    pg_prof_scope ps(ctx, "x_to_digits");
    x_to_digits_kernel<<<(unsigned)rows, 256, 0, ctx->stream>>>(
        x_dev, k, ggml_type == PG_GGML_Q4_0 ? 1 : 0, rows, xd.digits, xd.xs, xd.bsum);
    return pg_launch_check("x_to_digits");
}

pg_status pg_launch_gguf_gemv(pg_ctx *ctx, int ggml_type, size_t n_out, size_t k_in,
                              const uint8_t *qs, const uint16_t *d, const pg_gemv_batch &batch,
                              const pg_xdigits &xd, float *y) {
    if (batch.count == 0) return PG_OK;
    if (ggml_type == PG_GGML_Q4_0) return launch_gemv<4>(ctx, n_out, k_in, qs, d, batch, xd, y);
    return launch_gemv<8>(ctx, n_out, k_in, qs, d, batch, xd, y);
}

// Quantise `m` activation rows (device) into the arena and run the fused product.
pg_status pg_gguf_matmul_rows(pg_ctx *ctx, const float *x_dev, size_t m, const pg_gguf_tensor *w,
                              float *y_dev) {
    void *ws = nullptr;
    PG_TRY(pg_workspace(ctx, pg_xdigits_bytes(m, w->k_in), &ws));
    const pg_xdigits xd = pg_xdigits_carve(ws, m, w->k_in);
    PG_TRY(pg_launch_x_to_digits(ctx, x_dev, m, w->k_in, w->ggml_type, xd));
    pg_gemv_batch batch = {(int)m, nullptr, nullptr, nullptr, 1};
    return pg_launch_gguf_gemv(ctx, w->ggml_type, w->n_out, w->k_in, w->qs, w->d, batch, xd, y_dev);
}

PG_API pg_status pg_f16_to_f32(pg_ctx *ctx, const uint16_t *bits, size_t n, float *out) {
    PG_TRY(pg_use(ctx));
    if (n == 0) return PG_OK;
    PG_CHECK_ARG(bits && out, "pg_f16_to_f32: null pointer");
    pg_tmp din, dout;
    PG_TRY(din.alloc(n * 2));
    PG_TRY(dout.alloc(n * 4));
    PG_HIP(hipMemcpyAsync(din.p, bits, n * 2, hipMemcpyHostToDevice, ctx->stream));
    f16_to_f32_kernel<<<grid_for(n, 256), 256, 0, ctx->stream>>>(din.as<uint16_t>(), n, dout.as<uint32_t>());
    PG_TRY(pg_launch_check("f16_to_f32"));
    PG_HIP(hipMemcpyAsync(out, dout.p, n * 4, hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

static pg_status dequant_host(pg_ctx *ctx, const uint8_t *data, size_t num_elements, float *out,
                              int ggml_type, size_t block_bytes, const char *name) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(num_elements % 32 == 0, "%s: num_elements %zu is not a multiple of 32", name, num_elements);
    if (num_elements == 0) return PG_OK;
    PG_CHECK_ARG(data && out, "%s: null pointer", name);
    const size_t nblocks = num_elements / 32;
    pg_tmp din, dout;
    PG_TRY(din.alloc(nblocks * block_bytes));
    PG_TRY(dout.alloc(num_elements * sizeof(float)));
    PG_HIP(hipMemcpyAsync(din.p, data, nblocks * block_bytes, hipMemcpyHostToDevice, ctx->stream));
    const unsigned grid = grid_for(nblocks, 128);
    if (ggml_type == PG_GGML_Q8_0)
        dequant_q8_0_kernel<<<grid, 128, 0, ctx->stream>>>(din.as<uint8_t>(), nblocks, dout.as<float>());
    else if (ggml_type == PG_GGML_Q4_0)
        dequant_q4_0_kernel<<<grid, 128, 0, ctx->stream>>>(din.as<uint8_t>(), nblocks, dout.as<float>());
    else
        dequant_q4_1_kernel<<<grid, 128, 0, ctx->stream>>>(din.as<uint8_t>(), nblocks, dout.as<float>());
    PG_TRY(pg_launch_check(name));
    PG_HIP(hipMemcpyAsync(out, dout.p, num_elements * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

PG_API pg_status pg_dequant_q8_0(pg_ctx *ctx, const uint8_t *data, size_t num_elements, float *out) {
    return dequant_host(ctx, data, num_elements, out, PG_GGML_Q8_0, 34, "pg_dequant_q8_0");
}
PG_API pg_status pg_dequant_q4_0(pg_ctx *ctx, const uint8_t *data, size_t num_elements, float *out) {
    return dequant_host(ctx, data, num_elements, out, PG_GGML_Q4_0, 18, "pg_dequant_q4_0");
}
PG_API pg_status pg_dequant_q4_1(pg_ctx *ctx, const uint8_t *data, size_t num_elements, float *out) {
    return dequant_host(ctx, data, num_elements, out, PG_GGML_Q4_1, 20, "pg_dequant_q4_1");
}

PG_API pg_status pg_gguf_upload(pg_ctx *ctx, const void *blocks, int ggml_type, size_t n_out,
                                size_t k_in, pg_gguf_tensor **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(out != nullptr, "pg_gguf_upload: out is null");
    *out = nullptr;
    if (ggml_type == PG_GGML_Q4_1)
        return pg_fail(PG_EUNSUPPORTED, "pg_gguf_upload: Q4_1 has a dequantise kernel only");
    PG_CHECK_ARG(ggml_type == PG_GGML_Q4_0 || ggml_type == PG_GGML_Q8_0,
                 "pg_gguf_upload: ggml type %d is not a block-quantised type", ggml_type);
    PG_CHECK_ARG(n_out > 0 && k_in > 0 && blocks, "pg_gguf_upload: empty tensor or null pointer");
    PG_CHECK_ARG(k_in % 32 == 0, "pg_gguf_upload: k_in %zu is not a multiple of 32", k_in);
    PG_CHECK_ARG(n_out < (1ull << 31) && k_in < (1ull << 31) && n_out * (k_in / 32) < (1ull << 31),
                 "pg_gguf_upload: shape too large");
    const size_t nb = k_in / 32, nblocks = n_out * nb;
    const size_t bb = ggml_type == PG_GGML_Q4_0 ? 18 : 34, qb = bb - 2;
    pg_gguf_tensor *t = new (std::nothrow) pg_gguf_tensor();
    if (!t) return pg_fail(PG_ENOMEM, "host allocation failed");
    t->qs = nullptr;
    t->d = nullptr;
    t->ggml_type = ggml_type;
    t->n_out = n_out;
    t->k_in = k_in;
    pg_tmp raw;
    pg_status st = raw.alloc(nblocks * bb);
    hipError_t e = hipSuccess;
    if (st == PG_OK) {
        e = hipMalloc((void **)&t->qs, nblocks * qb);
        if (e == hipSuccess) e = hipMalloc((void **)&t->d, nblocks * sizeof(uint16_t));
        if (e == hipSuccess) e = hipMemcpyAsync(raw.p, blocks, nblocks * bb, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) {
            split_blocks_kernel<<<grid_for(nblocks, 256), 256, 0, ctx->stream>>>(raw.as<uint8_t>(), n_out, nb,
                                                                               ggml_type, t->qs, t->d);
            e = hipGetLastError();
        }
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess)
            st = pg_fail(e == hipErrorOutOfMemory ? PG_ENOMEM : PG_EDEVICE, "pg_gguf_upload: %s", hipGetErrorString(e));
    }
    if (st != PG_OK) { pg_gguf_free(ctx, t); return st; }
    *out = t;
    return PG_OK;
}

PG_API pg_status pg_gguf_shape(const pg_gguf_tensor *t, size_t *n_out, size_t *k_in, int *ggml_type) {
    PG_CHECK_ARG(t != nullptr, "pg_gguf_shape: null tensor");
    if (n_out) *n_out = t->n_out;
    if (k_in) *k_in = t->k_in;
    if (ggml_type) *ggml_type = t->ggml_type;
    return PG_OK;
}

PG_API void pg_gguf_free(pg_ctx *ctx, pg_gguf_tensor *t) {
    if (!t) return;
    if (ctx) {
        (void)hipSetDevice(ctx->device);
        (void)hipStreamSynchronize(ctx->stream);
    }
    if (t->qs) (void)hipFree(t->qs);
    if (t->d) (void)hipFree(t->d);
    delete t;
}

PG_API pg_status pg_gguf_matmul_dev(pg_ctx *ctx, const float *x_dev, size_t m,
                                    const pg_gguf_tensor *w, float *y_dev) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(w != nullptr, "pg_gguf_matmul: null weights");
    if (m == 0) return PG_OK;
    PG_CHECK_ARG(x_dev && y_dev, "pg_gguf_matmul: null pointer");
    PG_CHECK_ARG((uintptr_t)x_dev % 16 == 0, "pg_gguf_matmul: x must be 16-byte aligned");
    PG_CHECK_ARG(m < (1ull << 24), "pg_gguf_matmul: m = %zu too large", m);
    return pg_gguf_matmul_rows(ctx, x_dev, m, w, y_dev);
}

PG_API pg_status pg_gguf_matmul(pg_ctx *ctx, const float *x, size_t m, const pg_gguf_tensor *w,
                                float *y) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(w != nullptr, "pg_gguf_matmul: null weights");
    if (m == 0) return PG_OK;
    PG_CHECK_ARG(x && y, "pg_gguf_matmul: null pointer");
    pg_tmp dx, dy;
    PG_TRY(dx.alloc(m * w->k_in * sizeof(float)));
    PG_TRY(dy.alloc(m * w->n_out * sizeof(float)));
    PG_HIP(hipMemcpyAsync(dx.p, x, m * w->k_in * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_gguf_matmul_dev(ctx, dx.as<float>(), m, w, dy.as<float>()));
    PG_HIP(hipMemcpyAsync(y, dy.p, m * w->n_out * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}
