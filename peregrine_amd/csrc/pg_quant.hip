// quant::* entry points: weight / activation quantisation, dequantise, device
// residency of QuantizedTensor, and the W8A8 matmul dispatcher.
//
// Bit-exactness notes (all checked against the CPU oracle by the GPU tests):
//  - rounding is roundf (half away from zero), never rintf;
//  - weights divide by the scale (IEEE divide), activations multiply by the
//    reciprocal 1.0f/scale: two different roundings, kept as the reference has them;
//  - this file is compiled with -ffp-contract=off, f32 denormals stay enabled
//    and hipcc's default correctly-rounded f32 divide is relied on.
#include <new>
#include "pg_internal.h"
#include "pg_quant_dev.h"

namespace {

constexpr int QA_THREADS = 256;

__device__ __forceinline__ int quant_to_i8(float v) { return pg_quant_to_i8(v); }
__device__ __forceinline__ float wave_max(float v) { return pg_wave_max_f32(v); }
__device__ __forceinline__ float block_max_256(float v, float *red) { return pg_block_max_256(v, red); }

// One workgroup per row.  The row is read once into registers (up to
// 4*256*MAXV floats), reduced to its absmax, then rounded to i8 and written as
// packed dwords.  Columns [cols, q_stride) of the output row are zero-filled.
template <int MAXV>
__global__ __launch_bounds__(QA_THREADS) void quantize_rows_vec4_kernel(
    const float *__restrict__ a, size_t cols, int8_t *__restrict__ q, size_t q_stride,
    float *__restrict__ row_scales) {
    __shared__ float red[4];
    const size_t row = blockIdx.x;
    const float4 *ar = reinterpret_cast<const float4 *>(a + row * cols);
    const int nvec = (int)(cols >> 2);
    // Every load is issued before anything waits: vectors past the end of the row re-read
    // the last one (no branch between the loads) and are left out of the maximum.
    float4 v[MAXV];
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int idx = threadIdx.x + i * QA_THREADS;
        typedef float f4v __attribute__((ext_vector_type(4)));
        // (a plain load: the activations of a layer are read by several products in a row and
        // are usually still in the Infinity Cache; a non-temporal load would fetch them from HBM
        // every time)
        const f4v t = *(reinterpret_cast<const f4v *>(ar) + (idx < nvec ? idx : nvec - 1));
        v[i] = make_float4(t.x, t.y, t.z, t.w);
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int idx = threadIdx.x + i * QA_THREADS;
        const float m4 = fmaxf(fmaxf(fabsf(v[i].x), fabsf(v[i].y)), fmaxf(fabsf(v[i].z), fabsf(v[i].w)));
        amax = fmaxf(amax, idx < nvec ? m4 : 0.0f);
    }
    amax = block_max_256(amax, red);
    const float scale = (amax == 0.0f) ? 1.0f : amax / 127.0f;
    const float inv_scale = 1.0f / scale;
    if (threadIdx.x == 0) row_scales[row] = scale;
    int *qr = reinterpret_cast<int *>(q + row * q_stride);
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int idx = threadIdx.x + i * QA_THREADS;
        if (idx < nvec) {
            const int b0 = quant_to_i8(v[i].x * inv_scale) & 0xFF;
            const int b1 = quant_to_i8(v[i].y * inv_scale) & 0xFF;
            const int b2 = quant_to_i8(v[i].z * inv_scale) & 0xFF;
            const int b3 = quant_to_i8(v[i].w * inv_scale) & 0xFF;
            qr[idx] = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
        }
    }
    const int npad = (int)(q_stride >> 2);
    for (int idx = nvec + threadIdx.x; idx < npad; idx += QA_THREADS) qr[idx] = 0;
}

// Any shape: two passes over the row (the second one hits L2), scalar accesses.
__global__ __launch_bounds__(QA_THREADS) void quantize_rows_generic_kernel(
    const float *__restrict__ a, size_t cols, int8_t *__restrict__ q, size_t q_stride,
    float *__restrict__ row_scales) {
    __shared__ float red[4];
    const size_t row = blockIdx.x;
    const float *ar = a + row * cols;
    float amax = 0.0f;
    for (size_t k = threadIdx.x; k < cols; k += QA_THREADS) amax = fmaxf(amax, fabsf(ar[k]));
    amax = block_max_256(amax, red);
    const float scale = (amax == 0.0f) ? 1.0f : amax / 127.0f;
    const float inv_scale = 1.0f / scale;
    if (threadIdx.x == 0) row_scales[row] = scale;
    int8_t *qr = q + row * q_stride;
    for (size_t k = threadIdx.x; k < cols; k += QA_THREADS)
        qr[k] = (int8_t)quant_to_i8(ar[k] * inv_scale);
    for (size_t k = cols + threadIdx.x; k < q_stride; k += QA_THREADS) qr[k] = 0;
}

// ---- f32 rows as three signed byte digits ---------------------------------------------
// x[k] ~= s * X[k], X = 65536 d2 + 256 d1 + d0 with signed byte digits, |X| <= 8355711, s a power of two:
// 23 to 24 bits of fixed point per row, exact integer arithmetic on the matrix cores afterwards.
// planes[p][row][k] (p = 0: d0 .. 2: d2), rows of q_stride bytes, pad columns zero.
constexpr float DIG3_MAX = 8355711.0f;  // 127 * (65536 + 256 + 1)
__global__ __launch_bounds__(QA_THREADS) void rows_to_digits3_kernel(const float *__restrict__ a, size_t cols,
                                                                     int8_t *__restrict__ planes, size_t q_stride,
                                                                     size_t plane_bytes, float *__restrict__ row_scales) {
    __shared__ float red[4];
    const size_t row = blockIdx.x;
    const float *ar = a + row * cols;
    float amax = 0.0f;
    int bad = 0;
    for (size_t k = threadIdx.x; k < cols; k += QA_THREADS) {
        const float v = ar[k];
        amax = fmaxf(amax, fabsf(v));
        bad |= (v != v);
    }
    amax = block_max_256(amax, red);
    bad = __syncthreads_or(bad);
    const bool finite = !bad && amax <= 3.4028234663852886e38f;
    // power-of-two scale, so x -> X is exact whenever x has no bits below s
    // (integers stay integers), and s * X is exact again on the way back
    float s = 1.0f, inv = 1.0f;
    if (!finite) {
        s = __uint_as_float(0x7FC00000u);
        inv = 0.0f;
    } else if (amax > 0.0f) {
        int ex;
        (void)frexpf(amax, &ex);  // amax = f * 2^ex, f in [0.5, 1)
        int se = ex - 23;         // |x| / 2^se < 2^23 ...
        if (se < -126) se = -126;
        if (rintf(amax * ldexpf(1.0f, -se)) > DIG3_MAX) se += 1;  // ... but three signed bytes stop at 127 * 65793
        s = ldexpf(1.0f, se);
        inv = ldexpf(1.0f, -se);
    }
    if (threadIdx.x == 0) row_scales[row] = s;
    int8_t *p0 = planes + row * q_stride;
    for (size_t k = threadIdx.x; k < q_stride; k += QA_THREADS) {
        int X = 0;
        if (k < cols && finite) {
            const float t = fminf(fmaxf(rintf(ar[k] * inv), -DIG3_MAX), DIG3_MAX);
            X = (int)t;
        }
        const int d0 = ((X + 128) & 255) - 128;
        const int X1 = (X - d0) >> 8;
        const int d1 = ((X1 + 128) & 255) - 128;
        const int d2 = (X1 - d1) >> 8;
        p0[k] = (int8_t)d0;
        p0[plane_bytes + k] = (int8_t)d1;
        p0[2 * plane_bytes + k] = (int8_t)d2;
    }
}

// out[m, n] = (65536 I2 + 256 I1 + I0) * s[m] * w_scale[n], the integer exactly in f64.
__global__ void combine_digits3_kernel(const int32_t *__restrict__ acc, size_t plane_elems, const float *__restrict__ row_scales,
                                       const float *__restrict__ w_scales, size_t m, size_t n, float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= m * n) return;
    const size_t r = i / n, c = i - r * n;
    const double v = 65536.0 * (double)acc[2 * plane_elems + i] + 256.0 * (double)acc[plane_elems + i] + (double)acc[i];
    out[i] = (float)(v * (double)row_scales[r] * (double)w_scales[c]);
}

// ---- weight quantisation -----------------------------------------------------

__global__ void fill_u32_kernel(uint32_t *p, size_t n, uint32_t v) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// Per-column absmax with the reference's strict `>` (NaN never wins).  One
// thread per column, rows split over blockIdx.y; partial maxima are merged with
// an unsigned atomicMax on the bit pattern (order-independent for values >= 0).
constexpr int CM_ROWS_PER_BLOCK = 128;
__global__ __launch_bounds__(256) void col_absmax_kernel(const float *__restrict__ w, size_t rows,
                                                         size_t cols,
                                                         uint32_t *__restrict__ amax_bits) {
    const size_t n = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (n >= cols) return;
    const size_t r0 = (size_t)blockIdx.y * CM_ROWS_PER_BLOCK;
    const size_t r1 = r0 + CM_ROWS_PER_BLOCK < rows ? r0 + CM_ROWS_PER_BLOCK : rows;
    float cur = 0.0f;
    for (size_t r = r0; r < r1; ++r) {
        const float v = fabsf(w[r * cols + n]);
        if (v > cur) cur = v;
    }
    if (cur > 0.0f) atomicMax(amax_bits + n, __float_as_uint(cur));
}

__global__ void scales_from_amax_kernel(const uint32_t *__restrict__ amax_bits, size_t cols,
                                        size_t cols_pad, float *__restrict__ scales) {
    const size_t n = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= cols_pad) return;
    float s = 1.0f;
    if (n < cols) {
        const float amax = __uint_as_float(amax_bits[n]);
        s = (amax == 0.0f) ? 1.0f : amax / 127.0f;
    }
    scales[n] = s;
}

// 64x64 tile: q[k, n] = round(w[k, n] / scale[n]); optional dense q [rows, cols]
// and the K-contiguous transpose q_t[n * t_stride + k], staged through LDS so
// both global writes are row-contiguous.
__global__ __launch_bounds__(256) void quantize_weights_tile_kernel(
    const float *__restrict__ w, size_t rows, size_t cols, const float *__restrict__ scales,
    int8_t *__restrict__ q, int8_t *__restrict__ q_t, size_t t_stride) {
    __shared__ int8_t tile[64][65];
    const size_t k0 = (size_t)blockIdx.y * 64, n0 = (size_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // ty in 0..3
    const size_t n = n0 + tx;
    const float scale = (n < cols) ? scales[n] : 1.0f;
    for (int r = ty; r < 64; r += 4) {
        const size_t k = k0 + r;
        int8_t v = 0;
        if (k < rows && n < cols) {
            v = (int8_t)quant_to_i8(w[k * cols + n] / scale);
            if (q) q[k * cols + n] = v;
        }
        tile[r][tx] = v;
    }
    __syncthreads();
    if (q_t) {
        for (int c = ty; c < 64; c += 4) {
            const size_t nn = n0 + c, kk = k0 + tx;
            if (nn < cols && kk < rows) q_t[nn * t_stride + kk] = tile[tx][c];
        }
    }
}

// dst[c * dst_stride + r] = src[r * src_stride + c] for r < rows, c < cols.
__global__ __launch_bounds__(256) void transpose_i8_kernel(const int8_t *__restrict__ src,
                                                           size_t rows, size_t cols,
                                                           size_t src_stride,
                                                           int8_t *__restrict__ dst,
                                                           size_t dst_stride) {
    __shared__ int8_t tile[64][65];
    const size_t r0 = (size_t)blockIdx.y * 64, c0 = (size_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int r = ty; r < 64; r += 4)
        tile[r][tx] = (r0 + r < rows && c0 + tx < cols) ? src[(r0 + r) * src_stride + c0 + tx] : 0;
    __syncthreads();
    for (int c = ty; c < 64; c += 4)
        if (c0 + c < cols && r0 + tx < rows) dst[(c0 + c) * dst_stride + r0 + tx] = tile[tx][c];
}

__global__ void dequantize_kernel(const int8_t *__restrict__ q, const float *__restrict__ scales,
                                  size_t rows, size_t cols, float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * cols) return;
    out[i] = (float)q[i] * scales[i % cols];
}

inline unsigned grid_for(size_t n, unsigned block) { return (unsigned)((n + block - 1) / block); }

// amax -> scales, quantise, write q (optional) and q_t with the given stride.
pg_status quantize_weights_on_device(pg_ctx *ctx, const float *w_dev, size_t rows, size_t cols,
                                     int8_t *q_dev, int8_t *q_t_dev, size_t t_stride,
                                     float *scales_dev, size_t cols_pad) {
    pg_tmp amax;
    PG_TRY(amax.alloc(cols * sizeof(uint32_t)));
    fill_u32_kernel<<<grid_for(cols, 256), 256, 0, ctx->stream>>>(amax.as<uint32_t>(), cols, 0u);
    PG_TRY(pg_launch_check("fill_u32"));
    dim3 g1(grid_for(cols, 256), grid_for(rows, CM_ROWS_PER_BLOCK));
    col_absmax_kernel<<<g1, 256, 0, ctx->stream>>>(w_dev, rows, cols, amax.as<uint32_t>());
    PG_TRY(pg_launch_check("col_absmax"));
    scales_from_amax_kernel<<<grid_for(cols_pad, 256), 256, 0, ctx->stream>>>(
        amax.as<uint32_t>(), cols, cols_pad, scales_dev);
    PG_TRY(pg_launch_check("scales_from_amax"));
    dim3 g2(grid_for(cols, 64), grid_for(rows, 64));
    quantize_weights_tile_kernel<<<g2, 256, 0, ctx->stream>>>(w_dev, rows, cols, scales_dev, q_dev,
                                                              q_t_dev, t_stride);
    PG_TRY(pg_launch_check("quantize_weights_tile"));
    PG_HIP(hipStreamSynchronize(ctx->stream));  // amax is freed on return
    return PG_OK;
}

pg_status qtensor_alloc(pg_ctx *ctx, size_t rows, size_t cols, pg_qtensor **out) {
    pg_qtensor *t = new (std::nothrow) pg_qtensor();
    if (!t) return pg_fail(PG_ENOMEM, "host allocation failed");
    t->rows = rows;
    t->cols = cols;
    t->k_pad = pg_round_up(rows, PG_KPAD);
    t->n_pad = pg_round_up(cols, PG_NPAD);
    t->w_t = nullptr;
    t->scales = nullptr;
    const size_t bytes = t->k_pad * t->n_pad;
    hipError_t e = hipMalloc((void **)&t->w_t, bytes);
    if (e == hipSuccess) e = hipMalloc((void **)&t->scales, t->n_pad * sizeof(float));
    if (e == hipSuccess) e = hipMemsetAsync(t->w_t, 0, bytes, ctx->stream);
    if (e != hipSuccess) {
        if (t->w_t) (void)hipFree(t->w_t);
        if (t->scales) (void)hipFree(t->scales);
        delete t;
        return pg_fail(e == hipErrorOutOfMemory ? PG_ENOMEM : PG_EDEVICE,
                       "allocating a %zu x %zu quantised tensor failed: %s", rows, cols,
                       hipGetErrorString(e));
    }
    *out = t;
    return PG_OK;
}

}  // namespace

pg_status pg_launch_quantize_activations(pg_ctx *ctx, const float *a, size_t rows, size_t cols,
                                         int8_t *q, size_t q_stride, float *row_scales) {
    if (rows == 0) return PG_OK;
    const bool vec_ok = (cols % 4 == 0) && (q_stride % 4 == 0) &&
                        ((uintptr_t)a % 16 == 0) && ((uintptr_t)q % 4 == 0) && cols > 0;
    const size_t nvec = cols / 4;
    const dim3 grid((unsigned)rows);
#define PG_QROWS(V)                                                                                      \
    else if (vec_ok && nvec <= (V) * QA_THREADS)                                                         \
        PG_TRY(pg_launch(ctx, "quantize_rows", quantize_rows_vec4_kernel<V>, grid, dim3(QA_THREADS), 0, a, cols, q, \
                         q_stride, row_scales));
    if (cols == 0) PG_TRY(pg_launch(ctx, "quantize_rows", quantize_rows_generic_kernel, grid, dim3(QA_THREADS), 0, a, cols, q,
                                    q_stride, row_scales));
    PG_QROWS(2) PG_QROWS(4) PG_QROWS(6) PG_QROWS(8) PG_QROWS(11) PG_QROWS(14) PG_QROWS(16)
#undef PG_QROWS
    else
        PG_TRY(pg_launch(ctx, "quantize_rows", quantize_rows_generic_kernel, grid, dim3(QA_THREADS), 0, a, cols, q,
                         q_stride, row_scales));
    return pg_launch_check("quantize_rows");
}

PG_API pg_status pg_quantize_activations_dev(pg_ctx *ctx, const float *a_dev, size_t rows,
                                             size_t cols, int8_t *q_dev, float *row_scales_dev) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(rows == 0 || (a_dev && q_dev && row_scales_dev) || cols == 0,
                 "pg_quantize_activations_dev: null pointer");
    PG_CHECK_ARG(rows == 0 || (row_scales_dev != nullptr), "pg_quantize_activations_dev: null scales");
    PG_CHECK_ARG(rows < (1ull << 31), "pg_quantize_activations_dev: too many rows");
    return pg_launch_quantize_activations(ctx, a_dev, rows, cols, q_dev, cols, row_scales_dev);
}

PG_API pg_status pg_quantize_activations(pg_ctx *ctx, const float *a, size_t rows, size_t cols,
                                         int8_t *q, float *row_scales) {
    PG_TRY(pg_use(ctx));
    if (rows == 0) return PG_OK;
    PG_CHECK_ARG(row_scales && (cols == 0 || (a && q)), "pg_quantize_activations: null pointer");
    PG_CHECK_ARG(rows < (1ull << 31), "pg_quantize_activations: too many rows");
    const size_t n = rows * cols;
    pg_tmp da, dq, ds;
    PG_TRY(da.alloc(n * sizeof(float)));
    PG_TRY(dq.alloc(n));
    PG_TRY(ds.alloc(rows * sizeof(float)));
    if (n) PG_HIP(hipMemcpyAsync(da.p, a, n * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_launch_quantize_activations(ctx, da.as<float>(), rows, cols, dq.as<int8_t>(), cols,
                                          ds.as<float>()));
    if (n) PG_HIP(hipMemcpyAsync(q, dq.p, n, hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipMemcpyAsync(row_scales, ds.p, rows * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

PG_API pg_status pg_quantize_weights(pg_ctx *ctx, const float *w, size_t rows, size_t cols,
                                     int8_t *q, int8_t *q_t, float *scales) {
    PG_TRY(pg_use(ctx));
    const size_t n = rows * cols;
    if (cols == 0) return PG_OK;
    PG_CHECK_ARG(scales != nullptr, "pg_quantize_weights: scales is null");
    PG_CHECK_ARG(n == 0 || (w && q), "pg_quantize_weights: null pointer");
    pg_tmp dw, dq, dqt, ds;
    PG_TRY(dw.alloc(n * sizeof(float)));
    PG_TRY(dq.alloc(n));
    if (q_t) PG_TRY(dqt.alloc(n));
    PG_TRY(ds.alloc(cols * sizeof(float)));
    if (n) PG_HIP(hipMemcpyAsync(dw.p, w, n * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(quantize_weights_on_device(ctx, dw.as<float>(), rows, cols, dq.as<int8_t>(),
                                      q_t ? dqt.as<int8_t>() : nullptr, rows, ds.as<float>(), cols));
    if (n) PG_HIP(hipMemcpyAsync(q, dq.p, n, hipMemcpyDeviceToHost, ctx->stream));
    if (n && q_t) PG_HIP(hipMemcpyAsync(q_t, dqt.p, n, hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipMemcpyAsync(scales, ds.p, cols * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

PG_API pg_status pg_dequantize(pg_ctx *ctx, const int8_t *q, const float *scales, size_t rows,
                               size_t cols, float *out) {
    PG_TRY(pg_use(ctx));
    const size_t n = rows * cols;
    if (n == 0) return PG_OK;
    PG_CHECK_ARG(q && scales && out, "pg_dequantize: null pointer");
    pg_tmp dq, ds, dout;
    PG_TRY(dq.alloc(n));
    PG_TRY(ds.alloc(cols * sizeof(float)));
    PG_TRY(dout.alloc(n * sizeof(float)));
    PG_HIP(hipMemcpyAsync(dq.p, q, n, hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipMemcpyAsync(ds.p, scales, cols * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    dequantize_kernel<<<grid_for(n, 256), 256, 0, ctx->stream>>>(dq.as<int8_t>(), ds.as<float>(), rows,
                                                               cols, dout.as<float>());
    PG_TRY(pg_launch_check("dequantize"));
    PG_HIP(hipMemcpyAsync(out, dout.p, n * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

// A quantised weight from its row-major [rows, cols] integers already on the device.
pg_status pg_qtensor_from_device_q(pg_ctx *ctx, const int8_t *q_dev, const float *scales_host, size_t rows, size_t cols,
                                   pg_qtensor **out) {
    *out = nullptr;
    pg_qtensor *t = nullptr;
    PG_TRY(qtensor_alloc(ctx, rows, cols, &t));
    fill_u32_kernel<<<grid_for(t->n_pad, 256), 256, 0, ctx->stream>>>(reinterpret_cast<uint32_t *>(t->scales), t->n_pad,
                                                                    0x3F800000u);
    hipError_t e = hipMemcpyAsync(t->scales, scales_host, cols * sizeof(float), hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) {
        dim3 g(grid_for(cols, 64), grid_for(rows, 64));
        transpose_i8_kernel<<<g, 256, 0, ctx->stream>>>(q_dev, rows, cols, cols, t->w_t, t->k_pad);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        pg_qtensor_free(ctx, t);
        return pg_fail(PG_EDEVICE, "qtensor from device integers: %s", hipGetErrorString(e));
    }
    *out = t;
    return PG_OK;
}

PG_API pg_status pg_qtensor_upload(pg_ctx *ctx, const int8_t *q, const float *scales, size_t rows,
                                   size_t cols, pg_qtensor **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(out != nullptr, "pg_qtensor_upload: out is null");
    *out = nullptr;
    PG_CHECK_ARG(rows > 0 && cols > 0, "pg_qtensor_upload: empty tensor %zu x %zu", rows, cols);
    PG_CHECK_ARG(q && scales, "pg_qtensor_upload: null pointer");
    PG_CHECK_ARG(rows < (1ull << 31) && cols < (1ull << 31), "pg_qtensor_upload: shape too large");
    pg_tmp dq;
    PG_TRY(dq.alloc(rows * cols));
    PG_HIP(hipMemcpyAsync(dq.p, q, rows * cols, hipMemcpyHostToDevice, ctx->stream));
    return pg_qtensor_from_device_q(ctx, dq.as<int8_t>(), scales, rows, cols, out);
}

PG_API pg_status pg_qtensor_from_f32_dev(pg_ctx *ctx, const float *w_dev, size_t rows, size_t cols,
                                         pg_qtensor **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(out != nullptr, "pg_qtensor_from_f32: out is null");
    *out = nullptr;
    PG_CHECK_ARG(rows > 0 && cols > 0, "pg_qtensor_from_f32: empty tensor %zu x %zu", rows, cols);
    PG_CHECK_ARG(w_dev != nullptr, "pg_qtensor_from_f32: null pointer");
    PG_CHECK_ARG(rows < (1ull << 31) && cols < (1ull << 31), "pg_qtensor_from_f32: shape too large");
    pg_qtensor *t = nullptr;
    PG_TRY(qtensor_alloc(ctx, rows, cols, &t));
    pg_status st = quantize_weights_on_device(ctx, w_dev, rows, cols, nullptr, t->w_t, t->k_pad,
                                              t->scales, t->n_pad);
    if (st != PG_OK) { pg_qtensor_free(ctx, t); return st; }
    *out = t;
    return PG_OK;
}

PG_API pg_status pg_qtensor_from_f32(pg_ctx *ctx, const float *w, size_t rows, size_t cols,
                                     pg_qtensor **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(out != nullptr, "pg_qtensor_from_f32: out is null");
    *out = nullptr;
    PG_CHECK_ARG(rows > 0 && cols > 0 && w, "pg_qtensor_from_f32: empty tensor or null pointer");
    pg_tmp dw;
    PG_TRY(dw.alloc(rows * cols * sizeof(float)));
    PG_HIP(hipMemcpyAsync(dw.p, w, rows * cols * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    return pg_qtensor_from_f32_dev(ctx, dw.as<float>(), rows, cols, out);
}

PG_API pg_status pg_qtensor_download(pg_ctx *ctx, const pg_qtensor *t, int8_t *q, int8_t *q_t,
                                     float *scales) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(t != nullptr, "pg_qtensor_download: null tensor");
    const size_t rows = t->rows, cols = t->cols;
    if (q) {
        pg_tmp dq;
        PG_TRY(dq.alloc(rows * cols));
        dim3 g(grid_for(rows, 64), grid_for(cols, 64));
        // w_t is [cols, rows] with stride k_pad; transpose back to [rows, cols].
        transpose_i8_kernel<<<g, 256, 0, ctx->stream>>>(t->w_t, cols, rows, t->k_pad, dq.as<int8_t>(), cols);
        PG_TRY(pg_launch_check("transpose_i8"));
        PG_HIP(hipMemcpyAsync(q, dq.p, rows * cols, hipMemcpyDeviceToHost, ctx->stream));
        PG_HIP(hipStreamSynchronize(ctx->stream));
    }
    if (q_t)
        PG_HIP(hipMemcpy2DAsync(q_t, rows, t->w_t, t->k_pad, rows, cols, hipMemcpyDeviceToHost, ctx->stream));
    if (scales)
        PG_HIP(hipMemcpyAsync(scales, t->scales, cols * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

PG_API pg_status pg_qtensor_shape(const pg_qtensor *t, size_t *rows, size_t *cols) {
    PG_CHECK_ARG(t != nullptr, "pg_qtensor_shape: null tensor");
    if (rows) *rows = t->rows;
    if (cols) *cols = t->cols;
    return PG_OK;
}

PG_API void pg_qtensor_free(pg_ctx *ctx, pg_qtensor *t) {
    if (!t) return;
    if (ctx) {
        (void)hipSetDevice(ctx->device);
        (void)hipStreamSynchronize(ctx->stream);
    }
    if (t->w_t) (void)hipFree(t->w_t);
    if (t->scales) (void)hipFree(t->scales);
    delete t;
}

// ---- the W8A8 matmul -----------------------------------------------------------

// Rows of the quantised-activation scratch are padded to this many so the GEMM
// tiles never read past the arena.
// At or below this many activation rows the weight stream, not the matrix cores,
// bounds the product: use the dot-product GEMV kernel.
constexpr size_t PG_GEMV_MAX_M = 4;

// The product over device pointers.  Scratch (quantised rows, row scales, split-K partial planes)
// comes from the context's arena, or from `fixed` (of fixed_cap bytes) when that is given: then
// nothing is allocated and a request that does not fit is an error.
static pg_status matmul_quantized_on(pg_ctx *ctx, const float *a_dev, size_t m, size_t k, const pg_qtensor *w,
                                     float *out_dev, int32_t *acc_dev, void *fixed, size_t fixed_cap) {
    if (pg_gemv_w8a8_takes_f32_row(w, m, k, a_dev)) return pg_launch_gemv_w8a8_f32_row(ctx, a_dev, k, w, out_dev, acc_dev);
    const size_t m_pad = pg_round_up(m, PG_MPAD);
    const size_t a_bytes = m_pad * w->k_pad;
    // 5 .. 256 rows (batched decode, short prefill chunks): split-K product with i32 partial planes
    // behind the scales, where the unsplit tiles would leave most CUs idle
    // (up to 64 rows always; up to 256 only for long-K, narrow-N products like a down projection --
    // measured at 128 rows: 14336 -> 4096 35 -> 25 us split, but 4096 -> 4096 12.6 -> 19 us)
    int splits = 1;
    const bool skinny = pg_gemm_w8a8_takes_skinny(w, m);
    if (!skinny && m > PG_GEMV_MAX_M && (m <= 64 || (m <= 256 && w->k_pad >= 2 * w->cols)))
        PG_TRY(pg_launch_gemm_w8a8_few_rows(ctx, nullptr, w->k_pad, nullptr, w, m, nullptr, nullptr, nullptr, &splits));
    const size_t sz_scales = pg_round_up(m_pad * sizeof(float), 256);
    const size_t part_bytes = splits > 1 ? (size_t)splits * m * w->cols * sizeof(int32_t) : 0;
    const size_t need = a_bytes + sz_scales + part_bytes;
    void *ws = fixed;
    if (fixed) {
        if (need > fixed_cap)
            return pg_fail(PG_EINVAL, "this product needs %zu bytes of scratch (m = %zu, k = %zu, n = %zu); the fixed scratch holds %zu",
                           need, m, k, w->cols, fixed_cap);
    } else {
        PG_TRY(pg_workspace(ctx, need, &ws));
    }
    int8_t *a_i8 = static_cast<int8_t *>(ws);
    float *a_scales = reinterpret_cast<float *>(a_i8 + a_bytes);
    PG_TRY(pg_launch_quantize_activations(ctx, a_dev, m, k, a_i8, w->k_pad, a_scales));
    if (skinny) return pg_launch_gemm_w8a8_skinny(ctx, a_i8, w->k_pad, a_scales, w, m, out_dev, acc_dev);
    if (m <= PG_GEMV_MAX_M)
        return pg_launch_gemv_w8a8(ctx, a_i8, w->k_pad, a_scales, w, m, out_dev, acc_dev);
    if (splits > 1)
        return pg_launch_gemm_w8a8_few_rows(ctx, a_i8, w->k_pad, a_scales, w, m, out_dev, acc_dev,
                                            reinterpret_cast<int32_t *>(a_i8 + a_bytes + sz_scales), nullptr);
    return pg_launch_gemm_w8a8(ctx, a_i8, w->k_pad, a_scales, w, m, out_dev, acc_dev);
}

PG_API pg_status pg_matmul_quantized_dev(pg_ctx *ctx, const float *a_dev, size_t m, size_t k,
                                         const pg_qtensor *w, float *out_dev, int32_t *acc_dev) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(w != nullptr, "pg_matmul_quantized: null weights");
    PG_CHECK_ARG(w->rows == k, "pg_matmul_quantized: a has k = %zu but w has %zu rows", k, w->rows);
    if (m == 0) return PG_OK;
    PG_CHECK_ARG(a_dev && out_dev, "pg_matmul_quantized: null pointer");
    PG_CHECK_ARG(m < (1ull << 24), "pg_matmul_quantized: m = %zu too large", m);
    return matmul_quantized_on(ctx, a_dev, m, k, w, out_dev, acc_dev, nullptr, 0);
}

// ---- the same product for callers that cannot allocate ------------------------------------
// The scratch of pg_matmul_quantized_dev (quantised rows, row scales, split-K partial planes)
// lives in a file-scope device array instead of the context's growable arena.  Each GPU the
// library runs on holds its own copy of the array, at its own address, until the process ends;
// host code never passes the array's name to a kernel (on the host the name is only a stand-in
// for hipGetSymbolAddress), only the per-device address resolved below.
constexpr size_t PG_FIXED_SCRATCH_BYTES = 32u << 20;
static __device__ __align__(256) unsigned char scratch[PG_FIXED_SCRATCH_BYTES];
constexpr int PG_MAX_DEVICES = 64;
static void *g_fixed_scratch[PG_MAX_DEVICES];  // device address of `scratch` per device, null until resolved

// With ctx's device current: the address of this device's copy of the array.
static pg_status fixed_scratch_for(pg_ctx *ctx, void **out) {
    PG_CHECK_ARG(ctx->device >= 0 && ctx->device < PG_MAX_DEVICES, "device %d: the fixed scratch covers devices 0 .. %d", ctx->device,
                 PG_MAX_DEVICES - 1);
    void *p = g_fixed_scratch[ctx->device];
    if (!p) {
        PG_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return pg_fail(PG_EDEVICE, "hipGetSymbolAddress returned a null address for the fixed scratch");
        g_fixed_scratch[ctx->device] = p;
    }
    *out = p;
    return PG_OK;
}

PG_API pg_status pg_matmul_quantized_fixed_scratch_dev(pg_ctx *ctx, const float *a_dev, size_t m, size_t k,
                                                       const pg_qtensor *w, float *out_dev) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(w != nullptr, "pg_matmul_quantized_fixed_scratch: null weights");
    PG_CHECK_ARG(w->rows == k, "pg_matmul_quantized_fixed_scratch: a has k = %zu but w has %zu rows", k, w->rows);
    if (m == 0) return PG_OK;
    PG_CHECK_ARG(a_dev && out_dev, "pg_matmul_quantized_fixed_scratch: null pointer");
    PG_CHECK_ARG(m < (1ull << 24), "pg_matmul_quantized_fixed_scratch: m = %zu too large", m);
    void *fixed = nullptr;
    PG_TRY(fixed_scratch_for(ctx, &fixed));
    return matmul_quantized_on(ctx, a_dev, m, k, w, out_dev, nullptr, fixed, PG_FIXED_SCRATCH_BYTES);
}

PG_API size_t pg_fixed_scratch_bytes(void) { return PG_FIXED_SCRATCH_BYTES; }

// One activation matrix against several weights of equal K: the reference multiplies by
// column-concatenated weights (fuse_qkv src/models/llama/attention.rs:51-71, fuse_gate_up
// src/models/llama/decoder.rs:49-67) and slices the result; per-column weight scales and per-row
// activation scales make every output column independent of its neighbours, so the separate
// outputs here are bit for bit those of the single products.  The rows are quantised ONCE and,
// for more than 256 rows, the narrow products share one launch (the weights' column panels side
// by side in one tile space).
PG_API pg_status pg_matmul_quantized_multi_dev(pg_ctx *ctx, const float *a_dev, size_t m, size_t k,
                                               const pg_qtensor *const *w, size_t count, float *const *out_dev) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(count >= 1 && count <= (size_t)PG_GEMM_MAX_GROUP, "pg_matmul_quantized_multi: %zu weights (1 .. %d)", count,
                 PG_GEMM_MAX_GROUP);
    PG_CHECK_ARG(w != nullptr && out_dev != nullptr, "pg_matmul_quantized_multi: null table");
    for (size_t i = 0; i < count; ++i) {
        PG_CHECK_ARG(w[i] != nullptr, "pg_matmul_quantized_multi: weight %zu is null", i);
        PG_CHECK_ARG(w[i]->rows == k, "pg_matmul_quantized_multi: a has k = %zu but weight %zu has %zu rows", k, i, w[i]->rows);
        PG_CHECK_ARG(m == 0 || out_dev[i] != nullptr, "pg_matmul_quantized_multi: output %zu is null", i);
    }
    if (m == 0) return PG_OK;
    PG_CHECK_ARG(a_dev != nullptr, "pg_matmul_quantized_multi: null pointer");
    PG_CHECK_ARG(m < (1ull << 24), "pg_matmul_quantized_multi: m = %zu too large", m);
    bool one_row_group = m == 1 && count > 1;
    for (size_t i = 0; i < count && one_row_group; ++i) one_row_group = pg_gemv_w8a8_takes_f32_row(w[i], m, k, a_dev);
    if (one_row_group)  // one token: every weight's rows in one streaming launch that quantises the row itself
        return pg_launch_gemv_w8a8_f32_row_group(ctx, a_dev, k, w, out_dev, (int)count, nullptr);
    bool skinny_group = count > 1;
    for (size_t i = 0; i < count && skinny_group; ++i) skinny_group = pg_gemm_w8a8_takes_skinny(w[i], m) && w[i]->k_pad == w[0]->k_pad;
    if (skinny_group) {  // 2 .. 64 rows: quantised once, then the weights side by side in one launch
        const size_t k_pad = w[0]->k_pad, a_bytes = pg_round_up(m, PG_MPAD) * k_pad;
        void *ws = nullptr;
        PG_TRY(pg_workspace(ctx, a_bytes + pg_round_up(PG_MPAD * sizeof(float), 256), &ws));
        int8_t *a_i8 = static_cast<int8_t *>(ws);
        float *a_scales = reinterpret_cast<float *>(a_i8 + a_bytes);
        PG_TRY(pg_launch_quantize_activations(ctx, a_dev, m, k, a_i8, k_pad, a_scales));
        return pg_launch_gemm_w8a8_skinny_group(ctx, a_i8, k_pad, a_scales, w, out_dev, (int)count, m, nullptr);  // one launch for all
    }
    if (count == 1 || m <= 256) {  // few rows: the single products pick their own route (GEMV, split K)
        for (size_t i = 0; i < count; ++i) PG_TRY(pg_matmul_quantized_dev(ctx, a_dev, m, k, w[i], out_dev[i], nullptr));
        return PG_OK;
    }
    const size_t k_pad = w[0]->k_pad, m_pad = pg_round_up(m, PG_MPAD);
    const size_t a_bytes = m_pad * k_pad;
    void *ws = nullptr;
    PG_TRY(pg_workspace(ctx, a_bytes + pg_round_up(m_pad * sizeof(float), 256), &ws));
    int8_t *a_i8 = static_cast<int8_t *>(ws);
    float *a_scales = reinterpret_cast<float *>(a_i8 + a_bytes);
    PG_TRY(pg_launch_quantize_activations(ctx, a_dev, m, k, a_i8, k_pad, a_scales));
    // Weights that fill the chip with 256x256 tiles on their own run on their own (measured: gate and up
    // as two launches 2 x 112 us, as one launch of 896 tiles 242 us: the rounds that leave CUs idle run
    // faster); the narrow ones (q, k, v) share one launch, where k and v alone would leave most CUs idle.
    const pg_qtensor *small_w[PG_GEMM_MAX_GROUP];
    float *small_out[PG_GEMM_MAX_GROUP];
    int n_small = 0;
    for (size_t i = 0; i < count; ++i) {
        const size_t t256 = ((m + 255) / 256) * ((w[i]->cols + 255) / 256);
        if (t256 >= (size_t)ctx->num_cu) {
            PG_TRY(pg_launch_gemm_w8a8(ctx, a_i8, k_pad, a_scales, w[i], m, out_dev[i], nullptr));
        } else {
            small_w[n_small] = w[i];
            small_out[n_small++] = out_dev[i];
        }
    }
    if (n_small) PG_TRY(pg_launch_gemm_w8a8_group(ctx, a_i8, k_pad, a_scales, small_w, small_out, n_small, m));
    return PG_OK;
}

// Which tile the W8A8 matrix-core product last ran with on this context, and an override of the
// dispatcher's choice (0 = automatic; 1 = 64x64, 2 = 256x256, 3 = 128x256, 4 = 128x64,
// 5 = 128x128 output tiles).  For tests and tuning runs: every tile shape gives the same bits.
PG_API pg_status pg_gemm_w8a8_last_tile(const pg_ctx *ctx, int *bm, int *bn, int *k_splits) {
    PG_CHECK_ARG(ctx != nullptr, "null context");
    if (bm) *bm = ctx->gemm_last_bm;
    if (bn) *bn = ctx->gemm_last_bn;
    if (k_splits) *k_splits = ctx->gemm_last_splits;
    return PG_OK;
}

PG_API pg_status pg_gemm_w8a8_force_tile(pg_ctx *ctx, int tile) {
    PG_CHECK_ARG(ctx != nullptr, "null context");
    PG_CHECK_ARG(tile >= 0 && tile <= 5, "pg_gemm_w8a8_force_tile: tile %d (0 .. 5)", tile);
    ctx->gemm_force_tile = tile;
    return PG_OK;
}

PG_API pg_status pg_gemv_w8a8_force_shape(pg_ctx *ctx, int wavefronts, int rows_per_wavefront) {
    PG_CHECK_ARG(ctx != nullptr, "null context");
    PG_CHECK_ARG((wavefronts == 0 && rows_per_wavefront == 0) ||
                     ((wavefronts == 4 || wavefronts == 8 || wavefronts == 16) && (rows_per_wavefront == 1 || rows_per_wavefront == 2) &&
                      !(wavefronts == 16 && rows_per_wavefront == 2)),
                 "pg_gemv_w8a8_force_shape: %d wavefronts x %d rows (4 | 8 x 1 | 2, 16 x 1, or 0, 0 for automatic)", wavefronts, rows_per_wavefront);
    ctx->gemv_force_nw = wavefronts;
    ctx->gemv_force_rpw = rows_per_wavefront;
    return PG_OK;
}

// The reference's GPU numerics for the same call: f32 activations times dequantised weights,
// f32 accumulate (matmul_dequant_i8, src/metal/shaders.rs:2329-2375).  Here the activations
// become 23/24-bit fixed point per row (power-of-two scale) and the product runs three times on the int8 matrix
// cores (one pass per byte digit), exact in integers; the only roundings are the
// activation step (at most 2^-23 of the row's absmax, none for values that are multiples of the scale) and the final f64 -> f32.
PG_API pg_status pg_matmul_dequant_i8_dev(pg_ctx *ctx, const float *a_dev, size_t m, size_t k,
                                          const pg_qtensor *w, float *out_dev) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(w != nullptr, "pg_matmul_dequant_i8: null weights");
    PG_CHECK_ARG(w->rows == k, "pg_matmul_dequant_i8: a has k = %zu but w has %zu rows", k, w->rows);  // src/quant.rs:204
    if (m == 0) return PG_OK;
    PG_CHECK_ARG(a_dev && out_dev, "pg_matmul_dequant_i8: null pointer");
    PG_CHECK_ARG(m < (1ull << 24), "pg_matmul_dequant_i8: m = %zu too large", m);
    // a digit plane holds -128 .. 127 (the carry-free split yields -128), a weight -127 .. 127: 128 * 127 * k < 2^31
    PG_CHECK_ARG(k <= 132104, "pg_matmul_dequant_i8: k = %zu would overflow the i32 digit sums", k);
    const size_t m_pad = pg_round_up(m, PG_MPAD), n = w->cols;
    // With enough rows the two low digit planes run as ONE product over the planes stacked row-wise (they lie
    // back to back in the scratch, each m_pad rows; the accumulator planes are then m_pad rows apart) and
    // the third plane's product finishes the sum in its epilogue.
    const bool stacked = m >= 192;
    const size_t plane_bytes = m_pad * w->k_pad, plane_elems = (stacked ? m_pad : m) * n;
    // (the product's prologue reads a scale per stacked row, whether or not it writes f32: three planes' worth)
    const size_t sz_planes = pg_round_up(3 * plane_bytes, 256), sz_scales = pg_round_up(3 * m_pad * sizeof(float), 256);
    void *ws = nullptr;
    PG_TRY(pg_workspace(ctx, sz_planes + sz_scales + 3 * plane_elems * sizeof(int32_t), &ws));
    int8_t *planes = static_cast<int8_t *>(ws);
    float *row_scales = reinterpret_cast<float *>(planes + sz_planes);
    int32_t *acc = reinterpret_cast<int32_t *>(planes + sz_planes + sz_scales);
    PG_TRY(pg_launch(ctx, "rows_to_digits3", rows_to_digits3_kernel, dim3((unsigned)m), dim3(QA_THREADS), 0, a_dev, k, planes,
                     w->k_pad, plane_bytes, row_scales));
    if (stacked) {
        // the two low planes as one product, then the plane of weight 65536, whose epilogue joins the three
        // accumulators and scales them: no third accumulator plane and no combining launch
        PG_TRY(pg_launch_gemm_w8a8(ctx, planes, w->k_pad, row_scales, w, m_pad + m, nullptr, acc));
        return pg_launch_gemm_w8a8_combine(ctx, planes + 2 * plane_bytes, w->k_pad, row_scales, w, m, out_dev, acc, plane_elems);
    }
    for (int p = 0; p < 3; ++p) {
        if (m <= PG_GEMV_MAX_M)
            PG_TRY(pg_launch_gemv_w8a8(ctx, planes + p * plane_bytes, w->k_pad, row_scales, w, m, nullptr, acc + p * plane_elems));
        else
            PG_TRY(pg_launch_gemm_w8a8(ctx, planes + p * plane_bytes, w->k_pad, row_scales, w, m, nullptr, acc + p * plane_elems));
    }
    return pg_launch(ctx, "combine_digits3", combine_digits3_kernel, dim3(grid_for(plane_elems, 256)), dim3(256), 0, acc, plane_elems,
                     row_scales, w->scales, m, n, out_dev);
}

PG_API pg_status pg_matmul_dequant_i8(pg_ctx *ctx, const float *a, size_t m, size_t k, const pg_qtensor *w, float *out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(w != nullptr, "pg_matmul_dequant_i8: null weights");
    PG_CHECK_ARG(w->rows == k, "pg_matmul_dequant_i8: a has k = %zu but w has %zu rows", k, w->rows);
    if (m == 0) return PG_OK;
    PG_CHECK_ARG(a && out, "pg_matmul_dequant_i8: null pointer");
    pg_tmp da, dout;
    PG_TRY(da.alloc(m * k * sizeof(float)));
    PG_TRY(dout.alloc(m * w->cols * sizeof(float)));
    PG_HIP(hipMemcpyAsync(da.p, a, m * k * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_matmul_dequant_i8_dev(ctx, da.as<float>(), m, k, w, dout.as<float>()));
    PG_HIP(hipMemcpyAsync(out, dout.p, m * w->cols * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

PG_API pg_status pg_matmul_quantized(pg_ctx *ctx, const float *a, size_t m, size_t k,
                                     const pg_qtensor *w, float *out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(w != nullptr, "pg_matmul_quantized: null weights");
    PG_CHECK_ARG(w->rows == k, "pg_matmul_quantized: a has k = %zu but w has %zu rows", k, w->rows);
    if (m == 0) return PG_OK;
    PG_CHECK_ARG(a && out, "pg_matmul_quantized: null pointer");
    pg_tmp da, dout;
    PG_TRY(da.alloc(m * k * sizeof(float)));
    PG_TRY(dout.alloc(m * w->cols * sizeof(float)));
    PG_HIP(hipMemcpyAsync(da.p, a, m * k * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_matmul_quantized_dev(ctx, da.as<float>(), m, k, w, dout.as<float>(), nullptr));
    PG_HIP(hipMemcpyAsync(out, dout.p, m * w->cols * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}
