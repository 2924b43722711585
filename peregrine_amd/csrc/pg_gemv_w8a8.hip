// Decode-shaped W8A8 product (m <= 4 activation rows): a weight-streaming
// dot-product kernel.  HBM-bound: every weight byte is read exactly once with
// 128-bit loads, multiplied with v_dot4_i32_i8 against the quantised
// activation rows held in LDS, and reduced across the wavefront.
//
//   out[m, n] = (float)(sum_k a_i8[m, k] * w_t[n, k]) * a_scale[m] * w_scale[n]
//
// Integer sums are exact, so the lane/chunk order does not matter; the f32
// epilogue keeps the reference's multiplication order (src/quant.rs:163).
#include <limits.h>
#include "pg_internal.h"
#include "pg_quant_dev.h"
#include "pg_stream_addr.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int wave_sum_i32(int v) { return pg_wave_sum_i32(v); }

__device__ __forceinline__ int dot16(v4i w, v4i x, int acc) {
    acc = __builtin_amdgcn_sdot4(w.x, x.x, acc, false);
    acc = __builtin_amdgcn_sdot4(w.y, x.y, acc, false);
    acc = __builtin_amdgcn_sdot4(w.z, x.z, acc, false);
    acc = __builtin_amdgcn_sdot4(w.w, x.w, acc, false);
    return acc;
}

// One wavefront owns R consecutive weight rows (output columns); a workgroup is
// 4 wavefronts.  Lane l reads the 16-byte chunks l, l+64, ... of each row, so a
// wavefront load covers 1 KiB of contiguous weights.  w_t rows are padded to
// n_pad (a multiple of 4*R*gridDim granularity) and k_pad, so no load needs a
// bounds check; only the final store is masked by n.
template <int R, int M>
__global__ __launch_bounds__(256) void gemv_w8a8_kernel(
    const int8_t *__restrict__ w_t, int k_pad, const float *__restrict__ w_scales,
    const int8_t *__restrict__ a_i8, int a_stride, const float *__restrict__ a_scales, int n,
    float *__restrict__ out, int32_t *__restrict__ acc_out) {
    extern __shared__ v4i xs[];  // [M][k_pad / 16]
    const int nchunk = k_pad >> 4;
    for (int i = threadIdx.x; i < M * nchunk; i += 256) {
        const int m = i / nchunk, c = i - m * nchunk;
        xs[i] = reinterpret_cast<const v4i *>(a_i8 + (size_t)m * a_stride)[c];
    }
    __syncthreads();
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int row0 = (blockIdx.x * 4 + wave) * R;
    const v4i *wp = reinterpret_cast<const v4i *>(w_t + (size_t)row0 * k_pad);
    int acc[R][M];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[r][m] = 0;

#pragma unroll 2
    for (int c = lane; c < nchunk; c += 64) {
        v4i w[R];
#pragma unroll
        for (int r = 0; r < R; ++r) w[r] = __builtin_nontemporal_load(wp + (size_t)r * nchunk + c);
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const v4i x = xs[m * nchunk + c];
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r][m] = dot16(w[r], x, acc[r][m]);
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[r][m] = wave_sum_i32(acc[r][m]);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int col = row0 + r;
            if (col < n) {
                const float ws = w_scales[col];
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    if (out) out[(size_t)m * n + col] = (float)acc[r][m] * a_scales[m] * ws;
                    if (acc_out) acc_out[(size_t)m * n + col] = acc[r][m];
                }
            }
        }
    }
}


// M = 1 fast path for k_pad <= 16 KiB: no LDS and no barrier.  Each lane keeps its share of
// the quantised activation row (chunks lane, lane+64, ...) in registers; a wavefront walks
// RPW weight rows one after the other, so its loads are long contiguous runs (measured: 4 rows
// interleaved in one loop stream at 4.7 TB/s, one row at a time at 6.0 TB/s).
template <int NCH, int RPW>
__global__ __launch_bounds__(256) void gemv_w8a8_m1_kernel(
    const int8_t *__restrict__ w_t, int k_pad, const float *__restrict__ w_scales,
    const int8_t *__restrict__ a_i8, const float *__restrict__ a_scales, int n,
    float *__restrict__ out, int32_t *__restrict__ acc_out) {
    const int nchunk = k_pad >> 4;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int row0 = pg_m1_row0(blockIdx.x, wave, 4, RPW);
    const v4i *xp = reinterpret_cast<const v4i *>(a_i8);
    v4i x[NCH];
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        const int c = lane + 64 * j;
        x[j] = (c < nchunk) ? xp[c] : (v4i){0, 0, 0, 0};
    }
    const float a_scale = a_scales[0];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const int row = row0 + r;  // < n_pad by construction of the grid
        const v4i *wp = reinterpret_cast<const v4i *>(w_t + (size_t)row * k_pad);
        v4i w[NCH];
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            w[j] = __builtin_nontemporal_load(wp + pg_m1_weight_chunk(lane, j, nchunk));  // (past a short row: its first chunk, against zeros)
        }
        int acc = 0;
#pragma unroll
        for (int j = 0; j < NCH; ++j) acc = dot16(w[j], x[j], acc);  // x is zero beyond nchunk
        acc = wave_sum_i32(acc);
        if (lane == 0 && row < n) {
            if (out) out[row] = (float)acc * a_scale * w_scales[row];
            if (acc_out) acc_out[row] = acc;
        }
    }
}

// The same with the activation row still in f32 (quant::quantize_activations for one row,
// src/quant.rs:79-112, folded in): the workgroup requests its first weight rows, then finds the
// row's absmax, rounds the row to i8 into LDS with the arithmetic of quantize_rows_vec4_kernel
// (same scale, same reciprocal, same rounding: bit-identical integers), and every lane takes its
// chunks from there.  One launch per product instead of two: the separate one-row quantisation
// kernel costs about 4 us, as much as a third of the product itself.  k % 4 == 0.
// Up to PG_GEMM_MAX_GROUP weights of equal K against the same row in one launch (the reference's
// fused gate|up and q|k|v products at one token): weight g owns the workgroups wg0[g] .. wg0[g+1]-1
// (unused slots hold INT_MAX).  One weight is a group of one.
struct gemv_wgroup {
    const int8_t *w[PG_GEMM_MAX_GROUP];
    const float *ws[PG_GEMM_MAX_GROUP];
    float *out[PG_GEMM_MAX_GROUP];
    int n[PG_GEMM_MAX_GROUP];
    int wg0[PG_GEMM_MAX_GROUP];
};

// NW wavefronts per workgroup share one quantisation of the row: every workgroup repeats that
// arithmetic (about 14 vector instructions per element), so a long row is spread over more
// threads (K = 14336 on 256 threads is 56 elements each and 512 such workgroups: the vector
// units, not the weight stream, then set the pace; on 1024 threads it is 14 each and 256
// workgroups).
template <int NCH, int RPW, int NW>
__global__ __launch_bounds__(64 * NW) void gemv_w8a8_m1_f32x_kernel(
    const gemv_wgroup grp, int k_pad, const float *__restrict__ x_f32, int k, int32_t *__restrict__ acc_out) {
    constexpr int NT = 64 * NW, NV = (NCH * 256 + NT - 1) / NT;  // float4 of the row per thread
    __shared__ int xq[NCH * 256];  // the quantised row, zero beyond k: NCH KiB >= k_pad bytes
    __shared__ float red[NW];
    int g = 0;
#pragma unroll
    for (int i = 1; i < PG_GEMM_MAX_GROUP; ++i) g = (int)blockIdx.x >= grp.wg0[i] ? i : g;
    const int8_t *__restrict__ w_t = grp.w[g];
    const float *__restrict__ w_scales = grp.ws[g];
    float *__restrict__ out = grp.out[g];
    const int n = grp.n[g];
    const int nchunk = k_pad >> 4;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int row0 = pg_m1_row0((int)blockIdx.x - grp.wg0[g], wave, NW, RPW);
    auto load_row = [&](int row, v4i (&w)[NCH]) {
        const v4i *wp = reinterpret_cast<const v4i *>(w_t + (size_t)row * k_pad);
#pragma unroll
        for (int j = 0; j < NCH; ++j)
            w[j] = __builtin_nontemporal_load(wp + pg_m1_weight_chunk(lane, j, nchunk));  // (past a short row: its first chunk, against zeros)
    };
    // Loads return in issue order: the activation row (from L2) is requested first, so that its
    // quantisation can start as soon as it is there; every weight row of this wavefront (from HBM)
    // right behind it, all in flight together.
    const int nvec = k >> 2;
    const float4 *x4 = reinterpret_cast<const float4 *>(x_f32);
    float4 v[NV];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        v[i] = x4[pg_m1_x_vec(threadIdx.x, i, NT, nvec)];
    }
    v4i w[RPW][NCH];
#pragma unroll
    for (int r = 0; r < RPW; ++r) load_row(row0 + r, w[r]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int idx = threadIdx.x + NT * i;
        const float m4 = fmaxf(fmaxf(fabsf(v[i].x), fabsf(v[i].y)), fmaxf(fabsf(v[i].z), fabsf(v[i].w)));
        amax = fmaxf(amax, idx < nvec ? m4 : 0.0f);
    }
    // maximum over the workgroup; the barriers wait for LDS only (not __syncthreads(): that would
    // also wait for every weight row in flight)
    amax = pg_wave_max_f32(amax);
    if (lane == 0) red[wave] = amax;
    asm volatile("s_waitcnt lgkmcnt(0)\n s_barrier" ::: "memory");
    amax = red[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) amax = fmaxf(amax, red[i]);
    const float a_scale = (amax == 0.0f) ? 1.0f : amax / 127.0f;
    const float inv_scale = 1.0f / a_scale;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int idx = threadIdx.x + NT * i;
        const int b0 = pg_quant_to_i8(v[i].x * inv_scale) & 0xFF;
        const int b1 = pg_quant_to_i8(v[i].y * inv_scale) & 0xFF;
        const int b2 = pg_quant_to_i8(v[i].z * inv_scale) & 0xFF;
        const int b3 = pg_quant_to_i8(v[i].w * inv_scale) & 0xFF;
        if (NV * NT == NCH * 256 || idx < NCH * 256) xq[idx] = idx < nvec ? (b0 | (b1 << 8) | (b2 << 16) | (b3 << 24)) : 0;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n s_barrier" ::: "memory");
    int acc[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) acc[r] = 0;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        const v4i x = reinterpret_cast<const v4i *>(xq)[lane + 64 * j];  // zero beyond k
#pragma unroll
        for (int r = 0; r < RPW; ++r) acc[r] = dot16(w[r][j], x, acc[r]);
    }
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const int row = row0 + r;  // < n_pad by construction of the grid
        const int sum = wave_sum_i32(acc[r]);
        if (lane == 0 && row < n) {
            if (out) out[row] = (float)sum * a_scale * w_scales[row];
            if (acc_out) acc_out[row] = sum;
        }
    }
}

template <int NCH, int RPW, int NW>
pg_status launch_m1_f32x(pg_ctx *ctx, const float *x_f32, size_t k, const pg_qtensor *const *w, float *const *out, int count,
                         int32_t *acc) {
    gemv_wgroup grp;
    int wgs = 0;
    for (int i = 0; i < PG_GEMM_MAX_GROUP; ++i) {
        const bool used = i < count;
        grp.w[i] = used ? w[i]->w_t : nullptr;
        grp.ws[i] = used ? w[i]->scales : nullptr;
        grp.out[i] = used && out ? out[i] : nullptr;
        grp.n[i] = used ? (int)w[i]->cols : 0;
        grp.wg0[i] = used ? wgs : INT_MAX;
        if (used) wgs += (int)(w[i]->n_pad / (NW * RPW));  // n_pad is a multiple of 256
    }
    PG_TRY(pg_launch(ctx, "gemv_w8a8", gemv_w8a8_m1_f32x_kernel<NCH, RPW, NW>, dim3((unsigned)wgs), dim3(64 * NW), 0, grp,
                     (int)w[0]->k_pad, x_f32, (int)k, acc));
    return pg_launch_check("gemv_w8a8_m1_f32x");
}

// Wavefronts per workgroup by row length (16 elements of the row per thread or fewer); two weight
// rows per wavefront where that still leaves eight wavefronts per CU and the registers allow it
// (sixteen wavefronts per workgroup have 128 registers each: one row of up to 16 KiB in flight).
template <int NCH>
pg_status launch_m1_f32x_rows(pg_ctx *ctx, const float *x_f32, size_t k, const pg_qtensor *const *w, float *const *out, int count,
                              int32_t *acc) {
    size_t rows = 0;
    for (int i = 0; i < count; ++i) rows += w[i]->n_pad;
    if (ctx->gemv_force_nw) {  // pg_gemv_w8a8_force_shape: a test or a sweep names the instantiation
        const int nw = ctx->gemv_force_nw, rpw = ctx->gemv_force_rpw;
        if (nw == 4 && rpw == 1) return launch_m1_f32x<NCH, 1, 4>(ctx, x_f32, k, w, out, count, acc);
        if (nw == 4 && rpw == 2) return launch_m1_f32x<NCH, 2, 4>(ctx, x_f32, k, w, out, count, acc);
        if (nw == 8 && rpw == 1) return launch_m1_f32x<NCH, 1, 8>(ctx, x_f32, k, w, out, count, acc);
        if (nw == 8 && rpw == 2) return launch_m1_f32x<NCH, 2, 8>(ctx, x_f32, k, w, out, count, acc);
        if (nw == 16 && rpw == 1) return launch_m1_f32x<NCH, 1, 16>(ctx, x_f32, k, w, out, count, acc);
        return pg_fail(PG_EINVAL, "gemv_w8a8: no instantiation with %d wavefronts x %d rows", nw, rpw);
    }
    constexpr int NW = NCH <= 4 ? 4 : (NCH <= 8 ? 8 : 16);
    if constexpr (NW < 16) {
        if (rows / 2 >= (size_t)ctx->num_cu * 8) return launch_m1_f32x<NCH, 2, NW>(ctx, x_f32, k, w, out, count, acc);
    }
    return launch_m1_f32x<NCH, 1, NW>(ctx, x_f32, k, w, out, count, acc);
}

template <int NCH, int RPW>
pg_status launch_m1(pg_ctx *ctx, const int8_t *a_i8, const float *a_scales, const pg_qtensor *w,
                    float *out, int32_t *acc) {
    const unsigned grid = (unsigned)(w->n_pad / (4 * RPW));
    PG_TRY(pg_launch(ctx, "gemv_w8a8", gemv_w8a8_m1_kernel<NCH, RPW>, dim3(grid), dim3(256), 0, w->w_t,
                     (int)w->k_pad, w->scales, a_i8, a_scales, (int)w->cols, out, acc));
    return pg_launch_check("gemv_w8a8_m1");
}

template <int NCH>
pg_status launch_m1_rows(pg_ctx *ctx, const int8_t *a_i8, const float *a_scales, const pg_qtensor *w,
                         float *out, int32_t *acc) {
    // keep at least ~8 wavefronts per CU
    if (w->n_pad / 2 >= (size_t)ctx->num_cu * 8) return launch_m1<NCH, 2>(ctx, a_i8, a_scales, w, out, acc);
    return launch_m1<NCH, 1>(ctx, a_i8, a_scales, w, out, acc);
}

template <int R, int M>
pg_status launch(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                 const pg_qtensor *w, float *out, int32_t *acc) {
    const size_t lds = (size_t)M * w->k_pad;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)gemv_w8a8_kernel<R, M>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return pg_fail(PG_EDEVICE, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    }
    const unsigned grid = (unsigned)(w->n_pad / (4 * R));
    PG_TRY(pg_launch(ctx, "gemv_w8a8", gemv_w8a8_kernel<R, M>, dim3(grid), dim3(256), lds, w->w_t, (int)w->k_pad,
                     w->scales, a_i8, (int)a_stride, a_scales, (int)w->cols, out, acc));
    return pg_launch_check("gemv_w8a8");
}

template <int M>
pg_status launch_m(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                   const pg_qtensor *w, float *out, int32_t *acc) {
    // Aim for >= 8 wavefronts per CU: fewer rows per wavefront when the matrix is narrow.
    const size_t want_waves = (size_t)ctx->num_cu * 8;
    if (w->n_pad / 4 >= want_waves) return launch<4, M>(ctx, a_i8, a_stride, a_scales, w, out, acc);
    if (w->n_pad / 2 >= want_waves) return launch<2, M>(ctx, a_i8, a_stride, a_scales, w, out, acc);
    return launch<1, M>(ctx, a_i8, a_stride, a_scales, w, out, acc);
}

}  // namespace

bool pg_gemv_w8a8_takes_f32_row(const pg_qtensor *w, size_t m, size_t k, const float *x_f32) {
    return m == 1 && w->k_pad <= 16384 && k % 4 == 0 && k > 0 && (uintptr_t)x_f32 % 16 == 0;  // 128-bit loads of the row
}

pg_status pg_launch_gemv_w8a8_f32_row_group(pg_ctx *ctx, const float *x_f32, size_t k, const pg_qtensor *const *w,
                                            float *const *out, int count, int32_t *acc) {
    if (count < 1 || count > PG_GEMM_MAX_GROUP) return pg_fail(PG_EINVAL, "gemv_w8a8: %d weights in one launch (1 .. %d)", count, PG_GEMM_MAX_GROUP);
    for (int i = 1; i < count; ++i)
        if (w[i]->k_pad != w[0]->k_pad) return pg_fail(PG_EINVAL, "gemv_w8a8: the weights of one launch differ in K");
    const size_t nch = (w[0]->k_pad / 16 + 63) / 64;
    if (nch <= 4) return launch_m1_f32x_rows<4>(ctx, x_f32, k, w, out, count, acc);
    if (nch <= 8) return launch_m1_f32x_rows<8>(ctx, x_f32, k, w, out, count, acc);
    if (nch <= 14) return launch_m1_f32x_rows<14>(ctx, x_f32, k, w, out, count, acc);
    return launch_m1_f32x_rows<16>(ctx, x_f32, k, w, out, count, acc);
}

pg_status pg_launch_gemv_w8a8_f32_row(pg_ctx *ctx, const float *x_f32, size_t k, const pg_qtensor *w, float *out,
                                      int32_t *acc) {
    return pg_launch_gemv_w8a8_f32_row_group(ctx, x_f32, k, &w, &out, 1, acc);
}

pg_status pg_launch_gemv_w8a8(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride,
                              const float *a_scales, const pg_qtensor *w, size_t m, float *out,
                              int32_t *acc) {
    if ((size_t)m * w->k_pad > 150 * 1024)
        return pg_launch_gemm_w8a8(ctx, a_i8, a_stride, a_scales, w, m, out, acc);
    if (m == 1 && w->k_pad <= 16384) {
        const size_t nch = (w->k_pad / 16 + 63) / 64;
        if (nch <= 4) return launch_m1_rows<4>(ctx, a_i8, a_scales, w, out, acc);
        if (nch <= 8) return launch_m1_rows<8>(ctx, a_i8, a_scales, w, out, acc);
        if (nch <= 14) return launch_m1_rows<14>(ctx, a_i8, a_scales, w, out, acc);
        return launch_m1_rows<16>(ctx, a_i8, a_scales, w, out, acc);
    }
    switch (m) {
        case 1: return launch_m<1>(ctx, a_i8, a_stride, a_scales, w, out, acc);
        case 2: return launch_m<2>(ctx, a_i8, a_stride, a_scales, w, out, acc);
        case 3: return launch_m<3>(ctx, a_i8, a_stride, a_scales, w, out, acc);
        case 4: return launch_m<4>(ctx, a_i8, a_stride, a_scales, w, out, acc);
        default: return pg_launch_gemm_w8a8(ctx, a_i8, a_stride, a_scales, w, m, out, acc);
    }
}
