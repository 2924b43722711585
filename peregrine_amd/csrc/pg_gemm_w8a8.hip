// Prefill-shaped W8A8 product on the CDNA4 matrix cores.
//
//   acc[m, n] = sum_k a_i8[m, k] * w_t[n, k]              (i32, exact)
//   out[m, n] = ((float)acc * a_scale[m]) * w_scale[n]    (src/quant.rs:163)
//
// Both operands are K-contiguous, which is the natural operand layout of
// v_mfma_i32_32x32x32_i8: lane l supplies 16 consecutive k-bytes of row l%32
// (half-wave l/32 takes the upper 16 of each 32-wide k step).  The same
// (lane, byte) -> k mapping is used for A and B, so the sum is over matching k.
//
// Workgroup = 4 wavefronts in a 2x2 grid over a BM x BN output tile; each
// wavefront holds (BM/64) x (BN/64) accumulator tiles of 32x32.  K is consumed
// in steps of 64 bytes through two LDS stages filled by direct global->LDS
// loads (global_load_lds_dwordx4), so the fill of stage s+1 overlaps the MFMAs
// on stage s and no VGPRs are spent on staging.  Rows are 64 B in LDS; the 16 B
// chunks of a row are XOR-swizzled so that the 128-bit fragment reads of 8 or
// 16 consecutive rows fall in distinct bank groups.
#include "pg_internal.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BK = 64;  // bytes of K per LDS stage

typedef const void __attribute__((address_space(1))) *gptr_t;
typedef void __attribute__((address_space(3))) *lptr_t;

__device__ __forceinline__ void load_to_lds_16(const int8_t *src, char *lds_wave_base) {
    // Each lane moves 16 bytes; lane i lands at lds_wave_base + 16*i.
    __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)lds_wave_base, 16, 0, 0);
}

template <int BM, int BN>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(BM * BN > 256 * 128 ? 1 : 2)))
void gemm_w8a8_kernel(
    const int8_t *__restrict__ A, int lda, const int8_t *__restrict__ Bw, int ldb,
    const float *__restrict__ a_scales, const float *__restrict__ w_scales,
    float *__restrict__ out, int32_t *__restrict__ acc_out, int M, int N, int K, int tiles_m,
    int ntiles) {
    constexpr int TM = BM / 64, TN = BN / 64;  // 32x32 MFMA tiles per wavefront
    constexpr int WM = BM / 2, WN = BN / 2;    // wavefront tile
    constexpr int STAGE = (BM + BN) * BK;      // bytes per LDS stage
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous
    // run of tiles (m fastest) so the tiles sharing an L2 also share A/B panels.
    const int chunk = (ntiles + 7) / 8;
    const int t = (blockIdx.x % 8) * chunk + blockIdx.x / 8;
    if (t >= ntiles) return;
    const int m0 = (t % tiles_m) * BM, n0 = (t / tiles_m) * BN;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // ---- global -> LDS mapping: wave-load j fills LDS slots [64j, 64j+64) of a
    // panel, i.e. rows 16j..16j+15; lane -> (row, physical chunk).
    const int r16 = lane >> 2, pc = lane & 3;
    const int ld_sw = ((r16 >> 1) + 2 * wave + (r16 >> 3)) & 3;  // swizzle of row 16*(wave+4i)+r16
    const int ld_c = pc ^ ld_sw;                                  // logical chunk this lane fetches
    const int8_t *a_src = A + (size_t)(m0 + 16 * wave + r16) * lda + 16 * ld_c;
    const int8_t *b_src = Bw + (size_t)(n0 + 16 * wave + r16) * ldb + 16 * ld_c;

    // ---- LDS fragment offsets (bytes) for k-step 0/1 of a stage.
    const int l31 = lane & 31, half = lane >> 5;
    const int fr_sw = ((l31 >> 1) + (l31 >> 3)) & 3;
    int a_off[2], b_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const int phys = ((2 * ks + half) ^ fr_sw) * 16;
        a_off[ks] = (wm * WM + l31) * BK + phys;
        b_off[ks] = BM * BK + (wn * WN + l31) * BK + phys;
    }

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    auto issue = [&](int stage, int k0) {
        char *base = lds + stage * STAGE;
#pragma unroll
        for (int i = 0; i < TM; ++i)
            load_to_lds_16(a_src + (size_t)(64 * i) * lda + k0, base + (wave + 4 * i) * 1024);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            load_to_lds_16(b_src + (size_t)(64 * j) * ldb + k0,
                           base + BM * BK + (wave + 4 * j) * 1024);
    };
    auto compute = [&](int stage) {
        const char *base = lds + stage * STAGE;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            v4i af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                af[i] = *reinterpret_cast<const v4i *>(base + a_off[ks] + i * 32 * BK);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                bf[j] = *reinterpret_cast<const v4i *>(base + b_off[ks] + j * 32 * BK);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
    };

    const int KT = K / BK;
    issue(0, 0);
    for (int kt = 0; kt < KT; kt += 2) {
        // stage 0 holds k-tile kt
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (kt + 1 < KT) issue(1, (kt + 1) * BK);
        compute(0);
        if (kt + 1 < KT) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (kt + 2 < KT) issue(0, (kt + 2) * BK);
            compute(1);
        }
    }

    // ---- epilogue.  Accumulator register r of a 32x32 tile holds
    // row 8*(r/4) + 4*(lane/32) + r%4, column lane%32.
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * WN + 32 * j + l31;
            if (n >= N) continue;
            const float ws = w_scales[n];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * WM + 32 * i + 8 * (r >> 2) + 4 * half + (r & 3);
                if (m < M) {
                    const int a = acc[i][j][r];
                    out[(size_t)m * N + n] = (float)a * a_scales[m] * ws;
                    if (acc_out) acc_out[(size_t)m * N + n] = a;
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // one tile's stores at a time: bounded live ranges
        }
    }
}

template <int BM, int BN>
pg_status launch(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                 const pg_qtensor *w, size_t m, float *out, int32_t *acc) {
    const int tiles_m = (int)((m + BM - 1) / BM);
    const int tiles_n = (int)((w->cols + BN - 1) / BN);
    const int ntiles = tiles_m * tiles_n;
    const size_t lds = 2 * (size_t)(BM + BN) * BK;
    static bool attr_done = false;  // per instantiation
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute((const void *)gemm_w8a8_kernel<BM, BN>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return pg_fail(PG_EDEVICE, "hipFuncSetAttribute: %s", hipGetErrorString(e));
        attr_done = true;
    }
    const unsigned grid = (unsigned)(((ntiles + 7) / 8) * 8);
    {
        pg_prof_scope ps(ctx, "gemm_w8a8");
        gemm_w8a8_kernel<BM, BN><<<grid, 256, lds, ctx->stream>>>(
            a_i8, (int)a_stride, w->w_t, (int)w->k_pad, a_scales, w->scales, out, acc, (int)m,
            (int)w->cols, (int)w->k_pad, tiles_m, ntiles);
    }
    return pg_launch_check("gemm_w8a8");
}

}  // namespace

// a_i8 must have at least round_up(m, 256) rows of a_stride bytes (rows >= m may
// hold anything: they only feed accumulators that are never stored), a_stride ==
// w->k_pad with the K padding zero-filled.
pg_status pg_launch_gemm_w8a8(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride,
                              const float *a_scales, const pg_qtensor *w, size_t m, float *out,
                              int32_t *acc) {
    if (a_stride != w->k_pad) return pg_fail(PG_EINVAL, "gemm_w8a8: activation stride %zu != k_pad %zu", a_stride, w->k_pad);
    if ((uint64_t)a_stride * pg_round_up(m, 256) >= (1ull << 31) || (uint64_t)w->k_pad * w->n_pad >= (1ull << 40))
        return pg_fail(PG_EUNSUPPORTED, "gemm_w8a8: operand too large");
    const size_t n = w->cols;
    const size_t cus = (size_t)ctx->num_cu;
    auto tiles = [&](size_t bm, size_t bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn); };
    if (m <= 64) return launch<64, 64>(ctx, a_i8, a_stride, a_scales, w, m, out, acc);
    // Largest tile that still gives every CU work.
    if (tiles(256, 128) >= cus) return launch<256, 128>(ctx, a_i8, a_stride, a_scales, w, m, out, acc);
    return launch<128, 128>(ctx, a_i8, a_stride, a_scales, w, m, out, acc);
}
