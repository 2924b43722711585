// Ceilings of the part, measured with small kernels so that a roofline fraction can be read
// against what the hardware delivers under the same conditions (clocks under load, real HBM
// efficiency) as well as against the published peaks:
//   * int8 matrix-core rate with every operand in registers (no LDS, no memory),
//   * a pure 128-bit read stream over buffers larger than the last-level cache,
//   * the shader clock seen inside a W8A8 GEMM tile (pg_probe_gemm_clock, in pg_gemm_w8a8.hip).
#include "pg_internal.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// 8 wavefronts per workgroup, 2 x 4 accumulator tiles of 32x32 per wavefront: the register
// shape of the 256x256 GEMM tile.  clk_out[2 * wg] = shader cycles, [2 * wg + 1] = wall ticks.
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void probe_mfma_i8_kernel(int iters, const v4i *__restrict__ in, int *__restrict__ out, long long *__restrict__ clk_out) {
    v4i a[2], b[4];
#pragma unroll
    for (int i = 0; i < 2; ++i) a[i] = in[threadIdx.x + i * 512];
#pragma unroll
    for (int j = 0; j < 4; ++j) b[j] = in[threadIdx.x + (2 + j) * 512];
    v16i acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0);
        asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));  // keep the loop
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    int s = 0;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) s += acc[i][j][r];
    out[blockIdx.x * 512 + threadIdx.x] = s;
    if (threadIdx.x == 0) {
        clk_out[2 * blockIdx.x] = c1 - c0;
        clk_out[2 * blockIdx.x + 1] = w1 - w0;
    }
}

// Every workgroup streams a contiguous slice with 128-bit non-temporal loads, eight in flight
// per lane; the sum is stored only if it has an impossible value (keeps the loads alive).
__global__ __launch_bounds__(256) void probe_read_kernel(const v4i *__restrict__ src, size_t chunks_per_wg, int *__restrict__ out) {
    const v4i *p = src + (size_t)blockIdx.x * chunks_per_wg;
    v4i s = {0, 0, 0, 0};
    for (size_t c = threadIdx.x; c < chunks_per_wg; c += 8 * 256) {
        v4i v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const size_t i = c + (size_t)u * 256;
            v[u] = __builtin_nontemporal_load(p + (i < chunks_per_wg ? i : c));
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
    }
    if (s.x == 0x12345678 && s.y == 0x0BADF00D) out[0] = s.z + s.w;
}

// Pseudo-random bytes (an integer hash of the word index): matrix-core power, and with it the
// clock the part sustains, depends on how many operand bits toggle, so the probes do not run
// on constant data.
__global__ void probe_fill_kernel(uint32_t *__restrict__ p, size_t words) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= words) return;
    uint32_t x = (uint32_t)i * 0x9E3779B9u + 0x7F4A7C15u;
    x ^= x >> 16; x *= 0x85EBCA6Bu; x ^= x >> 13; x *= 0xC2B2AE35u; x ^= x >> 16;
    p[i] = x;
}

}  // namespace

pg_status pg_probe_fill_random(pg_ctx *ctx, void *dev, size_t bytes) {
    const size_t words = bytes / 4;
    if (!words) return PG_OK;
    probe_fill_kernel<<<dim3((unsigned)((words + 255) / 256)), dim3(256), 0, ctx->stream>>>(static_cast<uint32_t *>(dev), words);
    return pg_launch_check("probe_fill");
}

PG_API pg_status pg_probe_mfma_i8(pg_ctx *ctx, int iters, double *tops, double *clock_ghz) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(iters >= 1 && iters <= (1 << 20), "pg_probe_mfma_i8: iters %d", iters);
    const int wgs = ctx->num_cu;  // one workgroup of 8 wavefronts per CU: two per SIMD
    pg_tmp in, out, clk;
    PG_TRY(in.alloc(6 * 512 * sizeof(v4i)));
    PG_TRY(out.alloc((size_t)wgs * 512 * sizeof(int)));
    PG_TRY(clk.alloc((size_t)wgs * 2 * sizeof(long long)));
    PG_TRY(pg_probe_fill_random(ctx, in.p, 6 * 512 * sizeof(v4i)));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    PG_HIP(hipEventCreate(&e0));
    if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); return pg_fail(PG_EDEVICE, "hipEventCreate failed"); }
    pg_status st = PG_OK;
    float ms = 0.0f;
    for (int rep = 0; rep < 3 && st == PG_OK; ++rep) {  // the last repetition is the one reported
        hipError_t e = hipEventRecord(e0, ctx->stream);
        if (e == hipSuccess) {
            probe_mfma_i8_kernel<<<dim3(wgs), dim3(512), 0, ctx->stream>>>(iters, in.as<v4i>(), out.as<int>(), clk.as<long long>());
            e = hipGetLastError();
        }
        if (e == hipSuccess) e = hipEventRecord(e1, ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
        if (e != hipSuccess) st = pg_fail(PG_EDEVICE, "pg_probe_mfma_i8: %s", hipGetErrorString(e));
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    PG_TRY(st);
    std::vector<long long> h((size_t)wgs * 2);
    PG_HIP(hipMemcpy(h.data(), clk.p, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
    int wall_khz = 0;
    PG_HIP(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, ctx->device));
    double cyc = 0.0, wall = 0.0;
    for (int i = 0; i < wgs; ++i) { cyc += (double)h[2 * i]; wall += (double)h[2 * i + 1]; }
    // 8 wavefronts x 8 MFMAs x 32*32*32 multiply-adds x 2 ops per workgroup and iteration
    if (tops) *tops = (double)wgs * 8.0 * 8.0 * 65536.0 * iters / (ms * 1e-3) / 1e12;
    if (clock_ghz) *clock_ghz = wall > 0.0 && wall_khz > 0 ? cyc / (wall / (wall_khz * 1e3)) / 1e9 : 0.0;
    return PG_OK;
}

PG_API pg_status pg_probe_hbm_read(pg_ctx *ctx, size_t bytes_per_pass, int buffers, int passes, double *gbs) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(bytes_per_pass >= (1u << 20) && bytes_per_pass <= (1ull << 32), "pg_probe_hbm_read: %zu bytes per pass (1 MiB .. 4 GiB)", bytes_per_pass);
    PG_CHECK_ARG(buffers >= 1 && buffers <= 64 && passes >= 1 && passes <= 4096, "pg_probe_hbm_read: buffers %d, passes %d", buffers, passes);
    const size_t wgs = (size_t)ctx->num_cu * 8;
    const size_t chunks_per_wg = bytes_per_pass / 16 / wgs;
    const size_t pass_bytes = chunks_per_wg * wgs * 16;
    pg_tmp buf, out;
    PG_TRY(buf.alloc(pass_bytes * buffers));
    PG_TRY(out.alloc(256));
    PG_TRY(pg_probe_fill_random(ctx, buf.p, pass_bytes * buffers));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    PG_HIP(hipEventCreate(&e0));
    if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); return pg_fail(PG_EDEVICE, "hipEventCreate failed"); }
    auto run = [&](int n) {
        for (int i = 0; i < n; ++i)
            probe_read_kernel<<<dim3((unsigned)wgs), dim3(256), 0, ctx->stream>>>(
                reinterpret_cast<const v4i *>(buf.as<char>() + (size_t)(i % buffers) * pass_bytes), chunks_per_wg, out.as<int>());
    };
    run(buffers);  // warm-up: one pass over every buffer
    hipError_t e = hipEventRecord(e0, ctx->stream);
    run(passes);
    if (e == hipSuccess) e = hipGetLastError();
    if (e == hipSuccess) e = hipEventRecord(e1, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (e != hipSuccess) return pg_fail(PG_EDEVICE, "pg_probe_hbm_read: %s", hipGetErrorString(e));
    if (gbs) *gbs = (double)pass_bytes * passes / (ms * 1e-3) / 1e9;
    return PG_OK;
}
