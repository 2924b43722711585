// Ceilings of the part, measured with small kernels so that a roofline fraction can be read
// against what the hardware delivers under the same conditions (clocks under load, real HBM
// efficiency) as well as against the published peaks:
//   * int8 matrix-core rate with every operand in registers (no LDS, no memory),
//   * a pure 128-bit read stream over buffers larger than the last-level cache,
//   * the shader clock seen inside a W8A8 GEMM tile (pg_probe_gemm_clock, in pg_gemm_w8a8.hip).
#include "pg_internal.h"
#include "pg_stream_addr.h"

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

// Every workgroup streams a contiguous slice of `total` 16-byte chunks with 128-bit non-temporal loads, U in flight
// per lane (a lane past the end of the slice loads nothing); the sum is stored only if it has an impossible value
// (keeps the loads alive).
template <int U>
__global__ __launch_bounds__(1024) void probe_read_kernel(const v4i *__restrict__ src, size_t chunks_per_wg, size_t total, int *__restrict__ out) {
    const size_t first = (size_t)blockIdx.x * chunks_per_wg;
    const size_t n = first >= total ? 0 : (total - first < chunks_per_wg ? total - first : chunks_per_wg);
    const v4i *p = src + first;
    v4i s = {0, 0, 0, 0};
    for (size_t c = threadIdx.x; c < n; c += (size_t)U * blockDim.x) {
        v4i v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const size_t i = pg_probe_chunk(c, u, blockDim.x);
            v[u] = v4i{0, 0, 0, 0};
            if (i < n) v[u] = __builtin_nontemporal_load(p + i);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) s += v[u];
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

PG_API pg_status pg_probe_hbm_read_shaped(pg_ctx *ctx, size_t bytes_per_pass, int buffers, int passes, int workgroups,
                                          int threads, int loads_in_flight, double *gbs) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(bytes_per_pass >= (1u << 20) && bytes_per_pass <= (1ull << 32), "pg_probe_hbm_read: %zu bytes per pass (1 MiB .. 4 GiB)", bytes_per_pass);
    PG_CHECK_ARG(buffers >= 1 && buffers <= 64 && passes >= 1 && passes <= 4096, "pg_probe_hbm_read: buffers %d, passes %d", buffers, passes);
    PG_CHECK_ARG(workgroups >= 1 && workgroups <= 65536 && (threads == 256 || threads == 512 || threads == 1024) &&
                     (loads_in_flight == 4 || loads_in_flight == 8 || loads_in_flight == 16),
                 "pg_probe_hbm_read: %d workgroups of %d threads, %d loads in flight (256 | 512 | 1024 threads; 4 | 8 | 16 loads)", workgroups, threads, loads_in_flight);
    const size_t total = bytes_per_pass / 16, wgs = (size_t)workgroups;
    const size_t chunks_per_wg = (total + wgs - 1) / wgs;
    const size_t pass_bytes = total * 16;
    pg_tmp buf, out;
    PG_TRY(buf.alloc(pass_bytes * buffers));
    PG_TRY(out.alloc(256));
    PG_TRY(pg_probe_fill_random(ctx, buf.p, pass_bytes * buffers));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    PG_HIP(hipEventCreate(&e0));
    if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); return pg_fail(PG_EDEVICE, "hipEventCreate failed"); }
    auto run = [&](int n) {
        for (int i = 0; i < n; ++i) {
            const v4i *src = reinterpret_cast<const v4i *>(buf.as<char>() + (size_t)(i % buffers) * pass_bytes);
            if (loads_in_flight == 4) probe_read_kernel<4><<<dim3((unsigned)wgs), dim3(threads), 0, ctx->stream>>>(src, chunks_per_wg, total, out.as<int>());
            else if (loads_in_flight == 8) probe_read_kernel<8><<<dim3((unsigned)wgs), dim3(threads), 0, ctx->stream>>>(src, chunks_per_wg, total, out.as<int>());
            else probe_read_kernel<16><<<dim3((unsigned)wgs), dim3(threads), 0, ctx->stream>>>(src, chunks_per_wg, total, out.as<int>());
        }
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

// The default shape: eight workgroups of 256 threads per CU, eight loads in flight per lane.
PG_API pg_status pg_probe_hbm_read(pg_ctx *ctx, size_t bytes_per_pass, int buffers, int passes, double *gbs) {
    PG_TRY(pg_use(ctx));
    return pg_probe_hbm_read_shaped(ctx, bytes_per_pass, buffers, passes, ctx->num_cu * 8, 256, 8, gbs);
}
