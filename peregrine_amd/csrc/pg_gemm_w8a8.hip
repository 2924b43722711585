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
// Workgroup = NWM x NWN wavefronts over a BM x BN output tile; each wavefront
// holds (BM/NWM/32) x (BN/NWN/32) accumulator tiles of 32x32.  K is consumed in
// steps of BK bytes through NST LDS stages filled by direct global->LDS loads
// (global_load_lds_dwordx4): no VGPRs are spent on staging and the fill of later
// stages overlaps the MFMAs on the current one.
//
// LDS layout: a stage holds the A panel [BM rows][BK bytes] then the B panel
// [BN rows][BK bytes]; the 16-byte chunks of a row are XOR-swizzled so that the
// 128-bit fragment reads of 8 or 16 consecutive rows fall in distinct bank groups
// (measured: 122 B/clk/CU with the swizzle, 32-63 B/clk without).
//
// Main loop: fragments are double-buffered in registers.  The ds_reads of k-step
// ks+1 are interleaved with the MFMAs of k-step ks (sched_group_barrier pins the
// order); at the last k-step of a stage half of the MFMAs are issued, then the
// wavefront waits for the next stage (s_waitcnt vmcnt + raw s_barrier: the fence
// of __syncthreads would drain every outstanding prefetch), refills the stage it
// just finished and reads the next stage's first fragments under the remaining
// MFMAs.
#include <limits.h>
#include "pg_internal.h"
#include "pg_stream_addr.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef const void __attribute__((address_space(1))) *gptr_t;
typedef void __attribute__((address_space(3))) *lptr_t;

__device__ __forceinline__ void load_to_lds_16(const int8_t *src, char *lds_wave_base) {
    // Each lane moves 16 bytes; lane i lands at lds_wave_base + 16*i.
    __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)lds_wave_base, 16, 0, 0);
}


// Swizzle of the 16-byte chunk index within a row of BK bytes.
template <int BK> __device__ __forceinline__ int swz(int r);
template <> __device__ __forceinline__ int swz<64>(int r) { return ((r >> 1) + (r >> 3)) & 3; }
template <> __device__ __forceinline__ int swz<128>(int r) { return ((r >> 1) & 7) ^ ((r & 1) << 2); }

// The weights of one launch: up to PG_GEMM_MAX_GROUP tensors of equal K whose column panels are
// laid end to end in the launch's tile space (weight g owns the n-panels panel0[g] .. panel0[g+1]-1;
// unused slots hold INT_MAX).  One weight is a group of one.
struct gemm_wgroup {
    const int8_t *w[PG_GEMM_MAX_GROUP];
    const float *ws[PG_GEMM_MAX_GROUP];
    float *out[PG_GEMM_MAX_GROUP];
    int n[PG_GEMM_MAX_GROUP];
    int panel0[PG_GEMM_MAX_GROUP];
    // The last pass of the W8A32 product (one weight): with `comb` the accumulator is the digit of weight 65536
    // and the output is (65536 acc + 256 comb[comb_plane + i] + comb[i]) * a_scale * w_scale, the integer exact
    // and the scaling done in f64 (what combine_digits3_kernel computes from three stored planes).
    const int32_t *comb;
    long long comb_plane;
};

// CLK (the clock probe only): thread 0 of every workgroup also stores the shader cycles and the
// wall-clock ticks its K loop took, clk[2 * blockIdx.x] and clk[2 * blockIdx.x + 1].
template <int BM, int BN, int BK, int NST, int NWM, int NWN, int OCC, bool CLK = false, bool COMB = false>
__global__ __launch_bounds__(64 * NWM * NWN) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void gemm_w8a8_kernel(const int8_t *__restrict__ A, int lda, const gemm_wgroup grp, int ldb,
                      const float *__restrict__ a_scales, int32_t *__restrict__ acc_out, int M, int K,
                      int tiles_m, int ntiles, int kt_per_split, long long *__restrict__ clk) {
    constexpr int NW = NWM * NWN;
    constexpr int WM = BM / NWM, WN = BN / NWN;      // wavefront tile
    constexpr int TM = WM / 32, TN = WN / 32;        // 32x32 MFMA tiles per wavefront
    constexpr int CPR = BK / 16, RPL = 64 / CPR;     // chunks per row, rows per wave-load
    constexpr int LA = BM / RPL / NW, LB = BN / RPL / NW, LPS = LA + LB;  // wave-loads per wave per stage
    constexpr int STAGE = (BM + BN) * BK;            // bytes per LDS stage
    constexpr int KS = BK / 32;                      // k-steps per stage
    constexpr int NF = TM + TN, NMFMA = TM * TN;
    static_assert(LA >= 1 && LB >= 1 && KS % 2 == 0 && BM <= 64 * NW && BN <= 64 * NW, "unsupported tile configuration");
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous
    // run of tiles (m fastest) so the tiles sharing an L2 also share A/B panels.
    const int chunk = (ntiles + 7) / 8;
    const int t = (blockIdx.x % 8) * chunk + blockIdx.x / 8;
    if (t >= ntiles) return;
    const int np = t / tiles_m;  // n-panel of the launch; which weight owns it (uniform: scalar code)
    int g = 0;
#pragma unroll
    for (int i = 1; i < PG_GEMM_MAX_GROUP; ++i) g = np >= grp.panel0[i] ? i : g;
    const int8_t *__restrict__ Bw = grp.w[g];
    const float *__restrict__ w_scales = grp.ws[g];
    float *__restrict__ out = grp.out[g];
    const int N = grp.n[g];
    const int m0 = (t % tiles_m) * BM, n0 = (np - grp.panel0[g]) * BN;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / NWN, wn = wave % NWN;

    // ---- global -> LDS: wave-load j fills LDS slots [64j, 64j+64) of a panel, i.e.
    // rows RPL*j .. RPL*j+RPL-1; lane -> (row, physical chunk) fetches the logical chunk.
    const int lr = lane / CPR, pc = lane % CPR;
    int a_goff[LA], b_goff[LB];
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        const int row = RPL * (wave + NW * i) + lr;
        a_goff[i] = row * lda + 16 * (pc ^ swz<BK>(row));
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int row = RPL * (wave + NW * i) + lr;
        b_goff[i] = row * ldb + 16 * (pc ^ swz<BK>(row));
    }
    // A split product (few activation rows): blockIdx.y owns kt_per_split k-tiles of BK bytes and
    // writes its i32 partial sums to plane blockIdx.y of acc_out.  Otherwise gridDim.y == 1.
    const int kt0_split = blockIdx.y * kt_per_split;
    const int8_t *a_base = A + (size_t)m0 * lda + (size_t)kt0_split * BK;
    const int8_t *b_base = Bw + (size_t)n0 * ldb + (size_t)kt0_split * BK;
    if (acc_out) acc_out += (size_t)blockIdx.y * M * N;

    // ---- LDS fragment offsets (bytes) for each k-step of a stage.
    const int l31 = lane & 31, half = lane >> 5;
    int a_off[KS], b_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int ra = wm * WM + l31, rb = wn * WN + l31;
        a_off[ks] = ra * BK + (((2 * ks + half) ^ swz<BK>(ra)) * 16);
        b_off[ks] = BM * BK + rb * BK + (((2 * ks + half) ^ swz<BK>(rb)) * 16);
    }

    // The scales of this tile's rows and columns go to LDS (behind the stages) now, so that
    // the epilogue does not start with dependent global round trips.
    float *lds_as = reinterpret_cast<float *>(lds + NST * STAGE), *lds_ws = lds_as + BM;
    {
        const int t = threadIdx.x;
        if (t < BM) lds_as[t] = a_scales[m0 + t < M ? m0 + t : M - 1];
        if (t < BN) lds_ws[t] = w_scales[n0 + t < N ? n0 + t : N - 1];
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
        for (int i = 0; i < LA; ++i) load_to_lds_16(a_base + a_goff[i] + k0, base + (wave + NW * i) * 1024);
#pragma unroll
        for (int i = 0; i < LB; ++i)
            load_to_lds_16(b_base + b_goff[i] + k0, base + BM * BK + (wave + NW * i) * 1024);
    };
    v4i fa[2][TM], fb[2][TN];
    auto read_frags = [&](int buf, int stage, int ks) {
        const char *base = lds + stage * STAGE;
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[buf][i] = *reinterpret_cast<const v4i *>(base + a_off[ks] + i * 32 * BK);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[buf][j] = *reinterpret_cast<const v4i *>(base + b_off[ks] + j * 32 * BK);
    };
    auto mfmas = [&](int buf, int lo, int hi) {  // MFMAs lo..hi-1 of the TM x TN set, row-major
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                if (i * TN + j >= lo && i * TN + j < hi)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[buf][i], fb[buf][j], acc[i][j], 0, 0, 0);
    };
    // Before the barrier: this wavefront's LDS reads have returned (lgkmcnt) and all but
    // `ahead` of its youngest stage fills have landed (vmcnt).  After it, every wavefront's
    // share of the awaited stage is in LDS and the stage just consumed may be refilled.
    auto wait_barrier = [&](int ahead) {
#define PG_WB(N) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n s_barrier" ::"n"((N) * LPS > 63 ? 63 : (N) * LPS) : "memory")
        switch (ahead) {
            case 1: PG_WB(1); break;
            case 2: PG_WB(2); break;
            case 3: PG_WB(3); break;
            case 4: PG_WB(4); break;
            default: asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n s_barrier" ::: "memory"); break;
        }
#undef PG_WB
    };
    static_assert(NST >= 2 && NST <= 6, "wait_barrier covers up to 4 stages in flight beyond the awaited one");

    const int KT = (K / BK - kt0_split < kt_per_split) ? K / BK - kt0_split : kt_per_split;
    long long clk_c0 = 0, clk_w0 = 0;
    if constexpr (CLK) { clk_c0 = clock64(); clk_w0 = wall_clock64(); }
#pragma unroll
    for (int s = 0; s < NST - 1; ++s)
        if (s < KT) issue(s, s * BK);
    wait_barrier(KT - 1 < NST - 2 ? KT - 1 : NST - 2);
    if (NST - 1 < KT) issue(NST - 1, (NST - 1) * BK);
    read_frags(0, 0, 0);
    for (int kt0 = 0; kt0 < KT; kt0 += NST) {
#pragma unroll
        for (int s = 0; s < NST; ++s) {
            const int kt = kt0 + s;
            if (kt < KT) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const int cur = ks & 1, nxt = cur ^ 1;
                    if (ks + 1 < KS) {
                        read_frags(nxt, s, ks + 1);
                        mfmas(cur, 0, NMFMA);
                        if (NMFMA >= NF) {
#pragma unroll
                            for (int q = 0; q < NF; ++q) {
                                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
                                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
                            }
                            __builtin_amdgcn_sched_group_barrier(0x008, NMFMA - NF, 0);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    } else {
                        mfmas(cur, 0, NMFMA / 2);
                        __builtin_amdgcn_sched_barrier(0);
                        if (kt + 1 < KT) {
                            const int rem = KT - 2 - kt;  // stage fills younger than tile kt+1
                            wait_barrier(rem < NST - 2 ? rem : NST - 2);
                            if (kt + NST < KT) issue(s, (kt + NST) * BK);
                            read_frags(nxt, (s + 1) % NST, 0);
                        }
                        mfmas(cur, NMFMA / 2, NMFMA);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }
    }

    if constexpr (CLK) {
        if (threadIdx.x == 0) {
            clk[2 * blockIdx.x] = clock64() - clk_c0;
            clk[2 * blockIdx.x + 1] = wall_clock64() - clk_w0;
        }
    }
    // ---- epilogue.  Accumulator register r of a 32x32 tile holds
    // row 8*(r/4) + 4*(lane/32) + r%4, column lane%32.  (The scales were requested before the
    // K loop: loading them here would put several dependent memory round trips on every tile.)
    if (!COMB && out && !acc_out && m0 + BM <= M && n0 + BN <= N) {
        // A whole tile inside the matrix, f32 output only (every tile of the prefill shapes):
        // straight-line code, the 16 row scales of a 32-row tile as four 128-bit LDS reads.
        // The stores are non-temporal: this kernel never reads the output back, and 117 MB of
        // it per launch otherwise displace the operands of this and the next launch from L2
        // and the Infinity Cache (whole prefill layer 0.633 -> 0.59 ms).  The same hint on the
        // operand fills costs 7 - 15 %.
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            float as[16];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 v = *reinterpret_cast<const float4 *>(lds_as + wm * WM + 32 * i + 8 * g + 4 * half);
                as[4 * g] = v.x; as[4 * g + 1] = v.y; as[4 * g + 2] = v.z; as[4 * g + 3] = v.w;
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const float ws = lds_ws[wn * WN + 32 * j + l31];
                float *dst = out + (size_t)(m0 + wm * WM + 32 * i + 4 * half) * N + (n0 + wn * WN + 32 * j + l31);
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    __builtin_nontemporal_store((float)acc[i][j][r] * as[r] * ws, dst + (size_t)(8 * (r >> 2) + (r & 3)) * N);
                __builtin_amdgcn_sched_barrier(0);  // one tile's stores at a time: bounded live ranges
            }
        }
        return;
    }
    if (COMB && out && !acc_out && m0 + BM <= M && n0 + BN <= N) {
        // The W8A32 product's last pass on a whole tile: the two other digits' accumulators are fetched in the
        // order the stores go out (a lane's rows of one column, four at a time).
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            float as[16];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 v = *reinterpret_cast<const float4 *>(lds_as + wm * WM + 32 * i + 8 * g + 4 * half);
                as[4 * g] = v.x; as[4 * g + 1] = v.y; as[4 * g + 2] = v.z; as[4 * g + 3] = v.w;
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const double ws = (double)lds_ws[wn * WN + 32 * j + l31];
                const size_t base = (size_t)(m0 + wm * WM + 32 * i + 4 * half) * N + (n0 + wn * WN + 32 * j + l31);
#pragma unroll
                for (int r0 = 0; r0 < 16; r0 += 4) {  // four rows at a time (the 256x256 tile has no registers to spare)
                    int c0[4], c1[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const size_t idx = base + (size_t)(8 * ((r0 + r) >> 2) + ((r0 + r) & 3)) * N;
                        c0[r] = __builtin_nontemporal_load(grp.comb + idx);
                        c1[r] = __builtin_nontemporal_load(grp.comb + grp.comb_plane + idx);
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const double v = 65536.0 * (double)acc[i][j][r0 + r] + 256.0 * (double)c1[r] + (double)c0[r];
                        __builtin_nontemporal_store((float)(v * (double)as[r0 + r] * ws),
                                                    out + base + (size_t)(8 * ((r0 + r) >> 2) + ((r0 + r) & 3)) * N);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                __builtin_amdgcn_sched_barrier(0);  // one tile at a time: bounded live ranges
            }
        }
        return;
    }
    if (acc_out && !out && m0 + BM <= M && n0 + BN <= N) {  // the same for the integer-only output of the W8A32 passes
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                int32_t *dst = acc_out + (size_t)(m0 + wm * WM + 32 * i + 4 * half) * N + (n0 + wn * WN + 32 * j + l31);
#pragma unroll
                for (int r = 0; r < 16; ++r) __builtin_nontemporal_store(acc[i][j][r], dst + (size_t)(8 * (r >> 2) + (r & 3)) * N);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * WN + 32 * j + l31;
            if (n < N) {
                const float ws = lds_ws[wn * WN + 32 * j + l31];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = m0 + wm * WM + 32 * i + 8 * (r >> 2) + 4 * half + (r & 3);
                    if (m < M) {
                        const int a = acc[i][j][r];
                        const float as = lds_as[wm * WM + 32 * i + 8 * (r >> 2) + 4 * half + (r & 3)];
                        if (COMB && out) {
                            const size_t idx = (size_t)m * N + n;
                            const double v = 65536.0 * (double)a + 256.0 * (double)grp.comb[grp.comb_plane + idx] + (double)grp.comb[idx];
                            out[idx] = (float)(v * (double)as * (double)ws);
                        } else if (out) {
                            out[(size_t)m * N + n] = (float)a * as * ws;
                        }
                        if (acc_out) acc_out[(size_t)m * N + n] = a;
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // one tile's stores at a time: bounded live ranges
        }
    }
}

template <int BM, int BN, int BK, int NST, int NWM, int NWN, int OCC, bool COMB = false>
pg_status launch_group(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                       const pg_qtensor *const *w, float *const *out, int count, size_t m, int32_t *acc,
                       int splits = 1, int kt_per_split = 0, const int32_t *comb = nullptr, size_t comb_plane = 0) {
    const int tiles_m = (int)((m + BM - 1) / BM);
    gemm_wgroup grp;
    int panels = 0;
    for (int i = 0; i < PG_GEMM_MAX_GROUP; ++i) {
        const bool used = i < count;
        grp.w[i] = used ? w[i]->w_t : nullptr;
        grp.ws[i] = used ? w[i]->scales : nullptr;
        grp.out[i] = used && out ? out[i] : nullptr;
        grp.n[i] = used ? (int)w[i]->cols : 0;
        grp.panel0[i] = used ? panels : INT_MAX;
        if (used) panels += (int)((w[i]->cols + BN - 1) / BN);
    }
    grp.comb = comb;
    grp.comb_plane = (long long)comb_plane;
    const int ntiles = tiles_m * panels;
    const size_t lds = (size_t)NST * (BM + BN) * BK + (BM + BN) * sizeof(float);
    auto kern = gemm_w8a8_kernel<BM, BN, BK, NST, NWM, NWN, OCC, false, COMB>;
    PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));
    const unsigned grid = (unsigned)(((ntiles + 7) / 8) * 8);
    const size_t k_pad = w[0]->k_pad;
    if (splits == 1) kt_per_split = (int)(k_pad / BK);
    ctx->gemm_last_bm = BM;
    ctx->gemm_last_bn = BN;
    ctx->gemm_last_splits = splits;
    PG_TRY(pg_launch(ctx, "gemm_w8a8", kern, dim3(grid, (unsigned)splits), dim3(64 * NWM * NWN), lds, a_i8, (int)a_stride, grp,
                     (int)k_pad, a_scales, acc, (int)m, (int)k_pad, tiles_m, ntiles, kt_per_split, (long long *)nullptr));
    return pg_launch_check("gemm_w8a8");
}

template <int BM, int BN, int BK, int NST, int NWM, int NWN, int OCC>
pg_status launch(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                 const pg_qtensor *w, size_t m, float *out, int32_t *acc, int splits = 1, int kt_per_split = 0) {
    return launch_group<BM, BN, BK, NST, NWM, NWN, OCC>(ctx, a_i8, a_stride, a_scales, &w, &out, 1, m, acc, splits,
                                                        kt_per_split);
}

// out[m, n] = (float)(sum over the K splits of part[s][m, n]) * a_scale[m] * w_scale[n]: the integer sum is
// exact and order-free, the f32 epilogue is the one of the unsplit product (src/quant.rs:163).
__global__ __launch_bounds__(256) void splitk_finish_kernel(const int32_t *__restrict__ part, int splits, size_t plane,
                                                             const float *__restrict__ a_scales,
                                                             const float *__restrict__ w_scales, int n,
                                                             float *__restrict__ out, int32_t *__restrict__ acc_out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= plane) return;
    int acc = 0, s = 0;
    for (; s + 8 <= splits; s += 8) {  // eight independent loads in flight
        int v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(part + (size_t)(s + u) * plane + i);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; s < splits; ++s) acc += __builtin_nontemporal_load(part + (size_t)s * plane + i);
    const size_t r = i / n, c = i - r * n;
    if (out) out[i] = (float)acc * a_scales[r] * w_scales[c];
    if (acc_out) acc_out[i] = acc;
}

// ---- 2 .. 64 activation rows: one pass over the weights, no K split between workgroups -------------
// A workgroup owns 16 weight rows (output columns) and all of K: its NW wavefronts take one K run each and add
// their 16 x 16 i32 tiles through LDS at the end, so nothing is left for a second launch.  Operands of
// v_mfma_i32_16x16x64_i8 want lane -> (row lane % 16, 16 k at lane / 16): loaded that way from row-major memory,
// one instruction touches 64 cache lines a quarter at a time and the CU's vector cache, not HBM, sets the pace
// (19 us for 58.7 MB).  So every wavefront keeps a ring of its own in LDS, filled by direct global -> LDS loads in
// units of 128 k: one instruction brings 8 rows x 128 B (whole lines), chunk position p of row r holding the row's
// 16-byte chunk p ^ ((r >> 1) & 7), so that the fragment reads (16 rows, one chunk) fall into 16 different bank
// groups.  A unit of the ring holds the weight tile and MB tiles of quantised activation rows (from L2); NST - 1
// units are in flight while one is consumed.  No barrier in the loop: a wavefront reads only what it has loaded
// itself.  (The activations in fragment order straight into registers, with a deeper ring for the weights alone,
// measured slower: 13.0 against 11.8 us.)
// Every weight row is k_pad bytes from the next, so workgroups that all walked K from the start of their runs would
// ask the same memory channels at the same time: each starts at its own unit and wraps round its run (integer
// sums do not depend on the order).  The epilogue is the reference's (acc as f32) * a_scale[m] * w_scale[n]
// (src/quant.rs:163).  a_i8 has at least 16 MB rows of a_stride bytes (rows >= m feed accumulators never stored).
// NB: tiles of 16 weight rows per workgroup (2 for more than 16 activation rows: every activation fragment then
// meets two weight tiles, which halves what the CUs pull from L2).
// Up to PG_GEMM_MAX_GROUP weights of equal K in one launch (the fused q|k|v and gate|up products of models::llama):
// weight g owns the workgroups wg0[g] .. wg0[g + 1] - 1 (unused slots hold INT_MAX).
struct skinny_wgroup {
    const int8_t *w[PG_GEMM_MAX_GROUP];
    const float *ws[PG_GEMM_MAX_GROUP];
    float *out[PG_GEMM_MAX_GROUP];
    int n[PG_GEMM_MAX_GROUP];
    int wg0[PG_GEMM_MAX_GROUP];
};

template <int MB, int NB, int NW, int NST>
__global__ __launch_bounds__(64 * NW) void gemm_w8a8_skinny_kernel(const int8_t *__restrict__ a_i8, const skinny_wgroup grp,
                                                                    int k_pad, int m, const float *__restrict__ a_scales,
                                                                    int32_t *__restrict__ acc_out) {
    int g = 0;
#pragma unroll
    for (int i = 1; i < PG_GEMM_MAX_GROUP; ++i) g = (int)blockIdx.x >= grp.wg0[i] ? i : g;
    const int8_t *__restrict__ w_t = grp.w[g];
    const float *__restrict__ w_scales = grp.ws[g];
    float *__restrict__ out = grp.out[g];
    const int n = grp.n[g];
    constexpr int TILE = 2048, UNIT = (NB + MB) * TILE, LPS = 2 * (NB + MB);  // bytes per tile and unit; fills per unit
    static_assert((NST - 1) * LPS < 64 && NST <= 6, "the wait counter holds 63");
    extern __shared__ __attribute__((aligned(1024))) char lds[];  // NW rings of NST units; afterwards the wavefronts' tiles
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n0 = ((int)blockIdx.x - grp.wg0[g]) * 16 * NB;
    const int units = k_pad / 128, per = (units + NW - 1) / NW;
    const int u_begin = wave * per, u_end = u_begin + per < units ? u_begin + per : units;
    const int cnt = u_end - u_begin;
    char *ring = lds + (size_t)wave * NST * UNIT;
    // fill duty of this lane: rows 8 j + lane / 8 (j = 0, 1) of every tile, chunk (lane % 8) ^ ((row >> 1) & 7)
    const int8_t *src[NB + MB][2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int r = 8 * j + (lane >> 3), ch = (lane & 7) ^ ((r >> 1) & 7);
#pragma unroll
        for (int c = 0; c < NB; ++c) src[c][j] = w_t + pg_skinny_fill_offset(n0 + 16 * c + r, k_pad, 0, ch);  // (weight rows are padded to 256)
#pragma unroll
        for (int b = 0; b < MB; ++b) src[NB + b][j] = a_i8 + pg_skinny_fill_offset(16 * b + r, k_pad, 0, ch);
    }
    // fragment reads: row lane % 16, chunk 4 s + lane / 16 of k-step s
    const int fr = lane & 15, fsw = (fr >> 1) & 7;
    int rd[2];
#pragma unroll
    for (int st = 0; st < 2; ++st) rd[st] = fr * 128 + (((4 * st + (lane >> 4)) ^ fsw) * 16);
    const int rot = cnt > 0 ? (int)((blockIdx.x * 5u) % (unsigned)cnt) : 0;
    auto issue = [&](auto slot, int t) {  // t-th unit of the walk into ring slot `slot`
        const size_t kb = (size_t)pg_skinny_walk_unit(u_begin, cnt, t, rot) * 128;
        char *base = ring + decltype(slot)::value * UNIT;
#pragma unroll
        for (int q = 0; q < NB; ++q)  // the weights: used once, non-temporal
#pragma unroll
            for (int j = 0; j < 2; ++j)
                __builtin_amdgcn_global_load_lds((gptr_t)(src[q][j] + kb), (lptr_t)(base + q * TILE + j * 1024), 16, 0, 2);
#pragma unroll
        for (int q = NB; q < NB + MB; ++q)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                __builtin_amdgcn_global_load_lds((gptr_t)(src[q][j] + kb), (lptr_t)(base + q * TILE + j * 1024), 16, 0, 0);
    };
    v4i acc[NB][MB];
#pragma unroll
    for (int c = 0; c < NB; ++c)
#pragma unroll
        for (int b = 0; b < MB; ++b) acc[c][b] = v4i{0, 0, 0, 0};
    auto consume = [&](auto slot) {
        const char *base = ring + decltype(slot)::value * UNIT;
#pragma unroll
        for (int st = 0; st < 2; ++st) {
            v4i wf[NB];
#pragma unroll
            for (int c = 0; c < NB; ++c) wf[c] = *reinterpret_cast<const v4i *>(base + c * TILE + rd[st]);
#pragma unroll
            for (int b = 0; b < MB; ++b) {
                const v4i af = *reinterpret_cast<const v4i *>(base + (NB + b) * TILE + rd[st]);
#pragma unroll
                for (int c = 0; c < NB; ++c) acc[c][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, wf[c], acc[c][b], 0, 0, 0);
            }
        }
    };
    if (cnt > 0) {
        // prologue: NST - 1 units requested (fewer if the run is shorter)
#define PG_SK_PRO(U) if (U < NST - 1 && U < cnt) issue(std::integral_constant<int, (U < NST ? U : 0)>{}, U);
        PG_SK_PRO(0) PG_SK_PRO(1) PG_SK_PRO(2) PG_SK_PRO(3) PG_SK_PRO(4)
#undef PG_SK_PRO
        for (int t0 = 0; t0 < cnt; t0 += NST) {
#define PG_SK_STEP(U)                                                                                          \
            if (U < NST && t0 + U < cnt) {                                                                     \
                const int t = t0 + U;                                                                          \
                /* unit t is the oldest of those in flight: all but the NST - 2 younger ones have landed */   \
                if (t + NST - 2 < cnt) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NST - 2) * LPS) : "memory");  \
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                          \
                if (t + NST - 1 < cnt) issue(std::integral_constant<int, (U + NST - 1) % NST>{}, t + NST - 1); \
                __builtin_amdgcn_sched_barrier(0);                                                             \
                consume(std::integral_constant<int, (U < NST ? U : 0)>{});                                     \
                __builtin_amdgcn_sched_barrier(0);                                                             \
            }
            PG_SK_STEP(0) PG_SK_STEP(1) PG_SK_STEP(2) PG_SK_STEP(3) PG_SK_STEP(4) PG_SK_STEP(5)
#undef PG_SK_STEP
        }
    }
    __syncthreads();  // the rings are done with: their space takes the wavefronts' tiles
    int *red = reinterpret_cast<int *>(lds);  // [NW][NB * MB][4][64]
#pragma unroll
    for (int c = 0; c < NB; ++c)
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[((wave * NB * MB + c * MB + b) * 4 + i) * 64 + lane] = acc[c][b][i];
    __syncthreads();
    for (int e = threadIdx.x; e < NB * MB * 4 * 64; e += 64 * NW) {
        const int l = e & 63, i = (e >> 6) & 3, cb = e >> 8, c = cb / MB, b = cb - c * MB;
        int sum = 0;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += red[((w * NB * MB + cb) * 4 + i) * 64 + l];
        const int row = b * 16 + 4 * (l >> 4) + i, col = n0 + 16 * c + (l & 15);
        if (row < m && col < n) {
            const size_t o = (size_t)row * n + col;
            if (out) out[o] = (float)sum * a_scales[row] * w_scales[col];
            if (acc_out) acc_out[o] = sum;
        }
    }
}

// Tile choice (measured on MI355X at M = 2048): the larger the tile the fewer bytes each
// CU pulls from L2 per MFMA, but every CU needs a tile.  8 wavefronts per workgroup also
// double the rate at which one CU can stream from L2 (about 9 GB/s per wavefront).
// ctx->gemm_force_tile (pg_gemm_w8a8_force_tile) overrides the choice: 1 = 64x64, 2 = 256x256,
// 3 = 128x256, 4 = 128x64, 5 = 128x128.
pg_status gemm_dispatch(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                        const pg_qtensor *const *w, float *const *out, int count, size_t m, int32_t *acc,
                        const int32_t *comb = nullptr, size_t comb_plane = 0) {
    const size_t cus = (size_t)ctx->num_cu;
    auto tiles = [&](size_t bm, size_t bn) {
        size_t panels = 0;
        for (int i = 0; i < count; ++i) panels += (w[i]->cols + bn - 1) / bn;
        return ((m + bm - 1) / bm) * panels;
    };
    int pick = ctx->gemm_force_tile;
    if (pick == 0) {
        const size_t t256 = tiles(256, 256);
        if (m <= 64) pick = 1;
        // one and a half rounds of the largest tile or more -- or a single round that fills at least 70 %
        // of the CUs: the fused q|k|v product (192 tiles on 256 CUs) runs 56 us so against 65 us as
        // 384 half-size tiles (the CUs left idle let the busy ones clock higher)
        else if (t256 * 2 >= 3 * cus || (t256 <= cus && t256 * 10 >= 7 * cus)) pick = 2;
        else if (tiles(128, 256) >= cus) pick = 3;
        // Too few 128x128 tiles for the CUs (k/v projections, N = 1024): halve the tile instead of
        // leaving half of the chip idle (21.2 -> 16.5 us at 2048 x 4096 -> 1024).
        else if (tiles(128, 128) < cus) pick = 4;
        else pick = 5;
    }
    switch (pick) {
        case 1:
            if (comb) return launch_group<64, 64, 128, 2, 2, 2, 2, true>(ctx, a_i8, a_stride, a_scales, w, out, count, m, acc, 1, 0, comb, comb_plane);
            return launch_group<64, 64, 128, 2, 2, 2, 2>(ctx, a_i8, a_stride, a_scales, w, out, count, m, acc);
        case 2:
            if (comb) return launch_group<256, 256, 128, 2, 2, 4, 2, true>(ctx, a_i8, a_stride, a_scales, w, out, count, m, acc, 1, 0, comb, comb_plane);
            return launch_group<256, 256, 128, 2, 2, 4, 2>(ctx, a_i8, a_stride, a_scales, w, out, count, m, acc);
        case 3:
            if (comb) return launch_group<128, 256, 128, 2, 2, 4, 2, true>(ctx, a_i8, a_stride, a_scales, w, out, count, m, acc, 1, 0, comb, comb_plane);
            return launch_group<128, 256, 128, 2, 2, 4, 2>(ctx, a_i8, a_stride, a_scales, w, out, count, m, acc);
        case 4:
            if (comb) return launch_group<128, 64, 128, 3, 2, 2, 2, true>(ctx, a_i8, a_stride, a_scales, w, out, count, m, acc, 1, 0, comb, comb_plane);
            return launch_group<128, 64, 128, 3, 2, 2, 2>(ctx, a_i8, a_stride, a_scales, w, out, count, m, acc);
        case 5:
            if (comb) return launch_group<128, 128, 128, 3, 2, 2, 2, true>(ctx, a_i8, a_stride, a_scales, w, out, count, m, acc, 1, 0, comb, comb_plane);
            return launch_group<128, 128, 128, 3, 2, 2, 2>(ctx, a_i8, a_stride, a_scales, w, out, count, m, acc);
        default: return pg_fail(PG_EINVAL, "gemm_w8a8: unknown tile override %d", pick);
    }
}

}  // namespace

// Few activation rows (5 .. 256: batched decode, short prefill chunks): one or two tiles of activations against
// every weight row is far too few workgroups to stream the weights (64 on 256 CUs at N = 4096),
// so K is split until about two workgroups per CU exist; the partial i32 sums go to `part`
// ([splits][m][n]) and a second launch adds them and applies the scales.  Returns the number of
// splits through *splits_out when called with part == nullptr (sizing), else runs.
pg_status pg_launch_gemm_w8a8_few_rows(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                                       const pg_qtensor *w, size_t m, float *out, int32_t *acc, int32_t *part,
                                       int *splits_out) {
    const size_t n = w->cols, kt = w->k_pad / 128;
    const size_t bm = m <= 32 ? 32 : (m <= 64 ? 64 : 128);
    const size_t tiles = ((m + bm - 1) / bm) * ((n + 127) / 128);
    size_t splits = (2 * (size_t)ctx->num_cu + tiles - 1) / tiles;
    if (splits > kt / 2) splits = kt / 2;  // at least two k-tiles per workgroup
    if (splits > 16) splits = 16;
    if (splits < 1) splits = 1;
    const size_t kt_per = (kt + splits - 1) / splits;
    splits = (kt + kt_per - 1) / kt_per;   // no empty split
    if (splits_out) *splits_out = (int)splits;
    if (!part) return PG_OK;
    if (a_stride != w->k_pad) return pg_fail(PG_EINVAL, "gemm_w8a8: activation stride %zu != k_pad %zu", a_stride, w->k_pad);
    if (bm == 32)
        PG_TRY((launch<32, 128, 128, 3, 1, 4, 2>(ctx, a_i8, a_stride, a_scales, w, m, nullptr, part, (int)splits, (int)kt_per)));
    else if (bm == 64)
        PG_TRY((launch<64, 128, 128, 3, 2, 2, 2>(ctx, a_i8, a_stride, a_scales, w, m, nullptr, part, (int)splits, (int)kt_per)));
    else
        PG_TRY((launch<128, 128, 128, 3, 2, 2, 2>(ctx, a_i8, a_stride, a_scales, w, m, nullptr, part, (int)splits, (int)kt_per)));
    const size_t plane = m * n;
    return pg_launch(ctx, "gemm_w8a8_finish", splitk_finish_kernel, dim3((unsigned)((plane + 255) / 256)), dim3(256), 0,
                     (const int32_t *)part, (int)splits, plane, a_scales, (const float *)w->scales, (int)n, out, acc);
}

// 2 .. 64 rows in one launch (see gemm_w8a8_skinny_kernel).
// (33 .. 64 rows, us with the quantisation launch: 4096 -> 14336 24.7 against 30.3 split over K with a finishing pass,
// 4096 -> 4096 11.1 against 15.8, but 14336 -> 4096 27.8 against 26.2: long, narrow products keep the split.)
bool pg_gemm_w8a8_takes_skinny(const pg_qtensor *w, size_t m) { return m >= 2 && (m <= 32 || (m <= 64 && w->cols >= w->k_pad)) &&
           w->k_pad < (1ull << 30) && w->cols < (1ull << 30); }

// 2 .. 64 rows in one launch (see gemm_w8a8_skinny_kernel); `count` weights of equal K side by side.
pg_status pg_launch_gemm_w8a8_skinny_group(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                                           const pg_qtensor *const *w, float *const *out, int count, size_t m, int32_t *acc) {
    if (count < 1 || count > PG_GEMM_MAX_GROUP || (acc && count != 1))
        return pg_fail(PG_EINVAL, "gemm_w8a8 (few rows in one launch): %d weights (1 .. %d; the accumulators of one only)", count, PG_GEMM_MAX_GROUP);
    size_t cols = 0;
    for (int i = 0; i < count; ++i) {
        if (a_stride != w[i]->k_pad) return pg_fail(PG_EINVAL, "gemm_w8a8: activation stride %zu != k_pad %zu", a_stride, w[i]->k_pad);
        if (!pg_gemm_w8a8_takes_skinny(w[i], m)) return pg_fail(PG_EINVAL, "gemm_w8a8 (few rows in one launch): m = %zu", m);
        cols += w[i]->cols;
    }
    const size_t k_pad = w[0]->k_pad;
    // Wavefronts per workgroup (K runs): as many as keep every workgroup resident at once -- a second round of
    // workgroups would stream its weights after the first has drained.  The rings fill the CU's LDS: eight
    // wavefronts a CU with 16 to 18 KiB each up to 32 rows, four with 30 to 36 KiB where four activation tiles or
    // two weight tiles share a unit.  Two weight tiles a workgroup (more than 16 rows: halves what the CUs pull
    // from L2 for the activations) pay while that still gives every CU a workgroup (32 rows, us: 4096 -> 14336
    // 14.7 against 16.0, but 14336 -> 4096 20.0 against 16.0).
    const int mb = m <= 16 ? 1 : (m <= 32 ? 2 : 4);
    const int nb_tiles = (m > 16 && cols / 32 >= (size_t)ctx->num_cu) ? 2 : 1;
    const int nst = mb == 1 ? 4 : (mb == 2 && nb_tiles == 2 ? 4 : 3);
    const size_t ring = (size_t)nst * (nb_tiles + mb) * 2048;
    const int per_cu = ring * 8 <= 160 * 1024 ? 8 : 4;
    skinny_wgroup grp;
    int wgs = 0;
    for (int i = 0; i < PG_GEMM_MAX_GROUP; ++i) {
        const bool used = i < count;
        grp.w[i] = used ? w[i]->w_t : nullptr;
        grp.ws[i] = used ? w[i]->scales : nullptr;
        grp.out[i] = used ? out[i] : nullptr;
        grp.n[i] = used ? (int)w[i]->cols : 0;
        grp.wg0[i] = used ? wgs : INT_MAX;
        if (used) wgs += (int)((w[i]->cols + 16 * nb_tiles - 1) / (16 * nb_tiles));
    }
    const dim3 grid((unsigned)wgs);
    const size_t slots = (size_t)ctx->num_cu * per_cu, units = k_pad / 128;
    int nw = per_cu;
    while (nw > 1 && ((size_t)grid.x * nw > slots || units / nw < 4)) nw >>= 1;
#define PG_SKINNY_LAUNCH(MBB, NBB, NWW, NSTT)                                                                                \
    do {                                                                                                                     \
        auto kern = gemm_w8a8_skinny_kernel<MBB, NBB, NWW, NSTT>;                                                            \
        const size_t lds = (size_t)NWW * NSTT * (NBB + MBB) * 2048;                                                          \
        PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));                                                          \
        return pg_launch(ctx, "gemm_w8a8_few_rows", kern, grid, dim3(64 * NWW), lds, a_i8, grp, (int)k_pad, (int)m, a_scales, acc); \
    } while (0)
#define PG_SKINNY_NW8(MBB, NBB, NSTT)                       \
    switch (nw) {                                           \
        case 8: PG_SKINNY_LAUNCH(MBB, NBB, 8, NSTT);        \
        case 4: PG_SKINNY_LAUNCH(MBB, NBB, 4, NSTT);        \
        case 2: PG_SKINNY_LAUNCH(MBB, NBB, 2, NSTT);        \
        default: PG_SKINNY_LAUNCH(MBB, NBB, 1, NSTT);       \
    }
#define PG_SKINNY_NW4(MBB, NBB, NSTT)                       \
    switch (nw) {                                           \
        case 4: PG_SKINNY_LAUNCH(MBB, NBB, 4, NSTT);        \
        case 2: PG_SKINNY_LAUNCH(MBB, NBB, 2, NSTT);        \
        default: PG_SKINNY_LAUNCH(MBB, NBB, 1, NSTT);       \
    }
    if (mb == 1) PG_SKINNY_NW8(1, 1, 4)
    if (mb == 2 && nb_tiles == 1) PG_SKINNY_NW8(2, 1, 3)
    if (mb == 2) PG_SKINNY_NW4(2, 2, 4)
    if (nb_tiles == 1) PG_SKINNY_NW4(4, 1, 3)
    PG_SKINNY_NW4(4, 2, 3)
#undef PG_SKINNY_NW8
#undef PG_SKINNY_NW4
#undef PG_SKINNY_LAUNCH
}

pg_status pg_launch_gemm_w8a8_skinny(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                                     const pg_qtensor *w, size_t m, float *out, int32_t *acc) {
    return pg_launch_gemm_w8a8_skinny_group(ctx, a_i8, a_stride, a_scales, &w, &out, 1, m, acc);
}

// a_i8 must have at least round_up(m, 256) rows of a_stride bytes (rows >= m may
// hold anything: they only feed accumulators that are never stored), a_stride ==
// w->k_pad with the K padding zero-filled.
pg_status pg_launch_gemm_w8a8_group(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                                    const pg_qtensor *const *w, float *const *out, int count, size_t m) {
    if (count < 1 || count > PG_GEMM_MAX_GROUP) return pg_fail(PG_EINVAL, "gemm_w8a8: %d weights in one launch (1 .. %d)", count, PG_GEMM_MAX_GROUP);
    for (int i = 0; i < count; ++i) {
        if (a_stride != w[i]->k_pad) return pg_fail(PG_EINVAL, "gemm_w8a8: activation stride %zu != k_pad %zu", a_stride, w[i]->k_pad);
        if (w[i]->k_pad >= (1ull << 22) || m >= (1ull << 24) || w[i]->cols >= (1ull << 30))
            return pg_fail(PG_EUNSUPPORTED, "gemm_w8a8: shape exceeds the kernel's 32-bit tile offsets");
    }
    return gemm_dispatch(ctx, a_i8, a_stride, a_scales, w, out, count, m, nullptr);
}

pg_status pg_launch_gemm_w8a8(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride,
                              const float *a_scales, const pg_qtensor *w, size_t m, float *out,
                              int32_t *acc) {
    if (a_stride != w->k_pad) return pg_fail(PG_EINVAL, "gemm_w8a8: activation stride %zu != k_pad %zu", a_stride, w->k_pad);
    if (w->k_pad >= (1ull << 22) || m >= (1ull << 24) || w->cols >= (1ull << 30))
        return pg_fail(PG_EUNSUPPORTED, "gemm_w8a8: shape exceeds the kernel's 32-bit tile offsets");
    return gemm_dispatch(ctx, a_i8, a_stride, a_scales, &w, &out, 1, m, acc);
}

// The W8A32 product's last pass: `a_i8` is the digit plane of weight 65536, `comb` holds the accumulators of
// the other two ([2][comb_plane], the plane of weight 256 second); writes the finished f32 product.
pg_status pg_launch_gemm_w8a8_combine(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                                      const pg_qtensor *w, size_t m, float *out, const int32_t *comb, size_t comb_plane) {
    if (a_stride != w->k_pad) return pg_fail(PG_EINVAL, "gemm_w8a8: activation stride %zu != k_pad %zu", a_stride, w->k_pad);
    if (w->k_pad >= (1ull << 22) || m >= (1ull << 24) || w->cols >= (1ull << 30))
        return pg_fail(PG_EUNSUPPORTED, "gemm_w8a8: shape exceeds the kernel's 32-bit tile offsets");
    return gemm_dispatch(ctx, a_i8, a_stride, a_scales, &w, &out, 1, m, nullptr, comb, comb_plane);
}

// The shader clock inside the K loop of the 256x256 tile (the gate|up product's kernel): the
// product [m x k] . [k x n] on pseudo-random operands, every workgroup timing its own loop with
// the shader cycle counter and the constant-rate wall clock.
PG_API pg_status pg_probe_gemm_clock(pg_ctx *ctx, size_t m, size_t k, size_t n, double *clock_ghz, double *loop_us) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(m >= 256 && m <= 8192 && k >= 256 && k <= 32768 && n >= 256 && n <= 65536 && m % 256 == 0 && k % 128 == 0 && n % 256 == 0,
                 "pg_probe_gemm_clock: m %zu, n %zu must be multiples of 256 and k %zu of 128, within 8192 x 32768 x 65536", m, n, k);
    constexpr int BM = 256, BN = 256, BK = 128, NST = 2;
    const int tiles_m = (int)(m / BM), ntiles = tiles_m * (int)(n / BN);
    const unsigned grid = (unsigned)(((ntiles + 7) / 8) * 8);
    pg_tmp a, b, sc, out, clk;
    PG_TRY(a.alloc(m * k));
    PG_TRY(b.alloc(n * k));
    PG_TRY(sc.alloc((m > n ? m : n) * sizeof(float)));
    PG_TRY(out.alloc(m * n * sizeof(float)));
    PG_TRY(clk.alloc((size_t)grid * 2 * sizeof(long long)));
    PG_TRY(pg_probe_fill_random(ctx, a.p, m * k));
    PG_TRY(pg_probe_fill_random(ctx, b.p, n * k));
    PG_HIP(hipMemsetAsync(sc.p, 0, (m > n ? m : n) * sizeof(float), ctx->stream));
    PG_HIP(hipMemsetAsync(clk.p, 0, (size_t)grid * 2 * sizeof(long long), ctx->stream));
    gemm_wgroup grp;
    for (int i = 0; i < PG_GEMM_MAX_GROUP; ++i) {
        grp.w[i] = nullptr;
        grp.ws[i] = nullptr; grp.out[i] = nullptr; grp.n[i] = 0; grp.panel0[i] = INT_MAX;
    }
    grp.comb = nullptr;
    grp.comb_plane = 0;
    grp.w[0] = b.as<int8_t>(); grp.ws[0] = sc.as<float>(); grp.out[0] = out.as<float>(); grp.n[0] = (int)n; grp.panel0[0] = 0;
    const size_t lds = (size_t)NST * (BM + BN) * BK + (BM + BN) * sizeof(float);
    auto kern = gemm_w8a8_kernel<BM, BN, BK, NST, 2, 4, 2, true>;
    PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));
    for (int rep = 0; rep < 20; ++rep)  // the clock settles over the first launches; the last one is read
        PG_TRY(pg_launch(ctx, "gemm_w8a8_clock_probe", kern, dim3(grid), dim3(512), lds, a.as<int8_t>(), (int)k, grp, (int)k, sc.as<float>(),
                         (int32_t *)nullptr, (int)m, (int)k, tiles_m, ntiles, (int)(k / BK), clk.as<long long>()));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    std::vector<long long> h((size_t)grid * 2);
    PG_HIP(hipMemcpy(h.data(), clk.p, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
    int wall_khz = 0;
    PG_HIP(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, ctx->device));
    double cyc = 0.0, wall = 0.0;
    int used = 0;
    for (unsigned i = 0; i < grid; ++i)
        if (h[2 * i + 1] > 0) { cyc += (double)h[2 * i]; wall += (double)h[2 * i + 1]; ++used; }
    PG_CHECK_ARG(used > 0 && wall_khz > 0, "pg_probe_gemm_clock: no workgroup reported");
    const double secs = wall / (wall_khz * 1e3);
    if (clock_ghz) *clock_ghz = cyc / secs / 1e9;
    if (loop_us) *loop_us = secs / used * 1e6;
    return PG_OK;
}
