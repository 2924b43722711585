// Many-row product over Q4_0 / Q8_0 block weights on the f16 matrix cores:
//   y[t, n] = sum_b d[n, b] * sum_{k in block b} q[n, k] * x[t, k]
// (the M >> 1 dequant-matmul of models::llama, src/models/llama/model.rs:243-257 +
// src/tensor.rs:1342-1353: dequantise the weight, then Tensor::matmul).
//
// The weights stay exact: a Q4_0 quant q - 8 in [-8, 7] (a Q8_0 quant in [-127, 127]) is an
// f16 value, made in registers from the packed bytes, and a GGUF block is 32 consecutive k,
// exactly the K of one v_mfma_f32_16x16x32_f16.  The activation rows are split once into two
// f16 planes, x * 2^e = hi + lo (e per row, so that the row's largest magnitude lands in
// [2^14, 2^15): hi carries 11 bits, lo the next 11, what is dropped is below 2^-22 of the
// row's maximum).  Per block and 16x16 tile two chained MFMAs give T = (hi + lo) . q, products
// of f16 values summed in f32, and the accumulator takes acc += d[n, b] * T in f32: one VALU
// FMA per output and block where the int8 block product (pg_gguf_mm.hip) needs four
// instructions, which is what bounds that kernel at many rows.
//
// Workgroup = 8 wavefronts over NWM x NWN tiles of 128 rows x 64 weight rows: 256 x 256
// (2 x 4) or 128 x 512 (1 x 8).  K runs in stages of two blocks through two LDS stages filled
// by direct global->LDS loads: the two activation planes [rows][128 B] (16-byte chunks XOR
// swizzled as in the W8A8 kernel), the weights' packed bytes [weight rows][2 blocks] and their
// f16 scales.  One barrier per stage.  Inside a stage the wavefront walks 16 steps (2 blocks x
// 8 row tiles); at every step it issues 8 MFMAs (4 weight tiles x hi, lo) into one of two sets
// of T registers, and between them the 16 FMAs that fold the previous step's T into the
// accumulators, so neither unit waits for the other.  The second block's weights are unpacked
// under the first block's MFMAs.
//
// A K too short to fill the part with tiles is cut into chunks (blockIdx.y); the chunks' planes
// are summed in a fixed order by pg_launch_sum_parts.
#include <limits.h>
#include "pg_internal.h"
#include "pg_f16_planes.h"
#include "pg_stream_addr.h"

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef const void __attribute__((address_space(1))) *gptr_t;
typedef void __attribute__((address_space(3))) *lptr_t;

inline unsigned grid_for(size_t n, unsigned block) { return (unsigned)((n + block - 1) / block); }

__device__ __forceinline__ int swz128(int r) { return ((r >> 1) & 7) ^ ((r & 1) << 2); }

// ---- activation rows -> two f16 planes and the rows' inverse scales (pg_f16_planes.h) ----
__global__ __launch_bounds__(256) void rows_to_f16_planes_kernel(const float *__restrict__ x, int K, _Float16 *__restrict__ hi,
                                                                 _Float16 *__restrict__ lo, float *__restrict__ inv) {
    const size_t row = blockIdx.x;
    const float *xr = x + row * K;
    __shared__ float red[4];
    float amax = 0.0f;
    for (int i = threadIdx.x * 4; i < K; i += 1024) {
        const float4 v = *reinterpret_cast<const float4 *>(xr + i);
        amax = fmaxf(amax, fmaxf(fmaxf(pg_f16_mag(v.x), pg_f16_mag(v.y)), fmaxf(pg_f16_mag(v.z), pg_f16_mag(v.w))));
    }
    for (int o = 32; o; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const pg_f16_row_scale sc = pg_f16_row_scale_of(amax);
    if (threadIdx.x == 0) {
        inv[2 * row] = sc.i1;
        inv[2 * row + 1] = sc.i2;
    }
    for (int i = threadIdx.x * 4; i < K; i += 1024) {
        const float4 v = *reinterpret_cast<const float4 *>(xr + i);
        const float f[4] = {v.x, v.y, v.z, v.w};
        pg_f16_split4(f, sc, reinterpret_cast<uint2 *>(hi + row * K + i), reinterpret_cast<uint2 *>(lo + row * K + i));
    }
}

// 8 Q4_0 nibbles as stored at upload (two's complement of q - 8; nibble j = element j of the
// dword's 8) -> 8 f16 values q - 8.  0x6400 | q is the f16 1024 + q; minus 1032 it is q - 8.
__device__ __forceinline__ v8h nibbles_to_f16(uint32_t w) {
    w ^= 0x88888888u;
    const uint32_t a = w & 0x0F0F0F0Fu, b = (w >> 4) & 0x0F0F0F0Fu;
    const v2h bias = {(_Float16)1032.0f, (_Float16)1032.0f};
    union { uint32_t u[4]; v2h h[4]; v8h v; } r;
    r.u[0] = __builtin_amdgcn_perm(b, a, 0x0c040c00u) | 0x64006400u;
    r.u[1] = __builtin_amdgcn_perm(b, a, 0x0c050c01u) | 0x64006400u;
    r.u[2] = __builtin_amdgcn_perm(b, a, 0x0c060c02u) | 0x64006400u;
    r.u[3] = __builtin_amdgcn_perm(b, a, 0x0c070c03u) | 0x64006400u;
#pragma unroll
    for (int p = 0; p < 4; ++p) r.h[p] = r.h[p] - bias;
    return r.v;
}

// 8 Q8_0 quants (two dwords of int8, element order) -> 8 f16 values.  A byte q as q + 128 under 0x64 is the f16
// 1152 + q; the bytes 0x64 come from the selector's second source.
__device__ __forceinline__ v8h bytes_to_f16(uint32_t w0, uint32_t w1) {
    w0 ^= 0x80808080u;
    w1 ^= 0x80808080u;
    const v2h bias = {(_Float16)1152.0f, (_Float16)1152.0f};
    union { uint32_t u[4]; v2h h[4]; v8h v; } r;
    r.u[0] = __builtin_amdgcn_perm(w0, 0x64646464u, 0x00050004u);
    r.u[1] = __builtin_amdgcn_perm(w0, 0x64646464u, 0x00070006u);
    r.u[2] = __builtin_amdgcn_perm(w1, 0x64646464u, 0x00050004u);
    r.u[3] = __builtin_amdgcn_perm(w1, 0x64646464u, 0x00070006u);
#pragma unroll
    for (int p = 0; p < 4; ++p) r.h[p] = r.h[p] - bias;
    return r.v;
}

// The tensors of one launch: equal K, their panels of BN weight rows laid end to end in the launch's tile space.
struct hmm_group {
    const uint8_t *qs[PG_HMM_MAX_GROUP];
    const uint16_t *d[PG_HMM_MAX_GROUP];
    float *out[PG_HMM_MAX_GROUP];      // y, or the first K chunk's plane
    long long stride[PG_HMM_MAX_GROUP];  // floats from one K chunk's plane to the next
    int n[PG_HMM_MAX_GROUP];
    int panel0[PG_HMM_MAX_GROUP];      // first panel of tensor g (INT_MAX: unused)
};

constexpr int BKB = 2;  // blocks per stage

// QT = 8 (Q8_0): a weight row is two streams of 16-byte half blocks (elements 0 .. 15 and 16 .. 31 of every block,
// as the upload splits them); a stage holds 64 bytes a row, chunk 2 block + half at position chunk ^ ((row >> 2) & 3),
// so that the 64-bit fragment reads of 16 rows spread over all banks.
template <int QT, int NWM, int NWN>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gguf_hmm_kernel(const _Float16 *__restrict__ xh, const _Float16 *__restrict__ xl, const float *__restrict__ inv,
                        const hmm_group grp, int M, int nb, int tiles_m, int ntiles, int kt_per_split) {
    static_assert(NWM * NWN == 8, "eight wavefronts");
    constexpr int BM = 128 * NWM, BN = 64 * NWN;
    constexpr int WROW = QT == 8 ? 64 : 32;                   // bytes of packed weights per row and stage
    constexpr int LX = BM / 64, LW = (BN * WROW / 1024 + 7) / 8;  // wave-loads per wavefront and stage: one plane, weights
    constexpr int XP = BM * 128;                              // one activation plane of a stage
    constexpr int OFF_XL = XP, OFF_W = 2 * XP, OFF_D = OFF_W + 8 * LW * 1024, STAGE = OFF_D + 8 * 256;
    constexpr int LPS = 2 * LX + LW + 1;
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    // Workgroups are dealt round-robin to the 8 XCDs; each XCD gets a contiguous run of tiles
    // (row tiles fastest), so the tiles that share an L2 share weight panels.
    const int chunk = (ntiles + 7) / 8;
    const int t = (blockIdx.x % 8) * chunk + blockIdx.x / 8;
    if (t >= ntiles) return;
    const int np = t / tiles_m;
    int g = 0;
#pragma unroll
    for (int i = 1; i < PG_HMM_MAX_GROUP; ++i) g = np >= grp.panel0[i] ? i : g;
    const uint8_t *__restrict__ qs = grp.qs[g];
    const uint16_t *__restrict__ d = grp.d[g];
    const int N = grp.n[g];
    const int m0 = (t % tiles_m) * BM, n0 = (np - grp.panel0[g]) * BN;
    const int K = nb * 32;
    const int kt0 = blockIdx.y * kt_per_split;
    const int KT = nb / BKB - kt0 < kt_per_split ? nb / BKB - kt0 : kt_per_split;
    float *__restrict__ y = grp.out[g] + (size_t)blockIdx.y * grp.stride[g];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / NWN, wn = wave % NWN;
    const int l15 = lane & 15, q4 = lane >> 4;

    // ---- global -> LDS.  Activation planes: wave-load L covers rows 8L .. 8L+7 (lane -> row,
    // physical chunk; it fetches the logical chunk that belongs there).  Weights: wave-load L
    // covers rows 32L .. 32L+31, two 16-byte blocks a row, the block order flipped in every
    // second group of 8 rows (so that 16 rows' dword reads fall in 64 different banks).
    const char *xsrc[LX];
    {
        const int lr = lane >> 3, pc = lane & 7;
#pragma unroll
        for (int i = 0; i < LX; ++i) {
            const int row = 8 * (wave + 8 * i) + lr;
            xsrc[i] = reinterpret_cast<const char *>(xh) + pg_hmm_plane_offset(pg_hmm_clamp_row(m0 + row, M), K, kt0, pc ^ swz128(row));
        }
    }
    const ptrdiff_t lo_minus_hi = reinterpret_cast<const char *>(xl) - reinterpret_cast<const char *>(xh);
    const char *wsrc[LW];
#pragma unroll
    for (int i = 0; i < LW; ++i) {
        if constexpr (QT == 8) {
            const int row = 16 * (wave + 8 * i) + (lane >> 2);
            const int rc = row < BN ? row : BN - 1;
            const int c = (lane & 3) ^ ((row >> 2) & 3);  // logical chunk: 2 block + half
            wsrc[i] = reinterpret_cast<const char *>(qs) + pg_hmm_weight_offset_q8(pg_hmm_clamp_row(n0 + rc, N), c & 1, nb, kt0, c >> 1);
        } else {
            const int row = 32 * (wave + 8 * i) + (lane >> 1);
            const int rc = row < BN ? row : BN - 1;
            const int cb = (lane & 1) ^ ((row >> 3) & 1);
            wsrc[i] = reinterpret_cast<const char *>(qs) + pg_hmm_weight_offset(pg_hmm_clamp_row(n0 + rc, N), nb, kt0, cb);
        }
    }
    const char *dsrc;
    {
        const int row = wn * 64 + 2 * (lane & 31);   // this wavefront's own 64 weight rows, two per lane
        dsrc = reinterpret_cast<const char *>(d) + pg_hmm_scale_offset(pg_hmm_scale_row(n0 + row, N), nb, kt0, lane >> 5);
    }
    auto issue = [&](int stage, int kt) {   // kt: stage index within this workgroup's K chunk
        char *base = lds + stage * STAGE;
#pragma unroll
        for (int i = 0; i < LX; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(xsrc[i] + (size_t)kt * 128), (lptr_t)(base + (wave + 8 * i) * 1024), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < LX; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(xsrc[i] + lo_minus_hi + (size_t)kt * 128), (lptr_t)(base + OFF_XL + (wave + 8 * i) * 1024), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < LW; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(wsrc[i] + (size_t)kt * 32), (lptr_t)(base + OFF_W + (wave + 8 * i) * 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr_t)(dsrc + (size_t)kt * 32), (lptr_t)(base + OFF_D + wave * 256), 4, 0, 0);
    };

    // ---- fragment offsets: lane = (row l15, k group q4 of 8 elements)
    int a_off[2], w_off[2], d_off[2];
    {
        const int ra = wm * 128 + l15, rb = wn * 64 + l15;
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            a_off[b] = ra * 128 + (((4 * b + q4) ^ swz128(ra)) * 16);                    // + 16 rows per row tile
            if constexpr (QT == 8) w_off[b] = OFF_W + rb * 64 + 16 * ((2 * b + (q4 >> 1)) ^ ((rb >> 2) & 3)) + 8 * (q4 & 1);
            else w_off[b] = OFF_W + rb * 32 + 16 * (b ^ ((rb >> 3) & 1)) + 4 * q4;       // + 16 rows per weight tile
            d_off[b] = OFF_D + wave * 256 + (b * 32 + (l15 >> 1)) * 4 + (l15 & 1) * 2;   // + 32 bytes per weight tile
        }
    }

    v4f acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0, 0, 0, 0};

    issue(0, 0);
    if (KT > 1) {
        issue(1, 1);
        asm volatile("s_waitcnt vmcnt(%0)\n s_barrier" ::"n"(LPS) : "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(0)\n s_barrier" ::: "memory");
    }
    for (int kt = 0; kt < KT; ++kt) {
        const int s = kt & 1;
        const char *base = lds + s * STAGE;
        v8h fb[2][4];
        float df[2][4];
        uint32_t wraw[4][QT == 8 ? 2 : 1];
        _Float16 draw[4];
        auto read_w = [&](int b, int j, uint32_t (&raw)[QT == 8 ? 2 : 1]) {
            if constexpr (QT == 8) {
                const uint2 t = *reinterpret_cast<const uint2 *>(base + w_off[b] + j * 16 * WROW);
                raw[0] = t.x;
                raw[1] = t.y;
            } else {
                raw[0] = *reinterpret_cast<const uint32_t *>(base + w_off[b] + j * 16 * WROW);
            }
        };
        auto unpack = [&](const uint32_t (&raw)[QT == 8 ? 2 : 1]) -> v8h {
            if constexpr (QT == 8) return bytes_to_f16(raw[0], raw[1]);
            else return nibbles_to_f16(raw[0]);
        };
        v8h ah[2], al[2];
        v4f T[2][4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            read_w(0, j, wraw[j]);
            fb[0][j] = unpack(wraw[j]);
            df[0][j] = (float)*reinterpret_cast<const _Float16 *>(base + d_off[0] + j * 32);
            asm volatile("" : "+v"(df[0][j]));   // a plain f32 register: the FMAs below are v_fma_f32, not mixed-precision ones
        }
        ah[0] = *reinterpret_cast<const v8h *>(base + a_off[0]);
        al[0] = *reinterpret_cast<const v8h *>(base + OFF_XL + a_off[0]);
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const int b = q >> 3, cur = q & 1, nxt = cur ^ 1;
            if (q + 1 < 16) {
                const int b1 = (q + 1) >> 3, i1 = (q + 1) & 7;
                ah[nxt] = *reinterpret_cast<const v8h *>(base + a_off[b1] + i1 * 16 * 128);
                al[nxt] = *reinterpret_cast<const v8h *>(base + OFF_XL + a_off[b1] + i1 * 16 * 128);
            }
            if (q == 0) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    read_w(1, j, wraw[j]);
                    draw[j] = *reinterpret_cast<const _Float16 *>(base + d_off[1] + j * 32);
                }
            }
            if (q >= 2 && q < 6) {
                fb[1][q - 2] = unpack(wraw[q - 2]);
                df[1][q - 2] = (float)draw[q - 2];
                asm volatile("" : "+v"(df[1][q - 2]));
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) T[cur][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah[cur], fb[b][j], (v4f){0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j) T[cur][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al[cur], fb[b][j], T[cur][j], 0, 0, 0);
            if (q > 0) {
                const int bp = (q - 1) >> 3, ip = (q - 1) & 7;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[ip][j][r] = __builtin_fmaf(T[nxt][j][r], df[bp][j], acc[ip][j][r]);
                    asm volatile("" : "+v"(acc[ip][j]));   // keeps the FMAs in this step (they would sink to the end of the stage)
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);  // two VALU
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[7][j][r] = __builtin_fmaf(T[1][j][r], df[1][j], acc[7][j][r]);
            asm volatile("" : "+v"(acc[7][j]));
        }
        if (kt + 1 < KT) {
            // Only the next stage's fills are in flight: wait for mine and meet the others, who have then
            // also read this stage to the end; this stage takes the stage after next.
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n s_barrier" ::: "memory");
            if (kt + 2 < KT) issue(s, kt + 2);
        }
    }

    // ---- epilogue: register r of tile (i, j) is row 16 i + 4 q4 + r, weight row 16 j + l15
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = m0 + wm * 128 + 16 * i + 4 * q4 + r;
            if (m >= M) continue;
            const float s1 = inv[2 * m], s2 = inv[2 * m + 1];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + wn * 64 + 16 * j + l15;
                if (n < N) __builtin_nontemporal_store(acc[i][j][r] * s1 * s2, y + (size_t)m * N + n);
            }
        }
}

template <int QT, int NWM, int NWN> constexpr size_t hmm_lds_bytes() {
    return 2 * (size_t)(2 * 128 * NWM * 128 + 8 * ((64 * NWN * (QT == 8 ? 64 : 32) / 1024 + 7) / 8) * 1024 + 8 * 256);
}

}  // namespace

size_t pg_hmm_planes_bytes(size_t rows, size_t k) {
    return 2 * pg_round_up(rows * k * sizeof(_Float16), 256) + pg_round_up(2 * rows * sizeof(float), 256);
}

pg_hmm_planes pg_hmm_planes_carve(void *base, size_t rows, size_t k) {
    pg_hmm_planes p;
    char *c = static_cast<char *>(base);
    p.hi = c;
    c += pg_round_up(rows * k * sizeof(_Float16), 256);
    p.lo = c;
    c += pg_round_up(rows * k * sizeof(_Float16), 256);
    p.inv = reinterpret_cast<float *>(c);
    p.rows = rows;
    p.k = k;
    return p;
}

pg_status pg_launch_rows_to_f16_planes(pg_ctx *ctx, const float *x_dev, size_t rows, size_t k, const pg_hmm_planes &p) {
    if (rows == 0) return PG_OK;
    if (k % 4 != 0 || k > (size_t)INT_MAX) return pg_fail(PG_EINVAL, "rows_to_f16_planes: k = %zu", k);
    return pg_launch(ctx, "rows_to_f16_planes", rows_to_f16_planes_kernel, dim3((unsigned)rows), dim3(256), 0, x_dev, (int)k,
                     (_Float16 *)p.hi, (_Float16 *)p.lo, p.inv);
}

// Which products this kernel takes, and in how many K chunks.  `n_total` = weight rows of all the tensors of the
// launch.  A tile holds 256 x 256 outputs (128 x 512 up to 128 rows); a workgroup needs the CU to itself, so a
// launch wants about one workgroup per CU: short of that, K is cut into up to 8 chunks of at least 512.
bool pg_gguf_hmm_takes(const pg_ctx *ctx, int ggml_type, size_t m, size_t n_total, size_t k_in, int *ks_out) {
    if (ctx->hmm_mode == 2) return false;
    if ((ggml_type != PG_GGML_Q4_0 && ggml_type != PG_GGML_Q8_0) || k_in % 64 != 0 || k_in < 256 || k_in > ((size_t)1 << 24) || n_total < 2 || n_total > ((size_t)1 << 24) ||
        m < 2 || m > ((size_t)1 << 20))
        return false;
    const bool wide = m <= 128 || ggml_type == PG_GGML_Q8_0;  // (Q8_0: a stage of 256 x 256 does not fit the LDS twice)
    const size_t bm = wide ? 128 : 256, bn = wide ? 512 : 256;
    const size_t tiles = ((m + bm - 1) / bm) * ((n_total + bn - 1) / bn);
    size_t ks = (size_t)ctx->num_cu / tiles;
    const size_t stages = k_in / 64;
    while (ks > 1 && stages / ks < 8) --ks;
    if (ks > 8) ks = 8;
    if (ks < 1) ks = 1;
    const size_t per = (stages + ks - 1) / ks;
    ks = (stages + per - 1) / per;   // chunks of `per` stages: none is empty
    if (ks_out) *ks_out = (int)ks;
    if (ctx->hmm_mode == 1) return true;
    // Measured against the int8 block product (us, f16 route : int8 route, [K] -> [N] at M rows): 4096 -> 14336 at
    // 256 / 1024 / 4096 rows 97 : 105 / 241 : 329 / 981 : 1290; 14336 -> 4096 at 256 / 384 / 1024 126 : 101 /
    // 144 : 175 / 268 : 345; 4096 -> 4096 at 512 / 1024 / 4096 74 : 59 / 105 : 106 / 281 : 389; 8192 -> 28672 at
    // 64 / 96 / 1024 143 : 115 / 149 : 172 / 899 : 1326.  The f16 route wins from about 18 G multiply-adds on:
    // below that its tiles leave CUs idle or its K chunks cost a pass over their planes.
    // (Q8_0, always on 128 x 512 tiles: 4096 -> 14336 at 256 / 512 / 1024 rows 109 : 112 / 168 : 180 / 266 : 348, 14336 -> 4096 at
    // 256 / 512 / 1024 143 : 105 / 166 : 188 / 287 : 351, 4096 -> 4096 at 1024 / 2048 111 : 110 / 186 : 202: from about 24 G.)
    return m >= 96 && (double)m * (double)n_total * (double)k_in >= (ggml_type == PG_GGML_Q8_0 ? 2.4e10 : 1.8e10);
}

size_t pg_gguf_hmm_part_floats(size_t m, size_t n_total, int ks) { return ks > 1 ? (size_t)ks * m * n_total : 0; }

// ks > 1: the K chunks' planes go to `part` (tensor after tensor, ks planes of m x n_out each) and are summed into
// y[i]; with keep_parts they go to y[i] instead (ks planes, m * n_out floats apart) and stay unsummed.
pg_status pg_launch_gguf_hmm_group(pg_ctx *ctx, size_t k_in, const pg_gguf_tensor *const *w, float *const *y, int count, size_t m,
                                   const pg_hmm_planes &planes, int ks, float *part, bool keep_parts) {
    if (count < 1 || count > PG_HMM_MAX_GROUP) return pg_fail(PG_EINVAL, "gguf (f16 matrix cores): %d tensors (1 .. %d)", count, PG_HMM_MAX_GROUP);
    if (m == 0) return PG_OK;
    // (a Q4_1 tensor's nibbles and scales are laid out as a Q4_0 tensor's: its first term runs as the Q4_0 product)
    auto kind = [](int t) { return t == PG_GGML_Q4_1 ? PG_GGML_Q4_0 : t; };
    const int type = kind(w[0]->ggml_type);
    if (type != PG_GGML_Q4_0 && type != PG_GGML_Q8_0) return pg_fail(PG_EINVAL, "gguf (f16 matrix cores): ggml type %d", type);
    for (int i = 0; i < count; ++i)
        if (w[i]->k_in != k_in || kind(w[i]->ggml_type) != type) return pg_fail(PG_EINVAL, "gguf (f16 matrix cores): the tensors differ in K or type");
    if (k_in % 64 != 0 || planes.rows < m || planes.k != k_in) return pg_fail(PG_EINVAL, "gguf (f16 matrix cores): K = %zu, planes of %zu x %zu", k_in, planes.rows, planes.k);
    if (ks < 1 || (ks > 1 && !part && !keep_parts)) return pg_fail(PG_EINVAL, "gguf (f16 matrix cores): %d K chunks without a buffer for their planes", ks);
    const bool q8 = type == PG_GGML_Q8_0, wide = m <= 128 || q8;   // 128 x 512 tiles
    const size_t bm = wide ? 128 : 256, bn = wide ? 512 : 256;
    hmm_group grp;
    int panels = 0;
    size_t part_off = 0;
    for (int i = 0; i < PG_HMM_MAX_GROUP; ++i) {
        const bool used = i < count;
        grp.qs[i] = used ? w[i]->qs : nullptr;
        grp.d[i] = used ? w[i]->d : nullptr;
        grp.n[i] = used ? (int)w[i]->n_out : 0;
        grp.panel0[i] = used ? panels : INT_MAX;
        grp.out[i] = used ? (ks > 1 && !keep_parts ? part + part_off : y[i]) : nullptr;
        grp.stride[i] = used && ks > 1 ? (long long)(m * w[i]->n_out) : 0;
        if (used) {
            panels += (int)((w[i]->n_out + bn - 1) / bn);
            part_off += (size_t)ks * m * w[i]->n_out;
        }
    }
    const int tiles_m = (int)((m + bm - 1) / bm), ntiles = tiles_m * panels;
    const int stages = (int)(k_in / 64), kt_per = (stages + ks - 1) / ks;
    const int ks_real = (stages + kt_per - 1) / kt_per;
    if (ks_real != ks) return pg_fail(PG_EINVAL, "gguf (f16 matrix cores): %d K chunks of %d stages leave one empty", ks, kt_per);
    const dim3 grid((unsigned)((ntiles + 7) / 8 * 8), (unsigned)ks_real);
    const int nb = (int)(k_in / 32);
#define PG_HMM_LAUNCH(QTT, NWMM, NWNN)                                                                                          \
    do {                                                                                                                        \
        auto kern = gguf_hmm_kernel<QTT, NWMM, NWNN>;                                                                           \
        const size_t lds = hmm_lds_bytes<QTT, NWMM, NWNN>();                                                                    \
        PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));                                                             \
        PG_TRY(pg_launch(ctx, QTT == 8 ? "gguf_hmm_q8_0" : "gguf_hmm_q4_0", kern, grid, dim3(512), lds, (const _Float16 *)planes.hi, \
                         (const _Float16 *)planes.lo, (const float *)planes.inv, grp, (int)m, nb, tiles_m, ntiles, kt_per));    \
    } while (0)
    if (q8) PG_HMM_LAUNCH(8, 1, 8);
    else if (wide) PG_HMM_LAUNCH(4, 1, 8);
    else PG_HMM_LAUNCH(4, 2, 4);
#undef PG_HMM_LAUNCH
    if (ks > 1 && !keep_parts) {
        size_t off = 0;
        for (int i = 0; i < count; ++i) {
            const size_t plane = m * w[i]->n_out;
            PG_TRY(pg_launch_sum_parts(ctx, part + off, plane, ks_real, plane, y[i]));
            off += (size_t)ks * plane;
        }
    }
    return PG_OK;
}
