// MXFP4 weights (gpt_oss experts, examples/gpt_oss/moe.rs:5-117) on the scaled matrix-core
// instruction of gfx950, which takes FP4 (E2M1) codes and E8M0 block scales as they sit in the file.
//
// v_mfma_scale_f32_16x16x128_f8f6f4, D[16 x 16] += A[16 x 128] * B[128 x 16], with A in FP4 and B in
// FP8 (E4M3), every 32 consecutive k of a row of A / column of B scaled by 2^(byte - 127):
//   A  lane l holds row l % 16, k = 32 (l / 16) .. + 31: the 16 code bytes of one MXFP4 block, element e
//      in nibble e -- exactly the file's packing (byte i = elements 2i low, 2i + 1 high);
//   B  lane l holds column l % 16; its first 16 bytes are k = 16 (l / 16) .. + 15, its last 16 bytes
//      k = 64 + 16 (l / 16) .. + 15;
//   scale operands: one byte per lane (selected by op_sel), lane l = row or column l % 16, k block l / 16;
//   D  lane l holds column l % 16, rows 4 (l / 16) .. + 3.
// (Layouts read off the hardware with one-hot operands.)
//
// The weights are rows of A: 17 bytes per block are all the product reads.  An activation row is not
// representable in FP8, but a fixed-point rewriting of it is: per block x[k] = 2^se X[k], |X| < 2^23, and
// X = sum_j 32^j n_j with five balanced base-32 digits n_j in [-16, 16], each exact in E4M3.  Digit plane
// j of a row is one column of B with block scale byte 127 + se + 5 j, so the instruction itself applies
// both block scales and sums over K; the five columns of a row are added at the end.  Three activation
// rows (15 columns) share one pass over the weights.
#include "pg_internal.h"
#include "pg_stream_addr.h"
#include "pg_digits.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef const v4i __attribute__((address_space(1))) *gv4i_ptr;

constexpr int MX_PLANES = 5;  // digit planes per activation row
constexpr int MX_U = 8;       // chunks (of 4 blocks) per batch of weight loads in flight
constexpr int MX_MAX_T = 3;   // activation rows per pass over the weights

inline unsigned grid_for(size_t n, unsigned block) { return (unsigned)((n + block - 1) / block); }
inline size_t mx_chunks(size_t nb) { return pg_mx_chunks(nb); }  // chunks of 4 blocks per row, whole scale dwords

// ---- device layout of a tensor ------------------------------------------------------
// Fragment-major: for every group of 16 rows and every chunk of 4 blocks (128 k), the 64 lanes' 16 code
// bytes in lane order (one fully coalesced 1 KiB load per instruction), and per 4 chunks one dword per
// lane with the 4 scale bytes.  Rows and blocks past the tensor's end hold zero codes; blocks whose
// scale byte is 0 (the reference's f32::from_bits(0) = 0.0, the hardware's 2^-127) also get zero codes.
__global__ void mxfp4_fragments_kernel(const uint8_t *__restrict__ blocks, const uint8_t *__restrict__ scales, int n_out,
                                       int nb, int ncp, uint4 *__restrict__ qs, uint8_t *__restrict__ sc) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // (row group, chunk, lane)
    const size_t nrg = ((size_t)n_out + 15) / 16;
    if (i >= nrg * ncp * 64) return;
    const int lane = (int)(i & 63), c = (int)((i >> 6) % ncp);
    const size_t rg = (i >> 6) / ncp;
    const size_t row = rg * 16 + (lane & 15);
    const int blk = 4 * c + (lane >> 4);
    uint4 v = {0, 0, 0, 0};
    unsigned e = 127;
    if (row < (size_t)n_out && blk < nb) {
        e = scales[row * nb + blk];
        if (e != 0) {
            const uint8_t *src = blocks + (row * nb + blk) * 16;  // any alignment
            unsigned wv[4];
            for (int t = 0; t < 4; ++t) wv[t] = src[4 * t] | (src[4 * t + 1] << 8) | (src[4 * t + 2] << 16) | ((unsigned)src[4 * t + 3] << 24);
            v = make_uint4(wv[0], wv[1], wv[2], wv[3]);
        }
    }
    qs[i] = v;
    sc[((rg * (ncp / 4) + c / 4) * 64 + lane) * 4 + (c & 3)] = (uint8_t)e;
}

// ---- one activation block -> five E4M3 digit planes in LDS ---------------------------
// Eight consecutive lanes hold one block (f = elements 4 sub .. 4 sub + 3); all eight call together.
// dig: the row's first plane, planes `stride` bytes apart, k-th element of plane j at dig[j * stride + k];
// sb:  scale bytes, plane j / block b at sb[(j * 4 + b % 4) * ncp + b / 4].
__device__ __forceinline__ void mx_emit_digits(const float (&f)[4], int b, int sub, char *dig, int stride, uint8_t *sb, int ncp) {
    float amax = fmaxf(fmaxf(fabsf(f[0]), fabsf(f[1])), fmaxf(fabsf(f[2]), fabsf(f[3])));
    int bad = (f[0] != f[0]) | (f[1] != f[1]) | (f[2] != f[2]) | (f[3] != f[3]);
    amax = fmaxf(amax, __builtin_bit_cast(float, pg_dpp8<0xB1>(__builtin_bit_cast(int, amax))));
    bad |= pg_dpp8<0xB1>(bad);
    amax = fmaxf(amax, __builtin_bit_cast(float, pg_dpp8<0x4E>(__builtin_bit_cast(int, amax))));
    bad |= pg_dpp8<0x4E>(bad);
    amax = fmaxf(amax, __builtin_bit_cast(float, pg_dpp8<0x141>(__builtin_bit_cast(int, amax))));
    bad |= pg_dpp8<0x141>(bad);
    int se = 0;
    float inv = 1.0f;
    if (bad || !(amax <= 3.4028234663852886e38f)) {
        bad = 1;
        inv = 0.0f;
    } else if (amax > 0.0f) {
        int ex;
        (void)frexpf(amax, &ex);  // amax = f * 2^ex, f in [0.5, 1)
        se = ex - 23;             // |x| / 2^se < 2^23
        if (se < -126) se = -126;
        inv = ldexpf(1.0f, -se);
    }
    // Balanced base-32 digits, top down and all in f32 (every value is a small integer times a power of two,
    // so each step is exact): n_j = round(r / 32^j), r -= n_j 32^j; |n_j| <= 16.
    float r[4], d[MX_PLANES][4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float t = f[e] * inv;
        r[e] = (t != t) ? 0.0f : rintf(t);
    }
#pragma unroll
    for (int j = MX_PLANES - 1; j >= 1; --j) {
        const float down = __builtin_bit_cast(float, (127 - 5 * j) << 23), up = -__builtin_bit_cast(float, (127 + 5 * j) << 23);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            d[j][e] = rintf(r[e] * down);
            r[e] = fmaf(d[j][e], up, r[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) d[0][e] = r[e];
#pragma unroll
    for (int j = 0; j < MX_PLANES; ++j) {  // integers in [-16, 16] are exact in E4M3: the conversion's rounding never acts
        int packed = __builtin_amdgcn_cvt_pk_fp8_f32(d[j][0], d[j][1], 0, false);
        packed = __builtin_amdgcn_cvt_pk_fp8_f32(d[j][2], d[j][3], packed, true);
        *reinterpret_cast<int *>(dig + (size_t)j * stride + b * 32 + 4 * sub) = packed;
    }
    if (sub < MX_PLANES)  // a NaN / inf block poisons every product it enters: scale byte 255 is NaN
        sb[(sub * 4 + (b & 3)) * ncp + (b >> 2)] = (uint8_t)(bad ? 255 : 127 + se + 5 * sub);
}

// ---- the product ----------------------------------------------------------------------
// A workgroup of NW wavefronts = RG groups of 16 weight rows x KS = NW / RG slices of K, against T
// activation rows (blockIdx.y picks which); it first rewrites those rows (all of K) as digit planes in
// LDS while its first weight loads are in flight.  Each wavefront then walks its K slice in batches of
// MX_U chunks, the next batch requested before the current one is consumed, and the partial tiles of
// the KS slices and the 5 planes are added through LDS in a fixed order.
// PAIRS (T = 1): blockIdx.y is a (token, expert) pair of an MoE layer: the weights are the pair's expert's entry of
// two pointer tables, the activation row is pair / div, the output row the pair.
struct mx_pairs {
    const uint8_t *const *qs_tab;
    const uint32_t *const *sc_tab;
    const int *expert_of;  // [pairs]
    int div;
};

template <int T, int RG, int NW, bool PAIRS = false>
__global__ __launch_bounds__(64 * NW) void mxfp4_rows_kernel(const uint8_t *__restrict__ qs_frag, const uint32_t *__restrict__ sc_frag,
                                                                  const float *__restrict__ x, float *__restrict__ y,
                                                                  int n_out, int nb, int ncp, int m, const mx_pairs pr) {
    static_assert(!PAIRS || T == 1, "a pair is one activation row");
    constexpr int KS = NW / RG, COLS = MX_PLANES * T;
    size_t x_row0 = (size_t)blockIdx.y * T;  // first activation row of this workgroup
    if (PAIRS) {
        const int expert = pr.expert_of[blockIdx.y];
        qs_frag = pr.qs_tab[expert];
        sc_frag = pr.sc_tab[expert];
        x_row0 = blockIdx.y / (unsigned)pr.div;
    }
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int kp = ncp * 128, stride = kp + 16;  // plane stride = 16 (mod 256): the 16 columns of a 128-bit read fall into 16 different bank groups
    char *const dig = lds;
    uint8_t *const sb = reinterpret_cast<uint8_t *>(lds + (size_t)COLS * stride);
    float *const part = reinterpret_cast<float *>(lds + (size_t)COLS * stride + (((size_t)COLS * 4 * ncp + 15) & ~(size_t)15));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rgi = wave / KS, ksi = wave % KS;
    const int nrg = (n_out + 15) / 16;
    int rg = blockIdx.x * RG + rgi;
    rg = rg < nrg ? rg : nrg - 1;  // a spare wavefront repeats the last group; its result is not stored
    const int cps = ((ncp + KS - 1) / KS + 3) & ~3;  // chunks per K slice, whole scale dwords
    const int c0 = ksi * cps, c1 = (c0 + cps < ncp) ? c0 + cps : ncp;
    const gv4i_ptr qa = (gv4i_ptr)(uintptr_t)qs_frag + (size_t)rg * ncp * 64 + lane;
    const uint32_t *__restrict__ sa = sc_frag + (size_t)rg * (ncp / 4) * 64 + lane;

    v4i abuf[2][MX_U];
    uint32_t sabuf[2][MX_U / 4];
    auto load_batch = [&](v4i (&a)[MX_U], uint32_t (&s)[MX_U / 4], int cb) {
#pragma unroll
        for (int u = 0; u < MX_U; ++u) {
            const int c = cb + u;
            a[u] = __builtin_nontemporal_load(qa + (size_t)pg_mx_chunk(c, ncp) * 64);
        }
#pragma unroll
        for (int g = 0; g < MX_U / 4; ++g) {
            const int c = cb + 4 * g;
            s[g] = sa[(size_t)pg_mx_scale_word(c, ncp) * 64];
        }
    };
    // Loads return in issue order: the activation blocks of the first rounds (from L2) are requested
    // before the weights (from HBM), so that the digit arithmetic runs while the weights are in flight.
    const int sub = threadIdx.x & 7, nblk = 4 * ncp;
    // (No branch around a load: behind one the compiler waits for every load in flight, the weights too.
    // Block ids past the end load the last block again.)
    const int last = T * nblk - 1;
    auto row_of = [&](int id) { return T == 1 ? 0 : (id >= nblk) + (T > 2 && id >= 2 * nblk); };  // id / nblk
    auto x_valid = [&](int id) {
        const int t = row_of(id), b = id - t * nblk;
        return b < nb && x_row0 + t < (size_t)m;  // blocks nb .. 4 ncp - 1 and rows past m are zeros
    };
    auto load_x = [&](int id) {
        const int t = row_of(id), b = id - t * nblk;
        const size_t at = x_valid(id) ? ((x_row0 + t) * nb + b) * 8 + sub : 0;
        return reinterpret_cast<const float4 *>(x)[at];
    };
    auto emit = [&](int id, const float4 v) {
        const int t = row_of(id), b = id - t * nblk;
        const bool keep = x_valid(id);
        const float f[4] = {keep ? v.x : 0.0f, keep ? v.y : 0.0f, keep ? v.z : 0.0f, keep ? v.w : 0.0f};
        mx_emit_digits(f, b, sub, dig + (size_t)t * MX_PLANES * stride, stride, sb + (size_t)t * MX_PLANES * 4 * ncp, ncp);
    };
    constexpr int PER_ROUND = 8 * NW;  // blocks per round: 8 threads each
    constexpr int NPRE = 4;                  // rounds whose activation blocks are requested ahead of the weights
    const int g0 = threadIdx.x >> 3;
    float4 xv[NPRE];
#pragma unroll
    for (int r = 0; r < NPRE; ++r) {
        const int id = g0 + r * PER_ROUND;
        xv[r] = load_x(id < last ? id : last);
    }
    asm volatile("" ::: "memory");  // (keeps the compiler from moving these loads down to their uses)
    __builtin_amdgcn_sched_barrier(0);
    load_batch(abuf[0], sabuf[0], c0 < ncp ? c0 : 0);  // (an empty slice consumes nothing)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < NPRE; ++r) {
        const int id = g0 + r * PER_ROUND;
        if (id <= last) emit(id, xv[r]);  // whole 8-thread groups together
    }
    for (int id = g0 + NPRE * PER_ROUND; id <= last; id += PER_ROUND) emit(id, load_x(id));
    asm volatile("s_waitcnt lgkmcnt(0)\n s_barrier" ::: "memory");  // (not __syncthreads(): the weight loads stay in flight)

    // B side of this lane: column min(lane % 16, COLS - 1) (the spare columns repeat the last one and are dropped)
    const int col = (lane & 15) < COLS ? (lane & 15) : COLS - 1, q = lane >> 4;
    const char *const bcol = dig + (size_t)col * stride + 16 * q;
    const uint8_t *const sbl = sb + (size_t)(col * 4 + q) * ncp;
    v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
    auto consume = [&](const v4i (&a)[MX_U], const uint32_t (&s)[MX_U / 4], int cb) {
#pragma unroll
        for (int g = 0; g < MX_U / 4; ++g) {
            if (cb + 4 * g < c1) {  // the same for the whole wavefront
                const int sbv = *reinterpret_cast<const int *>(sbl + cb + 4 * g);
                const char *bp = bcol + (size_t)(cb + 4 * g) * 128;
                // (the byte selectors of the two scale operands are immediates)
#define PG_MX_STEP(U)                                                                                                   \
    do {                                                                                                                \
        const v4i b0 = *reinterpret_cast<const v4i *>(bp + (U) * 128), b1 = *reinterpret_cast<const v4i *>(bp + (U) * 128 + 64); \
        const v4i aw = a[4 * g + (U)];                                                                                  \
        const v8i A = {aw[0], aw[1], aw[2], aw[3], 0, 0, 0, 0};                                                         \
        const v8i B = {b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};                                         \
        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, acc, 4, 0, (U), (int)s[g], (U), sbv);              \
    } while (0)
                PG_MX_STEP(0);
                PG_MX_STEP(1);
                PG_MX_STEP(2);
                PG_MX_STEP(3);
#undef PG_MX_STEP
            }
        }
    };
    for (int cb = c0; cb < c1; cb += 2 * MX_U) {
        if (cb + MX_U < c1) load_batch(abuf[1], sabuf[1], cb + MX_U);
        __builtin_amdgcn_sched_barrier(0);
        consume(abuf[0], sabuf[0], cb);
        if (cb + 2 * MX_U < c1) load_batch(abuf[0], sabuf[0], cb + 2 * MX_U);
        __builtin_amdgcn_sched_barrier(0);
        if (cb + MX_U < c1) consume(abuf[1], sabuf[1], cb + MX_U);
    }

    // part[wave][lane][r]: column lane % 16, row 4 (lane / 16) + r of this wavefront's tile
    *reinterpret_cast<v4f *>(part + ((size_t)wave * 64 + lane) * 4) = acc;
    __syncthreads();
    if (threadIdx.x < RG * 16 * T) {
        const int t = threadIdx.x / (RG * 16), rr = threadIdx.x % (RG * 16), g = rr / 16, i = rr % 16;
        float sum = 0.0f;
#pragma unroll
        for (int j = MX_PLANES - 1; j >= 0; --j)
#pragma unroll
            for (int k = 0; k < KS; ++k)
                sum += part[((size_t)(g * KS + k) * 64 + 16 * (i >> 2) + t * MX_PLANES + j) * 4 + (i & 3)];
        const size_t row = ((size_t)blockIdx.x * RG + g) * 16 + i, item = (size_t)blockIdx.y * T + t;  // (PAIRS: the pair)
        if (row < (size_t)n_out && (PAIRS || item < (size_t)m)) y[item * n_out + row] = sum;
    }
}

size_t mx_lds_bytes(int t, int ncp, int nw = 16) {
    const size_t cols = (size_t)MX_PLANES * t;
    return cols * ((size_t)ncp * 128 + 16) + ((cols * 4 * ncp + 15) & ~(size_t)15) + (size_t)nw * 64 * 4 * sizeof(float);
}

template <int T, int RG, int NW>
pg_status launch_rows(pg_ctx *ctx, const pg_gguf_tensor *w, const float *x, float *y, size_t m, int ncp) {
    const size_t lds = mx_lds_bytes(T, ncp, NW);
    auto kern = mxfp4_rows_kernel<T, RG, NW>;
    PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));
    const dim3 grid(grid_for((w->n_out + 15) / 16, RG), grid_for(m, T));
    return pg_launch(ctx, "mxfp4_rows", kern, grid, dim3(64 * NW), lds, (const uint8_t *)w->qs,
                     reinterpret_cast<const uint32_t *>(w->d), x, y, (int)w->n_out, (int)(w->k_in / 32), ncp, (int)m, mx_pairs{});
}

// One launch for `pairs` (token, expert) pairs: pair p = row p / div of x against expert expert_of[p]; x has x_rows rows.
template <int RG, int NW>
pg_status launch_rows_pairs(pg_ctx *ctx, size_t n_out, size_t k_in, const float *x, size_t x_rows, float *y, size_t pairs, int ncp,
                            const mx_pairs &pr) {
    const size_t lds = mx_lds_bytes(1, ncp, NW);
    auto kern = mxfp4_rows_kernel<1, RG, NW, true>;
    PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));
    const dim3 grid(grid_for((n_out + 15) / 16, RG), (unsigned)pairs);
    return pg_launch(ctx, "mxfp4_rows_pairs", kern, grid, dim3(64 * NW), lds, (const uint8_t *)nullptr, (const uint32_t *)nullptr, x, y,
                     (int)n_out, (int)(k_in / 32), ncp, (int)x_rows, pr);
}

}  // namespace

// y[m, n_out] = x[m, k_in] . W^T for an MXFP4 tensor; x 16-byte aligned.
pg_status pg_launch_mxfp4_rows(pg_ctx *ctx, const float *x_dev, size_t m, const pg_gguf_tensor *w, float *y_dev) {
    if (m == 0) return PG_OK;
    const int nb = (int)(w->k_in / 32), ncp = (int)mx_chunks((size_t)nb);
    int t = m < (size_t)MX_MAX_T ? (int)m : MX_MAX_T;
    while (t > 1 && mx_lds_bytes(t, ncp) > (96u << 10)) --t;  // room for a second workgroup per CU
    if (mx_lds_bytes(t, ncp) > (160u << 10))
        return pg_fail(PG_EUNSUPPORTED, "mxfp4: k_in %zu does not fit the digit planes in LDS (up to 28160)", w->k_in);
    if ((m + t - 1) / t > 65535) return pg_fail(PG_EUNSUPPORTED, "mxfp4: more than %d activation rows", 65535 * t);
    // Every workgroup rewrites the activation rows as digits, so the fewer workgroups the less of that work.
    // Up to one group of 16 weight rows per CU: 16 wavefronts on it, K in 16 slices.  Beyond: 8 wavefronts
    // with the fewest row groups per workgroup (1, 2 or 4; K in 8, 4 or 2 slices) with which all
    // workgroups are resident at once (two per CU), four past that.
    const size_t groups = (w->n_out + 15) / 16 * ((m + t - 1) / t), slots = (size_t)ctx->num_cu * 2;
    const int shape = groups <= (size_t)ctx->num_cu ? 0 : (groups <= slots ? 1 : ((groups + 1) / 2 <= slots ? 2 : 4));
#define PG_MX_LAUNCH(TT)                                                                                              \
    (shape == 0 ? launch_rows<TT, 1, 16>(ctx, w, x_dev, y_dev, m, ncp)                                                \
     : shape == 1 ? launch_rows<TT, 1, 8>(ctx, w, x_dev, y_dev, m, ncp)                                               \
     : shape == 2 ? launch_rows<TT, 2, 8>(ctx, w, x_dev, y_dev, m, ncp) : launch_rows<TT, 4, 8>(ctx, w, x_dev, y_dev, m, ncp))
    switch (t) {
        case 1: return PG_MX_LAUNCH(1);
        case 2: return PG_MX_LAUNCH(2);
        default: return PG_MX_LAUNCH(3);
    }
#undef PG_MX_LAUNCH
}

namespace {

// ---- many activation rows: tiles on the scaled matrix-core instruction ------------------------
// From a few dozen rows on the product is matrix-core work, and the instruction still does all of it: the block
// scales of both sides are applied inside, so there is no rescaling of accumulators and nothing to dequantise.
// An activation block becomes MT_PLANES balanced base-32 digits per value (20 bits under the block's largest
// magnitude, |error| <= 2^-20 of it), each plane a B operand whose block scale carries the digit's weight; the
// planes accumulate into the same tile, so a row costs MT_PLANES instructions per 16 x 16 x 128 tile and no
// final sum.  A pre-pass writes the planes once, in the operand's own fragment order: per token group of 16
// and chunk of 128 k one record of MT_RECORD bytes,
//   [plane][half][64 lanes][16 B]   lane = token % 16 + 16 q holds k = 64 half + 16 q .. + 15 of the chunk
//   [64 lanes] scale dwords         lane = token % 16 + 16 (block of the chunk), byte j = plane j
constexpr int MT_PLANES = PG_MT_PLANES;
constexpr int MT_NW = PG_MT_NW;            // wavefronts per workgroup
constexpr int MT_FRAG = PG_MT_FRAG;        // bytes of one plane fragment
constexpr int MT_RECORD = PG_MT_RECORD;    // one token group's planes and scales of a chunk
constexpr int MT_UNITS = MT_RECORD / 16;   // in 16-byte units

// Experts' token lists, for the grouped products of an MoE layer: the token tiles (TB groups of 16 slots) of all
// experts follow one another, expert e's from tile goff[e]; slot i of an expert holds pair lists[e * stride + i].
struct mt_gather {
    const int *lists, *counts, *goff;  // [E][stride], [E], [E + 1]
    int stride, experts, tb, div;      // row of the source matrix = pair / div
};
// the expert whose tiles include token tile gt (gt < goff[experts])
__device__ __forceinline__ int mt_expert_of(const mt_gather &g, int gt) {
    int lo = 0, hi = g.experts;
    while (lo + 1 < hi) {
        const int mid = (lo + hi) >> 1;
        if (g.goff[mid] <= gt) lo = mid;
        else hi = mid;
    }
    return lo;
}

// First token tile of every expert: goff[e] = sum over e' < e of ceil(counts[e'] / (16 tb)); goff[experts] = all.
__global__ __launch_bounds__(64) void mxfp4_tile_offsets_kernel(const int *__restrict__ counts, int experts, int tb, int *__restrict__ goff) {
    if (threadIdx.x != 0) return;
    int run = 0;
    for (int e = 0; e < experts; ++e) {
        goff[e] = run;
        run += (counts[e] + 16 * tb - 1) / (16 * tb);
    }
    goff[experts] = run;
}

// One thread = 16 consecutive k of one token (half a block).  A wavefront = the 16 tokens of a group x two blocks x
// their halves, tokens on consecutive lanes: what it writes are whole 256-byte runs of the records, and the
// 256 bytes it reads of every token row are two full lines.
// GATHER: the token groups are the experts' slots (mt_gather) instead of the rows in order.
template <bool GATHER>
__global__ __launch_bounds__(256) void mxfp4_planes_kernel(const float *__restrict__ x, int m, int nb, int ncp, int token_groups,
                                                           char *__restrict__ bq, const mt_gather gat) {
    const size_t wv = ((size_t)blockIdx.x * 256 + threadIdx.x) >> 6;  // (token group, pair of blocks)
    const int lane = threadIdx.x & 63, col = lane & 15, sub = (lane >> 4) & 1, npair = 2 * ncp;
    const size_t tg = wv / npair;
    if (tg >= (size_t)token_groups) return;  // (whole wavefronts)
    const int b = 2 * (int)(wv % npair) + (lane >> 5);
    size_t t = tg * 16 + col;
    bool valid = t < (size_t)m && b < nb;
    if (GATHER) {
        const int gt = (int)(tg / gat.tb);
        if (gt >= gat.goff[gat.experts]) return;  // past the last expert's tiles (whole wavefronts)
        const int e = mt_expert_of(gat, gt);
        const int slot = ((gt - gat.goff[e]) * gat.tb + (int)(tg % gat.tb)) * 16 + col;
        valid = slot < gat.counts[e] && b < nb;
        t = valid ? (size_t)(gat.lists[(size_t)e * gat.stride + slot] / gat.div) : 0;
    }
    float f[16];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (valid) v = reinterpret_cast<const float4 *>(x)[(t * nb + b) * 8 + sub * 4 + e];
        f[4 * e] = v.x; f[4 * e + 1] = v.y; f[4 * e + 2] = v.z; f[4 * e + 3] = v.w;
    }
    float amax = 0.0f;
    int bad = 0;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        amax = fmaxf(amax, fabsf(f[e]));
        bad |= f[e] != f[e];
    }
    amax = fmaxf(amax, __shfl_xor(amax, 16, 64));  // the block's other half
    bad |= __shfl_xor(bad, 16, 64);
    int se = 0;
    float inv = 1.0f;
    if (bad || !(amax <= 3.4028234663852886e38f)) {
        bad = 1;
        inv = 0.0f;
    } else if (amax > 0.0f) {
        int ex;
        (void)frexpf(amax, &ex);          // amax = f * 2^ex, f in [0.5, 1)
        se = ex - (5 * MT_PLANES - 1);    // |x| / 2^se < 2^19 <= 16 (1 + 32 + 32^2 + 32^3)
        if (se < -126) se = -126;
        inv = ldexpf(1.0f, -se);
    }
    // Balanced base-32 digits, top down and all in f32 (every value is a small integer times a power of two, so
    // each step is exact): n_j = round(r / 32^j), r -= n_j 32^j; |n_j| <= 16.  Small integers keep the
    // instruction's own sum over k exact, which numbers spread over the format's exponent range do not (a split
    // into E4M3 values of decreasing size, four significant bits a plane, stopped at 2e-4 of the output's rms
    // however many planes it was given).
    int packed[MT_PLANES][4];
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
        float r[4], d[MT_PLANES][4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float tt = f[4 * e4 + e] * inv;
            r[e] = (tt != tt) ? 0.0f : rintf(tt);
        }
#pragma unroll
        for (int j = MT_PLANES - 1; j >= 1; --j) {
            const float down = __builtin_bit_cast(float, (127 - 5 * j) << 23), up = -__builtin_bit_cast(float, (127 + 5 * j) << 23);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                d[j][e] = rintf(r[e] * down);
                r[e] = fmaf(d[j][e], up, r[e]);
            }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) d[0][e] = r[e];
#pragma unroll
        for (int j = 0; j < MT_PLANES; ++j) {  // integers in [-16, 16] are exact in E4M3
            int pk = __builtin_amdgcn_cvt_pk_fp8_f32(d[j][0], d[j][1], 0, false);
            packed[j][e4] = __builtin_amdgcn_cvt_pk_fp8_f32(d[j][2], d[j][3], pk, true);
        }
    }
#pragma unroll
    for (int j = 0; j < MT_PLANES; ++j)
        *reinterpret_cast<v4i *>(bq + pg_mt_plane_store(tg, ncp, b, sub, col, j)) = v4i{packed[j][0], packed[j][1], packed[j][2], packed[j][3]};
    if (sub == 0) {  // a NaN / inf block poisons every product it enters: scale byte 255 is NaN
        unsigned word = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) word |= (unsigned)(j >= MT_PLANES ? 127 : (bad ? 255 : 127 + se + 5 * j)) << (8 * j);
        *reinterpret_cast<unsigned *>(bq + pg_mt_scale_store(tg, ncp, b, col)) = word;
    }
}

// A workgroup = MT_NW wavefronts x RA groups of 16 weight rows, against TB groups of 16 tokens, over one run of
// chunks (all of K, or one of `ks` runs whose partial tiles a later launch adds).  The weights go from memory
// straight into the A operand's registers (each wavefront streams its own rows: two chunks ahead for the widest
// row tile, a batch of four chunks ahead otherwise); the token records of a chunk are shared through LDS (staged
// through registers BD chunks ahead, two stages, one barrier per chunk).  Narrow tiles do little arithmetic per
// chunk, so what they need is requests in flight: the deeper staging is theirs.
// GROUPED: the token tiles are the experts' (mt_gather), the weights come from the expert's entry of two pointer
// tables, an output row is the pair the slot holds; one run of K; items walk the row tiles of one token tile first
// (that tile's records stay in the XCD's L2).
struct mt_experts {
    const uint8_t *const *qs_tab;
    const uint32_t *const *sc_tab;
};

template <int RA, int TB, int BD, bool GROUPED>
__global__ __launch_bounds__(64 * MT_NW) void mxfp4_tiles_kernel(const uint8_t *__restrict__ qs_frag, const uint32_t *__restrict__ sc_frag,
                                                                 const char *__restrict__ bq, float *__restrict__ y, int n_out,
                                                                 int ncp, int m, int n_tt, int ks, int cps, size_t part_stride,
                                                                 int items, int per_xcd, const mt_gather gat, const mt_experts ex) {
    constexpr int STAGE = TB * MT_RECORD, UNITS = TB * MT_UNITS, ROUNDS = (UNITS + 64 * MT_NW - 1) / (64 * MT_NW);
    constexpr bool RING = RA == 4;  // A two chunks ahead in a ring of two; else the next batch of four chunks
    static_assert(BD == 1 || BD == 2 || BD == 4, "the staging depth divides the unrolled batch");
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // every XCD (workgroup id % 8) walks its own run of work items, token tiles of one row tile and K run first:
    // that run's weights stay in the XCD's L2 while its token tiles pass
    const int item = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per_xcd || item >= items) return;
    int tt = item % n_tt, split = (item / n_tt) % ks, wt = item / (n_tt * ks), expert = 0, live = TB;
    if (GROUPED) {  // n_tt = the row tiles here; token tile 8 i + x belongs to XCD x (the unused tail tiles spread evenly)
        const int slot = (int)(blockIdx.x >> 3);
        wt = slot % n_tt;
        tt = (slot / n_tt) * 8 + (int)(blockIdx.x & 7);
        split = 0;
        if (tt >= gat.goff[gat.experts]) return;
        expert = mt_expert_of(gat, tt);
        qs_frag = ex.qs_tab[expert];
        sc_frag = ex.sc_tab[expert];
        // an expert's last tile is rarely full: token groups without a slot in use are skipped (their records hold zeros)
        const int left = gat.counts[expert] - (tt - gat.goff[expert]) * TB * 16;
        live = __builtin_amdgcn_readfirstlane(left >= TB * 16 ? TB : (left + 15) / 16);
    }
    const int kc0 = split * cps, kc1 = pg_mt_run_end(split, cps, ncp);  // whole batches of four chunks
    const int nrg = (n_out + 15) / 16;                       // >= RA (the launcher's choice of RA)
    const int rg_mine = (wt * MT_NW + wave) * RA;            // the row groups whose tiles this wavefront stores
    const int rg0 = pg_mt_first_row_group(rg_mine, RA, nrg);  // the ones it reads: a spare wavefront repeats the last ones
    const size_t a_stride = (size_t)ncp * 64;                // v4i per row group
    const gv4i_ptr qa = (gv4i_ptr)(uintptr_t)qs_frag + (size_t)rg0 * a_stride;
    const uint32_t *const sa = sc_frag + (size_t)rg0 * (ncp / 4) * 64;
    // this thread's share of a chunk's records: 16-byte unit u of the TB records, which lie ncp records apart
    const char *const b_base = bq + (size_t)tt * TB * ncp * MT_RECORD;
    unsigned b_off[ROUNDS];
#pragma unroll
    for (int i = 0; i < ROUNDS; ++i) b_off[i] = pg_mt_unit_offset((int)threadIdx.x + i * 64 * MT_NW, UNITS, ncp);
    v4i sr[BD][ROUNDS];
#define PG_MT_FETCH_B(SLOT, C)                                                                                          \
    do {                                                                                                                \
        _Pragma("unroll") for (int i = 0; i < ROUNDS; ++i)                                                              \
            sr[SLOT][i] = *reinterpret_cast<const v4i *>(b_base + b_off[i] + (unsigned)(C) * MT_RECORD);                \
    } while (0)
#define PG_MT_PUT_B(STG, SLOT)                                                                                          \
    do {                                                                                                                \
        _Pragma("unroll") for (int i = 0; i < ROUNDS; ++i) {                                                            \
            const int u = (int)threadIdx.x + i * 64 * MT_NW;                                                            \
            if (u < UNITS) *reinterpret_cast<v4i *>(lds + (STG) * STAGE + u * 16) = sr[SLOT][i];                        \
        }                                                                                                               \
    } while (0)
    v4i a[RING ? 2 : 4][RA], an[RING ? 1 : 4][RA];
    uint32_t sca[RA], sca_next[RA];
    auto fetch_a = [&](v4i (&dst)[RA], int c) {
#pragma unroll
        for (int r = 0; r < RA; ++r) dst[r] = __builtin_nontemporal_load(qa + (size_t)r * a_stride + (size_t)c * 64 + lane);
    };
    v4f acc[RA][TB];
#pragma unroll
    for (int r = 0; r < RA; ++r)
#pragma unroll
        for (int g = 0; g < TB; ++g) acc[r][g] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    PG_MT_FETCH_B(0, kc0);
    if (BD > 1) PG_MT_FETCH_B(BD > 1 ? 1 : 0, kc0 + 1);
    if (BD > 2) {
        PG_MT_FETCH_B(BD > 2 ? 2 : 0, kc0 + 2);
        PG_MT_FETCH_B(BD > 2 ? 3 : 0, kc0 + 3);
    }
#pragma unroll
    for (int u = 0; u < (RING ? 2 : 4); ++u) fetch_a(a[u], kc0 + u);
#pragma unroll
    for (int r = 0; r < RA; ++r) sca[r] = sa[((size_t)r * (ncp / 4) + (kc0 >> 2)) * 64 + lane];
    PG_MT_PUT_B(0, 0);
    if (kc0 + BD < kc1) PG_MT_FETCH_B(0, kc0 + BD);
    __syncthreads();
    for (int cb = kc0; cb < kc1; cb += 4) {
        const bool more = cb + 4 < kc1;
        if (more) {
#pragma unroll
            for (int r = 0; r < RA; ++r) sca_next[r] = sa[((size_t)r * (ncp / 4) + (cb >> 2) + 1) * 64 + lane];
            if (!RING) {
#pragma unroll
                for (int u = 0; u < 4; ++u) fetch_a(an[RING ? 0 : u], cb + 4 + u);
            }
        }
    // One plane of one token group: its two operand halves are read while the previous plane's instructions run.
    // (The byte selectors of the two scale operands are immediates: chunk within the dword, plane within the dword.)
#define PG_MT_READ(G, J, B0, B1)                                                                  \
    do {                                                                                          \
        B0 = *reinterpret_cast<const v4i *>(st + (G) * MT_RECORD + (J) * MT_FRAG + lane * 16);      \
        B1 = *reinterpret_cast<const v4i *>(st + (G) * MT_RECORD + (J) * MT_FRAG + 1024 + lane * 16); \
    } while (0)
#define PG_MT_MUL(U, G, J, B0, B1)                                                                                          \
    do {                                                                                                                    \
        const v8i B = {B0[0], B0[1], B0[2], B0[3], B1[0], B1[1], B1[2], B1[3]};                                             \
        _Pragma("unroll") for (int r = 0; r < RA; ++r) {                                                                    \
            const v4i aw = a[RING ? (U) & 1 : (U)][r];                                                                      \
            const v8i A = {aw[0], aw[1], aw[2], aw[3], 0, 0, 0, 0};                                                         \
            acc[r][G] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, acc[r][G], 4, 0, (U), (int)sca[r], (J), sbv[G]); \
            asm volatile("" : "+v"(acc[r][G]));  /* (or the compiler sinks every product to the end of the loop body) */  \
        }                                                                                                                   \
    } while (0)
#define PG_MT_GROUP(U, G)                                                 \
    do {                                                                  \
        if ((G) < TB && (!GROUPED || (G) < live)) {                       \
            PG_MT_READ(G, 1, y0, y1);                                     \
            PG_MT_MUL(U, G, 0, x0, x1);                                   \
            __builtin_amdgcn_sched_barrier(0);                            \
            PG_MT_READ(G, 2, x0, x1);                                     \
            PG_MT_MUL(U, G, 1, y0, y1);                                   \
            __builtin_amdgcn_sched_barrier(0);                            \
            PG_MT_READ(G, 3, y0, y1);                                     \
            PG_MT_MUL(U, G, 2, x0, x1);                                   \
            __builtin_amdgcn_sched_barrier(0);                            \
            if ((G) + 1 < TB) PG_MT_READ((G) + 1 < TB ? (G) + 1 : 0, 0, x0, x1); \
            PG_MT_MUL(U, G, 3, y0, y1);                                   \
            __builtin_amdgcn_sched_barrier(0);                            \
        }                                                                 \
    } while (0)
#define PG_MT_CHUNK(U)                                                                                   \
    do {                                                                                                 \
        const int c = cb + (U);                                                                          \
        const char *st = lds + ((U) & 1) * STAGE;                                                        \
        int sbv[TB];                                                                                     \
        _Pragma("unroll") for (int g = 0; g < TB; ++g)                                                   \
            sbv[g] = *reinterpret_cast<const int *>(st + g * MT_RECORD + MT_PLANES * MT_FRAG + lane * 4); \
        v4i x0, x1, y0, y1;                                                                              \
        PG_MT_READ(0, 0, x0, x1);                                                                        \
        __builtin_amdgcn_sched_barrier(0);                                                               \
        PG_MT_GROUP(U, 0);                                                                               \
        PG_MT_GROUP(U, 1);                                                                               \
        PG_MT_GROUP(U, 2);                                                                               \
        PG_MT_GROUP(U, 3);                                                                               \
        if (c + 1 < kc1) {                                                                               \
            PG_MT_PUT_B(((U) + 1) & 1, ((U) + 1) % BD);                                                  \
            if (c + 1 + BD < kc1) PG_MT_FETCH_B(((U) + 1) % BD, c + 1 + BD);                             \
        }                                                                                                \
        if (RING && c + 2 < kc1) fetch_a(a[RING ? (U) & 1 : 0], c + 2);                                  \
        __syncthreads();                                                                                 \
    } while (0)
        static_assert(MT_PLANES == 4 && TB <= 4, "the plane steps are written out");
        PG_MT_CHUNK(0);
        PG_MT_CHUNK(1);
        PG_MT_CHUNK(2);
        PG_MT_CHUNK(3);
#undef PG_MT_CHUNK
#undef PG_MT_GROUP
#undef PG_MT_MUL
#undef PG_MT_READ
        if (more) {
#pragma unroll
            for (int r = 0; r < RA; ++r) sca[r] = sca_next[r];
            if (!RING) {
#pragma unroll
                for (int u = 0; u < 4; ++u)
#pragma unroll
                    for (int r = 0; r < RA; ++r) a[RING ? 0 : u][r] = an[RING ? 0 : u][r];
            }
        }
    }
#undef PG_MT_FETCH_B
#undef PG_MT_PUT_B
    // D: lane holds token lane % 16 of its group, weight rows 4 (lane / 16) .. + 3 of the row group
    float *const out = y + (size_t)split * part_stride;
#pragma unroll
    for (int r = 0; r < RA; ++r) {
        if (rg_mine != rg0 && rg0 + r < rg_mine) continue;   // rows a spare wavefront only repeated
        if (rg_mine >= nrg) continue;
        const size_t row = (size_t)(rg0 + r) * 16 + 4 * (lane >> 4);
#pragma unroll
        for (int g = 0; g < TB; ++g) {
            size_t token = ((size_t)tt * TB + g) * 16 + (lane & 15);
            if (GROUPED) {
                const int slot = ((tt - gat.goff[expert]) * TB + g) * 16 + (lane & 15);
                if (slot >= gat.counts[expert]) continue;
                token = (size_t)gat.lists[(size_t)expert * gat.stride + slot];
            } else if (token >= (size_t)m) {
                continue;
            }
            float *o = out + token * n_out + row;
            if (row + 3 < (size_t)n_out && (n_out & 3) == 0) {
                *reinterpret_cast<v4f *>(o) = acc[r][g];
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (row + i < (size_t)n_out) o[i] = acc[r][g][i];
            }
        }
    }
}

using mt_plan = pg_mxfp4_tiles_plan;

template <int RA, int TB, int BD>
pg_status launch_tiles(pg_ctx *ctx, const pg_gguf_tensor *w, const char *bq, float *y, size_t m, int ncp, const mt_plan &p) {
    const size_t lds = 2 * (size_t)TB * MT_RECORD;
    auto kern = mxfp4_tiles_kernel<RA, TB, BD, false>;
    PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));
    const size_t items = p.n_wt * p.n_tt * p.ks, per_xcd = (items + 7) / 8;
    return pg_launch(ctx, "mxfp4_tiles", kern, dim3((unsigned)(8 * per_xcd)), dim3(64 * MT_NW), lds, (const uint8_t *)w->qs,
                     reinterpret_cast<const uint32_t *>(w->d), bq, y, (int)w->n_out, ncp, (int)m, (int)p.n_tt, p.ks, p.cps,
                     m * w->n_out, (int)items, (int)per_xcd, mt_gather{}, mt_experts{});
}

// The grouped form: `max_tiles` token tiles at most (the launch covers them all; those past the experts' last exit).
template <int RA, int TB, int BD>
pg_status launch_tiles_grouped(pg_ctx *ctx, size_t n_out, int ncp, const char *bq, float *y, size_t n_wt, size_t max_tiles,
                               const mt_gather &gat, const mt_experts &ex) {
    const size_t lds = 2 * (size_t)TB * MT_RECORD;
    auto kern = mxfp4_tiles_kernel<RA, TB, BD, true>;
    PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));
    const size_t per_xcd = (max_tiles + 7) / 8 * n_wt, items = 8 * per_xcd;
    return pg_launch(ctx, "mxfp4_tiles_grouped", kern, dim3((unsigned)(8 * per_xcd)), dim3(64 * MT_NW), lds, (const uint8_t *)nullptr,
                     (const uint32_t *)nullptr, bq, y, (int)n_out, ncp, 0, (int)n_wt, 1, ncp, (size_t)0, (int)items, (int)per_xcd, gat, ex);
}

}  // namespace

// The tile shape and K split for m rows of an [n_out, 32 nb] tensor: the widest row tile that still gives every CU a
// workgroup (and no wider than the tensor); with the narrowest still short of that, K in runs of at least 8 chunks.
pg_mxfp4_tiles_plan pg_mxfp4_tiles_plan_for(int num_cu, size_t n_out, size_t m, int ncp) {
    pg_mxfp4_tiles_plan p;
    p.tb = m <= 16 ? 1 : (m <= 32 ? 2 : 4);
    p.n_tt = (m + 16 * p.tb - 1) / (16 * p.tb);
    p.groups = p.n_tt * p.tb;
    const size_t nrg = (n_out + 15) / 16;
    p.ra = 4;
    while (p.ra > 1 && ((size_t)p.ra > nrg || (nrg + MT_NW * p.ra - 1) / (MT_NW * p.ra) * p.n_tt < (size_t)num_cu)) p.ra >>= 1;
    p.n_wt = (nrg + MT_NW * p.ra - 1) / (MT_NW * p.ra);
    const size_t tiles = p.n_wt * p.n_tt;
    p.ks = 1;
    if (tiles < (size_t)num_cu) p.ks = (int)std::min<size_t>(std::min<size_t>((size_t)num_cu / tiles, (size_t)ncp / 8), 16);
    if (p.ks < 1) p.ks = 1;
    p.cps = ((ncp / 4 + p.ks - 1) / p.ks) * 4;       // chunks per run: whole batches of four
    p.ks = (ncp + p.cps - 1) / p.cps;                // (no empty run)
    return p;
}

// Whether the tile kernel takes `m` activation rows of this tensor (otherwise the decode kernel's passes of three
// rows): from 16 rows, or 24 for a tensor under 2^25 weights, whose passes are short.
bool pg_mxfp4_tiles_takes(const pg_gguf_tensor *w, size_t m) {
    return w->ggml_type == PG_MXFP4 && m >= (w->n_out * w->k_in >= ((size_t)1 << 25) ? 16u : 24u) && m < ((size_t)1 << 27) &&
           w->n_out < ((size_t)1 << 27);
}

// y[m, n_out] = x[m, k_in] . W^T for an MXFP4 tensor over many rows; x 16-byte aligned.
pg_status pg_launch_mxfp4_tiles(pg_ctx *ctx, const float *x_dev, size_t m, const pg_gguf_tensor *w, float *y_dev) {
    const int nb = (int)(w->k_in / 32), ncp = (int)mx_chunks((size_t)nb);
    const mt_plan p = pg_mxfp4_tiles_plan_for(ctx->num_cu, w->n_out, m, ncp);
    PG_CHECK_ARG(p.n_wt * p.n_tt * p.ks < ((size_t)1 << 28), "mxfp4: %zu x %zu tiles", p.n_wt, p.n_tt);
    void *ws = nullptr;
    const size_t sz_b = pg_round_up(p.groups * ncp * (size_t)MT_RECORD, 256);
    const size_t sz_part = p.ks > 1 ? (size_t)p.ks * m * w->n_out * sizeof(float) : 0;
    PG_TRY(pg_workspace(ctx, sz_b + sz_part, &ws));
    char *bq = static_cast<char *>(ws);
    float *part = p.ks > 1 ? reinterpret_cast<float *>(bq + sz_b) : y_dev;
    const size_t threads = p.groups * 2 * (size_t)ncp * 64;  // a wavefront per token group and pair of blocks
    PG_CHECK_ARG((threads + 255) / 256 < ((size_t)1 << 31), "mxfp4: %zu rows x %zu is too much for one pre-pass", m, w->k_in);
    PG_TRY(pg_launch(ctx, "mxfp4_planes", mxfp4_planes_kernel<false>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, x_dev, (int)m, nb,
                     ncp, (int)p.groups, bq, mt_gather{}));
    // the staging depth: the less arithmetic a chunk holds, the more chunks ahead
#define PG_MT_LAUNCH(RA_, BD1, BD2, BD4) \
    (p.tb == 1 ? launch_tiles<RA_, 1, BD1>(ctx, w, bq, part, m, ncp, p) \
     : p.tb == 2 ? launch_tiles<RA_, 2, BD2>(ctx, w, bq, part, m, ncp, p) \
                 : launch_tiles<RA_, 4, BD4>(ctx, w, bq, part, m, ncp, p))
    PG_TRY(p.ra == 4 ? PG_MT_LAUNCH(4, 4, 2, 1) : (p.ra == 2 ? PG_MT_LAUNCH(2, 4, 4, 2) : PG_MT_LAUNCH(1, 4, 4, 4)));
#undef PG_MT_LAUNCH
    if (p.ks > 1) PG_TRY(pg_launch_sum_parts(ctx, part, m * w->n_out, p.ks, m * w->n_out, y_dev));
    return PG_OK;
}

// ---- ABI --------------------------------------------------------------------------------
// A block is 16 bytes of FP4 (E2M1) codes, byte k = elements 2k (low nibble) and 2k+1, plus
// one E8M0 scale byte: value = LUT[code] * 2^(scale - 127)   (examples/gpt_oss/moe.rs:5-53).
PG_API pg_status pg_mxfp4_upload(pg_ctx *ctx, const uint8_t *blocks, const uint8_t *scales, size_t out_dim,
                                 size_t in_dim, pg_gguf_tensor **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(out != nullptr, "pg_mxfp4_upload: out is null");
    *out = nullptr;
    PG_CHECK_ARG(out_dim > 0 && in_dim > 0 && blocks && scales, "pg_mxfp4_upload: empty tensor or null pointer");
    PG_CHECK_ARG(in_dim % 32 == 0, "pg_mxfp4_upload: in_dim %zu is not a multiple of 32", in_dim);
    PG_CHECK_ARG(out_dim < (1ull << 31) && in_dim < (1ull << 31) && out_dim * (in_dim / 32) < (1ull << 31),
                 "pg_mxfp4_upload: shape too large");
    const size_t nb = in_dim / 32, nblocks = out_dim * nb;
    const size_t ncp = mx_chunks(nb), nrg = (out_dim + 15) / 16;
    pg_gguf_tensor *t = new (std::nothrow) pg_gguf_tensor();
    if (!t) return pg_fail(PG_ENOMEM, "host allocation failed");
    t->qs = nullptr;
    t->d = nullptr;
    t->m = nullptr;
    t->qs_tiled = nullptr;
    t->ggml_type = PG_MXFP4;
    t->n_out = out_dim;
    t->k_in = in_dim;
    pg_tmp rb, rs;
    pg_status st = rb.alloc(nblocks * 16);
    if (st == PG_OK) st = rs.alloc(nblocks);
    hipError_t e = hipSuccess;
    if (st == PG_OK) {
        e = hipMalloc((void **)&t->qs, nrg * ncp * 64 * 16);
        if (e == hipSuccess) e = hipMalloc((void **)&t->d, nrg * (ncp / 4) * 64 * 4);
        if (e == hipSuccess) e = hipMemcpyAsync(rb.p, blocks, nblocks * 16, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) e = hipMemcpyAsync(rs.p, scales, nblocks, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) {
            mxfp4_fragments_kernel<<<grid_for(nrg * ncp * 64, 256), 256, 0, ctx->stream>>>(
                rb.as<uint8_t>(), rs.as<uint8_t>(), (int)out_dim, (int)nb, (int)ncp, reinterpret_cast<uint4 *>(t->qs),
                reinterpret_cast<uint8_t *>(t->d));
            e = hipGetLastError();
        }
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess)
            st = pg_fail(e == hipErrorOutOfMemory ? PG_ENOMEM : PG_EDEVICE, "pg_mxfp4_upload: %s", hipGetErrorString(e));
    }
    if (st != PG_OK) { pg_gguf_free(ctx, t); return st; }
    *out = t;
    return PG_OK;
}

PG_API pg_status pg_mxfp4_matmul(pg_ctx *ctx, const float *input, const uint8_t *blocks, const uint8_t *scales,
                                 size_t out_dim, size_t in_dim, float *output) {
    pg_gguf_tensor *t = nullptr;
    PG_TRY(pg_mxfp4_upload(ctx, blocks, scales, out_dim, in_dim, &t));
    const pg_status st = pg_gguf_matmul(ctx, input, 1, t, output);
    pg_gguf_free(ctx, t);
    return st;
}

// Mxfp4Expert  examples/gpt_oss/moe.rs:55-117, swiglu :145-154.
struct pg_mxfp4_expert {
    pg_gguf_tensor *mlp1, *mlp2;  // [2 * intermediate, hidden], [hidden, intermediate]
    float *bias1, *bias2;         // [2 * intermediate], [hidden] (one allocation)
    size_t hidden, intermediate;
    float alpha, clamp;
};

namespace {
// biased = h + bias1; gate = biased[2i].min(clamp); linear = biased[2i+1].clamp(-clamp, clamp);
// out[i] = gate * (1 / (1 + exp(-alpha * gate))) * (linear + 1)
__global__ __launch_bounds__(256) void mxfp4_bias_swiglu_kernel(const float *__restrict__ h, const float *__restrict__ bias,
                                                                size_t rows, size_t inter, float alpha, float clamp,
                                                                float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * inter) return;
    const size_t r = i / inter, c = i - r * inter;
    const float g0 = h[r * 2 * inter + 2 * c] + bias[2 * c], l0 = h[r * 2 * inter + 2 * c + 1] + bias[2 * c + 1];
    const float gate = fminf(g0, clamp);                                     // f32::min: a NaN operand loses
    const float linear = l0 != l0 ? l0 : fminf(fmaxf(l0, -clamp), clamp);    // f32::clamp keeps NaN
    const float activated = gate * (1.0f / (1.0f + expf(-alpha * gate)));
    out[i] = activated * (linear + 1.0f);
}

__global__ __launch_bounds__(256) void bias_add_kernel(const float *__restrict__ a, const float *__restrict__ bias,
                                                       size_t rows, size_t cols, float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < rows * cols) out[i] = a[i] + bias[i % cols];
}
}  // namespace

PG_API void pg_mxfp4_expert_free(pg_ctx *ctx, pg_mxfp4_expert *e) {
    if (!e) return;
    if (ctx) {
        (void)pg_use(ctx);
        (void)hipStreamSynchronize(ctx->stream);
    }
    pg_gguf_free(ctx, e->mlp1);
    pg_gguf_free(ctx, e->mlp2);
    if (e->bias1) (void)hipFree(e->bias1);
    delete e;
}

PG_API pg_status pg_mxfp4_expert_create(pg_ctx *ctx, size_t hidden, size_t intermediate, float alpha, float clamp,
                                        const uint8_t *mlp1_blocks, const uint8_t *mlp1_scales,
                                        const uint8_t *mlp2_blocks, const uint8_t *mlp2_scales, const float *mlp1_bias,
                                        const float *mlp2_bias, pg_mxfp4_expert **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(out != nullptr, "pg_mxfp4_expert_create: out is null");
    *out = nullptr;
    PG_CHECK_ARG(mlp1_bias && mlp2_bias, "pg_mxfp4_expert_create: null bias");
    pg_mxfp4_expert *e = new (std::nothrow) pg_mxfp4_expert{nullptr, nullptr, nullptr, nullptr, hidden, intermediate, alpha, clamp};
    if (!e) return pg_fail(PG_ENOMEM, "host allocation failed");
    pg_status st = pg_mxfp4_upload(ctx, mlp1_blocks, mlp1_scales, 2 * intermediate, hidden, &e->mlp1);
    if (st == PG_OK) st = pg_mxfp4_upload(ctx, mlp2_blocks, mlp2_scales, hidden, intermediate, &e->mlp2);
    if (st == PG_OK) {
        hipError_t he = hipMalloc((void **)&e->bias1, (2 * intermediate + hidden) * sizeof(float));
        if (he == hipSuccess) {
            e->bias2 = e->bias1 + 2 * intermediate;
            he = hipMemcpyAsync(e->bias1, mlp1_bias, 2 * intermediate * sizeof(float), hipMemcpyHostToDevice, ctx->stream);
        }
        if (he == hipSuccess) he = hipMemcpyAsync(e->bias2, mlp2_bias, hidden * sizeof(float), hipMemcpyHostToDevice, ctx->stream);
        if (he == hipSuccess) he = hipStreamSynchronize(ctx->stream);
        if (he != hipSuccess)
            st = pg_fail(he == hipErrorOutOfMemory ? PG_ENOMEM : PG_EDEVICE, "pg_mxfp4_expert_create: %s", hipGetErrorString(he));
    }
    if (st != PG_OK) { pg_mxfp4_expert_free(ctx, e); return st; }
    *out = e;
    return PG_OK;
}

// scratch_dev: [m, 3 * intermediate] floats (the mlp1 output, then the activated rows).
PG_API pg_status pg_mxfp4_expert_forward_dev(pg_ctx *ctx, const pg_mxfp4_expert *e, const float *x_dev, size_t m,
                                             float *scratch_dev, float *out_dev) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(e != nullptr, "pg_mxfp4_expert_forward: null expert");
    if (m == 0) return PG_OK;
    PG_CHECK_ARG(x_dev && scratch_dev && out_dev, "pg_mxfp4_expert_forward: null pointer");
    PG_CHECK_ARG((uintptr_t)x_dev % 16 == 0 && (uintptr_t)scratch_dev % 16 == 0,
                 "pg_mxfp4_expert_forward: x and scratch must be 16-byte aligned");
    PG_CHECK_ARG(m <= 65535, "pg_mxfp4_expert_forward: more than 65535 rows");
    const size_t inter = e->intermediate, hid = e->hidden;
    float *h = scratch_dev, *act = scratch_dev + m * 2 * inter;
    PG_TRY(pg_gguf_matmul_rows(ctx, x_dev, m, e->mlp1, h));
    PG_TRY(pg_launch(ctx, "mxfp4_bias_swiglu", mxfp4_bias_swiglu_kernel, dim3(grid_for(m * inter, 256)), dim3(256), 0,
                     (const float *)h, (const float *)e->bias1, m, inter, e->alpha, e->clamp, act));
    PG_TRY(pg_gguf_matmul_rows(ctx, act, m, e->mlp2, out_dev));
    return pg_launch(ctx, "bias_add", bias_add_kernel, dim3(grid_for(m * hid, 256)), dim3(256), 0, (const float *)out_dev,
                     (const float *)e->bias2, m, hid, out_dev);
}

PG_API pg_status pg_mxfp4_expert_forward(pg_ctx *ctx, const pg_mxfp4_expert *e, const float *x, size_t m, float *out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(e != nullptr, "pg_mxfp4_expert_forward: null expert");
    if (m == 0) return PG_OK;
    PG_CHECK_ARG(x && out, "pg_mxfp4_expert_forward: null pointer");
    pg_tmp dx, ds, dout;
    PG_TRY(dx.alloc(m * e->hidden * sizeof(float)));
    PG_TRY(ds.alloc(m * 3 * e->intermediate * sizeof(float)));
    PG_TRY(dout.alloc(m * e->hidden * sizeof(float)));
    PG_HIP(hipMemcpyAsync(dx.p, x, m * e->hidden * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_mxfp4_expert_forward_dev(ctx, e, dx.as<float>(), m, ds.as<float>(), dout.as<float>()));
    PG_HIP(hipMemcpyAsync(out, dout.p, m * e->hidden * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}


// ---- the MoE layer over MXFP4 experts, grouped ------------------------------------------------
// MoELayer::forward after its router  examples/gpt_oss/moe.rs:286-352: the reference walks the tokens and calls
// Mxfp4Expert::forward once per (token, chosen expert).  Here every expert's tokens form token tiles of the tile
// kernel, all experts in one launch per product: routing lists, the pairs' activation rows gathered into digit
// records, mlp1 of all experts, bias + swiglu per pair, records again, mlp2, and out[t] = sum_k w[t,k] (y + bias2)
// in k order.
namespace {

// biased = h + bias1[expert]; the gpt-oss swiglu (examples/gpt_oss/moe.rs:155-166) per pair
__global__ __launch_bounds__(256) void mxfp4_moe_swiglu_kernel(const float *__restrict__ h, const float *const *__restrict__ bias_tab,
                                                               const int *__restrict__ topk_idx, size_t pairs, size_t inter,
                                                               float alpha, float clamp, float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= pairs * inter) return;
    const size_t p = i / inter, c = i - p * inter;
    const float *bias = bias_tab[topk_idx[p]];
    const float g0 = h[p * 2 * inter + 2 * c] + bias[2 * c], l0 = h[p * 2 * inter + 2 * c + 1] + bias[2 * c + 1];
    const float gate = fminf(g0, clamp);                                     // f32::min: a NaN operand loses
    const float linear = l0 != l0 ? l0 : fminf(fmaxf(l0, -clamp), clamp);    // f32::clamp keeps NaN
    const float activated = gate * (1.0f / (1.0f + expf(-alpha * gate)));
    out[i] = activated * (linear + 1.0f);
}

// output[t] += weight * (out + mlp2_bias) over the token's experts in the order given  (examples/gpt_oss/moe.rs:104-108, 330-334)
__global__ __launch_bounds__(256) void mxfp4_moe_combine_kernel(const float *__restrict__ yb, const float *const *__restrict__ bias_tab,
                                                                const int *__restrict__ topk_idx, const float *__restrict__ topk_p,
                                                                size_t tokens, size_t hidden, int top_k, float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= tokens * hidden) return;
    const size_t t = i / hidden, c = i - t * hidden;
    float acc = 0.0f;
    for (int k = 0; k < top_k; ++k) {
        const size_t p = t * top_k + k;
        const float result = yb[p * hidden + c] + bias_tab[topk_idx[p]][c];
        const float prod = topk_p[p] * result;
        acc = acc + prod;
    }
    out[i] = acc;
}

// One grouped product: rows `src` (pair / div) of the experts' slots -> records -> tiles against tensor table `which`.
pg_status moe_product(pg_ctx *ctx, const float *src, size_t k_in, size_t n_out, int tb, size_t max_tiles, mt_gather gat, int div,
                      const void **tab, size_t experts, int which, char *bq, float *y) {
    const int nb = (int)(k_in / 32), ncp = (int)mx_chunks((size_t)nb);
    gat.div = div;
    const size_t groups = max_tiles * tb, threads = groups * 2 * (size_t)ncp * 64;
    PG_CHECK_ARG((threads + 255) / 256 < ((size_t)1 << 31), "mxfp4 moe: too many pairs x %zu for one pre-pass", k_in);
    PG_TRY(pg_launch(ctx, "mxfp4_planes_gather", mxfp4_planes_kernel<true>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, src, 0, nb,
                     ncp, (int)groups, bq, gat));
    const size_t nrg = (n_out + 15) / 16;
    int ra = 4;
    while (ra > 1 && ((size_t)ra > nrg || (nrg + MT_NW * ra - 1) / (MT_NW * ra) * max_tiles < 2 * (size_t)ctx->num_cu)) ra >>= 1;
    const size_t n_wt = (nrg + MT_NW * ra - 1) / (MT_NW * ra);
    PG_CHECK_ARG(n_wt * max_tiles < ((size_t)1 << 28), "mxfp4 moe: %zu x %zu tiles", n_wt, max_tiles);
    const mt_experts ex = {reinterpret_cast<const uint8_t *const *>(tab + (size_t)(2 * which) * experts),
                           reinterpret_cast<const uint32_t *const *>(tab + (size_t)(2 * which + 1) * experts)};
#define PG_MTG(RA_, BD1, BD2, BD4) \
    (tb == 1 ? launch_tiles_grouped<RA_, 1, BD1>(ctx, n_out, ncp, bq, y, n_wt, max_tiles, gat, ex) \
     : tb == 2 ? launch_tiles_grouped<RA_, 2, BD2>(ctx, n_out, ncp, bq, y, n_wt, max_tiles, gat, ex) \
               : launch_tiles_grouped<RA_, 4, BD4>(ctx, n_out, ncp, bq, y, n_wt, max_tiles, gat, ex))
    return ra == 4 ? PG_MTG(4, 4, 2, 1) : (ra == 2 ? PG_MTG(2, 4, 4, 2) : PG_MTG(1, 4, 4, 4));
#undef PG_MTG
}

// The same product pair by pair on the decode kernel (few pairs).
bool pairs_fit(int ncp) { return mx_lds_bytes(1, ncp) <= (160u << 10); }
pg_status moe_product_pairs(pg_ctx *ctx, const float *src, size_t src_rows, size_t k_in, size_t n_out, size_t pairs, int div,
                            const void **tab, size_t experts, int which, const int *topk_idx, float *y) {
    const int ncp = (int)mx_chunks(k_in / 32);
    const mx_pairs pr = {reinterpret_cast<const uint8_t *const *>(tab + (size_t)(2 * which) * experts),
                         reinterpret_cast<const uint32_t *const *>(tab + (size_t)(2 * which + 1) * experts), topk_idx, div};
    // as pg_launch_mxfp4_rows chooses: 16 wavefronts on a row group while there is at most one group per CU, else 8
    // on the fewest row groups that keep every workgroup resident at once
    const size_t groups = (n_out + 15) / 16 * pairs, slots = (size_t)ctx->num_cu * 2;
    if (groups <= (size_t)ctx->num_cu) return launch_rows_pairs<1, 16>(ctx, n_out, k_in, src, src_rows, y, pairs, ncp, pr);
    if (groups <= slots) return launch_rows_pairs<1, 8>(ctx, n_out, k_in, src, src_rows, y, pairs, ncp, pr);
    if ((groups + 1) / 2 <= slots) return launch_rows_pairs<2, 8>(ctx, n_out, k_in, src, src_rows, y, pairs, ncp, pr);
    return launch_rows_pairs<4, 8>(ctx, n_out, k_in, src, src_rows, y, pairs, ncp, pr);
}

}  // namespace

PG_API pg_status pg_mxfp4_moe_ffn_routed_dev(pg_ctx *ctx, const float *x_dev, size_t T, const int32_t *expert_idx_dev,
                                             const float *weight_dev, size_t top_k, const pg_mxfp4_expert *const *experts, size_t E,
                                             float *out_dev) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(E >= 1 && E <= (size_t)PG_MOE_MAX_EXPERTS, "pg_mxfp4_moe_ffn: %zu experts (1..%d supported)", E, PG_MOE_MAX_EXPERTS);
    PG_CHECK_ARG(top_k >= 1 && top_k <= E, "pg_mxfp4_moe_ffn: top_k %zu of %zu experts", top_k, E);
    PG_CHECK_ARG(experts && experts[0], "pg_mxfp4_moe_ffn: null expert table");
    const size_t hidden = experts[0]->hidden, inter = experts[0]->intermediate;
    const float alpha = experts[0]->alpha, clamp = experts[0]->clamp;
    for (size_t e = 0; e < E; ++e) {
        PG_CHECK_ARG(experts[e] != nullptr, "pg_mxfp4_moe_ffn: expert %zu is null", e);
        PG_CHECK_ARG(experts[e]->hidden == hidden && experts[e]->intermediate == inter && experts[e]->alpha == alpha &&
                         experts[e]->clamp == clamp, "pg_mxfp4_moe_ffn: expert %zu differs in shape, alpha or clamp", e);
    }
    if (T == 0) return PG_OK;
    PG_CHECK_ARG(x_dev && expert_idx_dev && weight_dev && out_dev, "pg_mxfp4_moe_ffn: null pointer");
    PG_CHECK_ARG((uintptr_t)x_dev % 16 == 0, "pg_mxfp4_moe_ffn: x must be 16-byte aligned");
    PG_CHECK_ARG(T * top_k < (1ull << 20), "pg_mxfp4_moe_ffn: too many (token, expert) pairs");
    const size_t P = T * top_k;
    // token tiles: groups of 16 slots, as many to a tile as an expert's average share suggests
    const int tb = P / E <= 16 ? 1 : (P / E <= 32 ? 2 : 4);
    const size_t max_tiles = P / (16 * (size_t)tb) + E;  // sum over experts of ceil(count / (16 tb)) stays below
    const int ncp1 = (int)mx_chunks(hidden / 32), ncp2 = (int)mx_chunks(inter / 32);
    const size_t sz_idx = pg_round_up(P * sizeof(int), 256), sz_p = pg_round_up(P * sizeof(float), 256);
    const size_t sz_lists = pg_round_up(E * T * sizeof(int), 256), sz_counts = pg_round_up((2 * E + 1) * sizeof(int), 256);
    const size_t sz_rec = pg_round_up(max_tiles * tb * (size_t)std::max(ncp1, ncp2) * MT_RECORD, 256);
    const size_t sz_h = pg_round_up(P * 2 * inter * sizeof(float), 256), sz_act = pg_round_up(P * inter * sizeof(float), 256);
    const size_t sz_y = pg_round_up(P * hidden * sizeof(float), 256);
    void *ws = nullptr;
    PG_TRY(pg_workspace(ctx, sz_idx + sz_p + sz_lists + sz_counts + sz_rec + sz_h + sz_act + sz_y, &ws));
    char *p = static_cast<char *>(ws);
    int *topk_idx = reinterpret_cast<int *>(p); p += sz_idx;
    float *topk_p = reinterpret_cast<float *>(p); p += sz_p;
    int *lists = reinterpret_cast<int *>(p); p += sz_lists;
    int *counts = reinterpret_cast<int *>(p), *goff = counts + E; p += sz_counts;
    char *rec = p; p += sz_rec;
    float *h = reinterpret_cast<float *>(p); p += sz_h;
    float *act = reinterpret_cast<float *>(p); p += sz_act;
    float *yb = reinterpret_cast<float *>(p);
    // [mlp1 codes | mlp1 scales | mlp2 codes | mlp2 scales | bias1 | bias2], E each
    const void *host_tab[6 * PG_MOE_MAX_EXPERTS];
    for (size_t e = 0; e < E; ++e) {
        host_tab[0 * E + e] = experts[e]->mlp1->qs; host_tab[1 * E + e] = experts[e]->mlp1->d;
        host_tab[2 * E + e] = experts[e]->mlp2->qs; host_tab[3 * E + e] = experts[e]->mlp2->d;
        host_tab[4 * E + e] = experts[e]->bias1;    host_tab[5 * E + e] = experts[e]->bias2;
    }
    const void **tab = nullptr;
    PG_TRY(pg_moe_cached_table(ctx, host_tab, 6 * E, &tab));
    // With few pairs hardly two of them meet in an expert, and a pair is a one-row product: the decode kernel, one
    // workgroup column per pair (exact activations; no expert lists).  Otherwise the experts' token tiles on the tile kernel.
    const bool by_pairs = P <= 2 * E && P <= 64 && pairs_fit(ncp1) && pairs_fit(ncp2);
    PG_TRY(pg_launch_moe_routing(ctx, nullptr, expert_idx_dev, weight_dev, T, E, top_k, topk_idx, topk_p, by_pairs ? nullptr : lists, counts));
    if (!by_pairs)
        PG_TRY(pg_launch(ctx, "mxfp4_tile_offsets", mxfp4_tile_offsets_kernel, dim3(1), dim3(64), 0, (const int *)counts, (int)E, tb, goff));
    const mt_gather gat = {lists, counts, goff, (int)T, (int)E, tb, 1};
    if (by_pairs)
        PG_TRY(moe_product_pairs(ctx, x_dev, T, hidden, 2 * inter, P, (int)top_k, tab, E, 0, topk_idx, h));
    else
        PG_TRY(moe_product(ctx, x_dev, hidden, 2 * inter, tb, max_tiles, gat, (int)top_k, tab, E, 0, rec, h));
    PG_TRY(pg_launch(ctx, "mxfp4_moe_swiglu", mxfp4_moe_swiglu_kernel, dim3(grid_for(P * inter, 256)), dim3(256), 0, (const float *)h,
                     reinterpret_cast<const float *const *>(tab + 4 * E), (const int *)topk_idx, P, inter, alpha, clamp, act));
    if (by_pairs)
        PG_TRY(moe_product_pairs(ctx, act, P, inter, hidden, P, 1, tab, E, 1, topk_idx, yb));
    else
        PG_TRY(moe_product(ctx, act, inter, hidden, tb, max_tiles, gat, 1, tab, E, 1, rec, yb));
    return pg_launch(ctx, "mxfp4_moe_combine", mxfp4_moe_combine_kernel, dim3(grid_for(T * hidden, 256)), dim3(256), 0, (const float *)yb,
                     reinterpret_cast<const float *const *>(tab + 5 * E), (const int *)topk_idx, (const float *)topk_p, T, hidden,
                     (int)top_k, out_dev);
}

PG_API pg_status pg_mxfp4_moe_ffn_routed(pg_ctx *ctx, const float *x, size_t T, const int32_t *expert_idx, const float *weight,
                                         size_t top_k, const pg_mxfp4_expert *const *experts, size_t E, float *out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(experts && experts[0], "pg_mxfp4_moe_ffn: null expert table");
    if (T == 0) return PG_OK;
    PG_CHECK_ARG(x && expert_idx && weight && out, "pg_mxfp4_moe_ffn: null pointer");
    PG_CHECK_ARG(E >= 1 && E <= (size_t)PG_MOE_MAX_EXPERTS && top_k >= 1 && top_k <= E, "pg_mxfp4_moe_ffn: top_k %zu of %zu experts", top_k, E);
    // the reference indexes self.experts[expert_idx] (examples/gpt_oss/moe.rs:104-108) and would panic on an index out
    // of range; its top-k never names an expert twice for a token, which the grouped products rely on
    for (size_t t = 0; t < T; ++t)
        for (size_t k = 0; k < top_k; ++k) {
            const int32_t e = expert_idx[t * top_k + k];
            PG_CHECK_ARG(e >= 0 && (size_t)e < E, "pg_mxfp4_moe_ffn: token %zu names expert %d of %zu", t, (int)e, E);
            for (size_t j = 0; j < k; ++j)
                PG_CHECK_ARG(expert_idx[t * top_k + j] != e, "pg_mxfp4_moe_ffn: token %zu names expert %d twice", t, (int)e);
        }
    const size_t hidden = experts[0]->hidden;
    pg_tmp dx, di, dw, dout;
    PG_TRY(dx.alloc(T * hidden * sizeof(float)));
    PG_TRY(di.alloc(T * top_k * sizeof(int32_t)));
    PG_TRY(dw.alloc(T * top_k * sizeof(float)));
    PG_TRY(dout.alloc(T * hidden * sizeof(float)));
    PG_HIP(hipMemcpyAsync(dx.p, x, T * hidden * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipMemcpyAsync(di.p, expert_idx, T * top_k * sizeof(int32_t), hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipMemcpyAsync(dw.p, weight, T * top_k * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_mxfp4_moe_ffn_routed_dev(ctx, dx.as<float>(), T, di.as<int32_t>(), dw.as<float>(), top_k, experts, E, dout.as<float>()));
    PG_HIP(hipMemcpyAsync(out, dout.p, T * hidden * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}
