// Skinny / grouped product over GGUF block-quantised weights on the int8 matrix cores:
//   y[pair, n] = sum_b  d[n, b] * xs[tok, b] * sum_{k in block b} q[n, k] * X[tok, k]
// for up to 32 activation rows ("tokens") per workgroup, so the weights are read from HBM
// once per group of tokens instead of once per token (M > 1 dequant-matmul of models::llama,
// src/models/llama/model.rs:243-257 + src/tensor.rs:1342-1353, and the per-expert products
// of the MoE FFN, examples/grok1/moe.rs:91-104).
//
// A GGUF block is 32 consecutive k, exactly the K of one v_mfma_i32_32x32x32_i8: per block
// and 32x32 (weight rows x tokens) tile, two MFMAs give the exact integer dots of the
// weights with the high and the low byte digit of the fixed-point activations
// X = 256 * hi + lo (|X| <= 32639, per-block scale xs = absmax / 32639), and the tile is scaled by
// d[n, b] * xs[tok, b] and accumulated in f32.  Weight rows sit on the accumulator
// registers, tokens on lanes.
//
// Workgroup = 4 wavefronts = 128 weight rows x 32 tokens x one K chunk.  Everything is
// staged through LDS with direct global->LDS loads, two stages of 4 blocks ahead of the one
// being consumed: each wavefront's own 32 weight rows and their f16 block scales, and the
// token digits and scales of the stage, which the four wavefronts share.
#include <limits.h>
#include "pg_internal.h"
#include "pg_stream_addr.h"
#include "pg_digits.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef const void __attribute__((address_space(1))) *gptr_t;
typedef void __attribute__((address_space(3))) *lptr_t;
typedef const v4i __attribute__((address_space(1))) *gv4i_ptr;

inline unsigned grid_for(size_t n, unsigned block) { return (unsigned)((n + block - 1) / block); }

constexpr int NBU = 4;                              // blocks per stage
// LDS stage layout.  Every fill is arranged so that neighbouring lanes fetch neighbouring
// 16-byte chunks of global memory (whole 64- or 128-byte runs per request); the chunk order
// inside a run is XOR-swizzled so that the 128-bit LDS reads of 16 neighbouring lanes fall
// into 16 different 16-byte bank groups (gfx950 serves a 128-bit read over 256 bytes of banks a
// pass: with 8 distinct groups per 8 lanes only, lanes l and l + 8 collided and every such read
// took 8 cycles instead of 4).  For the digits that means: tokens 8 .. 15 (mod 16) keep their two
// planes in swapped places.
constexpr int DIG_STAGE = 64 * 128;                 // [token][plane] units of 128 B: 4 blocks x 2 halves  8 KiB
constexpr int D_STAGE = 4 * 256;                    // [wave][row group of 8][j][8 f16]                     1 KiB
constexpr int XS_STAGE = 32 * 16;                   // [token][4 block scales]                              512 B
constexpr int OFF_D = DIG_STAGE, OFF_XS = OFF_D + D_STAGE, OFF_W = OFF_XS + XS_STAGE;
template <int QT> struct MMCfg {
    static constexpr int W_WAVE = QT == 8 ? 64 * 64 : 32 * 64;  // per wavefront: [stream][4 blocks][16 B]
    static constexpr int W_FILLS = W_WAVE / 1024;               // weight fills per wavefront and stage
    static constexpr int STAGE = OFF_W + 4 * W_WAVE;            // 25.5 KiB (Q8_0) / 17.5 KiB (Q4_0)
    // Two LDS stages (one in flight beyond the one consumed), so that THREE workgroups share a CU (three wavefronts
    // a SIMD, 168 registers each).  Against two workgroups of three stages the expert products ran 2 % faster, the
    // 16-row product 6 % and the 1024-row o projection 7 %: a third wavefront fills the issue slots the other two
    // leave while they wait, which counts for more than the deeper ring.  (Three stages of the smaller Q4_0 stage,
    // 3 x 52.5 KiB a CU, measured like two workgroups: they do not fit three at a time.)
    static constexpr int RING = 2;
    static constexpr int AHEAD = RING - 1;
    static constexpr int LPS = 2 + 1 + 1 + W_FILLS;             // LDS fills per wavefront and stage
};

// ---- activation rows -> two byte-digit planes (pg_emit_mm_digits, pg_digits.h) ----------
template <bool NIB>
__global__ __launch_bounds__(256) void x_to_mm_digits_kernel(const float *__restrict__ x, int nb, int nbp,
                                                             int8_t *__restrict__ digits, float *__restrict__ xs,
                                                             float *__restrict__ xsum) {
    const size_t row = blockIdx.y;
    const int b = blockIdx.x * 32 + (threadIdx.x >> 3), sub = threadIdx.x & 7;
    if (b >= nb) return;  // whole 8-thread groups leave together
    const float4 v = reinterpret_cast<const float4 *>(x + (row * nb + b) * 32)[sub];
    const float f[4] = {v.x, v.y, v.z, v.w};
    pg_emit_mm_digits<NIB>(f, row, b, sub, nb, nbp, digits, xs, xsum);
}

// Q4_1's second term on many rows: y[t][n] += sum_b (8 d[n][b] + m[n][b]) * xsum[t][b] (the first, d sum (q - 8) x,
// is the Q4_0 product on the same nibbles).  Workgroup = 256 / NQ weight rows x 16 tokens; thread = (row, one of NQ
// runs of blocks), 16 tokens in registers; the tokens' block sums wait in LDS as [b][16]; the runs are added in
// ascending order.  NQ = 4 for few tokens (more workgroups, shorter loops), 1 for many (the block sums staged once
// per 256 rows).
constexpr int Q41_TT = 16;
template <int NQ>
__global__ __launch_bounds__(256) void q41_offset_kernel(const uint16_t *__restrict__ d, const uint16_t *__restrict__ m, int n_out,
                                                         int nb, const float *__restrict__ xsum, int nbp, int rows,
                                                         float *__restrict__ y) {
    constexpr int RPW = 256 / NQ;
    extern __shared__ __attribute__((aligned(16))) float s_tile[];  // [nb][Q41_TT], then [NQ - 1][RPW][Q41_TT] partial sums
    const int t0 = blockIdx.y * Q41_TT, lrow = threadIdx.x % RPW, quarter = threadIdx.x / RPW;
    const int n = blockIdx.x * RPW + lrow;
    for (int i = threadIdx.x; i < nb * Q41_TT; i += 256) {
        const int t = i / nb, b = i - t * nb;  // (consecutive threads: consecutive blocks of one token)
        s_tile[b * Q41_TT + t] = t0 + t < rows ? xsum[(size_t)(t0 + t) * nbp + b] : 0.0f;
    }
    __syncthreads();
    float acc[Q41_TT];
#pragma unroll
    for (int t = 0; t < Q41_TT; ++t) acc[t] = 0.0f;
    const int nc = n < n_out ? n : n_out - 1;
    const size_t tile = (size_t)(nc >> 3) * nb * 8 + (nc & 7);
    const int per = (nb + NQ - 1) / NQ, b_lo = quarter * per, b_hi = b_lo + per < nb ? b_lo + per : nb;
    for (int b = b_lo; b < b_hi; ++b) {
        _Float16 dh, mh;
        const uint16_t db = d[tile + (size_t)b * 8], mb = m[tile + (size_t)b * 8];
        __builtin_memcpy(&dh, &db, 2);
        __builtin_memcpy(&mh, &mb, 2);
        const float c = fmaf(8.0f, (float)dh, (float)mh);
#pragma unroll
        for (int t4 = 0; t4 < Q41_TT / 4; ++t4) {
            const float4 sv = *reinterpret_cast<const float4 *>(s_tile + b * Q41_TT + 4 * t4);
            acc[4 * t4] = fmaf(c, sv.x, acc[4 * t4]); acc[4 * t4 + 1] = fmaf(c, sv.y, acc[4 * t4 + 1]);
            acc[4 * t4 + 2] = fmaf(c, sv.z, acc[4 * t4 + 2]); acc[4 * t4 + 3] = fmaf(c, sv.w, acc[4 * t4 + 3]);
        }
    }
    if constexpr (NQ > 1) {
        float *part = s_tile + nb * Q41_TT;
        if (quarter > 0) {
#pragma unroll
            for (int t = 0; t < Q41_TT; ++t) part[((quarter - 1) * RPW + lrow) * Q41_TT + t] = acc[t];
        }
        __syncthreads();
        if (quarter > 0) return;
#pragma unroll
        for (int qv = 0; qv < NQ - 1; ++qv)
#pragma unroll
            for (int t = 0; t < Q41_TT; ++t) acc[t] += part[(qv * RPW + lrow) * Q41_TT + t];
    }
    if (n >= n_out) return;
#pragma unroll
    for (int t = 0; t < Q41_TT; ++t)
        if (t0 + t < rows) y[(size_t)(t0 + t) * n_out + n] += acc[t];
}

// Two's-complement nibbles (as stored at upload) of one dword -> four signed bytes holding
// 16 * (q - 8): a nibble moved to the top of its byte IS that value, no sign extension
// needed.  left = 4 takes the low nibble of every byte, left = 0 the high one.
__device__ __forceinline__ int nibbles_to_i8x16(int v, int left) {
    return (int)(((unsigned)v << left) & 0xF0F0F0F0u);
}

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
    _Float16 v;
    const uint16_t hb = (uint16_t)h;
    __builtin_memcpy(&v, &hb, 2);
    return (float)v;
}

// grid: x = tiles of 128 weight rows, y = expert * tiles_per_expert + token tile, z = K chunk.
// `chunk` (blocks per K chunk) is a multiple of NBU and no chunk is empty.
// out: [K chunks][total pairs][n_out] (plain y with one chunk).
// (Three wavefronts per SIMD, 168 registers each: the MFMA results are written to ordinary VGPRs,
// not to accumulation registers that would have to be copied out first.)
// NT: the weight fills carry the non-temporal hint.  Right for the expert products, where a
// weight byte is used by one or two workgroups and 1.7 GB of them per launch would otherwise
// push the activations, digits and partial sums of the neighbouring kernels out of the caches
// (MoE step 1.22 -> 1.17 ms); wrong for a prefill, where 32 token tiles re-read every weight.
template <int QT, bool NT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void gguf_mm_kernel(const uint8_t *__restrict__ qs0, const uint16_t *__restrict__ d0,
                                                      pg_mm_group grp, int n_out_arg, int nb, int nbp, int chunk,
                                                      const int8_t *__restrict__ digits, const float *__restrict__ xs,
                                                      float *__restrict__ out_arg, size_t part_stride_arg) {
    extern __shared__ __attribute__((aligned(1024))) char lds[];  // RING * STAGE bytes
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l31 = lane & 31, hh = lane >> 5;

    // Which 128 weight rows (bx) and which token tile (by).  With many token tiles (a prefill)
    // the launch is one-dimensional and XCD-aware: workgroup id = 8 * j + xcd, and the j-th
    // workgroup of an XCD is member j % 32 of super-tile (j / 32) * 8 + xcd, a super-tile being
    // 4 row groups x 8 token tiles whose weights and digits (about 3 MB) stay in that XCD's L2
    // while its 32 workgroups run: each weight row group is fetched once per 8 token tiles
    // instead of once per tile.
    int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
    if (grp.xcd_ks) {
        // K chunks dealt to XCDs (workgroup id % 8 = XCD): chunk z runs on the 8 / ks XCDs with
        // id % ks == z, so an XCD's L2 holds only its chunk of the activation digits, and the
        // workgroups of an XCD walk the row groups of one token tile after another.
        const int xcd = blockIdx.x & 7, per = 8 / grp.xcd_ks;
        const int j = (blockIdx.x >> 3) * per + xcd / grp.xcd_ks;
        if (j >= grp.remap_rg * grp.remap_tiles) return;
        bz = xcd % grp.xcd_ks;
        bx = j % grp.remap_rg;
        by = j / grp.remap_rg;
    } else if (grp.remap_rg) {
        const int nrgb = (grp.remap_rg + 3) / 4, ntb = (grp.remap_tiles + 7) / 8;
        const int jj = blockIdx.x >> 3, st = (jj >> 5) * 8 + (blockIdx.x & 7), w = jj & 31;
        if (st >= nrgb * ntb) return;
        bx = (st % nrgb) * 4 + (w & 3);
        by = (st / nrgb) * 8 + (w >> 2);
        if (bx >= grp.remap_rg || by >= grp.remap_tiles) return;
    }
    int e = 0, tt = by;
    if (grp.counts) {
        e = by / grp.tiles_per_expert;
        tt = by - e * grp.tiles_per_expert;
    }
    const int count = grp.counts ? grp.counts[e] : grp.max_count;
    if (tt * 32 >= count) return;  // the same for every thread of the workgroup
    const uint8_t *qs_any = grp.qs_table ? grp.qs_table[e] : qs0;
    const uint16_t *d_any = grp.d_table ? grp.d_table[e] : d0;
    int n_out = n_out_arg;
    float *__restrict__ out = out_arg;
    size_t part_stride = part_stride_arg;
    if (grp.nseg) {  // which tensor of the launch this row group belongs to
        int t = 0;
        while (t + 1 < grp.nseg && bx >= grp.seg_first[t + 1]) ++t;
        bx -= grp.seg_first[t];
        qs_any = grp.seg_qs[t];
        d_any = grp.seg_d[t];
        n_out = grp.seg_n[t];
        out = grp.seg_out[t];
        part_stride = grp.seg_stride[t];
    }

    constexpr int STAGE = MMCfg<QT>::STAGE, W_WAVE = MMCfg<QT>::W_WAVE, W_FILLS = MMCfg<QT>::W_FILLS;
    // Activation row of a token slot of this tile (spare slots shadow the tile's first token).
    auto xrow_of = [&](int tok) -> size_t {
        const int slot = tt * 32 + tok;
        const int slot_c = slot < count ? slot : tt * 32;
        const int pr = grp.lists ? grp.lists[(size_t)e * grp.list_stride + slot_c] : slot_c;
        return (size_t)(pr / grp.x_row_div);
    };
    // Orientation of the 32x32 result tile: TOKENS on the accumulator-register axis (register r
    // of lanes with hh = lane/32 holds token slot 8*(r/4) + 4*hh + r%4), WEIGHT ROWS on the lanes.
    // A tile with few tokens then needs only the first NR registers scaled and accumulated:
    // NR = 4 covers 8 token slots, 8 covers 16, 16 all 32.
    const int ntok = count - tt * 32 < 32 ? count - tt * 32 : 32;

    // Fill duties of this lane.
    // digits: fill n = 2*wave + u covers units 8n .. 8n+7, unit = 2*token + plane; the lane
    // fetches chunk (lane & 7) ^ (token & 7) of the unit's 128 bytes, chunk = 2*block + half.
    const int8_t *dig_src[2];
    int dig_jb[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int unit = (2 * wave + u) * 8 + (lane >> 3), tok = unit >> 1, pl = (unit & 1) ^ ((tok >> 3) & 1);
        const int ch = (lane & 7) ^ (tok & 7);
        dig_jb[u] = ch >> 1;
        dig_src[u] = digits + xrow_of(tok) * pg_mm_row_bytes(nb) + (size_t)pl * nb * 32 + (ch & 1) * 16;
    }
    // xs: lanes 0..7 of wavefront w fetch the 4 block scales of tokens 8w .. 8w+7
    const float *xs_src = xs + xrow_of(8 * wave + (lane & 7)) * (size_t)nbp;
    // weights: fill q covers streams 16q .. 16q+15 (Q8_0: stream = 32*half + row, Q4_0: stream = row);
    // the lane fetches block (lane & 3) ^ swizzle of the stream's 4 blocks.
    const int row0 = bx * 128 + wave * 32;
    const int w_jb = (lane & 3) ^ ((lane >> 4) & 3);  // (stream >> 2) & 3, stream = 16q + (lane >> 2)
    const int8_t *w_src[W_FILLS];
#pragma unroll
    for (int q = 0; q < W_FILLS; ++q) {
        const int st = 16 * q + (lane >> 2);
        const int wrow = row0 + (st & 31) < n_out ? row0 + (st & 31) : n_out - 1;  // clamped; masked at the store
        w_src[q] = reinterpret_cast<const int8_t *>(qs_any) +
                   (QT == 8 ? ((size_t)wrow * 2 + (st >> 5)) * nb * 16 : (size_t)wrow * nb * 16);
        // Tile-major copy: [row group][4 blocks][wavefront][fill][lane] 16-byte chunks, the very
        // order of the fills below, padded with zero rows and blocks: a stage of a workgroup is
        // 4 * W_WAVE contiguous bytes (row groups pg_tiled_group_bytes apart).
        if (grp.tiled)
            w_src[q] = reinterpret_cast<const int8_t *>(qs_any) +
                       (size_t)bx * pg_tiled_group_bytes(nb, QT == 8) + wave * W_WAVE + q * 1024 + lane * 16;
    }
    // f16 scales of this wavefront's 32 rows: lane -> (group lane/16, block (lane/4)%4, dword lane%4)
    const int ngroups = (n_out + 7) / 8;
    int dg = (row0 >> 3) + (lane >> 4);
    dg = dg < ngroups ? dg : ngroups - 1;
    const char *d_grp = reinterpret_cast<const char *>(d_any) + (size_t)dg * nb * 16 + (lane & 3) * 4;
    const int d_jb = (lane >> 2) & 3;

    const int b_begin = bz * chunk;
    const int b_end = b_begin + chunk < nb ? b_begin + chunk : nb;
    const int nst = (b_end - b_begin + NBU - 1) / NBU;

    // Every load of the K loop is a direct global->LDS fill, so the only memory waits in the
    // loop are the explicit ones below (two stages stay in flight across the barrier).
    // (The ring slot is a compile-time constant everywhere so that the compiler can tell the
    // stage being filled from the stage being read and adds no waits of its own.)
    auto issue = [&](auto ring_slot, int s) {
        const int b0 = b_begin + s * NBU;
        char *base = lds + decltype(ring_slot)::value * STAGE;
        auto blk = [&](int j) { return (size_t)(b0 + j < b_end ? b0 + j : b_end - 1); };  // past the end: a valid, unused block
#pragma unroll
        for (int u = 0; u < 2; ++u)
            __builtin_amdgcn_global_load_lds((gptr_t)(dig_src[u] + blk(dig_jb[u]) * 32), (lptr_t)(base + (2 * wave + u) * 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr_t)(d_grp + blk(d_jb) * 16), (lptr_t)(base + OFF_D + wave * 256), 4, 0, 0);
        if (lane < 8)
            __builtin_amdgcn_global_load_lds((gptr_t)(xs_src + b0), (lptr_t)(base + OFF_XS + wave * 128), 16, 0, 0);
        const size_t w_off = grp.tiled ? (size_t)(b0 >> 2) * (4 * W_WAVE) : blk(w_jb) * 16;
#pragma unroll
        for (int q = 0; q < W_FILLS; ++q)
            __builtin_amdgcn_global_load_lds((gptr_t)(w_src[q] + w_off), (lptr_t)(base + OFF_W + wave * W_WAVE + q * 1024), 16, 0, NT ? 2 : 0);
    };

    float acc[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

    // One block of the stage at `base`: operands from LDS, two MFMAs, scale-and-accumulate.
    // Split into three phases so that the full-stage path can overlap them across blocks.
    const int w_rd = OFF_W + wave * W_WAVE + (QT == 8 ? lane : l31) * 64, w_sw = ((QT == 8 ? lane : l31) >> 2) & 3;
    const int dig_rd = l31 * 256, dig_sw = l31 & 7, dig_hi = ((l31 >> 3) & 1) * 128;  // tokens 8 .. 15 (mod 16) keep their planes swapped
    const int d_rd = OFF_D + wave * 256 + (l31 >> 3) * 64 + (l31 & 7) * 2;  // this lane's weight row: [group of 8][j][8 f16]
    auto read_ab = [&](const char *base, int j, v4i (&ab)[3]) {
        ab[0] = *reinterpret_cast<const v4i *>(base + w_rd + ((j ^ w_sw) * 16));
        ab[1] = *reinterpret_cast<const v4i *>(base + dig_rd + dig_hi + (((2 * j + hh) ^ dig_sw) * 16));
        ab[2] = *reinterpret_cast<const v4i *>(base + dig_rd + (128 - dig_hi) + (((2 * j + hh) ^ dig_sw) * 16));
    };
    // the block's weight scale of this lane's row
    // (read as integers: a float-typed LDS read makes the compiler wait for every fill in flight)
    auto read_d = [&](const char *base, int j, unsigned &dbits) {
        dbits = *reinterpret_cast<const unsigned short *>(base + d_rd + j * 16);
    };
    auto mfmas = [&](const v4i (&ab)[3], v16i &ihi, v16i &ilo) {
        v4i a = ab[0];
        if constexpr (QT == 4) {
#pragma unroll
            for (int t = 0; t < 4; ++t) a[t] = nibbles_to_i8x16(a[t], 4 - 4 * hh);
        }
        v16i zero;
#pragma unroll
        for (int r = 0; r < 16; ++r) zero[r] = 0;
        ihi = __builtin_amdgcn_mfma_i32_32x32x32_i8(ab[1], a, zero, 0, 0, 0);  // rows = tokens, columns = weight rows
        ilo = __builtin_amdgcn_mfma_i32_32x32x32_i8(ab[2], a, zero, 0, 0, 0);
    };
    auto scale_acc = [&](auto nr, const v16i &ihi, const v16i &ilo, unsigned dbits, const int (&sx)[16][4], int j) {
        float dv = half_bits_to_float(dbits);
        if constexpr (QT == 4) dv *= 0.0625f;  // the weight operand was 16 * (q - 8)
#pragma unroll
        for (int r = 0; r < decltype(nr)::value; ++r) {
            // |integer| < 2^31: rounded to 24 bits, then scaled (two roundings of 2^-24, far below the digit step)
            const float fx = (float)(ihi[r] * 256 + ilo[r]) * __int_as_float(sx[r][j]);
            acc[r] = fmaf(dv, fx, acc[r]);
        }
    };
    auto compute = [&](auto nr, auto ring_slot, int s) {
        const int b0 = b_begin + s * NBU;
        const char *base = lds + decltype(ring_slot)::value * STAGE;
        // activation scales of this lane's NR token slots for the stage's four blocks
        // (vector element -> named int: a bit cast applied directly to a vector element
        // expression was compiled as a cast of element 0)
        int sx[16][4];
#pragma unroll
        for (int r = 0; r < decltype(nr)::value; ++r) {
            const v4i t = *reinterpret_cast<const v4i *>(base + OFF_XS + (8 * (r >> 2) + 4 * hh + (r & 3)) * 16);
            const int t0 = t[0], t1 = t[1], t2 = t[2], t3 = t[3];
            sx[r][0] = t0; sx[r][1] = t1; sx[r][2] = t2; sx[r][3] = t3;
        }
        v4i ab[2][3];
        unsigned dd[2];
        v16i ihi[2], ilo[2];
        if (b0 + NBU <= b_end) {  // full stage (wavefront-uniform)
            // Software pipeline over the 4 blocks: while block j is scaled and accumulated on
            // the vector ALU, the MFMAs of block j+1 run and the LDS reads of block j+2 return.
            read_ab(base, 0, ab[0]);
            read_d(base, 0, dd[0]);
            read_ab(base, 1, ab[1]);
            mfmas(ab[0], ihi[0], ilo[0]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < NBU; ++j) {
                if (j + 1 < NBU) {
                    mfmas(ab[(j + 1) & 1], ihi[(j + 1) & 1], ilo[(j + 1) & 1]);
                    __builtin_amdgcn_sched_barrier(0);  // younger LDS reads must not be waited for here
                    read_d(base, j + 1, dd[(j + 1) & 1]);
                }
                if (j + 2 < NBU) read_ab(base, j + 2, ab[j & 1]);
                __builtin_amdgcn_sched_barrier(0);
                scale_acc(nr, ihi[j & 1], ilo[j & 1], dd[j & 1], sx, j);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int j = 0; j < NBU - 1; ++j)
                if (b0 + j < b_end) {
                    read_ab(base, j, ab[0]);
                    read_d(base, j, dd[0]);
                    mfmas(ab[0], ihi[0], ilo[0]);
                    scale_acc(nr, ihi[0], ilo[0], dd[0], sx, j);
                }
        }
    };

    // ---- the other orientation, for tiles with more than 16 tokens: weight rows on the
    // accumulator-register axis (register r <-> row 8*(r/4) + 4*hh + r%4), tokens on the lanes.
    // All 16 registers are needed either way, and this way round the activation scales are one
    // LDS read per stage instead of sixteen.
    auto read_d_rows = [&](const char *base, int j, v2i (&dd)[4]) {
#pragma unroll
        for (int g = 0; g < 4; ++g)  // rows 8g + 4*hh + {0..3}  <->  accumulator registers 4g .. 4g+3
            dd[g] = *reinterpret_cast<const v2i *>(base + OFF_D + wave * 256 + (g * 4 + j) * 16 + hh * 8);
    };
    auto mfmas_rows = [&](const v4i (&ab)[3], v16i &ihi, v16i &ilo) {  // rows = weight rows, columns = tokens
        v4i a = ab[0];
        if constexpr (QT == 4) {
#pragma unroll
            for (int t = 0; t < 4; ++t) a[t] = nibbles_to_i8x16(a[t], 4 - 4 * hh);
        }
        v16i zero;
#pragma unroll
        for (int r = 0; r < 16; ++r) zero[r] = 0;
        ihi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, ab[1], zero, 0, 0, 0);
        ilo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, ab[2], zero, 0, 0, 0);
    };
    auto scale_acc_rows = [&](const v16i &ihi, const v16i &ilo, const v2i (&dd)[4], float sj) {
        if constexpr (QT == 4) sj *= 0.0625f;  // the weight operand was 16 * (q - 8)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int r = 4 * g + q;
                const uint32_t pairbits = (uint32_t)dd[g][q >> 1];
                const float dv = half_bits_to_float((q & 1) ? pairbits >> 16 : pairbits & 0xFFFFu);
                // |integer| < 2^31: rounded to 24 bits, then scaled (two roundings of 2^-24, far below the digit step)
                const float fx = (float)(ihi[r] * 256 + ilo[r]) * sj;
                acc[r] = fmaf(dv, fx, acc[r]);
            }
    };
    auto compute_rows = [&](auto ring_slot, int s) {
        const int b0 = b_begin + s * NBU;
        const char *base = lds + decltype(ring_slot)::value * STAGE;
        // Read as integers: a float-typed LDS read makes the compiler wait for every LDS fill in
        // flight (it cannot tell the stages apart), an int-typed one leaves the waits to us.
        const v4i sxi = *reinterpret_cast<const v4i *>(base + OFF_XS + l31 * 16);
        // (element -> named int -> float: a bit cast applied directly to a vector element
        // expression was compiled as a cast of element 0)
        const int sx0 = sxi[0], sx1 = sxi[1], sx2 = sxi[2], sx3 = sxi[3];
        const float sx[4] = {__int_as_float(sx0), __int_as_float(sx1), __int_as_float(sx2), __int_as_float(sx3)};
        v4i ab[2][3];
        v2i dd[2][4];
        v16i ihi[2], ilo[2];
        if (b0 + NBU <= b_end) {  // full stage (wavefront-uniform)
            // Software pipeline over the 4 blocks: while block j is scaled and accumulated on
            // the vector ALU, the MFMAs of block j+1 run and the LDS reads of block j+2 return.
            read_ab(base, 0, ab[0]);
            read_d_rows(base, 0, dd[0]);
            read_ab(base, 1, ab[1]);
            mfmas_rows(ab[0], ihi[0], ilo[0]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < NBU; ++j) {
                if (j + 1 < NBU) {
                    mfmas_rows(ab[(j + 1) & 1], ihi[(j + 1) & 1], ilo[(j + 1) & 1]);
                    __builtin_amdgcn_sched_barrier(0);  // younger LDS reads must not be waited for here
                    read_d_rows(base, j + 1, dd[(j + 1) & 1]);
                }
                if (j + 2 < NBU) read_ab(base, j + 2, ab[j & 1]);
                __builtin_amdgcn_sched_barrier(0);
                scale_acc_rows(ihi[j & 1], ilo[j & 1], dd[j & 1], sx[j]);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int j = 0; j < NBU - 1; ++j)
                if (b0 + j < b_end) {
                    read_ab(base, j, ab[0]);
                    read_d_rows(base, j, dd[0]);
                    mfmas_rows(ab[0], ihi[0], ilo[0]);
                    scale_acc_rows(ihi[0], ilo[0], dd[0], sx[j]);
                }
        }
    };

    auto wait_barrier = [&](bool one_ahead) {
        if (one_ahead) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n s_barrier" ::"n"(MMCfg<QT>::LPS) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n s_barrier" ::: "memory");
    };

    constexpr int RING = MMCfg<QT>::RING, AHEAD = MMCfg<QT>::AHEAD;
    issue(std::integral_constant<int, 0>{}, 0);
    if (AHEAD > 1 && nst > 1) issue(std::integral_constant<int, 1 % RING>{}, 1);
    auto k_loop = [&](auto nr) {
        for (int s0 = 0; s0 < nst; s0 += RING) {
#define PG_MM_STEP(U)                                                                     \
            if (s0 + U < nst) {                                                           \
                const int s = s0 + U;                                                     \
                wait_barrier(AHEAD > 1 && s + 1 < nst);                                   \
                if (s + AHEAD < nst) issue(std::integral_constant<int, (U + AHEAD) % RING>{}, s + AHEAD); \
                compute(nr, std::integral_constant<int, U>{}, s);                         \
            }
            PG_MM_STEP(0)
            PG_MM_STEP(1)
            if constexpr (RING > 2) { PG_MM_STEP(2) }
#undef PG_MM_STEP
        }
    };
    if (ntok > 16) {  // the same choice for the whole workgroup
        for (int s0 = 0; s0 < nst; s0 += RING) {
#define PG_MM_STEP(U)                                                                     \
            if (s0 + U < nst) {                                                           \
                const int s = s0 + U;                                                     \
                wait_barrier(AHEAD > 1 && s + 1 < nst);                                   \
                if (s + AHEAD < nst) issue(std::integral_constant<int, (U + AHEAD) % RING>{}, s + AHEAD); \
                compute_rows(std::integral_constant<int, U>{}, s);                        \
            }
            PG_MM_STEP(0)
            PG_MM_STEP(1)
            if constexpr (RING > 2) { PG_MM_STEP(2) }
#undef PG_MM_STEP
        }
        const bool tok_ok = tt * 32 + l31 < count;  // the token whose outputs this lane accumulated
        if (!tok_ok) return;
        const int pair = grp.lists ? grp.lists[(size_t)e * grp.list_stride + tt * 32 + l31] : tt * 32 + l31;
        float *y = out + bz * part_stride + (size_t)pair * n_out;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int r0 = row0 + 8 * g + 4 * hh;
            if (r0 + 3 < n_out && (n_out & 3) == 0) {
                *reinterpret_cast<float4 *>(y + r0) = make_float4(acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]);
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (r0 + q < n_out) y[r0 + q] = acc[4 * g + q];
            }
        }
        return;
    }
    if (ntok <= 8) k_loop(std::integral_constant<int, 4>{});
    else k_loop(std::integral_constant<int, 8>{});

    // lanes hold consecutive weight rows: each token's 32 outputs leave as one 128-byte run
    const int row = row0 + l31;
    if (row >= n_out) return;
    float *ybase = out + bz * part_stride + row;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int tok = 8 * (r >> 2) + 4 * hh + (r & 3);
        if (tok < ntok) {
            const int slot = tt * 32 + tok;
            const int pair = grp.lists ? grp.lists[(size_t)e * grp.list_stride + slot] : slot;
            ybase[(size_t)pair * n_out] = acc[r];
        }
    }
}

// ---- up to 16 activation rows over a Q4_0 or Q8_0 tensor in one launch after the digits ------------------------
// The product above splits K between workgroups where one token tile meets a wide tensor, and a third launch adds
// the planes.  Here a workgroup owns 16 NB weight rows and all of K: its NW wavefronts take one run of K each, every
// wavefront with an LDS ring of its own (no barrier in the loop: it reads only what it loaded itself), and their
// f32 tiles are added through LDS in a fixed order at the end.  A unit of the ring is 8 blocks (256 k): the weight
// tiles as whole 128-byte lines per row (8 rows an instruction, 16-byte chunk p of row r at position
// p ^ ((r >> 1) & 7)), their f16 scales, the two digit planes of the 16 token rows (256 bytes a row and plane,
// chunk c of token t at position c ^ t) and the tokens' block scales; NST - 1 units are in flight while one is
// consumed.  v_mfma_i32_16x16x32_i8 takes one block per instruction: lane -> (token or weight row lane % 16, 8 k at
// lane / 16), result lane -> weight row lane % 16, tokens 4 (lane / 16) + i.  The weights are read in the row-major
// planes every tensor has (no tile-major copy).  Each workgroup starts its walk through K at its own unit.
// MT: token rows the ring holds (4, 8 or 16: the digits are most of a unit, and the fewer there are the more units
// fit in flight); token slots from MT on read the rows of slots 0 .. MT - 1 again and are never stored.
// QT = 8 (Q8_0): a weight row is two streams (bytes 0 .. 15 and 16 .. 31 of its blocks, as the upload splits them), 32
// streams a tile, kept in LDS half-major (stream slot 16 half + row) so that the fragment reads of 16 rows and one
// half stay free of bank conflicts; no nibbles to unpack.
// Up to three tensors of equal K in one launch (q|k|v, gate|up of models::llama): tensor g owns the workgroups
// wg0[g] .. wg0[g + 1] - 1 (unused slots hold INT_MAX).
template <int QT, int NB, int MT, int NW, int NST>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2, MT <= 8 ? 4 : 2))) void gguf_skinny_kernel(const pg_skinny_group grp, int nb, int nbp, int m,
                                                                    const int8_t *__restrict__ digits, const float *__restrict__ xs) {
    int tg = 0;
#pragma unroll
    for (int i = 1; i < 3; ++i) tg = (int)blockIdx.x >= grp.wg0[i] ? i : tg;
    const uint8_t *__restrict__ qs = grp.qs[tg];
    const uint16_t *__restrict__ dsc = grp.d[tg];
    float *__restrict__ y = grp.y[tg];
    const float *__restrict__ res = grp.res[tg];
    const int n_out = grp.n[tg];
    constexpr int WF = QT == 8 ? 4 : 2, W_T = WF * 1024, D_T = 256, DIG = MT * 512, XS_B = 512, GQ = MT / 2;  // WF, GQ: weight, digit fills per unit
    constexpr int OFF_DS = NB * W_T, OFF_DG = OFF_DS + NB * D_T, OFF_X = OFF_DG + DIG, UNIT = OFF_X + XS_B;
    constexpr int LPS = WF * NB + 1 + GQ + 1;  // fills per unit
    static_assert((NST - 1) * LPS < 64 && NST <= 6 && NB <= 2, "the wait counter holds 63");
    extern __shared__ __attribute__((aligned(1024))) char lds[];  // NW rings of NST units; afterwards the wavefronts' tiles
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n0 = ((int)blockIdx.x - grp.wg0[tg]) * 16 * NB;
    const int units = nb / 8, per = (units + NW - 1) / NW;
    const int u_begin = wave * per, u_end = u_begin + per < units ? u_begin + per : units;
    const int cnt = u_end - u_begin;
    char *ring = lds + (size_t)wave * NST * UNIT;
    const size_t row_bytes = pg_mm_row_bytes(nb);

    // fill duties of this lane
    const uint8_t *w_src[NB][WF];  // stream slot 8 j + lane / 8 of tile c (Q4_0: slot = row; Q8_0: slot = 16 half + row), chunk (lane % 8) ^ ((row >> 1) & 7); rows past the end: the last
#pragma unroll
    for (int c = 0; c < NB; ++c)
#pragma unroll
        for (int j = 0; j < WF; ++j) {
            const int slot = 8 * j + (lane >> 3), r = slot & 15, half = slot >> 4, ch = (lane & 7) ^ ((r >> 1) & 7);
            const int row = pg_gemv_clamp_row(n0 + 16 * c + r, n_out);
            w_src[c][j] = qs + pg_gskinny_weight_offset(QT == 8 ? (size_t)row * 2 + half : (size_t)row, nb, 0, ch);
        }
    // scales: lanes 0 .. 16 NB - 1: scale tile (n0 / 8 + lane / 8), blocks of the unit lane % 8 (16 bytes = 8 rows x f16)
    const int ntile = (n_out + 7) / 8;
    const int dt = pg_gskinny_scale_tile(n0, lane, ntile);
    const char *d_src = reinterpret_cast<const char *>(dsc) + pg_gskinny_scale_offset(dt, nb, 0, lane);
    // digits: instruction q covers runs 4 q .. 4 q + 3, run = 2 token + plane; lane -> run 4 q + lane / 16, position lane % 16
    const int8_t *g_src[GQ];
#pragma unroll
    for (int q = 0; q < GQ; ++q) {
        const int run = 4 * q + (lane >> 4), tok = run >> 1, pl = run & 1;
        const int ch = (lane & 15) ^ tok;
        g_src[q] = digits + (size_t)(tok < m ? tok : 0) * row_bytes + (size_t)pl * nb * 32 + ch * 16;
    }
    // token scales: lanes 0 .. 2 MT - 1: token lane / 2, blocks 4 (lane % 2) .. + 3 of the unit
    const float *x_src = xs + (size_t)((lane >> 1) < m ? (lane >> 1) : 0) * nbp + 4 * (lane & 1);

    const int rot = cnt > 0 ? (int)((blockIdx.x * 5u) % (unsigned)cnt) : 0;
    auto issue = [&](auto slot, int t) {
        const size_t unit = (size_t)pg_skinny_walk_unit(u_begin, cnt, t, rot);
        char *base = ring + decltype(slot)::value * UNIT;
#pragma unroll
        for (int c = 0; c < NB; ++c)
#pragma unroll
            for (int j = 0; j < WF; ++j)
                __builtin_amdgcn_global_load_lds((gptr_t)(w_src[c][j] + unit * 128), (lptr_t)(base + c * W_T + j * 1024), 16, 0, 2);
        if (lane < 16 * NB) __builtin_amdgcn_global_load_lds((gptr_t)(d_src + unit * 128), (lptr_t)(base + OFF_DS), 16, 0, 0);
#pragma unroll
        for (int q = 0; q < GQ; ++q)
            __builtin_amdgcn_global_load_lds((gptr_t)(g_src[q] + unit * 256), (lptr_t)(base + OFF_DG + q * 1024), 16, 0, 0);
        if (lane < 2 * MT) __builtin_amdgcn_global_load_lds((gptr_t)(x_src + unit * 8), (lptr_t)(base + OFF_X), 16, 0, 0);
    };

    // fragment reads of this lane
    const int fr = lane & 15, g4 = lane >> 4, ft = fr & (MT - 1);
    const int w_rd = ((QT == 8 ? 16 * (g4 >> 1) : 0) + fr) * 128 + 8 * (g4 & 1), w_sw = (fr >> 1) & 7;  // + ((j ^ w_sw) * 16): bytes 8 (g4 & 1) .. of block j
    const int dg_rd = OFF_DG + ft * 512 + 8 * (g4 & 1);                     // + plane * 256 + (((2 j + (g4 >> 1)) ^ ft) * 16)
    const int ds_rd = OFF_DS + (fr >> 3) * 128 + (fr & 7) * 2;              // + tile c * 256 + j * 16: this lane's weight row
    const int x_rd = OFF_X + ((4 * g4) & (MT - 1)) * 32;                    // tokens 4 g4 .. + 3, 8 floats each
    const int left = 4 - 4 * (g4 >> 1);                                     // low nibbles for the even elements' half

    // Up to 8 token rows (QUAD): v_mfma_i32_4x4x4_i8 instead, sixteen independent 4 x 4 x 4 products an instruction.
    // Product b of a lane quad takes weight rows 4 (b % 4) .. + 3 against four tokens for FOUR DIFFERENT blocks of K
    // (block lane / 16 of a group of four): lane -> weight row lane % 16 of block lane / 16, its eight operand
    // dwords the block's 32 k; the token operand comes from lane % 4's token (one more set of instructions for
    // tokens 4 .. 7).  The result registers are the four tokens of the lane's own row and block, so nothing of the
    // 16 x 16 tile is padding: per block and 16 rows a quarter of the instructions of the form above, which spends
    // them on 16 token slots whatever the count.  A lane sums blocks lane / 16, + 4, ...; the four partial sums of a
    // row meet in the final pass through LDS.
    constexpr bool QUAD = MT <= 8;
    constexpr int NQ = QUAD ? MT / 4 : 1, NS = NB * NQ;  // accumulator sets: weight tiles x token quads
    float acc[NS][4];
#pragma unroll
    for (int c = 0; c < NS; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[c][i] = 0.0f;

    auto consume_quad = [&](auto slot) {
        const char *base = ring + decltype(slot)::value * UNIT;
        const int tq = lane & 3;  // the token (of each set) whose digits this lane hands to its quad
#pragma unroll
        for (int J = 0; J < 2; ++J) {
            const int blk = 4 * J + g4;
            // the lane's rows (one a tile) and block: 32 weight bytes each as eight dwords in the order of the digit halves
            int wk[NB][8];
            float dv[NB];
#pragma unroll
            for (int c = 0; c < NB; ++c) {
                const char *wt = base + c * W_T;
                if constexpr (QT == 4) {
                    const v4i wr = *reinterpret_cast<const v4i *>(wt + fr * 128 + ((blk ^ w_sw) * 16));
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        wk[c][p] = nibbles_to_i8x16(wr[p], 4);      // low nibbles: the even elements (digit half 0)
                        wk[c][4 + p] = nibbles_to_i8x16(wr[p], 0);  // high nibbles: the odd ones (half 1)
                    }
                } else {
                    const v4i w0 = *reinterpret_cast<const v4i *>(wt + fr * 128 + ((blk ^ w_sw) * 16));
                    const v4i w1 = *reinterpret_cast<const v4i *>(wt + (16 + fr) * 128 + ((blk ^ w_sw) * 16));
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        wk[c][p] = w0[p];
                        wk[c][4 + p] = w1[p];
                    }
                }
                dv[c] = half_bits_to_float(*reinterpret_cast<const unsigned short *>(base + ds_rd + c * D_T + blk * 16));
            }
#pragma unroll
            for (int s2 = 0; s2 < NQ; ++s2) {
                const int tok = 4 * s2 + tq;
                const char *dg = base + OFF_DG + tok * 512;
                const v4i h0 = *reinterpret_cast<const v4i *>(dg + (((2 * blk) ^ tok) * 16));
                const v4i h1 = *reinterpret_cast<const v4i *>(dg + (((2 * blk + 1) ^ tok) * 16));
                const v4i l0 = *reinterpret_cast<const v4i *>(dg + 256 + (((2 * blk) ^ tok) * 16));
                const v4i l1 = *reinterpret_cast<const v4i *>(dg + 256 + (((2 * blk + 1) ^ tok) * 16));
                int sx[4];  // the scales of tokens 4 s2 .. + 3 for this lane's block (read as integers: see gguf_mm_kernel)
#pragma unroll
                for (int i = 0; i < 4; ++i) sx[i] = *reinterpret_cast<const int *>(base + OFF_X + (4 * s2 + i) * 32 + blk * 4);
#pragma unroll
                for (int c = 0; c < NB; ++c) {
                    v4i ihi = {0, 0, 0, 0}, ilo = {0, 0, 0, 0};
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        ihi = __builtin_amdgcn_mfma_i32_4x4x4i8(h0[p], wk[c][p], ihi, 0, 0, 0);  // rows = tokens, columns = weight rows
                        ilo = __builtin_amdgcn_mfma_i32_4x4x4i8(l0[p], wk[c][p], ilo, 0, 0, 0);
                    }
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        ihi = __builtin_amdgcn_mfma_i32_4x4x4i8(h1[p], wk[c][4 + p], ihi, 0, 0, 0);
                        ilo = __builtin_amdgcn_mfma_i32_4x4x4i8(l1[p], wk[c][4 + p], ilo, 0, 0, 0);
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float fx = (float)(ihi[i] * 256 + ilo[i]) * __int_as_float(sx[i]);
                        acc[c * NQ + s2][i] = fmaf(dv[c], fx, acc[c * NQ + s2][i]);
                    }
                }
            }
        }
    };

    auto consume = [&](auto slot) {
        if constexpr (QUAD) {
            consume_quad(slot);
            return;
        }
        const char *base = ring + decltype(slot)::value * UNIT;
        // the scales of this lane's four tokens for the unit's eight blocks (read as integers: see gguf_mm_kernel)
        int sx[4][8];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const v4i t = *reinterpret_cast<const v4i *>(base + x_rd + i * 32 + h * 16);
                const int t0 = t[0], t1 = t[1], t2 = t[2], t3 = t[3];
                sx[i][4 * h] = t0; sx[i][4 * h + 1] = t1; sx[i][4 * h + 2] = t2; sx[i][4 * h + 3] = t3;
            }
        // Software pipeline over the unit's 8 blocks: while block j is scaled and accumulated on the vector ALU,
        // the MFMAs of block j + 1 run and the LDS reads of block j + 2 return (one wavefront a SIMD: nothing else
        // would fill those waits).
        long dh[2], dl[2];
        v2i wraw[2][NB];
        unsigned db[2][NB];
        v4i ihi[2][NB], ilo[2][NB];
        auto read = [&](int buf, int j) {
            const int dpos = (((2 * j + (g4 >> 1)) ^ ft) * 16);
            dh[buf] = *reinterpret_cast<const long *>(base + dg_rd + dpos);
            dl[buf] = *reinterpret_cast<const long *>(base + dg_rd + 256 + dpos);
#pragma unroll
            for (int c = 0; c < NB; ++c) wraw[buf][c] = *reinterpret_cast<const v2i *>(base + c * W_T + w_rd + ((j ^ w_sw) * 16));
        };
        auto read_d = [&](int buf, int j) {  // the blocks' weight scales of this lane's rows
#pragma unroll
            for (int c = 0; c < NB; ++c) db[buf][c] = *reinterpret_cast<const unsigned short *>(base + ds_rd + c * D_T + j * 16);
        };
        auto mfmas = [&](int buf, int c) {
            const v4i zero = {0, 0, 0, 0};
            {
                v2i wq = wraw[buf][c];
                if constexpr (QT == 4) {
                    wq[0] = nibbles_to_i8x16(wq[0], left);
                    wq[1] = nibbles_to_i8x16(wq[1], left);
                }
                const long wl = __builtin_bit_cast(long, wq);
                ihi[buf][c] = __builtin_amdgcn_mfma_i32_16x16x32_i8(dh[buf], wl, zero, 0, 0, 0);  // rows = tokens, columns = weight rows
                ilo[buf][c] = __builtin_amdgcn_mfma_i32_16x16x32_i8(dl[buf], wl, zero, 0, 0, 0);
            }
        };
        auto scale = [&](int buf, int j, int c) {
            {
                const float dv = half_bits_to_float(db[buf][c]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float fx = (float)(ihi[buf][c][i] * 256 + ilo[buf][c][i]) * __int_as_float(sx[i][j]);
                    acc[c][i] = fmaf(dv, fx, acc[c][i]);
                }
            }
        };
        read(0, 0);
        read_d(0, 0);
        read(1, 1);
#pragma unroll
        for (int c = 0; c < NB; ++c) mfmas(0, c);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            // tile by tile: the two MFMAs of block j + 1 are issued, then block j of the same tile is scaled while
            // they run (instructions issue in order: MFMAs back to back would hold the vector work behind them)
            // (the LDS reads of block j + 2 go first and have the whole step to return; their buffers held block j,
            // whose MFMAs were issued a step ago)
            if (j + 1 < 8) read_d((j + 1) & 1, j + 1);
            if (j + 2 < 8) read(j & 1, j + 2);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int c = 0; c < NB; ++c) {
                if (j + 1 < 8) {
                    mfmas((j + 1) & 1, c);
                    __builtin_amdgcn_sched_barrier(0);
                }
                scale(j & 1, j, c);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    if (cnt > 0) {
#define PG_GS_PRO(U) if (U < NST - 1 && U < cnt) issue(std::integral_constant<int, (U < NST ? U : 0)>{}, U);
        PG_GS_PRO(0) PG_GS_PRO(1) PG_GS_PRO(2) PG_GS_PRO(3) PG_GS_PRO(4)
#undef PG_GS_PRO
        for (int t0 = 0; t0 < cnt; t0 += NST) {
#define PG_GS_STEP(U)                                                                                          \
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
            PG_GS_STEP(0) PG_GS_STEP(1) PG_GS_STEP(2) PG_GS_STEP(3) PG_GS_STEP(4) PG_GS_STEP(5)
#undef PG_GS_STEP
        }
    }
    __syncthreads();  // the rings are done with: their space takes the wavefronts' tiles
    float *red = reinterpret_cast<float *>(lds);  // [NW][NS][4][64]
#pragma unroll
    for (int c = 0; c < NS; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[((wave * NS + c) * 4 + i) * 64 + lane] = acc[c][i];
    __syncthreads();
    if constexpr (QUAD) {
        for (int e = threadIdx.x; e < NS * 4 * 16; e += 64 * NW) {
            const int r = e & 15, i = (e >> 4) & 3, c = e >> 6;  // c = tile * NQ + token quad
            float sum = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; ++w)  // ascending runs of K, within a run the four block classes in order
#pragma unroll
                for (int q = 0; q < 4; ++q) sum += red[((w * NS + c) * 4 + i) * 64 + 16 * q + r];
            const int tok = 4 * (c % NQ) + i, row = n0 + 16 * (c / NQ) + r;
            if (tok < m && row < n_out) {
                const float v = QT == 4 ? sum * 0.0625f : sum;  // (Q4_0: the weight operand was 16 * (q - 8))
                y[(size_t)tok * n_out + row] = res ? res[(size_t)tok * n_out + row] + v : v;
            }
        }
        return;
    }
    for (int e = threadIdx.x; e < NB * 4 * 64; e += 64 * NW) {
        const int l = e & 63, i = (e >> 6) & 3, c = e >> 8;
        float sum = red[(c * 4 + i) * 64 + l];
#pragma unroll
        for (int w = 1; w < NW; ++w) sum += red[((w * NB + c) * 4 + i) * 64 + l];  // ascending runs of K
        const int tok = 4 * (l >> 4) + i, row = n0 + 16 * c + (l & 15);
        if (tok < m && row < n_out) {
            const float v = QT == 4 ? sum * 0.0625f : sum;  // (Q4_0: the weight operand was 16 * (q - 8))
            y[(size_t)tok * n_out + row] = res ? res[(size_t)tok * n_out + row] + v : v;
        }
    }
}

// y[i] = part[0][i] + part[1][i] + ... in a fixed order.
__global__ void sum_parts_kernel(const float *__restrict__ part, size_t n, int ks, size_t stride, float *__restrict__ y) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float acc = part[i];
    for (int s = 1; s < ks; ++s) acc += part[(size_t)s * stride + i];
    y[i] = acc;
}

}  // namespace

pg_status pg_launch_sum_parts(pg_ctx *ctx, const float *part, size_t n, int ks, size_t stride, float *y) {
    if (n == 0) return PG_OK;
    return pg_launch(ctx, "gguf_mm_sum_parts", sum_parts_kernel, dim3(grid_for(n, 256)), dim3(256), 0, part, n, ks, stride, y);
}

size_t pg_mmdigits_bytes(size_t rows, size_t k) {
    const size_t nb = k / 32, nbp = pg_round_up(nb, 4);
    return rows * pg_mm_row_bytes(nb) + 2 * pg_round_up(rows * nbp * sizeof(float), 256);
}

pg_mmdigits pg_mmdigits_carve(void *base, size_t rows, size_t k) {
    const size_t nb = k / 32;
    pg_mmdigits md;
    char *p = static_cast<char *>(base);
    md.digits = reinterpret_cast<int8_t *>(p);
    p += rows * pg_mm_row_bytes(nb);
    md.xs = reinterpret_cast<float *>(p);
    p += pg_round_up(rows * pg_round_up(nb, 4) * sizeof(float), 256);
    md.xsum = reinterpret_cast<float *>(p);
    md.rows = rows;
    md.k = k;
    return md;
}

pg_status pg_launch_x_to_mm_digits(pg_ctx *ctx, const float *x_dev, size_t rows, size_t k, int ggml_type,
                                   const pg_mmdigits &md) {
    if (rows == 0) return PG_OK;
    if (rows > 65535) return pg_fail(PG_EUNSUPPORTED, "x_to_mm_digits: more than 65535 activation rows");
    const int nb = (int)(k / 32), nbp = (int)pg_round_up(nb, 4);
    const dim3 grid(grid_for(nb, 32), (unsigned)rows);
    if (ggml_type == PG_GGML_Q4_0 || ggml_type == PG_GGML_Q4_1)
        return pg_launch(ctx, "x_to_mm_digits", x_to_mm_digits_kernel<true>, grid, dim3(256), 0, x_dev, nb, nbp, md.digits, md.xs,
                         ggml_type == PG_GGML_Q4_1 ? md.xsum : (float *)nullptr);
    return pg_launch(ctx, "x_to_mm_digits", x_to_mm_digits_kernel<false>, grid, dim3(256), 0, x_dev, nb, nbp, md.digits, md.xs,
                     (float *)nullptr);
}

pg_status pg_launch_q41_offset(pg_ctx *ctx, const pg_gguf_tensor *w, const pg_mmdigits &md, size_t rows, float *y) {
    const int nb = (int)(w->k_in / 32), nbp = (int)pg_round_up(nb, 4);
    const bool few = rows <= 64;
    const size_t lds = ((size_t)nb + (few ? 3 * 64 : 0)) * Q41_TT * sizeof(float);
    if (lds > 128 * 1024) return pg_fail(PG_EUNSUPPORTED, "gguf_matmul: Q4_1 rows of %zu on the matrix-core route", w->k_in);
    PG_TRY(pg_allow_dynamic_lds(ctx, few ? (const void *)q41_offset_kernel<4> : (const void *)q41_offset_kernel<1>, 128 * 1024));
    if ((rows + Q41_TT - 1) / Q41_TT > 65535) return pg_fail(PG_EUNSUPPORTED, "gguf_matmul: too many activation rows");
    const dim3 grid(grid_for(w->n_out, few ? 64 : 256), (unsigned)((rows + Q41_TT - 1) / Q41_TT));
    if (few)
        return pg_launch(ctx, "gguf_q4_1_offsets", q41_offset_kernel<4>, grid, dim3(256), lds, (const uint16_t *)w->d,
                         (const uint16_t *)w->m, (int)w->n_out, nb, (const float *)md.xsum, nbp, (int)rows, y);
    return pg_launch(ctx, "gguf_q4_1_offsets", q41_offset_kernel<1>, grid, dim3(256), lds, (const uint16_t *)w->d,
                     (const uint16_t *)w->m, (int)w->n_out, nb, (const float *)md.xsum, nbp, (int)rows, y);
}

// Digits of `act_rows` activation rows that no XCD's L2 (4 MiB) can keep while every workgroup
// of a token tile reads them: then K is split so that a chunk's share does fit, and the chunks
// are dealt to XCDs (see the kernel).  Without the split a K = 32768 product over 128 rows
// fetches its 8 MiB of digits once per 128-row group: 1.2x the weight bytes in total.
static bool digits_exceed_l2(size_t act_rows, size_t nb) { return act_rows * pg_mm_row_bytes(nb) > (2u << 20); }

int pg_gguf_mm_splitk(const pg_ctx *ctx, size_t n_out, size_t k_in, size_t groups, size_t act_rows, bool grouped,
                      int *chunk_out, bool *xcd_chunks) {
    const size_t nb = k_in / 32;
    const size_t wgs = ((n_out + 127) / 128) * (groups ? groups : 1);
    // A short K is split only as far as every workgroup is still resident at once: a second round of
    // workgroups would pay the start-up latency again.  (Three workgroups fit on a CU; splitting for
    // three a CU instead of two measured the same on the 16-row product, with more partial planes to sum.)
    const size_t slots = 2 * (size_t)ctx->num_cu;
    size_t ks = slots / wgs;
    if (ks > 8) ks = 8;
    if (ks < 1) ks = 1;
    bool by_xcd = false;
    // (Plain products over 16 token tiles and more are not split: they run as super-tiles.)
    if ((grouped || groups < 16) && digits_exceed_l2(act_rows, nb)) {
        size_t c = 2;
        while (c < 8 && act_rows * pg_mm_row_bytes(nb) > c * (size_t)(2u << 20)) c *= 2;
        // worth it while the partial sums (written and read back) stay under a tenth of the weights
        const bool cheap = c * act_rows * 8 * 10 <= nb * 34 * (grouped ? groups : 1);  // per weight row
        if (c >= ks && nb / c >= 8 * NBU && cheap) {
            ks = c;
            by_xcd = true;
        }
    }
    size_t chunk = pg_round_up((nb + ks - 1) / ks, NBU);
    if (chunk < 2 * NBU) chunk = 2 * NBU;
    const size_t ks_real = (nb + chunk - 1) / chunk;
    if (ks_real != ks) by_xcd = false;  // the deal needs 2, 4 or 8 chunks exactly
    if (chunk_out) *chunk_out = (int)chunk;
    if (xcd_chunks) *xcd_chunks = by_xcd;
    return (int)ks_real;
}

// Up to 16 rows over a Q4_0 or Q8_0 tensor whose K is a multiple of 256: the one-launch product (see the kernel).
// With 9 .. 16 token rows (the 16 x 16 x 32 form) the kernel is bound by instruction issue (about 500 instructions per
// 8 blocks and weight tile, most of them the per-block scaling of 16 token slots), seven wavefronts fit a CU at two
// units a ring, and it beats digits + product over K chunks + their sum only where those are short of workgroups
// (14336 -> 4096: 18.2 against 24.3 us; 4096 -> 4096: 8.8 against 13.3; but 4096 -> 14336: 21.5 against 20.0 - 22.0).
// Up to 8 token rows (the 4 x 4 x 4 form) a quarter of those instructions remain and the kernel is bound by how many
// bytes its rings keep in flight: 4 x 4096 -> 14336 takes 9.0 us (with its arithmetic switched off 8.6 - 9.1; in the
// 16 x 16 x 32 form it took 11.9).
bool pg_gguf_skinny_takes(const pg_ctx *ctx, int ggml_type, size_t m, size_t n_out, size_t k_in) {
    return (ggml_type == PG_GGML_Q4_0 || ggml_type == PG_GGML_Q8_0) && m >= 2 && (m <= 8 || (m <= 16 && n_out / 32 < (size_t)ctx->num_cu)) &&
           k_in % 256 == 0 && k_in >= 1024 && n_out >= 1 && n_out < (1u << 30) && k_in < (1u << 24);
}

pg_status pg_launch_gguf_skinny_group(pg_ctx *ctx, int ggml_type, size_t k_in, const pg_gguf_tensor *const *w, float *const *y, int count,
                                      size_t m, const pg_mmdigits &md, const float *residual) {
    if (count < 1 || count > 3) return pg_fail(PG_EINVAL, "gguf (few rows in one launch): %d tensors (1 .. 3)", count);
    size_t n_total = 0;
    for (int i = 0; i < count; ++i) {
        if (w[i]->k_in != k_in || w[i]->ggml_type != ggml_type) return pg_fail(PG_EINVAL, "gguf (few rows in one launch): the tensors differ in K or type");
        n_total += w[i]->n_out;
    }
    if (!pg_gguf_skinny_takes(ctx, ggml_type, m, n_total, k_in)) return pg_fail(PG_EINVAL, "gguf (few rows in one launch): [%zu x %zu] x %zu", m, k_in, n_total);
    const int nb = (int)(k_in / 32), nbp = (int)pg_round_up(nb, 4);
    const bool q8 = ggml_type == PG_GGML_Q8_0;
    // Wavefronts (runs of K) per workgroup: as many as keep every workgroup resident at once.  The rings: units of
    // 4.75 / 6.75 / 10.75 KiB for 4 / 8 / 16 token rows (Q8_0: 2 KiB more), as many stages as let eight wavefronts
    // share a CU's LDS (16 token rows: two stages and six or seven wavefronts; three stages and four were slower).
    // Two weight tiles a workgroup (32 rows) where that still leaves a workgroup for every CU: the digits, which
    // every workgroup fetches for all of K, then cost half as much per weight byte.
    const int tiles = (m <= 8 && n_total / 32 >= (size_t)ctx->num_cu) ? 2 : 1;
    const size_t unit_bytes = (size_t)tiles * ((q8 ? 4096 : 2048) + 256) + (m <= 4 ? 4 : (m <= 8 ? 8 : 16)) * 512 + 512;
    const int stages = 2;  // (three stages on fewer wavefronts: 10.7 - 10.9 against 9.0 us on 4 x 4096 -> 14336)
    const size_t lds_cu = 160u << 10;
    pg_skinny_group grp;
    int wgs = 0;
    for (int i = 0; i < 3; ++i) {
        const bool used = i < count;
        grp.qs[i] = used ? w[i]->qs : nullptr;
        grp.d[i] = used ? w[i]->d : nullptr;
        grp.y[i] = used ? y[i] : nullptr;
        grp.res[i] = i == 0 ? residual : nullptr;
        grp.n[i] = used ? (int)w[i]->n_out : 0;
        grp.wg0[i] = used ? wgs : INT_MAX;
        if (used) wgs += (int)((w[i]->n_out + 16 * tiles - 1) / (16 * tiles));
    }
    const dim3 grid((unsigned)wgs);
    // LDS is handed out per workgroup: nw wavefronts' rings each; up to 16 wavefronts a CU (4 a SIMD)
    const size_t units = (size_t)nb / 8;
    auto fits = [&](int nw_) {
        if (m > 8) return (size_t)grid.x * nw_ <= (size_t)ctx->num_cu * (q8 ? 6 : 7);
        const size_t per_cu = std::min<size_t>(lds_cu / ((size_t)nw_ * stages * unit_bytes), 16 / nw_);
        return (size_t)grid.x <= (size_t)ctx->num_cu * per_cu;
    };
    int nw = m <= 8 ? 8 : 4;
    while (nw > 1 && (!fits(nw) || units / nw < 4)) nw >>= 1;
#define PG_GSK_LAUNCH(QTT, NBB, MTT, NWW, NSTT)                                                                                \
    do {                                                                                                                       \
        auto kern = gguf_skinny_kernel<QTT, NBB, MTT, NWW, NSTT>;                                                              \
        const size_t lds = (size_t)NWW * NSTT * (NBB * ((QTT == 8 ? 4096 : 2048) + 256) + MTT * 512 + 512);                    \
        PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));                                                            \
        return pg_launch(ctx, QTT == 8 ? "gguf_q8_0_few_rows_mm" : "gguf_q4_0_few_rows_mm", kern, grid, dim3(64 * NWW), lds,  \
                         grp, nb, nbp, (int)m, (const int8_t *)md.digits, (const float *)md.xs);                               \
    } while (0)
#define PG_GSK_NW8(QTT, NBB, MTT, NSTT)                     \
    switch (nw) {                                           \
        case 8: PG_GSK_LAUNCH(QTT, NBB, MTT, 8, NSTT);      \
        case 4: PG_GSK_LAUNCH(QTT, NBB, MTT, 4, NSTT);      \
        case 2: PG_GSK_LAUNCH(QTT, NBB, MTT, 2, NSTT);      \
        default: PG_GSK_LAUNCH(QTT, NBB, MTT, 1, NSTT);     \
    }
#define PG_GSK_NW4(QTT, MTT, NSTT)                        \
    switch (nw) {                                         \
        case 4: PG_GSK_LAUNCH(QTT, 1, MTT, 4, NSTT);      \
        case 2: PG_GSK_LAUNCH(QTT, 1, MTT, 2, NSTT);      \
        default: PG_GSK_LAUNCH(QTT, 1, MTT, 1, NSTT);     \
    }
    if (q8) {
        if (m <= 4) { if (tiles == 2) PG_GSK_NW8(8, 2, 4, 2) else PG_GSK_NW8(8, 1, 4, 2) }
        if (m <= 8) { if (tiles == 2) PG_GSK_NW8(8, 2, 8, 2) else PG_GSK_NW8(8, 1, 8, 2) }
        PG_GSK_NW4(8, 16, 2)
    }
    if (m <= 4) { if (tiles == 2) PG_GSK_NW8(4, 2, 4, 2) else PG_GSK_NW8(4, 1, 4, 2) }
    if (m <= 8) { if (tiles == 2) PG_GSK_NW8(4, 2, 8, 2) else PG_GSK_NW8(4, 1, 8, 2) }
    PG_GSK_NW4(4, 16, 2)
#undef PG_GSK_NW8
#undef PG_GSK_NW4
#undef PG_GSK_LAUNCH
}

pg_status pg_launch_gguf_mm(pg_ctx *ctx, int ggml_type, size_t n_out, size_t k_in, const uint8_t *qs,
                            const uint16_t *d, const pg_mm_group &grp, size_t total_pairs, const pg_mmdigits &md,
                            float *y, float *part, bool keep_parts) {
    if (total_pairs == 0) return PG_OK;
    const int nb = (int)(k_in / 32), nbp = (int)pg_round_up(nb, 4);
    const size_t experts = grp.counts ? (size_t)grp.num_experts : 1;
    int chunk = 0;
    const size_t gy = experts * (size_t)grp.tiles_per_expert;
    // token tiles that certainly hold work: all of them without expert lists, one per expert with
    bool by_xcd = false;
    const int ks = pg_gguf_mm_splitk(ctx, n_out, k_in, grp.counts ? experts : gy, md.rows, grp.counts != nullptr, &chunk, &by_xcd);
    if (ks > 1 && !part) return pg_fail(PG_EINVAL, "gguf_mm: split-K needs a partial-sum buffer");
    if (grp.nseg && ((ks > 1 && !keep_parts) || grp.counts || !grp.tiled))
        return pg_fail(PG_EINVAL, "gguf_mm: several tensors in one launch leave their K chunks unsummed, take no expert lists and read tile-major copies");
    if (gy > 65535) return pg_fail(PG_EUNSUPPORTED, "gguf_mm: too many token tiles");
    dim3 grid(grid_for(n_out, 128), (unsigned)gy, (unsigned)ks);
    pg_mm_group g2 = grp;
    g2.remap_rg = g2.remap_tiles = 0;
    if (!grp.counts && ks == 1 && gy >= 16) {  // a plain product over many token tiles: see the kernel
        g2.remap_rg = (int)grid.x;
        g2.remap_tiles = (int)gy;
        const size_t supertiles = (size_t)((grid.x + 3) / 4) * ((gy + 7) / 8);
        grid = dim3((unsigned)((supertiles + 7) / 8 * 8 * 32), 1, 1);
    }
    g2.xcd_ks = 0;
    if (by_xcd) {
        g2.xcd_ks = ks;
        g2.remap_rg = (int)grid.x;
        g2.remap_tiles = (int)gy;
        const size_t per = 8 / (size_t)ks, tiles = (size_t)grid.x * gy;
        grid = dim3((unsigned)((tiles + per - 1) / per * 8), 1, 1);
    }
    float *dst = ks > 1 ? part : y;
    const size_t stride = total_pairs * n_out;
    const size_t lds = ggml_type == PG_GGML_Q4_0 ? (size_t)MMCfg<4>::RING * MMCfg<4>::STAGE : (size_t)MMCfg<8>::RING * MMCfg<8>::STAGE;
    auto launch = [&](auto kern, const char *name) -> pg_status {
        PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));
        return pg_launch(ctx, name, kern, grid, dim3(256), lds, qs, d, g2, (int)n_out, nb, nbp, chunk, md.digits, md.xs, dst,
                         stride);
    };
    const bool nt = grp.counts != nullptr;
    if (ggml_type == PG_GGML_Q4_0) PG_TRY(nt ? launch(gguf_mm_kernel<4, true>, "gguf_mm_q4_0") : launch(gguf_mm_kernel<4, false>, "gguf_mm_q4_0"));
    else PG_TRY(nt ? launch(gguf_mm_kernel<8, true>, "gguf_mm_q8_0") : launch(gguf_mm_kernel<8, false>, "gguf_mm_q8_0"));
    if (ks > 1 && !keep_parts)
        PG_TRY(pg_launch(ctx, "gguf_mm_sum_parts", sum_parts_kernel, dim3(grid_for(stride, 256)), dim3(256), 0, part, stride, ks,
                         stride, y));
    return PG_OK;
}
