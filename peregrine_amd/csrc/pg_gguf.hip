// gguf::* entry points: f16 conversion, block dequantisation, and the fused
// dequantise-matmul over GGUF Q4_0 / Q8_0 weights kept quantised in HBM.
//
// Fused product, y[m, n] = sum_k x[m, k] * (q[n, k] * d[n, k/32]):
//  * each block of 32 activations is first rewritten as fixed point, x[k] = s * X[k] with s
//    a power of two taken from the block's absmax (absolute error <= 2^-19 (Q4_0) or 2^-23
//    (Q8_0) of the block's max|x| per element, at or below what an f32 accumulation commits
//    anyway), and X is split into signed digits: five 4-bit digits for Q4_0, three bytes
//    for Q8_0;
//  * the inner sums over one block, sum_k q * digit_j, are then exact integer dot products
//    on packed data with no per-element unpack or int->float conversion: Q4_0 nibbles are
//    stored with their top bit flipped at upload, which makes each nibble the two's
//    complement of (q - 8), so v_dot8_i32_i4 multiplies 8 weights by 8 activation digits per
//    instruction straight from the packed bytes; Q8_0 uses v_dot4_i32_i8;
//  * the digit sums are recombined exactly in integers, converted once and scaled by
//    d * s in f32 once per block.
// The result differs from the reference's dequantise-then-f32-matmul only by rounding noise
// (relative tolerance 1e-3 is the contract; the tests hold this path to 2e-5).
#include <mutex>
#include <new>
#include "pg_internal.h"
#include "pg_stream_addr.h"
#include "pg_digits.h"

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
// Q4_0: qs[(n*nb + b)*16 .. +16] = the block's 16 nibble bytes, each nibble's top bit flipped.
// Q8_0: qs[((n*2 + h)*nb + b)*16 .. +16] = bytes 16h..16h+15 of the block's 32 i8.
// d[((n/8)*nb + b)*8 + n%8] = the block's f16 scale: tiles of 8 rows, so one 128-bit load
// gives a lane the scales of its block for 8 consecutive weight rows (rows past n_out: 0).
// Q4_1: as Q4_0, plus the block's f16 offset in m[] (tiled like d); q - 8 goes to the dot
// product and the 8 is folded into the offset term at run time.
__global__ void split_blocks_kernel(const uint8_t *__restrict__ raw, size_t n_out, size_t nb,
                                    int ggml_type, uint8_t *__restrict__ qs,
                                    uint16_t *__restrict__ d, uint16_t *__restrict__ m) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t n_pad = (n_out + 7) / 8 * 8;
    if (i >= n_pad * nb) return;
    const size_t n = i / nb, b = i - n * nb;
    uint16_t *dd = d + ((n / 8) * nb + b) * 8 + (n % 8);
    if (n >= n_out) {
        *dd = 0;
        if (m) m[((n / 8) * nb + b) * 8 + (n % 8)] = 0;
        return;
    }
    if (ggml_type == PG_GGML_Q4_1) {
        const uint8_t *blk = raw + i * 20;
        *dd = ld_u16(blk);
        m[((n / 8) * nb + b) * 8 + (n % 8)] = ld_u16(blk + 2);
        for (int j = 0; j < 16; ++j) qs[i * 16 + j] = blk[4 + j] ^ 0x88;
    } else if (ggml_type == PG_GGML_Q4_0) {
        const uint8_t *blk = raw + i * 18;
        *dd = ld_u16(blk);
        for (int j = 0; j < 16; ++j) qs[i * 16 + j] = blk[2 + j] ^ 0x88;  // nibble -> (q - 8) in two's complement
    } else {
        const uint8_t *blk = raw + i * 34;
        *dd = ld_u16(blk);
        for (int h = 0; h < 2; ++h)
            for (int j = 0; j < 16; ++j) qs[((n * 2 + h) * nb + b) * 16 + j] = blk[2 + 16 * h + j];
    }
}

// ---- activation blocks -> fixed point digits ------------------------------------------
// For every block of 32 activations: x[k] = s * X[k] with s a power of two chosen from the
// block's absmax.  Output for activation row m (all of it in the scratch arena):
//   xs[m][b]            the block's scale s (NaN if the block holds a NaN or inf)
//   digits[m][j][b]     16 bytes per (plane j, block b); lanes that own consecutive blocks
//                       read consecutive 16-byte chunks.
//     Q4_0 (NIB): |X| < 2^18, X = sum_j 16^j n_j with five signed 4-bit digits; plane j holds
//                 n_j of the block's 32 elements, element e in nibble e (the order the
//                 weight bytes pack them: byte i = elements 2i (low) and 2i+1 (high)).
//     Q8_0:       |X| < 2^22, X = 65536 a0 + 256 a1 + a2 with signed byte digits; plane
//                 2j+h holds a_j of elements 16h..16h+15.
// 8 consecutive threads own one block (4 elements each); a workgroup covers 32 blocks.
template <bool NIB>
__global__ __launch_bounds__(256) void x_to_digits_kernel(const float *__restrict__ x, int nb,
                                                          int8_t *__restrict__ digits,
                                                          float *__restrict__ xs, float *__restrict__ xsum) {
    const size_t row = blockIdx.y;
    const int b = blockIdx.x * 32 + (threadIdx.x >> 3), sub = threadIdx.x & 7;
    if (b >= nb) return;  // whole 8-thread groups leave together
    const float4 v = reinterpret_cast<const float4 *>(x + (row * nb + b) * 32)[sub];
    const float f[4] = {v.x, v.y, v.z, v.w};
    pg_emit_digits<NIB>(f, row, b, sub, nb, digits, xs, xsum);
}

// ---- M = 1 fused dequant-GEMV ------------------------------------------------------
// One wavefront per workgroup, no LDS, no barrier.  Lane l owns blocks l, l+64, ... (BPL
// of them per K segment of 64*BPL blocks): its activation digits, block sums and block
// scales for those blocks sit in registers while the wavefront walks R*NG weight rows, R at
// a time, requesting the next R rows before it consumes the current ones.  One wavefront
// load of weights covers 64 consecutive blocks (1 KiB) of one row.
// sum over one block of (weight) * (activation fixed-point value X), exact, as an i32.
// Q4_0: w = 16 bytes of biased nibbles, xn[j] = plane j (32 signed nibbles).
__device__ __forceinline__ int block_dot_q4(const v4i w, const v4i (&xn)[5]) {
    int acc = 0;
#pragma unroll
    for (int j = 4; j >= 0; --j) {  // Horner over the 4-bit digits: acc = 16*acc + I_j
        int ij = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t) ij = __builtin_amdgcn_sdot8(w[t], xn[j][t], ij, false);
        acc = acc * 16 + ij;
    }
    return acc;  // |acc| <= 32 * 8 * 2^18 = 2^26
}
// Q8_0: w0/w1 = the block's 32 i8, x[j][h] = byte digit j of half h.  Returns the high and
// low parts separately (65536 * i0 would overflow i32 when added to the rest).
__device__ __forceinline__ void block_dot_q8(const v4i w0, const v4i w1, const v4i (&x)[6], int &hi, int &lo) {
    int i[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        i[j] = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            i[j] = __builtin_amdgcn_sdot4(w0[t], x[2 * j][t], i[j], false);
            i[j] = __builtin_amdgcn_sdot4(w1[t], x[2 * j + 1][t], i[j], false);
        }
    }
    hi = i[0];
    lo = i[1] * 256 + i[2];
}

// Hardware f16 -> f32 (exact for every non-NaN input).
__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}

__device__ __forceinline__ float wave_sum_f32(float v) { return pg_wave_sum_f32(v); }

typedef const v4i __attribute__((address_space(1))) *gv4i_ptr;  // loads known to be global, not flat

constexpr int GGUF_LDSX_UNITS = 3072;  // XM 2: 16-byte units of digits and scales a workgroup carries into LDS in one go

template <int QT, int BPL, int R>
struct RowLoads {
    v4i w[R][BPL][QT == 8 ? 2 : 1];
};

// blockIdx.x = group of RW consecutive weight rows (RW divides 8: one scale tile),
// blockIdx.y = batch item (activation row / MoE pair).  With a table, item i multiplies by
// expert table[expert_of[i]] and reads activation row i / x_row_div; without one, every item
// uses (qs0, d0).  R rows are in flight at a time (NG = RW / R groups, double-buffered).
// Q41 (with QT = 4): every block also has an offset m; its term (8 d + m) * sum_k x_k uses the
// block sums written with the digits.
// XM, where the activation digits come from:
//   0  from memory, every wavefront its own reads (the rows come as digits, one row per item / x_row_div);
//   1  the one activation row, the same for every item, arrives in f32 (x_f32) and the workgroup -- NW
//      wavefronts, each with its own RW rows -- rewrites it as digits into LDS itself, after every
//      wavefront has requested its first weight rows: one launch instead of two, and the digit arithmetic
//      (18 vector operations per element, shared by NW wavefronts) runs while those first loads are in
//      flight.  NORM: that row is RMSNorm(x_f32) with the weights epi.gamma (src/nn.rs:560-652): the digits
//      are those of x * gamma, the sum of squares rides on the digits' barrier, and the scalar factor
//      multiplies the product: the norm costs no launch and no extra barrier;
//   2  from memory, but once per workgroup, into LDS, for its NW wavefronts: with few rows per wavefront
//      under a long row (K = 14336 is 36 KB of digits, more than the CU's vector cache) every wavefront
//      would otherwise pull the whole of them through L2 again.
// EPI (one item, NW * RW = 32: a workgroup owns one block of 32 output rows) makes the output the digit
// input of the NEXT product, so that the one-token step of models::llama needs no launch in between:
//   1  y (+ residual) is stored as usual, and also as digits of y * gamma (the RMSNorm weights,
//      src/nn.rs:560-652) with the block's sum of y^2 in ss_out[block]: the normalisation factor is a
//      scalar, which the next product applies to its result (POST);
//   2  the workgroup multiplies by two tensors (gate, then up = epi.qs1 / d1) and leaves only the digits
//      of silu(gate) * up (src/models/llama/decoder.rs:143-150).
// POST: the product is multiplied by 1 / sqrt(sum(ss_in[0 .. ss_n)) * ss_inv_dim + eps) before anything else.
template <int QT, int BPL, int RW, int R, bool Q41 = false, int XM = 0, int NW = 1, int EPI = 0, bool POST = false, bool NORM = false>
__global__ __launch_bounds__(64 * NW) void gguf_gemv_kernel(
    const uint8_t *__restrict__ qs0, const uint16_t *__restrict__ d0, pg_gemv_batch batch,
    int n_out, int nb, const int8_t *__restrict__ digits_base, const float *__restrict__ xs_base,
    float *__restrict__ y_base, const float *__restrict__ residual_base, const uint16_t *__restrict__ m0,
    const float *__restrict__ xsum_base, const float *__restrict__ x_f32, pg_gemv_epi epi) {
    constexpr int SEG = 64 * BPL;  // blocks per K segment
    constexpr bool XF32 = XM == 1, LDSX = XM == 2;
    constexpr int NT = EPI == 2 ? 2 : 1;  // tensors per workgroup
    constexpr int NG = RW / R, NGT = NG * NT;
    static_assert(EPI == 0 || (XM == 0 && !Q41 && NW * RW == 32), "an output block of 32 rows per workgroup");
    static_assert(EPI != 0 || XM != 0 || NW == 1, "several wavefronts per workgroup only where they share something");
    constexpr int NH = QT == 8 ? 2 : 1;
    constexpr int NP = QT == 8 ? 6 : 5;  // digit planes
    static_assert(XM == 0 || !Q41, "the LDS forms hold no block sums");
    static_assert(!NORM || (XM == 1 && !POST), "the norm is folded in where the row arrives in f32");
    extern __shared__ __attribute__((aligned(16))) char lds_digits[];  // XM 1, 2: [6 planes][nb][16 B], then nb scales
    const int item = blockIdx.y;
    const uint8_t *qs_any = qs0;
    const uint16_t *d_any = d0;
    if (batch.qs_table) {
        const int e = batch.expert_of[item];
        qs_any = batch.qs_table[e];
        d_any = batch.d_table[e];
    }
    const gv4i_ptr qs = (gv4i_ptr)(uintptr_t)qs_any;
    const gv4i_ptr dsc = (gv4i_ptr)(uintptr_t)d_any;
    const gv4i_ptr qs_t[2] = {qs, (gv4i_ptr)(uintptr_t)epi.qs1};
    const gv4i_ptr dsc_t[2] = {dsc, (gv4i_ptr)(uintptr_t)epi.d1};
    const size_t xrow = (size_t)(item / batch.x_row_div);
    const gv4i_ptr digits = (gv4i_ptr)(uintptr_t)(digits_base + xrow * (size_t)nb * 96);
    const float *__restrict__ xs = xs_base + xrow * (size_t)nb;
    const gv4i_ptr msc = (gv4i_ptr)(uintptr_t)m0;
    const float *__restrict__ xsum = Q41 ? xsum_base + xrow * (size_t)nb : nullptr;
    float *__restrict__ y = y_base + (size_t)item * n_out;
    const int lane = threadIdx.x & 63;
    const int row0 = (blockIdx.x * NW + (threadIdx.x >> 6)) * RW;
    int8_t *const ldig = reinterpret_cast<int8_t *>(lds_digits);
    float *const lxs = reinterpret_cast<float *>(lds_digits + (size_t)nb * 96);
    float acc[NGT][R];  // group g: tensor g / NG, rows (g % NG) * R ..
#pragma unroll
    for (int g = 0; g < NGT; ++g)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[g][r] = 0.0f;
    float post = 1.0f;
    float ssv[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // POST: requested first, needed last (ss_n <= 256)
    if constexpr (POST) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (lane + 64 * i < epi.ss_n) ssv[i] = epi.ss_in[lane + 64 * i];
    }
    float4 gm = {0.0f, 0.0f, 0.0f, 0.0f};     // EPI 1: the norm weights of the workgroup's block, likewise
    if constexpr (EPI == 1) {
        if (threadIdx.x < 8) gm = reinterpret_cast<const float4 *>(epi.gamma)[blockIdx.x * 8 + threadIdx.x];
    }

    for (int seg0 = 0; seg0 < nb; seg0 += SEG) {
        const int seg_n = (nb - seg0 < SEG) ? nb - seg0 : SEG;
        int blk[BPL];  // this lane's blocks; lanes past the segment end re-read block seg0 with a zero scale
#pragma unroll
        for (int p = 0; p < BPL; ++p) blk[p] = pg_gemv_lane_block(seg0, lane, p, seg_n);
        auto load_rows = [&](RowLoads<QT, BPL, R> &L, int g) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int row = pg_gemv_clamp_row(row0 + (g % NG) * R + r, n_out);  // clamped; masked at the store
#pragma unroll
                for (int p = 0; p < BPL; ++p)
#pragma unroll
                    for (int h = 0; h < NH; ++h)
                        L.w[r][p][h] = __builtin_nontemporal_load(qs_t[NT == 1 ? 0 : g / NG] + pg_gemv_weight_unit(row, h, NH, nb, blk[p]));
            }
        };
        // Loads return in issue order, so the (L2 / L1 resident) digits, block sums and scales
        // of this lane's blocks are requested first and the HBM weight rows right behind them:
        // the arithmetic on row r can then start as soon as row r lands, while later rows are
        // still in flight.
        v4i xd[BPL][NP];
        float sb[BPL];
        v4i dtile[NT][BPL];  // f16 scales of this lane's blocks for the 8 rows of the tile
        v4i mtile[BPL];  // Q4_1: their f16 offsets
        float sxs[BPL];  // Q4_1: scale * block sum of the activation block
        RowLoads<QT, BPL, R> L[2];
        if constexpr (LDSX) {
            // Loads return in issue order: the digits (from L2) are requested first, the weight rows (from HBM)
            // right behind them, and only the digits are waited for before the workgroup's one barrier.
            constexpr int CPT = GGUF_LDSX_UNITS / (64 * NW);  // 16-byte units per thread: digit planes, then the block scales
            const bool live = row0 < n_out;
            const int nd = NP * nb, nu = nd + (nb >> 2);
            v4i cp[CPT];
            if (seg0 == 0) {
#pragma unroll
                for (int c = 0; c < CPT; ++c) {
                    const int u = (int)threadIdx.x + c * 64 * NW;
                    cp[c] = u < nd ? digits[u] : ((gv4i_ptr)(uintptr_t)xs)[u < nu ? u - nd : 0];
                }
            }
            if (live) {
#pragma unroll
                for (int p = 0; p < BPL; ++p) dtile[0][p] = dsc[pg_gemv_scale_unit(row0, nb, blk[p])];
                load_rows(L[0], 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (seg0 == 0) {
#pragma unroll
                for (int c = 0; c < CPT; ++c) {
                    const int u = (int)threadIdx.x + c * 64 * NW;
                    if (u < nd) *reinterpret_cast<v4i *>(ldig + (size_t)u * 16) = cp[c];
                    else if (u < nu) *reinterpret_cast<v4i *>(reinterpret_cast<char *>(lxs) + (size_t)(u - nd) * 16) = cp[c];
                }
                asm volatile("s_waitcnt lgkmcnt(0)\n s_barrier" ::: "memory");  // (the weight loads stay in flight)
            }
            if (!live) return;  // after the workgroup's only barrier
#pragma unroll
            for (int p = 0; p < BPL; ++p) {
#pragma unroll
                for (int j = 0; j < NP; ++j) xd[p][j] = *reinterpret_cast<const v4i *>(ldig + ((size_t)j * nb + blk[p]) * 16);
                sb[p] = lxs[blk[p]];
            }
        } else if constexpr (XF32) {
            // Loads return in issue order: the row (a few KiB, from L2) is requested first so that the digit
            // arithmetic can start as soon as it is there, the weight rows (from HBM) right behind it so
            // that they fly meanwhile.  (A wavefront whose rows all lie past n_out -- the last workgroup's
            // spare ones -- only helps with the digits.)
            const bool live = row0 < n_out;
            const int sub = threadIdx.x & 7, bfirst = (int)threadIdx.x >> 3;
            float4 xv[4], gv[4];
            float ssq = 0.0f;
            auto fetch = [&](int b0) {
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int b = b0 + u * 8 * NW;
                    xv[u] = reinterpret_cast<const float4 *>(x_f32)[(size_t)pg_gemv_x_block(b, nb) * 8 + sub];
                    if constexpr (NORM) gv[u] = reinterpret_cast<const float4 *>(epi.gamma)[(size_t)pg_gemv_x_block(b, nb) * 8 + sub];
                }
            };
            if (seg0 == 0) fetch(bfirst);
            if (live) {
#pragma unroll
                for (int p = 0; p < BPL; ++p) dtile[0][p] = dsc[pg_gemv_scale_unit(row0, nb, blk[p])];
                load_rows(L[0], 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (seg0 == 0) {  // the row as digits, once per workgroup: 8 threads per block of 32, 4 elements each
                for (int b0 = bfirst; b0 < nb; b0 += 32 * NW) {  // four blocks per thread and round
                    if (b0 != bfirst) fetch(b0);
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int b = b0 + u * 8 * NW;
                        if (b < nb) {  // whole 8-thread groups together
                            float f[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w};
                            if constexpr (NORM) {
                                ssq += f[0] * f[0] + f[1] * f[1] + f[2] * f[2] + f[3] * f[3];
                                f[0] *= gv[u].x; f[1] *= gv[u].y; f[2] *= gv[u].z; f[3] *= gv[u].w;
                            }
                            pg_emit_digits<QT == 4>(f, 0, b, sub, nb, ldig, lxs);
                        }
                    }
                }
                float *red = lxs + nb;  // NORM: the wavefronts' sums of squares, behind the block scales
                if constexpr (NORM) {
                    ssq = wave_sum_f32(ssq);
                    if (lane == 0) red[threadIdx.x >> 6] = ssq;
                }
                // (not __syncthreads(): that would also wait for every weight load in flight)
                asm volatile("s_waitcnt lgkmcnt(0)\n s_barrier" ::: "memory");
                if constexpr (NORM) {
                    float ss = 0.0f;
#pragma unroll
                    for (int w = 0; w < NW; ++w) ss += red[w];
                    post = 1.0f / sqrtf(ss * epi.ss_inv_dim + epi.eps);
                }
            }
            if (!live) return;  // after the workgroup's only barrier
#pragma unroll
            for (int p = 0; p < BPL; ++p) {
#pragma unroll
                for (int j = 0; j < NP; ++j) xd[p][j] = *reinterpret_cast<const v4i *>(ldig + ((size_t)j * nb + blk[p]) * 16);
                sb[p] = lxs[blk[p]];
            }
        } else {
#pragma unroll
            for (int p = 0; p < BPL; ++p) {
#pragma unroll
                for (int j = 0; j < NP; ++j) xd[p][j] = digits[(size_t)j * nb + blk[p]];
                sb[p] = xs[blk[p]];
#pragma unroll
                for (int t = 0; t < NT; ++t) dtile[t][p] = dsc_t[t][(size_t)(row0 >> 3) * nb + blk[p]];
                if constexpr (Q41) {
                    mtile[p] = msc[(size_t)(row0 >> 3) * nb + blk[p]];
                    sxs[p] = xsum[blk[p]];
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            load_rows(L[0], 0);
        }
        __builtin_amdgcn_sched_barrier(0);  // every load is issued before any arithmetic
#pragma unroll
        for (int p = 0; p < BPL; ++p) {
            sb[p] *= (lane + 64 * p < seg_n ? 1.0f : 0.0f);
            if constexpr (Q41) sxs[p] *= sb[p];
        }
#pragma unroll
        for (int g = 0; g < NGT; ++g) {
            if (g + 1 < NGT) {
                load_rows(L[(g + 1) & 1], g + 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            const RowLoads<QT, BPL, R> &C = L[g & 1];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int tr = (row0 & 7) + (g % NG) * R + r;  // row within the scale tile
#pragma unroll
                for (int p = 0; p < BPL; ++p) {
                    float f;  // sum_k (weight) * X over the block
                    if constexpr (QT == 4) {
                        f = (float)block_dot_q4(C.w[r][p][0], reinterpret_cast<const v4i(&)[5]>(xd[p]));
                    } else {
                        int hi, lo;
                        block_dot_q8(C.w[r][p][0], C.w[r][p][NH - 1], reinterpret_cast<const v4i(&)[6]>(xd[p]), hi, lo);
                        f = fmaf((float)hi, 65536.0f, (float)lo);  // both terms exact in f32
                    }
                    const uint32_t pair = (uint32_t)dtile[g / NG][p][tr >> 1];
                    const float dv = half_bits_to_float((uint16_t)((tr & 1) ? pair >> 16 : pair & 0xFFFFu));
                    const float ds = dv * sb[p];
                    acc[g][r] = fmaf(ds, f, acc[g][r]);
                    if constexpr (Q41) {
                        const uint32_t mp = (uint32_t)mtile[p][tr >> 1];
                        const float mv = half_bits_to_float((uint16_t)((tr & 1) ? mp >> 16 : mp & 0xFFFFu));
                        acc[g][r] = fmaf(fmaf(8.0f, dv, mv), sxs[p], acc[g][r]);  // q = (q - 8) + 8
                    }
                }
            }
        }
    }
    __shared__ float res[NT][EPI != 0 ? 32 : 1];  // EPI: the workgroup's 32 outputs (per tensor)
    if constexpr (POST) post = 1.0f / sqrtf(wave_sum_f32((ssv[0] + ssv[1]) + (ssv[2] + ssv[3])) * epi.ss_inv_dim + epi.eps);
#pragma unroll
    for (int g = 0; g < NGT; ++g)
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float v = wave_sum_f32(acc[g][r]);
            if constexpr (POST || NORM) v *= post;
            const int row = row0 + (g % NG) * R + r;
            if constexpr (EPI != 2) {
                if (lane == 0 && row < n_out) {
                    if (residual_base) v = residual_base[(size_t)item * n_out + row] + v;
                    y[row] = v;
                }
            }
            if constexpr (EPI != 0) {
                if (lane == 0) res[g / NG][row - blockIdx.x * 32] = v;
            }
        }
    if constexpr (EPI != 0) {  // n_out is a multiple of 32 here
        __syncthreads();
        if (threadIdx.x < 8) {  // one block of 32: eight lanes, four elements each
            const int sub = threadIdx.x, e0 = sub * 4;
            float f[4];
            if constexpr (EPI == 1) {
                const float h[4] = {res[0][e0], res[0][e0 + 1], res[0][e0 + 2], res[0][e0 + 3]};
                f[0] = h[0] * gm.x; f[1] = h[1] * gm.y; f[2] = h[2] * gm.z; f[3] = h[3] * gm.w;
                float ss = h[0] * h[0] + h[1] * h[1] + h[2] * h[2] + h[3] * h[3];
                ss += __builtin_bit_cast(float, pg_dpp8<0xB1>(__builtin_bit_cast(int, ss)));
                ss += __builtin_bit_cast(float, pg_dpp8<0x4E>(__builtin_bit_cast(int, ss)));
                ss += __builtin_bit_cast(float, pg_dpp8<0x141>(__builtin_bit_cast(int, ss)));
                if (sub == 0) epi.ss_out[blockIdx.x] = ss;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float gv = res[0][e0 + e];
                    f[e] = gv / (1.0f + expf(-gv)) * res[NT - 1][e0 + e];
                }
            }
            pg_emit_digits<QT == 4>(f, 0, blockIdx.x, sub, n_out / 32, epi.out_digits, epi.out_xs);
        }
    }
}

// Two to four activation rows in f32 over one Q4_0 tensor, in ONE launch and one pass over the weights
// (src/tensor.rs:1342-1353 on dequantised weights, M of 2 to 4): the workgroup -- NW wavefronts with RW weight rows
// each -- rewrites all the rows as digits into LDS (per row the planes, then the block scales) while
// its first weight rows are in flight (row a at a * nb * 100 bytes rounded up to 16); a weight row then meets every activation row from registers, the digits
// of one activation row at a time coming back from LDS (10 reads of 16 bytes per row and BPL blocks against
// 20 R BPL dot instructions).  The matrix-core route for these counts is three launches (digits, product over four
// K chunks, their sum): 17 to 20 us on 4096 -> 14336 where the weights stream in 8.  Same digits, same integer
// dots and the same order of sums as the one-row kernel: a row's result equals that kernel's bit for bit.
template <int BPL, int RW, int R, int NW, int AR>
__global__ __launch_bounds__(64 * NW) void gguf_gemv_fewrows_kernel(const uint8_t *__restrict__ qs0, const uint16_t *__restrict__ d0,
                                                                     int n_out, int nb, const float *__restrict__ x_f32,
                                                                     float *__restrict__ y) {
    constexpr int SEG = 64 * BPL, NG = RW / R, MAXA = AR, ar = AR;
    extern __shared__ __attribute__((aligned(16))) char lds_digits[];
    const gv4i_ptr qs = (gv4i_ptr)(uintptr_t)qs0;
    const gv4i_ptr dsc = (gv4i_ptr)(uintptr_t)d0;
    const int lane = threadIdx.x & 63;
    const int row0 = (blockIdx.x * NW + (threadIdx.x >> 6)) * RW;
    const bool live = row0 < n_out;
    const size_t row_bytes = ((size_t)nb * 100 + 15) & ~(size_t)15;
    float acc[MAXA][RW];
#pragma unroll
    for (int a = 0; a < MAXA; ++a)
#pragma unroll
        for (int r = 0; r < RW; ++r) acc[a][r] = 0.0f;

    for (int seg0 = 0; seg0 < nb; seg0 += SEG) {
        const int seg_n = (nb - seg0 < SEG) ? nb - seg0 : SEG;
        int blk[BPL];  // this lane's blocks; lanes past the segment end re-read block seg0 with a zero scale
#pragma unroll
        for (int p = 0; p < BPL; ++p) blk[p] = pg_gemv_lane_block(seg0, lane, p, seg_n);
        auto load_rows = [&](RowLoads<4, BPL, R> &L, int g) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int row = pg_gemv_clamp_row(row0 + g * R + r, n_out);  // clamped; masked at the store
#pragma unroll
                for (int p = 0; p < BPL; ++p) L.w[r][p][0] = __builtin_nontemporal_load(qs + pg_gemv_weight_unit(row, 0, 1, nb, blk[p]));
            }
        };
        v4i dtile[BPL];
        RowLoads<4, BPL, R> L[2];
        if (seg0 == 0) {
            // Loads return in issue order: the first activation blocks (from L2) are requested first, the weight
            // rows (from HBM) right behind them, so that the digit arithmetic runs while the weights fly.
            const int sub = threadIdx.x & 7, bfirst = (int)threadIdx.x >> 3, total = ar * nb;  // (row, block) pairs, row-major
            float4 xv[4];
            auto fetch = [&](int i0) {
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int i = i0 + u * 8 * NW;
                    xv[u] = reinterpret_cast<const float4 *>(x_f32)[(size_t)(i < total ? i : 0) * 8 + sub];
                }
            };
            fetch(bfirst);
            if (live) {
#pragma unroll
                for (int p = 0; p < BPL; ++p) dtile[p] = dsc[pg_gemv_scale_unit(row0, nb, blk[p])];
                load_rows(L[0], 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            for (int i0 = bfirst; i0 < total; i0 += 32 * NW) {
                if (i0 != bfirst) fetch(i0);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int i = i0 + u * 8 * NW;
                    if (i < total) {  // whole 8-thread groups together
                        const int a = i / nb, b = i - a * nb;
                        const float f[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w};
                        // block-major in LDS: a block's five planes side by side (80 bytes), its scale at float 5 b behind
                        // them -- the plane-major writer with one block per plane and block index 5 b
                        int8_t *base = reinterpret_cast<int8_t *>(lds_digits + a * row_bytes);
                        pg_emit_digits<true>(f, 0, 5 * b, sub, 1, base, reinterpret_cast<float *>(base + (size_t)nb * 80));
                    }
                }
            }
            // (not __syncthreads(): that would also wait for every weight load in flight)
            asm volatile("s_waitcnt lgkmcnt(0)\n s_barrier" ::: "memory");
            if (!live) return;  // after the workgroup's only barrier
        } else {
#pragma unroll
            for (int p = 0; p < BPL; ++p) dtile[p] = dsc[pg_gemv_scale_unit(row0, nb, blk[p])];
            load_rows(L[0], 0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            if (g + 1 < NG) {
                load_rows(L[(g + 1) & 1], g + 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            const RowLoads<4, BPL, R> &C = L[g & 1];
#pragma unroll
            for (int a = 0; a < MAXA; ++a) {
                {
                    __builtin_amdgcn_sched_barrier(0);  // (one activation row's reads at a time: registers)
                    const char *base = lds_digits + a * row_bytes;
#pragma unroll
                    for (int p = 0; p < BPL; ++p) {  // (one block's digits at a time: 20 registers, not 20 BPL)
                        v4i xd[5];
#pragma unroll
                        for (int j = 0; j < 5; ++j) xd[j] = *reinterpret_cast<const v4i *>(base + blk[p] * 80 + j * 16);
                        const float sb = reinterpret_cast<const float *>(base + nb * 80)[5 * blk[p]] * (lane + 64 * p < seg_n ? 1.0f : 0.0f);
#pragma unroll
                        for (int r = 0; r < R; ++r) {
                            const int tr = (row0 & 7) + g * R + r;  // row within the scale tile
                            const float f = (float)block_dot_q4(C.w[r][p][0], xd);
                            const uint32_t pair = (uint32_t)dtile[p][tr >> 1];
                            const float dv = half_bits_to_float((uint16_t)((tr & 1) ? pair >> 16 : pair & 0xFFFFu));
                            acc[a][g * R + r] = fmaf(dv * sb, f, acc[a][g * R + r]);
                        }
                    }
                }
            }
        }
    }
#pragma unroll
    for (int a = 0; a < MAXA; ++a) {
#pragma unroll
            for (int r = 0; r < RW; ++r) {
                const float v = wave_sum_f32(acc[a][r]);
                if (lane == 0 && row0 + r < n_out) y[(size_t)a * n_out + row0 + r] = v;
            }
        }
}

template <int QT, int BPL, bool Q41>
pg_status launch_gemv_bpl(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d,
                          const pg_gemv_batch &batch, const pg_xdigits &xd, float *y, const float *residual,
                          const uint16_t *m) {
    const int nb = (int)(k_in / 32);
    // rows in flight per wavefront: bounded by registers (16 B of weights per row and block)
    constexpr int NH = QT == 8 ? 2 : 1;
    constexpr int R8 = BPL * NH <= 2 ? 8 : (BPL * NH <= 4 ? 4 : 2);
    const size_t want = (size_t)ctx->num_cu * 6;  // wavefronts wanted in the grid
#define PG_GGUF_GEMV_LAUNCH(RWW, RR)                                                               \
    do {                                                                                           \
        const dim3 grid(grid_for(n_out, RWW), (unsigned)batch.count);                              \
        PG_TRY(pg_launch(ctx, QT == 4 ? (Q41 ? "gguf_gemv_q4_1" : "gguf_gemv_q4_0") : "gguf_gemv_q8_0", \
                         gguf_gemv_kernel<QT, BPL, RWW, RR, Q41>, grid, dim3(64), 0, qs, d, batch, \
                         (int)n_out, nb, xd.digits, xd.xs, y, residual, m, (const float *)xd.xsum, (const float *)nullptr, pg_gemv_epi{})); \
    } while (0)
    if (n_out / 8 * batch.count >= want) PG_GGUF_GEMV_LAUNCH(8, R8);
    else if (n_out / 4 * batch.count >= want) PG_GGUF_GEMV_LAUNCH(4, (R8 < 4 ? R8 : 4));
    else if (!Q41 && BPL == 4 && nb % 4 == 0 && (size_t)nb * (QT == 8 ? 6 : 5) + nb / 4 <= (size_t)GGUF_LDSX_UNITS) {
        // two rows per wavefront under a long row: eight wavefronts share one copy of the digits in LDS
        auto kern = gguf_gemv_kernel<QT, BPL, 2, 2, false, 2, 8>;  // (four wavefronts of four rows: 10.8 against 9.0 us on 4096 x 14336)
        const size_t lds = (size_t)nb * 96 + (size_t)nb * sizeof(float);
        PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));
        PG_TRY(pg_launch(ctx, QT == 4 ? "gguf_gemv_q4_0" : "gguf_gemv_q8_0", kern, dim3(grid_for(n_out, 16), (unsigned)batch.count), dim3(512),
                         lds, qs, d, batch, (int)n_out, nb, xd.digits, xd.xs, y, residual, m, (const float *)nullptr, (const float *)nullptr,
                         pg_gemv_epi{}));
    } else PG_GGUF_GEMV_LAUNCH(2, 2);
#undef PG_GGUF_GEMV_LAUNCH
    return PG_OK;
}

// Products whose output is the next product's digit input (see EPI at the kernel): a workgroup owns
// 32 output rows as 32 / RW wavefronts.
template <int QT, int BPL, int EPI, bool POST>
pg_status launch_gemv_epi_bpl(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d, const pg_xdigits &xd,
                              float *y, const float *residual, const pg_gemv_epi &epi) {
    const int nb = (int)(k_in / 32);
    const pg_gemv_batch one = {1, nullptr, nullptr, nullptr, 1};
    constexpr int NH = QT == 8 ? 2 : 1;
    constexpr int R8 = BPL * NH <= 2 ? 8 : (BPL * NH <= 4 ? 4 : 2);
    const size_t want = (size_t)ctx->num_cu * 6;  // wavefronts wanted in the grid
    const size_t rows = n_out * (EPI == 2 ? 2 : 1);
#define PG_GGUF_GEMV_E_LAUNCH(RWW, RR)                                                                                            \
    PG_TRY(pg_launch(ctx, EPI == 1 ? (QT == 4 ? "gguf_gemv_q4_0_norm_digits" : "gguf_gemv_q8_0_norm_digits")                      \
                              : (QT == 4 ? "gguf_gemv_q4_0_swiglu_digits" : "gguf_gemv_q8_0_swiglu_digits"),                      \
                     gguf_gemv_kernel<QT, BPL, RWW, RR, false, 0, 32 / RWW, EPI, POST>, dim3((unsigned)(n_out / 32)),             \
                     dim3(64 * (32 / RWW)), 0, qs, d, one, (int)n_out, nb, xd.digits, xd.xs, y, residual, (const uint16_t *)nullptr, \
                     (const float *)nullptr, (const float *)nullptr, epi))
    if constexpr (BPL * NH > 2) {  // (8 or 16 wavefronts would leave too few registers each for rows this long)
        PG_GGUF_GEMV_E_LAUNCH(8, R8);
    } else {
        if (rows / 8 >= want) PG_GGUF_GEMV_E_LAUNCH(8, R8);
        else if (rows / 4 >= want / 2) PG_GGUF_GEMV_E_LAUNCH(4, (R8 < 4 ? R8 : 4));
        else PG_GGUF_GEMV_E_LAUNCH(2, 2);
    }
#undef PG_GGUF_GEMV_E_LAUNCH
    return PG_OK;
}

template <int EPI, bool POST>
pg_status launch_gemv_epi(pg_ctx *ctx, int ggml_type, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d, const pg_xdigits &xd,
                          float *y, const float *residual, const pg_gemv_epi &epi) {
    size_t bpl = (k_in / 32 + 63) / 64;
    if (bpl > 4) bpl = 4;
    if (ggml_type != PG_GGML_Q4_0 && ggml_type != PG_GGML_Q8_0)
        return pg_fail(PG_EUNSUPPORTED, "gguf_gemv: only Q4_0 and Q8_0 products leave their output as digits");
    const bool q4 = ggml_type == PG_GGML_Q4_0;
    switch (bpl) {
        case 1: return q4 ? launch_gemv_epi_bpl<4, 1, EPI, POST>(ctx, n_out, k_in, qs, d, xd, y, residual, epi)
                          : launch_gemv_epi_bpl<8, 1, EPI, POST>(ctx, n_out, k_in, qs, d, xd, y, residual, epi);
        case 2: return q4 ? launch_gemv_epi_bpl<4, 2, EPI, POST>(ctx, n_out, k_in, qs, d, xd, y, residual, epi)
                          : launch_gemv_epi_bpl<8, 2, EPI, POST>(ctx, n_out, k_in, qs, d, xd, y, residual, epi);
        case 3: return q4 ? launch_gemv_epi_bpl<4, 3, EPI, POST>(ctx, n_out, k_in, qs, d, xd, y, residual, epi)
                          : launch_gemv_epi_bpl<8, 3, EPI, POST>(ctx, n_out, k_in, qs, d, xd, y, residual, epi);
        default: return q4 ? launch_gemv_epi_bpl<4, 4, EPI, POST>(ctx, n_out, k_in, qs, d, xd, y, residual, epi)
                           : launch_gemv_epi_bpl<8, 4, EPI, POST>(ctx, n_out, k_in, qs, d, xd, y, residual, epi);
    }
}

// One row still in f32: the one-launch form (four or eight wavefronts per workgroup share the digits).
template <int QT, int BPL, int NW>
pg_status launch_gemv_f32x_bpl(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d, const float *x_f32,
                               float *y) {
    constexpr int NH = QT == 8 ? 2 : 1;
    constexpr int R8 = BPL * NH <= 2 ? 8 : (BPL * NH <= 4 ? 4 : 2);
    const int nb = (int)(k_in / 32);
    const size_t lds = (size_t)nb * 96 + (size_t)nb * sizeof(float);
    const pg_gemv_batch one = {1, nullptr, nullptr, nullptr, 1};
    const size_t want = (size_t)ctx->num_cu * 6;
    const char *name = QT == 4 ? "gguf_gemv_q4_0" : "gguf_gemv_q8_0";
#define PG_GGUF_GEMV_X_LAUNCH(RWW, RR)                                                                             \
    do {                                                                                                           \
        auto kern = gguf_gemv_kernel<QT, BPL, RWW, RR, false, true, NW>;                                       \
        PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));                                                \
        PG_TRY(pg_launch(ctx, name, kern, dim3(grid_for(n_out, RWW * NW)), dim3(64 * NW), lds, qs, d, one, (int)n_out, nb, \
                         (const int8_t *)nullptr, (const float *)nullptr, y, (const float *)nullptr,               \
                         (const uint16_t *)nullptr, (const float *)nullptr, x_f32, pg_gemv_epi{}));                    \
    } while (0)
    if (n_out / 8 >= want) PG_GGUF_GEMV_X_LAUNCH(8, R8);
    else if (n_out / 4 >= want) PG_GGUF_GEMV_X_LAUNCH(4, (R8 < 4 ? R8 : 4));
    else PG_GGUF_GEMV_X_LAUNCH(2, 2);
#undef PG_GGUF_GEMV_X_LAUNCH
    return PG_OK;
}

// The same over any number of items (all multiply the one row), with RMSNorm folded in.
template <int BPL>
pg_status launch_gemv_norm_bpl(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d, const pg_gemv_batch &batch,
                               const float *x_f32, const pg_gemv_epi &epi, float *y) {
    constexpr int NW = 8, R8 = BPL <= 2 ? 8 : (BPL <= 4 ? 4 : 2);  // (measured on 6 x 1024 rows of 4096: 7.6 us; four wavefronts 8.2)
    const int nb = (int)(k_in / 32);
    const size_t lds = (size_t)nb * 96 + (size_t)nb * sizeof(float) + NW * sizeof(float);
    const size_t want = (size_t)ctx->num_cu * 6;
#define PG_GGUF_GEMV_N_LAUNCH(RWW, RR)                                                                                           \
    do {                                                                                                                         \
        auto kern = gguf_gemv_kernel<4, BPL, RWW, RR, false, 1, NW, 0, false, true>;                                             \
        PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));                                                              \
        PG_TRY(pg_launch(ctx, "gguf_gemv_q4_0_rmsnorm", kern, dim3(grid_for(n_out, RWW * NW), (unsigned)batch.count), dim3(64 * NW), lds, \
                         qs, d, batch, (int)n_out, nb, (const int8_t *)nullptr, (const float *)nullptr, y, (const float *)nullptr, \
                         (const uint16_t *)nullptr, (const float *)nullptr, x_f32, epi));                                        \
    } while (0)
    if constexpr (BPL > 2) {  // (more rows in flight would spill registers)
        PG_GGUF_GEMV_N_LAUNCH(2, 2);
    } else {
        if (n_out / 8 * batch.count >= want) PG_GGUF_GEMV_N_LAUNCH(8, R8);
        else if (n_out / 4 * batch.count >= want) PG_GGUF_GEMV_N_LAUNCH(4, (R8 < 4 ? R8 : 4));
        else PG_GGUF_GEMV_N_LAUNCH(2, 2);
    }
#undef PG_GGUF_GEMV_N_LAUNCH
    return PG_OK;
}

template <int QT>
pg_status launch_gemv_f32x(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d, const float *x_f32, float *y) {
    size_t bpl = (k_in / 32 + 63) / 64;
    if (bpl > 4) bpl = 4;
    // Every workgroup makes the whole row's digits: the fewer, larger workgroups the less of that work
    // in total -- eight wavefronts each where that still leaves a workgroup for a good part of the CUs.
    const bool wide = n_out / 64 >= (size_t)ctx->num_cu / 6;
    switch (bpl) {
        case 1: return wide ? launch_gemv_f32x_bpl<QT, 1, 8>(ctx, n_out, k_in, qs, d, x_f32, y) : launch_gemv_f32x_bpl<QT, 1, 4>(ctx, n_out, k_in, qs, d, x_f32, y);
        case 2: return wide ? launch_gemv_f32x_bpl<QT, 2, 8>(ctx, n_out, k_in, qs, d, x_f32, y) : launch_gemv_f32x_bpl<QT, 2, 4>(ctx, n_out, k_in, qs, d, x_f32, y);
        case 3: return wide ? launch_gemv_f32x_bpl<QT, 3, 8>(ctx, n_out, k_in, qs, d, x_f32, y) : launch_gemv_f32x_bpl<QT, 3, 4>(ctx, n_out, k_in, qs, d, x_f32, y);
        default: return wide ? launch_gemv_f32x_bpl<QT, 4, 8>(ctx, n_out, k_in, qs, d, x_f32, y) : launch_gemv_f32x_bpl<QT, 4, 4>(ctx, n_out, k_in, qs, d, x_f32, y);
    }
}

// Bytes of LDS the few-rows kernel needs; its launch shapes follow the one-row form's.
inline size_t fewrows_lds(size_t m, size_t k_in) { return m * pg_round_up((k_in / 32) * 100, 16); }

template <int BPL, int AR>
pg_status launch_gemv_fewrows_bpl(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d, const float *x_f32,
                                  float *y) {
    constexpr size_t m = AR;
    constexpr int NW = 8, R8 = BPL <= 1 ? 8 : 4;  // rows in flight: bounded by registers
    const int nb = (int)(k_in / 32);
    const size_t lds = fewrows_lds(m, k_in), want = (size_t)ctx->num_cu * 6;
#define PG_GGUF_FEWROWS_LAUNCH(RWW, RR)                                                                                          \
    do {                                                                                                                         \
        auto kern = gguf_gemv_fewrows_kernel<BPL, RWW, RR, NW, AR>;                                                              \
        PG_TRY(pg_allow_dynamic_lds(ctx, (const void *)kern, lds));                                                              \
        PG_TRY(pg_launch(ctx, "gguf_gemv_q4_0_few_rows", kern, dim3(grid_for(n_out, RWW * NW)), dim3(64 * NW), lds, qs, d,     \
                         (int)n_out, nb, x_f32, y));                                                                             \
    } while (0)
    if constexpr (BPL <= 2) {
        if (n_out / 8 >= want) {
            PG_GGUF_FEWROWS_LAUNCH(8, R8);
            return PG_OK;
        }
    }
    if (n_out / 4 >= want) PG_GGUF_FEWROWS_LAUNCH(4, 4);
    else PG_GGUF_FEWROWS_LAUNCH(2, 2);
#undef PG_GGUF_FEWROWS_LAUNCH
    return PG_OK;
}

template <int QT, bool Q41 = false>
pg_status launch_gemv(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d,
                      const pg_gemv_batch &batch, const pg_xdigits &xd, float *y, const float *residual,
                      const uint16_t *m) {
    const size_t nb = k_in / 32;
    size_t bpl = (nb + 63) / 64;
    if (bpl > 4) bpl = 4;  // longer rows run as several K segments of 256 blocks
    switch (bpl) {
        case 1: return launch_gemv_bpl<QT, 1, Q41>(ctx, n_out, k_in, qs, d, batch, xd, y, residual, m);
        case 2: return launch_gemv_bpl<QT, 2, Q41>(ctx, n_out, k_in, qs, d, batch, xd, y, residual, m);
        case 3: return launch_gemv_bpl<QT, 3, Q41>(ctx, n_out, k_in, qs, d, batch, xd, y, residual, m);
        default: return launch_gemv_bpl<QT, 4, Q41>(ctx, n_out, k_in, qs, d, batch, xd, y, residual, m);
    }
}

}  // namespace

size_t pg_xdigits_bytes(size_t rows, size_t k) {
    const size_t nb = k / 32;
    return pg_round_up(3 * rows * k, 256) + 2 * pg_round_up(rows * nb * sizeof(float), 256);
}

pg_xdigits pg_xdigits_carve(void *base, size_t rows, size_t k) {
    const size_t nb = k / 32;
    pg_xdigits xd;
    char *p = static_cast<char *>(base);
    xd.digits = reinterpret_cast<int8_t *>(p);
    p += pg_round_up(3 * rows * k, 256);
    xd.xs = reinterpret_cast<float *>(p);
    p += pg_round_up(rows * nb * sizeof(float), 256);
    xd.xsum = reinterpret_cast<float *>(p);
    xd.rows = rows;
    xd.k = k;
    return xd;
}

pg_status pg_launch_x_to_digits(pg_ctx *ctx, const float *x_dev, size_t rows, size_t k,
                                int ggml_type, const pg_xdigits &xd) {
    if (rows == 0) return PG_OK;
    if (rows > 65535) return pg_fail(PG_EUNSUPPORTED, "x_to_digits: more than 65535 activation rows");
    const int nb = (int)(k / 32);
    const dim3 grid(grid_for(nb, 32), (unsigned)rows);
    if (ggml_type == PG_GGML_Q4_0 || ggml_type == PG_GGML_Q4_1)
        PG_TRY(pg_launch(ctx, "x_to_digits", x_to_digits_kernel<true>, grid, dim3(256), 0, x_dev, nb, xd.digits, xd.xs,
                         ggml_type == PG_GGML_Q4_1 ? xd.xsum : (float *)nullptr));
    else
        PG_TRY(pg_launch(ctx, "x_to_digits", x_to_digits_kernel<false>, grid, dim3(256), 0, x_dev, nb, xd.digits, xd.xs,
                         (float *)nullptr));
    return pg_launch_check("x_to_digits");
}

pg_status pg_launch_gguf_gemv_rmsnorm(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d,
                                      const pg_gemv_batch &batch, const float *x_f32, const float *gamma, float eps, float *y) {
    if (batch.count == 0) return PG_OK;
    if (batch.count > 65535) return pg_fail(PG_EUNSUPPORTED, "gguf_gemv: more than 65535 batch items");
    if (k_in % 32 != 0 || k_in > 8192 || !gamma || (((uintptr_t)gamma | (uintptr_t)x_f32) % 16) != 0)
        return pg_fail(PG_EINVAL, "gguf_gemv (RMSNorm folded in): k_in %zu (a multiple of 32, at most 8192) or an argument does not fit", k_in);
    pg_gemv_epi epi = {};
    epi.gamma = gamma; epi.eps = eps; epi.ss_inv_dim = 1.0f / (float)k_in;
    switch ((k_in / 32 + 63) / 64) {
        case 1: return launch_gemv_norm_bpl<1>(ctx, n_out, k_in, qs, d, batch, x_f32, epi, y);
        case 2: return launch_gemv_norm_bpl<2>(ctx, n_out, k_in, qs, d, batch, x_f32, epi, y);
        case 3: return launch_gemv_norm_bpl<3>(ctx, n_out, k_in, qs, d, batch, x_f32, epi, y);
        default: return launch_gemv_norm_bpl<4>(ctx, n_out, k_in, qs, d, batch, x_f32, epi, y);
    }
}

pg_status pg_launch_gguf_gemv_norm_digits(pg_ctx *ctx, int ggml_type, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d,
                                          const pg_xdigits &xd, float *y, const float *residual, const float *gamma,
                                          const pg_xdigits &out, float *ss_out) {
    if (n_out % 32 != 0 || k_in % 32 != 0 || !gamma || (uintptr_t)gamma % 16 != 0 || !ss_out || !y)
        return pg_fail(PG_EINVAL, "gguf_gemv (digits of the normalised output): [%zu, %zu] or an argument does not fit", n_out, k_in);
    pg_gemv_epi epi = {};
    epi.gamma = gamma; epi.out_digits = out.digits; epi.out_xs = out.xs; epi.ss_out = ss_out;
    return launch_gemv_epi<1, false>(ctx, ggml_type, n_out, k_in, qs, d, xd, y, residual, epi);
}

pg_status pg_launch_gguf_gemv_swiglu_digits(pg_ctx *ctx, int ggml_type, size_t n_out, size_t k_in, const uint8_t *qs_gate, const uint16_t *d_gate,
                                            const uint8_t *qs_up, const uint16_t *d_up, const pg_xdigits &xd, const float *ss_in,
                                            size_t ss_n, size_t ss_dim, float eps, const pg_xdigits &out) {
    if (n_out % 32 != 0 || k_in % 32 != 0 || !ss_in || ss_n == 0 || ss_dim == 0)
        return pg_fail(PG_EINVAL, "gguf_gemv (digits of SiLU(gate) * up): [%zu, %zu] or an argument does not fit", n_out, k_in);
    pg_gemv_epi epi = {};
    epi.qs1 = qs_up; epi.d1 = d_up; epi.out_digits = out.digits; epi.out_xs = out.xs;
    if (ss_n > 256) return pg_fail(PG_EUNSUPPORTED, "gguf_gemv (digits of SiLU(gate) * up): more than 256 partial sums");
    epi.ss_in = ss_in; epi.ss_n = (int)ss_n; epi.ss_inv_dim = 1.0f / (float)ss_dim; epi.eps = eps;
    return launch_gemv_epi<2, true>(ctx, ggml_type, n_out, k_in, qs_gate, d_gate, xd, nullptr, nullptr, epi);
}

pg_status pg_launch_gguf_gemv(pg_ctx *ctx, int ggml_type, size_t n_out, size_t k_in,
                              const uint8_t *qs, const uint16_t *d, const pg_gemv_batch &batch,
                              const pg_xdigits &xd, float *y, const float *residual, const uint16_t *m) {
    if (batch.count == 0) return PG_OK;
    if (batch.count > 65535) return pg_fail(PG_EUNSUPPORTED, "gguf_gemv: more than 65535 batch items");
    if (ggml_type == PG_GGML_Q4_1) {
        if (!m || batch.qs_table) return pg_fail(PG_EINVAL, "gguf_gemv: Q4_1 needs its offsets and runs without expert tables");
        return launch_gemv<4, true>(ctx, n_out, k_in, qs, d, batch, xd, y, residual, m);
    }
    if (ggml_type == PG_GGML_Q4_0) return launch_gemv<4>(ctx, n_out, k_in, qs, d, batch, xd, y, residual, nullptr);
    if (ggml_type == PG_MXFP4) return pg_fail(PG_EUNSUPPORTED, "gguf_gemv: MXFP4 tensors have their own kernel");
    return launch_gemv<8>(ctx, n_out, k_in, qs, d, batch, xd, y, residual, nullptr);
}

// y[row] = product over one activation row given in f32 (16-byte aligned): one launch, digits made inside.
// Every workgroup repeats the digit arithmetic for the whole row, so the form pays where there are few
// workgroups and the separate digit launch (2.4 us in a chain of launches) weighs most: Q4_0 with up to
// 8192 weight rows (measured one launch against two: 4096 -> 4096 5.5 against 6.7 us, 14336 -> 4096 11.5
// against 12.8 us; but 4096 -> 14336 10.9 against 10.3 us, and Q8_0 there 19.3 against 14.6 us).
// k_in up to 32768 (the row's digits live in LDS).
// Two rows at once, three over a small tensor (Q4_0, K up to 8192; all their digits fit in LDS).  The kernel's time
// grows by the arithmetic of every further row and by the digits of K m elements that every workgroup makes; the
// matrix-core routes' hardly at all, but they start with a launch for the digits: us, rows 2 / 3 / 4, against
// digits + one matrix-core launch at 4 rows: 4096 -> 14336 12.2 / 16.2 / 19.9 against 14.4; 4096 -> 4096 6.7 / 8.6 /
// 10.4 against 8.2; 14336 -> 4096 17.8 / 24.1 / - against 14.3.  Since the matrix-core route for up to 8 rows moved to
// 4 x 4 x 4 products (4096 -> 14336 11.0 us, 14336 -> 4096 11.8, 4096 -> 4096 7.7, 4096 -> 6144 8.4 at 2 .. 4 rows)
// this kernel keeps two rows over small tensors only (4096 -> 4096: 6.8).
bool pg_gguf_gemv_takes_few_rows(int ggml_type, size_t m, size_t n_out, size_t k_in, const float *x_f32) {
    return ggml_type == PG_GGML_Q4_0 && m == 2 && n_out * k_in <= ((size_t)1 << 24) && k_in >= 32 && k_in <= 8192 &&
           fewrows_lds(m, k_in) <= 150 * 1024 && (uintptr_t)x_f32 % 16 == 0;
}

pg_status pg_launch_gguf_gemv_few_rows(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d, const float *x_f32,
                                       size_t m, float *y) {
#define PG_FEWROWS_BPL(B) launch_gemv_fewrows_bpl<B, 2>(ctx, n_out, k_in, qs, d, x_f32, y)
    if (m != 2) return pg_fail(PG_EINVAL, "gguf_gemv (few rows): %zu rows", m);
    switch ((k_in / 32 + 63) / 64) {
        case 1: return PG_FEWROWS_BPL(1);
        case 2: return PG_FEWROWS_BPL(2);
        case 3: return PG_FEWROWS_BPL(3);
        default: return PG_FEWROWS_BPL(4);
    }
#undef PG_FEWROWS_BPL
}

bool pg_gguf_gemv_takes_f32_row(int ggml_type, size_t n_out, size_t k_in, const float *x_f32) {
    return ggml_type == PG_GGML_Q4_0 && n_out <= 8192 && k_in >= 32 && k_in <= 32768 && (uintptr_t)x_f32 % 16 == 0;
}

pg_status pg_launch_gguf_gemv_f32_row(pg_ctx *ctx, int ggml_type, size_t n_out, size_t k_in, const uint8_t *qs,
                                      const uint16_t *d, const float *x_f32, float *y) {
    if (ggml_type != PG_GGML_Q4_0) return pg_fail(PG_EUNSUPPORTED, "gguf_gemv: the one-launch row product holds Q4_0 code only");
    return launch_gemv_f32x<4>(ctx, n_out, k_in, qs, d, x_f32, y);
}

// The tile-major copy of a tensor's quant plane that gguf_mm_kernel fetches: 16-byte chunks in
// the order [group of 128 rows][group of 4 blocks][wavefront][fill][lane], where the lane of a
// fill stands for (stream 16*fill + lane/4, block (lane%4) ^ ((lane/8)%4)) exactly as in the
// kernel's fill duties; rows past n_out and blocks past k_in/32 are zeros.
template <int QT>
__global__ void tile_weights_kernel(const uint8_t *__restrict__ qs, int n_out, int nb, uint8_t *__restrict__ tiled) {
    constexpr int CH = (QT == 8 ? 4096 : 2048) / 16, FILLS = CH / 64;  // chunks and fills per wavefront and stage
    const int nsg = (nb + 3) / 4, rg = blockIdx.y;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;    // chunk within the row group
    if (i >= (size_t)nsg * 4 * CH) return;
    const int lane = (int)(i & 63), q = (int)((i >> 6) % FILLS), wave = (int)((i / CH) & 3), sg = (int)(i / (4 * CH));
    const int st = 16 * q + (lane >> 2), j = (lane & 3) ^ ((lane >> 4) & 3);
    const int row = rg * 128 + wave * 32 + (st & 31), half = st >> 5, block = sg * 4 + j;
    uint4 v = {0, 0, 0, 0};
    if (row < n_out && block < nb)
        v = *reinterpret_cast<const uint4 *>(qs + (QT == 8 ? ((size_t)row * 2 + half) * nb + block : (size_t)row * nb + block) * 16);
    *reinterpret_cast<uint4 *>(tiled + rg * pg_tiled_group_bytes(nb, QT == 8) + i * 16) = v;
}

static std::mutex g_tiled_mutex;

pg_status pg_gguf_ensure_tiled(pg_ctx *ctx, const pg_gguf_tensor *w) {
    // One maker at a time, and the pointer is published only once the copy is complete, so another
    // context, stream or thread that finds it set may read it at once.
    std::lock_guard<std::mutex> lock(g_tiled_mutex);
    if (w->qs_tiled) return PG_OK;
    if (w->ggml_type != PG_GGML_Q4_0 && w->ggml_type != PG_GGML_Q8_0 && w->ggml_type != PG_GGML_Q4_1)
        return pg_fail(PG_EUNSUPPORTED, "gguf: no tile-major copy for ggml type %d", w->ggml_type);
    const int nb = (int)(w->k_in / 32);
    const bool q8 = w->ggml_type == PG_GGML_Q8_0;
    const size_t groups = (w->n_out + 127) / 128, group_bytes = pg_tiled_group_bytes(nb, q8);
    const size_t bytes = groups * group_bytes, chunks = (group_bytes - 4352) / 16;
    if (groups > 65535) return pg_fail(PG_EUNSUPPORTED, "gguf: too many weight rows for a tile-major copy");
    uint8_t *p = nullptr;
    hipError_t e = hipMalloc((void **)&p, bytes);
    if (e != hipSuccess)
        return pg_fail(e == hipErrorOutOfMemory ? PG_ENOMEM : PG_EDEVICE, "gguf tile-major copy (%zu bytes): %s", bytes, hipGetErrorString(e));
    const dim3 grid(grid_for(chunks, 256), (unsigned)groups);
    pg_status st = q8 ? pg_launch(ctx, "gguf_tile_weights", tile_weights_kernel<8>, grid, dim3(256), 0, (const uint8_t *)w->qs,
                                  (int)w->n_out, nb, p)
                      : pg_launch(ctx, "gguf_tile_weights", tile_weights_kernel<4>, grid, dim3(256), 0, (const uint8_t *)w->qs,
                                  (int)w->n_out, nb, p);
    if (st == PG_OK && hipStreamSynchronize(ctx->stream) != hipSuccess) st = pg_fail(PG_EDEVICE, "gguf tile-major copy: the stream failed");
    if (st != PG_OK) { (void)hipFree(p); return st; }
    w->qs_tiled = p;
    return PG_OK;
}

// `count` products of one block type (Q4_0 or Q8_0) over the same many rows on the f16 matrix cores: the rows become two f16 planes once,
// tensors of the same launch shape share a launch (up to PG_HMM_MAX_GROUP).
static pg_status pg_gguf_hmm_rows(pg_ctx *ctx, const float *x_dev, size_t m, const pg_gguf_tensor *const *w, float *const *y_dev,
                                  int count, int ks) {
    const size_t k_in = w[0]->k_in;
    size_t n_total = 0;
    for (int i = 0; i < count; ++i) n_total += w[i]->n_out;
    const size_t sz_p = pg_hmm_planes_bytes(m, k_in), sz_part = pg_round_up(pg_gguf_hmm_part_floats(m, n_total, ks) * sizeof(float), 256);
    void *ws = nullptr;
    PG_TRY(pg_workspace(ctx, sz_p + sz_part, &ws));
    const pg_hmm_planes planes = pg_hmm_planes_carve(ws, m, k_in);
    float *part = ks > 1 ? reinterpret_cast<float *>(static_cast<char *>(ws) + sz_p) : nullptr;
    PG_TRY(pg_launch_rows_to_f16_planes(ctx, x_dev, m, k_in, planes));
    return pg_launch_gguf_hmm_group(ctx, k_in, w, y_dev, count, m, planes, ks, part);
}

// Quantise `m` activation rows (device) into the arena and run the fused product: the
// streaming GEMV for one row, the matrix-core kernel (weights read once) for more.
pg_status pg_gguf_matmul_rows(pg_ctx *ctx, const float *x_dev, size_t m, const pg_gguf_tensor *w,
                              float *y_dev) {
    void *ws = nullptr;
    if (w->ggml_type == PG_MXFP4) {
        // The MXFP4 kernel is a decode kernel (three rows per pass over the weights).  From 16 rows on (24 for a
        // tensor under 2^25 weights, where the passes are short) the tile kernel on the same instruction takes over:
        // the weights once per 64 rows, the rows as four planes of base-32 digits.
        if (pg_mxfp4_tiles_takes(w, m)) return pg_launch_mxfp4_tiles(ctx, x_dev, m, w, y_dev);
        return pg_launch_mxfp4_rows(ctx, x_dev, m, w, y_dev);
    }
    int hks = 1;
    if (ctx->hmm_mode == 1 && pg_gguf_hmm_takes(ctx, w->ggml_type, m, w->n_out, w->k_in, &hks))  // forced (pg_gguf_hmm_force)
        return pg_gguf_hmm_rows(ctx, x_dev, m, &w, &y_dev, 1, hks);
    // a K of a few blocks needs the streaming kernel's finer fixed point; so do up to seven rows of Q4_1 (its
    // matrix-core route is three launches more than the streaming one: 27 against 19 us at four rows of 4096 ->
    // 14336, 35 against 59 at sixteen) and Q4_1 rows too long for the offset kernel
    if (m == 1 && pg_gguf_gemv_takes_f32_row(w->ggml_type, w->n_out, w->k_in, x_dev))
        return pg_launch_gguf_gemv_f32_row(ctx, w->ggml_type, w->n_out, w->k_in, w->qs, w->d, x_dev, y_dev);
    if (pg_gguf_gemv_takes_few_rows(w->ggml_type, m, w->n_out, w->k_in, x_dev))
        return pg_launch_gguf_gemv_few_rows(ctx, w->n_out, w->k_in, w->qs, w->d, x_dev, m, y_dev);
    const bool q41 = w->ggml_type == PG_GGML_Q4_1;
    if (m == 1 || (q41 && (m < 8 || w->k_in > 32768)) || w->k_in / 32 < PG_MM_MIN_BLOCKS) {
        if (m > 65535) return pg_fail(PG_EUNSUPPORTED, "gguf_matmul: more than 65535 rows through the streaming kernel (Q4_1 or k_in < %zu)", PG_MM_MIN_BLOCKS * 32);
        PG_TRY(pg_workspace(ctx, pg_xdigits_bytes(m, w->k_in), &ws));
        const pg_xdigits xd = pg_xdigits_carve(ws, m, w->k_in);
        PG_TRY(pg_launch_x_to_digits(ctx, x_dev, m, w->k_in, w->ggml_type, xd));
        pg_gemv_batch batch = {(int)m, nullptr, nullptr, nullptr, 1};
        return pg_launch_gguf_gemv(ctx, w->ggml_type, w->n_out, w->k_in, w->qs, w->d, batch, xd, y_dev, nullptr, w->m);
    }
    if (pg_gguf_skinny_takes(ctx, w->ggml_type, m, w->n_out, w->k_in)) {  // up to 16 rows: digits, then one launch
        PG_TRY(pg_workspace(ctx, pg_mmdigits_bytes(m, w->k_in), &ws));
        const pg_mmdigits md = pg_mmdigits_carve(ws, m, w->k_in);
        PG_TRY(pg_launch_x_to_mm_digits(ctx, x_dev, m, w->k_in, w->ggml_type, md));
        return pg_launch_gguf_skinny_group(ctx, w->ggml_type, w->k_in, &w, &y_dev, 1, m, md);
    }
    if (pg_gguf_hmm_takes(ctx, w->ggml_type, m, w->n_out, w->k_in, &hks))  // many rows of Q4_0 / Q8_0: the f16 matrix cores
        return pg_gguf_hmm_rows(ctx, x_dev, m, &w, &y_dev, 1, hks);
    if (q41 && w->k_in <= 32768 && pg_gguf_hmm_takes(ctx, PG_GGML_Q4_0, m, w->n_out, w->k_in, &hks)) {
        // Q4_1 at that size: the first term d sum (q - 8) x as the Q4_0 product on the f16 matrix cores, then the
        // offsets times the rows' block sums (which the digit launch writes beside its planes)
        PG_TRY(pg_gguf_hmm_rows(ctx, x_dev, m, &w, &y_dev, 1, hks));
        PG_TRY(pg_workspace(ctx, pg_mmdigits_bytes(m, w->k_in), &ws));   // (the product is done with the arena)
        const pg_mmdigits md = pg_mmdigits_carve(ws, m, w->k_in);
        PG_TRY(pg_launch_x_to_mm_digits(ctx, x_dev, m, w->k_in, w->ggml_type, md));
        return pg_launch_q41_offset(ctx, w, md, m, y_dev);
    }
    const int ks = pg_gguf_mm_splitk(ctx, w->n_out, w->k_in, (m + 31) / 32, m, false, nullptr);
    const size_t sz_d = pg_mmdigits_bytes(m, w->k_in);
    const size_t sz_part = ks > 1 ? pg_round_up((size_t)ks * m * w->n_out * sizeof(float), 256) : 0;
    PG_TRY(pg_workspace(ctx, sz_d + sz_part, &ws));
    const pg_mmdigits md = pg_mmdigits_carve(ws, m, w->k_in);
    float *part = ks > 1 ? reinterpret_cast<float *>(static_cast<char *>(ws) + sz_d) : nullptr;
    PG_TRY(pg_launch_x_to_mm_digits(ctx, x_dev, m, w->k_in, w->ggml_type, md));
    pg_mm_group grp = {1, nullptr, nullptr, nullptr, nullptr, 0, (int)((m + 31) / 32), (int)m, 1};
    PG_TRY(pg_gguf_ensure_tiled(ctx, w));
    grp.tiled = 1;
    // Q4_1: the Q4_0 product on the same nibbles and scales, then the blocks' offsets times the rows' block sums
    PG_TRY(pg_launch_gguf_mm(ctx, q41 ? PG_GGML_Q4_0 : w->ggml_type, w->n_out, w->k_in, w->qs_tiled, w->d, grp, m, md, y_dev, part));
    return q41 ? pg_launch_q41_offset(ctx, w, md, m, y_dev) : PG_OK;
}

// Several products over the same activation rows (q/k/v, gate/up): the rows are rewritten
// as digits once per ggml type in use instead of once per product.  All k_in are equal.
pg_status pg_gguf_matmul_rows_multi(pg_ctx *ctx, const float *x_dev, size_t m, const pg_gguf_tensor *const *w,
                                    float *const *y_dev, int count) {
    if (count <= 0 || m == 0) return PG_OK;
    const size_t k_in = w[0]->k_in;
    for (int i = 1; i < count; ++i)
        if (w[i]->k_in != k_in) return pg_fail(PG_EINVAL, "gguf_matmul_multi: the products differ in k_in");
    void *ws = nullptr;
    int digits_type = -1;
    bool any_mxfp4 = false, any_q41 = false;
    for (int i = 0; i < count; ++i) {
        any_mxfp4 |= w[i]->ggml_type == PG_MXFP4;
        any_q41 |= w[i]->ggml_type == PG_GGML_Q4_1;
    }
    if (any_mxfp4 || any_q41 || (m > 1 && k_in / 32 < PG_MM_MIN_BLOCKS)) {  // no shared route: product by product
        for (int i = 0; i < count; ++i) PG_TRY(pg_gguf_matmul_rows(ctx, x_dev, m, w[i], y_dev[i]));
        return PG_OK;
    }
    if (m == 1) {
        PG_TRY(pg_workspace(ctx, pg_xdigits_bytes(m, k_in), &ws));
        const pg_xdigits xd = pg_xdigits_carve(ws, m, k_in);
        const pg_gemv_batch batch = {1, nullptr, nullptr, nullptr, 1};
        for (int i = 0; i < count; ++i) {
            const int want = w[i]->ggml_type == PG_GGML_Q4_0 ? PG_GGML_Q4_0 : PG_GGML_Q8_0;  // nibble or byte digits
            if (want != digits_type) {
                PG_TRY(pg_launch_x_to_digits(ctx, x_dev, m, k_in, want, xd));
                digits_type = want;
            }
            PG_TRY(pg_launch_gguf_gemv(ctx, w[i]->ggml_type, w[i]->n_out, k_in, w[i]->qs, w[i]->d, batch, xd, y_dev[i]));
        }
        return PG_OK;
    }
    {   // many rows, one block type: one launch on the f16 matrix cores
        bool one_type = count <= PG_HMM_MAX_GROUP;
        size_t n_total = 0;
        for (int i = 0; i < count; ++i) {
            one_type &= w[i]->ggml_type == w[0]->ggml_type;
            n_total += w[i]->n_out;
        }
        int hks = 1;
        if (one_type && pg_gguf_hmm_takes(ctx, w[0]->ggml_type, m, n_total, k_in, &hks)) return pg_gguf_hmm_rows(ctx, x_dev, m, w, y_dev, count, hks);
    }
    const size_t sz_d = pg_mmdigits_bytes(m, k_in);
    size_t sz_part = 0;
    for (int i = 0; i < count; ++i) {
        const int ks = pg_gguf_mm_splitk(ctx, w[i]->n_out, k_in, (m + 31) / 32, m, false, nullptr);
        const size_t sz = ks > 1 ? pg_round_up((size_t)ks * m * w[i]->n_out * sizeof(float), 256) : 0;
        if (sz > sz_part) sz_part = sz;
    }
    PG_TRY(pg_workspace(ctx, sz_d + sz_part, &ws));
    const pg_mmdigits md = pg_mmdigits_carve(ws, m, k_in);
    float *part_base = reinterpret_cast<float *>(static_cast<char *>(ws) + sz_d);
    pg_mm_group grp = {1, nullptr, nullptr, nullptr, nullptr, 0, (int)((m + 31) / 32), (int)m, 1};
    grp.tiled = 1;
    for (int i = 0; i < count; ++i) {
        PG_TRY(pg_gguf_ensure_tiled(ctx, w[i]));
        if (w[i]->ggml_type != digits_type) {
            PG_TRY(pg_launch_x_to_mm_digits(ctx, x_dev, m, k_in, w[i]->ggml_type, md));
            digits_type = w[i]->ggml_type;
        }
        const int ks = pg_gguf_mm_splitk(ctx, w[i]->n_out, k_in, (m + 31) / 32, m, false, nullptr);
        PG_TRY(pg_launch_gguf_mm(ctx, w[i]->ggml_type, w[i]->n_out, k_in, w[i]->qs_tiled, w[i]->d, grp, m, md, y_dev[i],
                                 ks > 1 ? part_base : nullptr));
    }
    return PG_OK;
}

PG_API pg_status pg_gguf_hmm_force(pg_ctx *ctx, int mode) {
    PG_CHECK_ARG(ctx != nullptr, "null context");
    PG_CHECK_ARG(mode >= 0 && mode <= 2, "pg_gguf_hmm_force: mode %d (0 = automatic, 1 = wherever it can run, 2 = never)", mode);
    ctx->hmm_mode = mode;
    return PG_OK;
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
    PG_CHECK_ARG(ggml_type == PG_GGML_Q4_0 || ggml_type == PG_GGML_Q4_1 || ggml_type == PG_GGML_Q8_0,
                 "pg_gguf_upload: ggml type %d is not a block-quantised type", ggml_type);
    PG_CHECK_ARG(n_out > 0 && k_in > 0 && blocks, "pg_gguf_upload: empty tensor or null pointer");
    PG_CHECK_ARG(k_in % 32 == 0, "pg_gguf_upload: k_in %zu is not a multiple of 32", k_in);
    PG_CHECK_ARG(n_out < (1ull << 31) && k_in < (1ull << 31) && n_out * (k_in / 32) < (1ull << 31),
                 "pg_gguf_upload: shape too large");
    const size_t nb = k_in / 32, nblocks = n_out * nb;
    const size_t bb = ggml_type == PG_GGML_Q4_0 ? 18 : (ggml_type == PG_GGML_Q4_1 ? 20 : 34), qb = ggml_type == PG_GGML_Q8_0 ? 32 : 16;
    pg_gguf_tensor *t = new (std::nothrow) pg_gguf_tensor();
    if (!t) return pg_fail(PG_ENOMEM, "host allocation failed");
    t->qs = nullptr;
    t->d = nullptr;
    t->m = nullptr;
    t->qs_tiled = nullptr;
    t->ggml_type = ggml_type;
    t->n_out = n_out;
    t->k_in = k_in;
    pg_tmp raw;
    pg_status st = raw.alloc(nblocks * bb);
    hipError_t e = hipSuccess;
    if (st == PG_OK) {
        e = hipMalloc((void **)&t->qs, nblocks * qb);
        if (e == hipSuccess) e = hipMalloc((void **)&t->d, (n_out + 7) / 8 * 8 * nb * sizeof(uint16_t));
        if (e == hipSuccess && ggml_type == PG_GGML_Q4_1) e = hipMalloc((void **)&t->m, (n_out + 7) / 8 * 8 * nb * sizeof(uint16_t));
        if (e == hipSuccess) e = hipMemcpyAsync(raw.p, blocks, nblocks * bb, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) {
            split_blocks_kernel<<<grid_for((n_out + 7) / 8 * 8 * nb, 256), 256, 0, ctx->stream>>>(raw.as<uint8_t>(), n_out, nb,
                                                                               ggml_type, t->qs, t->d, t->m);
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
    if (t->m) (void)hipFree(t->m);
    if (t->qs_tiled) (void)hipFree(t->qs_tiled);
    delete t;
}

// Load-time step: the derived copy that a product over up to `max_rows` activation rows would otherwise make
// on its first call (pg_gguf_ensure_tiled: an allocation, a launch and a wait) is made now,
// so that the `_dev` products, the Llama block and the expert FFN over this tensor neither allocate nor wait --
// the place of the reference's own load-time rearrangement (load_transposed_weight, src/models/llama/model.rs:243-257).
PG_API pg_status pg_gguf_prepare(pg_ctx *ctx, const pg_gguf_tensor *w, size_t max_rows) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(w != nullptr, "pg_gguf_prepare: null tensor");
    if (max_rows < 2 || w->k_in / 32 < PG_MM_MIN_BLOCKS) return PG_OK;  // one row, or a K of a few blocks: the streaming kernels read the planes as uploaded
    if (w->ggml_type == PG_MXFP4) return PG_OK;  // every MXFP4 product reads the planes as uploaded
    if (w->ggml_type == PG_GGML_Q4_0 || w->ggml_type == PG_GGML_Q8_0 || w->ggml_type == PG_GGML_Q4_1)
        return pg_gguf_ensure_tiled(ctx, w);
    return PG_OK;
}

// The reverse: frees the derived copies (after the stream has drained); the next product that needs one makes it again.
PG_API pg_status pg_gguf_drop_prepared(pg_ctx *ctx, const pg_gguf_tensor *w) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(w != nullptr, "pg_gguf_drop_prepared: null tensor");
    PG_HIP(hipStreamSynchronize(ctx->stream));
    if (w->qs_tiled) { (void)hipFree(w->qs_tiled); w->qs_tiled = nullptr; }
    return PG_OK;
}

// Device bytes the tensor holds now: the planes as uploaded and the derived copies (0 if none was made).
PG_API pg_status pg_gguf_device_bytes(const pg_gguf_tensor *w, size_t *uploaded, size_t *derived) {
    PG_CHECK_ARG(w != nullptr, "pg_gguf_device_bytes: null tensor");
    const size_t nb = w->k_in / 32, blocks = w->n_out * nb;
    auto tiled_bytes = [](const pg_gguf_tensor *t) {
        return t->qs_tiled ? ((t->n_out + 127) / 128) * pg_tiled_group_bytes((int)(t->k_in / 32), t->ggml_type == PG_GGML_Q8_0) : (size_t)0;
    };
    if (uploaded) *uploaded = blocks * (w->ggml_type == PG_GGML_Q8_0 ? 34 : (w->ggml_type == PG_GGML_Q4_1 ? 20 : (w->ggml_type == PG_MXFP4 ? 17 : 18)));
    if (derived) *derived = tiled_bytes(w);
    return PG_OK;
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
