// Internal definitions shared by the HIP translation units of libperegrine_hip.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#include <string>
#include <tuple>
#include <type_traits>
#include <utility>
#include <vector>
#include "peregrine_hip.h"

#define PG_API extern "C" __attribute__((visibility("default")))

struct pg_prof_rec {
    const char *name;
    hipEvent_t start, stop;
    size_t threads;  // work-items of the launch (grid x block)
};
struct pg_prof_total {
    std::string name;
    double total_ms;
    size_t launches;
    std::vector<std::pair<size_t, size_t>> grids;  // distinct launch sizes (work-items) and how many launches had each
};

// One device + one stream + one growable scratch arena.
struct pg_ctx {
    int device;
    hipStream_t stream;
    bool owns_stream;
    void *ws;        // scratch arena (quantised activations, partial results)
    size_t ws_bytes;
    int num_cu;
    bool profiling;                     // per-kernel HIP events (pg_profile_begin/end)
    std::vector<pg_prof_rec> prof;      // one record per launch while profiling
    std::vector<pg_prof_total> totals;  // aggregated by pg_profile_end
    // MoE expert pointer tables, one per distinct set of experts seen (a model's MoE layers
    // alternate): a repeated call with a known set neither copies nor synchronises.
    struct moe_table {
        std::vector<const void *> host;
        void *dev;
    };
    std::vector<moe_table> moe_tabs;
    // Kernels whose dynamic LDS limit was raised on this context's device (pg_allow_dynamic_lds).
    std::vector<std::pair<const void *, size_t>> lds_raised;  // kernels whose dynamic-LDS limit was raised, and to what
    // W8A8 GEMM dispatch: the tile of the most recent launch (pg_gemm_w8a8_last_tile) and an
    // optional override of the dispatcher's choice (pg_gemm_w8a8_force_tile; 0 = automatic).
    int gemm_last_bm = 0, gemm_last_bn = 0, gemm_last_splits = 0;
    int gemm_force_tile = 0;
    int gemv_force_nw = 0, gemv_force_rpw = 0;  // pg_gemv_w8a8_force_shape (0 = the dispatcher chooses)
    int hmm_mode = 0;  // pg_gguf_hmm_force: 0 = the dispatcher chooses, 1 = the f16 matrix-core product wherever it can run, 2 = never
};

// Device-resident quantised weight, K-contiguous and zero-padded:
//   w_t    [n_pad, k_pad] i8, w_t[n*k_pad + k] = q[k, n]; padding is 0
//   scales [n_pad] f32 (padding 1.0)
struct pg_qtensor {
    int8_t *w_t;
    float *scales;
    size_t rows, cols;    // rows = K, cols = N (the reference's naming)
    size_t k_pad, n_pad;  // multiples of PG_KPAD / PG_NPAD
};

// GGUF block tensor split into planes at upload:
//   qs     [n_out, k_in/32, QB] quant bytes (QB = 16 for Q4_0, 32 for Q8_0)
//   d      [ceil(n_out/8), k_in/32, 8]  f16 block scales, tiled by 8 weight rows
struct pg_gguf_tensor {
    uint8_t *qs;
    uint16_t *d;
    uint16_t *m;  // Q4_1 only: the blocks' f16 offsets, tiled like d; else null
    // Q4_0 / Q8_0: a second copy of qs in the order gguf_mm_kernel's workgroups fetch it
    // (pg_gguf_ensure_tiled makes it on the tensor's first product over more than one row).
    mutable uint8_t *qs_tiled;
    int ggml_type;
    size_t n_out, k_in;
};

// The matrix-core block product carries 16-bit fixed-point activations per block: fine when a
// dot product averages over many blocks, too coarse when one or two blocks make the whole sum
// (an outlier in the block then costs every other element ~2^-16 of the outlier).  Products
// whose K spans fewer blocks than this run the streaming kernel (18 / 22-bit activations),
// one item per activation row.
// attention::StandardKVCache (src/attention.rs:8-15) on the device: k, v = [num_kv_heads][capacity][head_dim] f32.
struct pg_kv_cache {
    float *k, *v;
    size_t len, capacity, num_kv_heads, head_dim;
};
constexpr size_t PG_MM_MIN_BLOCKS = 5;
constexpr int PG_GEMM_MAX_GROUP = 4;  // weights one W8A8 launch can carry (fused q|k|v, gate|up)
constexpr size_t PG_KPAD = 128;  // device K stride is a multiple of this
constexpr size_t PG_NPAD = 256;  // device weight rows are padded to this
constexpr size_t PG_MPAD = 256;  // quantised activation rows in the workspace are padded to this

static inline size_t pg_round_up(size_t v, size_t m) { return (v + m - 1) / m * m; }

// Error plumbing --------------------------------------------------------------
pg_status pg_fail(pg_status st, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define PG_CHECK_ARG(cond, ...)                                   \
    do {                                                          \
        if (!(cond)) return pg_fail(PG_EINVAL, __VA_ARGS__);      \
    } while (0)

#define PG_HIP(call)                                                              \
    do {                                                                          \
        hipError_t e_ = (call);                                                   \
        if (e_ != hipSuccess)                                                     \
            return pg_fail(e_ == hipErrorOutOfMemory ? PG_ENOMEM : PG_EDEVICE,    \
                           "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                           __FILE__, __LINE__);                                   \
    } while (0)

#define PG_TRY(call)                    \
    do {                                \
        pg_status s_ = (call);          \
        if (s_ != PG_OK) return s_;     \
    } while (0)

// Make ctx's device current for the calling thread.
pg_status pg_use(pg_ctx *ctx);
// Scratch arena of at least `bytes` (256-byte aligned); contents undefined.
pg_status pg_workspace(pg_ctx *ctx, size_t bytes, void **out);
// Check the launch just made.
pg_status pg_launch_check(const char *what);
// Let `kernel` use `bytes` of dynamic LDS on this context's device (the attribute is set once
// per context: it belongs to the device's copy of the kernel).
pg_status pg_allow_dynamic_lds(pg_ctx *ctx, const void *kernel, size_t bytes);

// Launch `kernel` on the context's stream.  While profiling (pg_profile_begin/end) the
// dispatch carries a start and a stop event: hipExtLaunchKernel stamps them with the
// kernel's own begin and end times (what a kernel trace reports), not with the time the
// stream reaches a separately recorded event.
template <typename... KArgs, size_t... I>
inline void pg_arg_ptrs(std::tuple<KArgs...> &t, void **out, std::index_sequence<I...>) {
    ((out[I] = static_cast<void *>(&std::get<I>(t))), ...);
}
template <typename... KArgs, typename... Args>
inline pg_status pg_launch(pg_ctx *ctx, const char *name, void (*kernel)(KArgs...), dim3 grid, dim3 block,
                           size_t lds, Args &&...args) {
    static_assert(sizeof...(KArgs) == sizeof...(Args), "argument count differs from the kernel's");
    hipEvent_t start = nullptr, stop = nullptr;
    if (ctx->profiling) {
        if (hipEventCreate(&start) != hipSuccess) start = nullptr;
        if (start && hipEventCreate(&stop) != hipSuccess) { (void)hipEventDestroy(start); start = stop = nullptr; }
        if (start)
            ctx->prof.push_back({name, start, stop, (size_t)grid.x * grid.y * grid.z * block.x * block.y * block.z});
    }
    std::tuple<KArgs...> tup{static_cast<KArgs>(args)...};
    void *ptrs[sizeof...(KArgs) ? sizeof...(KArgs) : 1];
    pg_arg_ptrs(tup, ptrs, std::index_sequence_for<KArgs...>{});
    const hipError_t e = hipExtLaunchKernel(reinterpret_cast<const void *>(kernel), grid, block, ptrs, lds,
                                            ctx->stream, start, stop, 0);
    if (e != hipSuccess) return pg_fail(PG_EDEVICE, "launch of %s failed: %s", name, hipGetErrorString(e));
    return PG_OK;
}

// RAII device temporary for the host-pointer entry points.
struct pg_tmp {
    void *p = nullptr;
    ~pg_tmp() { if (p) (void)hipFree(p); }
    pg_status alloc(size_t bytes) {
        hipError_t e = hipMalloc(&p, bytes ? bytes : 1);
        if (e != hipSuccess) { p = nullptr; return pg_fail(PG_ENOMEM, "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e)); }
        return PG_OK;
    }
    template <class T> T *as() const { return static_cast<T *>(p); }
};

// Fills device memory with pseudo-random bytes (the probes' operands), stream ordered.
pg_status pg_probe_fill_random(pg_ctx *ctx, void *dev, size_t bytes);

// Kernel launchers implemented per translation unit (device pointers, stream ordered).
pg_status pg_launch_quantize_activations(pg_ctx *ctx, const float *a, size_t rows, size_t cols,
                                         int8_t *q, size_t q_stride, float *row_scales);
pg_status pg_launch_gemm_w8a8(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride,
                              const float *a_scales, const pg_qtensor *w, size_t m,
                              float *out, int32_t *acc);
// The same activation rows against up to PG_GEMM_MAX_GROUP weights of equal K in ONE launch: the
// weights' column panels form one tile space (a fused QKV or gate|up product without a fused
// copy of the weights).  out[i] is [m, w[i]->cols].
pg_status pg_launch_gemm_w8a8_group(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                                    const pg_qtensor *const *w, float *const *out, int count, size_t m);
// 5 .. 64 activation rows: K split over workgroups, i32 partial sums in `part`, then one finishing
// launch.  With part == nullptr only reports the number of splits (for sizing `part`).
pg_status pg_launch_gemm_w8a8_combine(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                                      const pg_qtensor *w, size_t m, float *out, const int32_t *comb, size_t comb_plane);
bool pg_gemm_w8a8_takes_skinny(const pg_qtensor *w, size_t m);
pg_status pg_launch_gemm_w8a8_skinny_group(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                                           const pg_qtensor *const *w, float *const *out, int count, size_t m, int32_t *acc);
pg_status pg_launch_gemm_w8a8_skinny(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                                     const pg_qtensor *w, size_t m, float *out, int32_t *acc);
pg_status pg_launch_gemm_w8a8_few_rows(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride, const float *a_scales,
                                       const pg_qtensor *w, size_t m, float *out, int32_t *acc, int32_t *part,
                                       int *splits_out);
pg_status pg_launch_gemv_w8a8(pg_ctx *ctx, const int8_t *a_i8, size_t a_stride,
                              const float *a_scales, const pg_qtensor *w, size_t m,
                              float *out, int32_t *acc);
// One activation row still in f32: quantised inside the product's own launch (same integers and
// scale as pg_launch_quantize_activations would give).  Only where the predicate holds.
bool pg_gemv_w8a8_takes_f32_row(const pg_qtensor *w, size_t m, size_t k, const float *x_f32);
pg_status pg_launch_gemv_w8a8_f32_row(pg_ctx *ctx, const float *x_f32, size_t k, const pg_qtensor *w, float *out,
                                      int32_t *acc);
// The same row against up to PG_GEMM_MAX_GROUP weights of equal K in one launch.
pg_status pg_launch_gemv_w8a8_f32_row_group(pg_ctx *ctx, const float *x_f32, size_t k, const pg_qtensor *const *w,
                                            float *const *out, int count, int32_t *acc);
// Activation rows rewritten as three byte-digit planes (see pg_gguf.hip).
struct pg_xdigits {
    int8_t *digits;  // [rows][6 planes][k/32 blocks][16 bytes] (Q4_0 uses 5 planes, Q8_0 all 6)
    float *xs;       // [rows][k/32] power-of-two block scales
    float *xsum;     // [rows][k/32] sum of each block's fixed-point values (written for Q4_1 only)
    size_t rows, k;
};

// Sum over the 64 lanes of a wavefront, returned in every lane (DPP within rows of 16
// lanes, then the four row totals through scalar registers).
__device__ __forceinline__ float pg_wave_sum_f32(float v) {
    auto dpp_add = [](float x, auto ctrl) {
        const int y = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xf, 0xf, false);
        return x + __builtin_bit_cast(float, y);
    };
    v = dpp_add(v, std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
    v = dpp_add(v, std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]
    v = dpp_add(v, std::integral_constant<int, 0x141>{});  // row_half_mirror
    v = dpp_add(v, std::integral_constant<int, 0x140>{});  // row_mirror
    const int b = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
}

__device__ __forceinline__ int pg_wave_sum_i32(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false);
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false);
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, false);
    v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xf, 0xf, false);
    return __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) +
           __builtin_amdgcn_readlane(v, 32) + __builtin_amdgcn_readlane(v, 48);
}
size_t pg_xdigits_bytes(size_t rows, size_t k);
pg_xdigits pg_xdigits_carve(void *base, size_t rows, size_t k);
pg_status pg_launch_x_to_digits(pg_ctx *ctx, const float *x_dev, size_t rows, size_t k,
                                int ggml_type, const pg_xdigits &xd);
// A batch of independent M = 1 products: item i uses activation row i / x_row_div and,
// when a table is given, the weights of expert expert_of[i].
struct pg_gemv_batch {
    int count;
    const uint8_t *const *qs_table;
    const uint16_t *const *d_table;
    const int *expert_of;
    int x_row_div;
};
// What a product whose output feeds the next product does besides (see gguf_gemv_kernel).
struct pg_gemv_epi {
    const float *gamma;      // RMSNorm weights of the output row
    int8_t *out_digits;      // the output (times gamma, or SiLU(gate) * up) as digits
    float *out_xs;
    float *ss_out;           // [n_out / 32] sums of squares of the output, one per block
    const float *ss_in;      // the input row's sums of squares: the product is divided by its RMS
    int ss_n;
    float ss_inv_dim, eps;
    const uint8_t *qs1;      // the second tensor (up) of the SiLU(gate) * up form
    const uint16_t *d1;
};
// y[item][row] = product (+ residual[item][row] when `residual` is given).
pg_status pg_launch_gguf_gemv(pg_ctx *ctx, int ggml_type, size_t n_out, size_t k_in,
                              const uint8_t *qs, const uint16_t *d, const pg_gemv_batch &batch,
                              const pg_xdigits &xd, float *y, const float *residual = nullptr,
                              const uint16_t *m = nullptr);
// Q4_0, one f32 row shared by every item: y[item] = W[item] . RMSNorm(x_f32; gamma, eps), the norm folded
// into the product's launch.  k_in at most 8192; x_f32 and gamma 16-byte aligned.
pg_status pg_launch_gguf_gemv_rmsnorm(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d,
                                      const pg_gemv_batch &batch, const float *x_f32, const float *gamma, float eps, float *y);
// Q4_0 or Q8_0, one row: y = product (+ residual) as usual, and besides `out` = the digits of y * gamma and
// ss_out[n_out / 32] = the sums of squares of y by block: RMSNorm(y) without a launch, its scalar factor
// left to the consumer.  n_out a multiple of 32.
pg_status pg_launch_gguf_gemv_norm_digits(pg_ctx *ctx, int ggml_type, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d,
                                          const pg_xdigits &xd, float *y, const float *residual, const float *gamma,
                                          const pg_xdigits &out, float *ss_out);
// Q4_0 or Q8_0 (gate and up alike), one row: out = digits of SiLU(g) * u with g, u = the products by gate and up, both divided by the
// RMS of the input row (ss_in: ss_n partial sums of squares over ss_dim elements, eps).
pg_status pg_launch_gguf_gemv_swiglu_digits(pg_ctx *ctx, int ggml_type, size_t n_out, size_t k_in, const uint8_t *qs_gate, const uint16_t *d_gate,
                                            const uint8_t *qs_up, const uint16_t *d_up, const pg_xdigits &xd, const float *ss_in,
                                            size_t ss_n, size_t ss_dim, float eps, const pg_xdigits &out);
// One activation row still in f32: digits made inside the product's own launch.  Only where the predicate holds.
bool pg_gguf_gemv_takes_f32_row(int ggml_type, size_t n_out, size_t k_in, const float *x_f32);
pg_status pg_launch_gguf_gemv_f32_row(pg_ctx *ctx, int ggml_type, size_t n_out, size_t k_in, const uint8_t *qs,
                                      const uint16_t *d, const float *x_f32, float *y);
bool pg_gguf_gemv_takes_few_rows(int ggml_type, size_t m, size_t n_out, size_t k_in, const float *x_f32);
pg_status pg_launch_gguf_gemv_few_rows(pg_ctx *ctx, size_t n_out, size_t k_in, const uint8_t *qs, const uint16_t *d, const float *x_f32,
                                       size_t m, float *y);
// Activation rows as two byte-digit planes for the matrix-core product (see pg_gguf_mm.hip).
struct pg_mmdigits {
    int8_t *digits;  // [rows][2 planes][k/32 blocks][2 halves][16 bytes], rows padded to an odd number of 256-byte lines
    float *xs;       // [rows][k/32 rounded up to 4] block scales
    float *xsum;     // [rows][k/32 rounded up to 4] plain block sums of x (written for Q4_1 products only)
    size_t rows, k;
};
size_t pg_mmdigits_bytes(size_t rows, size_t k);
pg_mmdigits pg_mmdigits_carve(void *base, size_t rows, size_t k);
bool pg_gguf_skinny_takes(const pg_ctx *ctx, int ggml_type, size_t m, size_t n_out, size_t k_in);
struct pg_skinny_group {  // the tensors of one few-rows launch (gguf_skinny_kernel)
    const uint8_t *qs[3];
    const uint16_t *d[3];
    float *y[3];
    const float *res[3];  // where set: y = res + product (same shape as y)
    int n[3];
    int wg0[3];
};
pg_status pg_launch_gguf_skinny_group(pg_ctx *ctx, int ggml_type, size_t k_in, const pg_gguf_tensor *const *w, float *const *y, int count,
                                      size_t m, const pg_mmdigits &md, const float *residual = nullptr);  // residual: added to tensor 0's product
pg_status pg_launch_x_to_mm_digits(pg_ctx *ctx, const float *x_dev, size_t rows, size_t k, int ggml_type,
                                   const pg_mmdigits &md);
// Q4_1 on the matrix-core route: the product is the Q4_0 product on the same nibbles and scales plus
// y[t][n] += sum_b (8 d + m)[n][b] * (sum of x over block b of row t); this adds the second term (md.xsum
// as pg_launch_x_to_mm_digits leaves it for PG_GGML_Q4_1).  k_in up to 32768.
pg_status pg_launch_q41_offset(pg_ctx *ctx, const pg_gguf_tensor *w, const pg_mmdigits &md, size_t rows, float *y);
// Which activation rows multiply which weights.  Without `counts`: one weight tensor and pairs
// 0 .. max_count-1.  With `counts`: expert e owns counts[e] pairs, listed (in ascending order) in
// lists[e * list_stride ..]; its weights are qs_table[e] / d_table[e].  Pair p reads activation
// row p / x_row_div and writes output row p.  tiles_per_expert = ceil(max pairs per expert / 32).
struct pg_mm_group {
    int num_experts;
    const uint8_t *const *qs_table;
    const uint16_t *const *d_table;
    const int *lists;
    const int *counts;
    int list_stride;
    int tiles_per_expert;
    int max_count;
    int x_row_div;
    int remap_rg, remap_tiles;  // set by the launcher (row groups and token tiles of an XCD-aware 1-D launch), else 0
    int tiled;                  // the qs pointers are tile-major copies (pg_gguf_tensor::qs_tiled)
    int xcd_ks;                 // set by the launcher: K chunks dealt to XCDs (2, 4 or 8), else 0
    // Several tensors of equal K in one launch (q|k|v, gate|up): the launch's 128-row groups are the tensors'
    // groups one after the other; tensor t starts at group seg_first[t], has seg_n[t] rows, its own tile-major
    // copy, scales and output (planes seg_stride[t] floats apart).  nseg = 0: the one tensor of the arguments.
    int nseg;
    int seg_first[3], seg_n[3];
    const uint8_t *seg_qs[3];
    const uint16_t *seg_d[3];
    float *seg_out[3];
    size_t seg_stride[3];
};
// Bytes from one 128-row group of a tile-major copy to the next: the group's stages (16 KiB
// each for Q8_0, 8 KiB for Q4_0) plus 4352 bytes, so that workgroups walking their groups in
// step do not all address the same memory channels (a bare power-of-two stride would).
__host__ __device__ static inline size_t pg_tiled_group_bytes(int nb, bool q8) {
    return (size_t)((nb + 3) / 4) * (q8 ? 16384 : 8192) + 4352;
}
// Makes w->qs_tiled if it is missing (one allocation and one kernel on the context's stream).
pg_status pg_gguf_ensure_tiled(pg_ctx *ctx, const pg_gguf_tensor *w);
// Number of K chunks the product is split into (partial sums: [chunks][pairs][n_out] floats);
// `groups` = token tiles that certainly hold work (all tiles of a plain product, one per expert).
// `act_rows` = activation rows the product reads, `grouped` = with expert lists.
int pg_gguf_mm_splitk(const pg_ctx *ctx, size_t n_out, size_t k_in, size_t groups, size_t act_rows, bool grouped,
                      int *chunk_out, bool *xcd_chunks = nullptr);
pg_status pg_launch_gguf_mm(pg_ctx *ctx, int ggml_type, size_t n_out, size_t k_in, const uint8_t *qs,
                            const uint16_t *d, const pg_mm_group &grp, size_t total_pairs, const pg_mmdigits &md,
                            float *y, float *part, bool keep_parts = false);  // keep_parts: the K chunks' planes are left in `part` unsummed
// y[i] = part[0][i] + ... + part[ks - 1][i] (planes `stride` floats apart), in that order.
// Huffman pieces shared by the coded weights and the coded KV cache (pg_huffman.hip).
struct pg_huffman_dev_stream {
    const uint8_t *bytes_dev;   // the stream
    size_t bytes, symbols;
    const uint16_t *lut_dev;    // its decode table, pg_huffman_lut_entries() entries
    size_t out_off;             // where its symbols go in the output
};
bool pg_huffman_host_table(const uint64_t *freqs, uint8_t *bit_lengths, uint32_t *codes);
size_t pg_huffman_lut_entries();
pg_status pg_huffman_host_lut(const uint8_t *bit_lengths, uint16_t *lut);
pg_status pg_huffman_decode_device_streams(pg_ctx *ctx, const pg_huffman_dev_stream *streams, size_t count, int8_t *out_dev);
pg_status pg_launch_sum_parts(pg_ctx *ctx, const float *part, size_t n, int ks, size_t stride, float *y);
// The many-row Q4_0 product on the f16 matrix cores (pg_gguf_hmm.hip).  The activation rows as two f16 planes
// [rows][k] (x * 2^e = hi + lo, e per row) and the rows' 2^-e as two f32 factors each.
constexpr int PG_HMM_MAX_GROUP = 4;  // tensors one launch can carry (q|k|v, gate|up)
struct pg_hmm_planes {
    void *hi, *lo;
    float *inv;  // [rows][2]
    size_t rows, k;
};
size_t pg_hmm_planes_bytes(size_t rows, size_t k);
pg_hmm_planes pg_hmm_planes_carve(void *base, size_t rows, size_t k);
pg_status pg_launch_rows_to_f16_planes(pg_ctx *ctx, const float *x_dev, size_t rows, size_t k, const pg_hmm_planes &p);
// Whether a product of m rows with n_total weight rows (all the tensors of the launch) runs there, and in how many
// K chunks (*ks_out; their planes need pg_gguf_hmm_part_floats floats).
bool pg_gguf_hmm_takes(const pg_ctx *ctx, int ggml_type, size_t m, size_t n_total, size_t k_in, int *ks_out);
size_t pg_gguf_hmm_part_floats(size_t m, size_t n_total, int ks);
pg_status pg_launch_gguf_hmm_group(pg_ctx *ctx, size_t k_in, const pg_gguf_tensor *const *w, float *const *y, int count, size_t m,
                                   const pg_hmm_planes &planes, int ks, float *part, bool keep_parts = false);
// y[m, n_out] = x[m, k_in] . dequant(w)^T on device pointers (uses the scratch arena).
// MXFP4 tensors (pg_mxfp4.hip): qs holds the code bytes in matrix-core fragment order, d the E8M0 scale
// bytes (four per dword); every product over them runs pg_launch_mxfp4_rows.
pg_status pg_launch_mxfp4_rows(pg_ctx *ctx, const float *x_dev, size_t m, const pg_gguf_tensor *w, float *y_dev);
// Many rows: the tile kernel on the same instruction (activations as three digit planes, weights read once per 64 rows).
// MoE pieces shared by the block-tensor experts (pg_moe.hip) and the MXFP4 experts (pg_mxfp4.hip).
constexpr int PG_MOE_MAX_EXPERTS = 256;
pg_status pg_moe_cached_table(pg_ctx *ctx, const void *const *host_tab, size_t n, const void ***dev_tab);
pg_status pg_launch_moe_routing(pg_ctx *ctx, const float *router_logits_dev, const int *idx_dev, const float *weight_dev, size_t T,
                                size_t E, size_t top_k, int *topk_idx, float *topk_p, int *lists, int *counts);
struct pg_mxfp4_tiles_plan {
    int ra, tb;            // groups of 16 weight rows per wavefront, groups of 16 tokens per workgroup
    int ks, cps;           // runs of K and chunks per run
    size_t n_wt, n_tt;     // row tiles, token tiles
    size_t groups;         // token groups the records are written for (n_tt * tb)
};
pg_mxfp4_tiles_plan pg_mxfp4_tiles_plan_for(int num_cu, size_t n_out, size_t m, int ncp);
bool pg_mxfp4_tiles_takes(const pg_gguf_tensor *w, size_t m);
pg_status pg_launch_mxfp4_tiles(pg_ctx *ctx, const float *x_dev, size_t m, const pg_gguf_tensor *w, float *y_dev);
pg_status pg_gguf_matmul_rows(pg_ctx *ctx, const float *x_dev, size_t m, const pg_gguf_tensor *w,
                              float *y_dev);
// `count` such products over the same rows (equal k_in), the rows rewritten as digits once.
pg_status pg_gguf_matmul_rows_multi(pg_ctx *ctx, const float *x_dev, size_t m, const pg_gguf_tensor *const *w,
                                    float *const *y_dev, int count);
