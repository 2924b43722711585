// Grouped MoE expert FFN over block-quantised (Q8_0 / Q4_0) experts, entirely
// stream-ordered on the device (no host round trip for the routing):
//   1. route: softmax over the E router logits of each token, top-k by stable
//      descending order (ties -> lower expert index)   examples/grok1/moe.rs:76-89
//   2. gate / up products of every (token, k) pair against its expert's weights
//   3. h = act(g) * u                                   grok1/moe.rs:27-34, deepseek/moe.rs:55-59
//   4. down product of every pair
//   5. out[t] = 0 + p_0 * y_0 + p_1 * y_1 ... in k order, multiply then add
//      (examples/grok1/moe.rs:99-104), raw softmax probabilities.
#include "pg_internal.h"
#include <algorithm>

namespace {

inline unsigned grid_for(size_t n, unsigned block) { return (unsigned)((n + block - 1) / block); }

constexpr int MAX_EXPERTS = PG_MOE_MAX_EXPERTS;

// One thread per token.
__global__ void route_topk_kernel(const float *__restrict__ logits, int T, int E, int top_k,
                                  int *__restrict__ topk_idx, float *__restrict__ topk_p) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= T) return;
    const float *x = logits + (size_t)t * E;
    float mx = -INFINITY;
    for (int e = 0; e < E; ++e)
        if (x[e] > mx) mx = x[e];
    float sum = 0.0f;
    for (int e = 0; e < E; ++e) sum += expf(x[e] - mx);
    // k passes of "largest remaining, lowest index on ties" == stable descending sort
    unsigned taken[MAX_EXPERTS / 32];
    for (int i = 0; i < MAX_EXPERTS / 32; ++i) taken[i] = 0u;
    for (int k = 0; k < top_k; ++k) {
        int best = -1;
        float bp = 0.0f;
        for (int e = 0; e < E; ++e) {
            if (taken[e >> 5] & (1u << (e & 31))) continue;
            const float p = expf(x[e] - mx) / sum;
            if (best < 0 || p > bp) { best = e; bp = p; }
        }
        taken[best >> 5] |= 1u << (best & 31);
        topk_idx[(size_t)t * top_k + k] = best;
        topk_p[(size_t)t * top_k + k] = bp;
    }
}

// A routing that the caller made (another gate: examples/deepseek/moe.rs:111-215, examples/gpt_oss/moe.rs:298-330)
// is copied into the same arrays.  The grouped products assume what every top-k gate delivers: a token's experts are
// distinct and inside 0 .. E - 1.  An entry that breaks this is replaced by the lowest expert the token does not use
// yet, with weight 0, so that nothing downstream can index outside a table whatever the buffers hold (the entry's
// own contribution is then 0 times a finite product).  One thread per token.
__global__ void copy_routing_kernel(const int *__restrict__ idx_in, const float *__restrict__ w_in, int T, int E, int top_k,
                                    int *__restrict__ topk_idx, float *__restrict__ topk_p) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= T) return;
    unsigned taken[MAX_EXPERTS / 32];
    for (int i = 0; i < MAX_EXPERTS / 32; ++i) taken[i] = 0u;
    for (int k = 0; k < top_k; ++k) {
        int e = idx_in[(size_t)t * top_k + k];
        float w = w_in[(size_t)t * top_k + k];
        if (e < 0 || e >= E || (taken[e >> 5] & (1u << (e & 31)))) {
            e = 0;
            while (taken[e >> 5] & (1u << (e & 31))) ++e;  // top_k <= E: a free expert exists
            w = 0.0f;
        }
        taken[e >> 5] |= 1u << (e & 31);
        topk_idx[(size_t)t * top_k + k] = e;
        topk_p[(size_t)t * top_k + k] = w;
    }
}

// Per expert, the (token, k) pairs routed to it, in ascending pair order.  One wavefront per
// expert: ballot + prefix count over 64 pairs at a time.
__global__ __launch_bounds__(64) void expert_lists_kernel(const int *__restrict__ topk_idx, int P, int stride,
                                                          int *__restrict__ lists, int *__restrict__ counts) {
    const int e = blockIdx.x, lane = threadIdx.x;
    int base = 0;
    for (int p0 = 0; p0 < P; p0 += 64) {
        const int p = p0 + lane;
        const bool mine = p < P && topk_idx[p] == e;
        const unsigned long long mask = __ballot(mine);
        if (mine) lists[(size_t)e * stride + base + __popcll(mask & ((1ull << lane) - 1ull))] = p;
        base += __popcll(mask);
    }
    if (lane == 0) counts[e] = base;
}

__device__ __forceinline__ float act_silu(float x) {
    const float sig = 1.0f / (1.0f + expf(-x));
    return x * sig;
}
__device__ __forceinline__ float act_gelu_tanh(float x) {
    const float c = sqrtf(2.0f / 3.14159265358979323846f);
    const float inner = c * (x + 0.044715f * x * x * x);
    return 0.5f * x * (1.0f + tanhf(inner));
}

__global__ void act_mul_kernel(const float *__restrict__ g, const float *__restrict__ u, size_t n,
                               int act, float *__restrict__ h) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float a = (act == PG_ACT_GELU_TANH) ? act_gelu_tanh(g[i]) : act_silu(g[i]);
    h[i] = a * u[i];
}

// `shared` (optional): the shared experts' output, added last (y.add(&z), examples/deepseek/moe.rs:298-300).
__global__ void combine_kernel(const float *__restrict__ yb, const float *__restrict__ topk_p, int T,
                               int d, int top_k, const float *__restrict__ shared, float *__restrict__ out) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)T * d) return;
    const size_t t = i / d, c = i - t * d;
    float acc = 0.0f;
    for (int k = 0; k < top_k; ++k) {
        const float prod = topk_p[t * top_k + k] * yb[(t * top_k + k) * d + c];
        acc = acc + prod;
    }
    out[i] = shared ? acc + shared[i] : acc;
}

}  // namespace

// A table of device pointers (an expert set's planes) in a device buffer kept with the context, one per distinct
// table; uploaded (blocking: the source is the caller's stack frame) only on a table's first use.
pg_status pg_moe_cached_table(pg_ctx *ctx, const void *const *host_tab, size_t n, const void ***dev_tab) {
    for (size_t i = 0; i < ctx->moe_tabs.size(); ++i) {
        auto &t = ctx->moe_tabs[i];
        if (t.host.size() == n && memcmp(t.host.data(), host_tab, n * sizeof(void *)) == 0) {
            *dev_tab = static_cast<const void **>(t.dev);
            if (i + 1 != ctx->moe_tabs.size()) std::rotate(ctx->moe_tabs.begin() + i, ctx->moe_tabs.begin() + i + 1, ctx->moe_tabs.end());  // most recent last
            return PG_OK;
        }
    }
    // Least recently used out first.  A layer has two sets (row-major planes for one token, tile-major ones for
    // more), and a model alternates its layers: 512 sets hold both for 256 layers (the reference's Grok-1 has 64,
    // examples/grok1/model.rs:35), so a decode loop after a prefill misses on no layer.
    if (ctx->moe_tabs.size() >= 512) {  // a bounded cache: drop a set once nothing can still read it
        PG_HIP(hipStreamSynchronize(ctx->stream));
        (void)hipFree(ctx->moe_tabs.front().dev);
        ctx->moe_tabs.erase(ctx->moe_tabs.begin());
    }
    void *dev = nullptr;
    PG_HIP(hipMalloc(&dev, n * sizeof(void *)));
    const hipError_t ce = hipMemcpy(dev, host_tab, n * sizeof(void *), hipMemcpyHostToDevice);
    if (ce != hipSuccess) {
        (void)hipFree(dev);
        return pg_fail(PG_EDEVICE, "uploading an expert table: %s", hipGetErrorString(ce));
    }
    ctx->moe_tabs.push_back({std::vector<const void *>(host_tab, host_tab + n), dev});
    *dev_tab = static_cast<const void **>(dev);
    return PG_OK;
}

// The routing of T tokens as the expert products want it: topk_idx / topk_p [T * top_k] (from the router's logits,
// grok1's softmax -> top-k, or a copy of the caller's own choice with out-of-range and repeated experts made
// harmless), and per expert the (token, k) pairs routed to it in ascending order (lists [E][T], counts [E]).
pg_status pg_launch_moe_routing(pg_ctx *ctx, const float *router_logits_dev, const int *idx_dev, const float *weight_dev, size_t T,
                                size_t E, size_t top_k, int *topk_idx, float *topk_p, int *lists, int *counts) {
    if (router_logits_dev)
        PG_TRY(pg_launch(ctx, "moe_route_topk", route_topk_kernel, dim3(grid_for(T, 64)), dim3(64), 0,
                         router_logits_dev, (int)T, (int)E, (int)top_k, topk_idx, topk_p));
    else
        PG_TRY(pg_launch(ctx, "moe_copy_routing", copy_routing_kernel, dim3(grid_for(T, 64)), dim3(64), 0,
                         idx_dev, weight_dev, (int)T, (int)E, (int)top_k, topk_idx, topk_p));
    if (!lists) return PG_OK;  // (a caller that works pair by pair)
    return pg_launch(ctx, "moe_expert_lists", expert_lists_kernel, dim3((unsigned)E), dim3(64), 0, (const int *)topk_idx,
                     (int)(T * top_k), (int)T, lists, counts);
}

// The expert FFN behind both entry points: the routing comes from `router_logits_dev` (grok1's softmax -> top-k) or,
// when that is null, from `idx_dev` / `weight_dev` as the caller's gate made them.
static pg_status moe_ffn_core(pg_ctx *ctx, const float *x_dev, size_t T, const float *router_logits_dev,
                              const int *idx_dev, const float *weight_dev, size_t E, size_t top_k,
                              const pg_gguf_tensor *const *gate, const pg_gguf_tensor *const *up,
                              const pg_gguf_tensor *const *down, int act, const float *shared_dev, float *out_dev) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(E >= 1 && E <= MAX_EXPERTS, "pg_moe_ffn: %zu experts (1..%d supported)", E, MAX_EXPERTS);
    PG_CHECK_ARG(top_k >= 1 && top_k <= E, "pg_moe_ffn: top_k %zu of %zu experts", top_k, E);
    PG_CHECK_ARG(act == PG_ACT_SILU || act == PG_ACT_GELU_TANH, "pg_moe_ffn: unknown activation %d", act);
    PG_CHECK_ARG(gate && up && down && gate[0] && up[0] && down[0], "pg_moe_ffn: null expert table");
    const size_t d = gate[0]->k_in, ffn = gate[0]->n_out;
    const int type = gate[0]->ggml_type;
    PG_CHECK_ARG(type == PG_GGML_Q4_0 || type == PG_GGML_Q8_0, "pg_moe_ffn: experts must be Q4_0 or Q8_0 block tensors");
    for (size_t e = 0; e < E; ++e) {
        PG_CHECK_ARG(gate[e] && up[e] && down[e], "pg_moe_ffn: expert %zu has a null tensor", e);
        PG_CHECK_ARG(gate[e]->k_in == d && gate[e]->n_out == ffn && up[e]->k_in == d &&
                         up[e]->n_out == ffn && down[e]->k_in == ffn && down[e]->n_out == d,
                     "pg_moe_ffn: expert %zu shapes do not match [ffn=%zu, d=%zu]", e, ffn, d);
        PG_CHECK_ARG(gate[e]->ggml_type == type && up[e]->ggml_type == type && down[e]->ggml_type == type,
                     "pg_moe_ffn: expert %zu mixes block types", e);
    }
    if (T == 0) return PG_OK;
    PG_CHECK_ARG(x_dev && (router_logits_dev || (idx_dev && weight_dev)) && out_dev, "pg_moe_ffn: null pointer");
    PG_CHECK_ARG((uintptr_t)x_dev % 16 == 0, "pg_moe_ffn: x must be 16-byte aligned");
    PG_CHECK_ARG(T * top_k < (1ull << 20), "pg_moe_ffn: too many (token, expert) pairs");
    const size_t P = T * top_k;

    // Which products take the streaming kernel (18 / 22-bit activations, one item per pair) instead
    // of the matrix-core one (16-bit activations per block):
    //  * a product whose own K spans only a few blocks (as everywhere);
    //  * all three when the experts are narrow (ffn < 512).  An error of 2^-16 of a block's
    //    absmax in g or u is multiplied by the partner factor in h = act(g) * u; where that factor
    //    is an outlier (|g| of 10 and more happens) the one h element carries an absolute error far
    //    above the others', and the down product only averages it away over many terms: its share
    //    of an output's error falls as 1 / sqrt(ffn) (measured 1.4e-3 of the row rms at ffn 64,
    //    below 2e-4 from ffn 2048 up).  Narrow experts are tiny products; the price is nil.
    const bool narrow = ffn < 512 && P <= 65535;
    // 3. one token: its top_k pairs meet top_k different experts with one activation row each, which is the
    //    streaming kernel's case (Grok-1-sized experts, Q8_0, top 2: 315 -> 227 us, the three products at 6.3 TB/s;
    //    from two tokens on pairs share experts and the matrix-core kernel, which reads an expert once, wins)
    const bool one_token = T == 1;
    const bool up_stream = narrow || one_token || d / 32 < PG_MM_MIN_BLOCKS, down_stream = narrow || one_token || ffn / 32 < PG_MM_MIN_BLOCKS;
    PG_CHECK_ARG(!(up_stream || down_stream) || P <= 65535, "pg_moe_ffn: too many pairs for experts this small");

    // Arena layout.
    const int ks_up = up_stream ? 1 : pg_gguf_mm_splitk(ctx, ffn, d, E, T, true, nullptr);
    const int ks_down = down_stream ? 1 : pg_gguf_mm_splitk(ctx, d, ffn, E, P, true, nullptr);
    const size_t part_floats = std::max(ks_up > 1 ? (size_t)ks_up * P * ffn : 0, ks_down > 1 ? (size_t)ks_down * P * d : 0);
    const size_t sz_idx = pg_round_up(P * sizeof(int), 256);
    const size_t sz_p = pg_round_up(P * sizeof(float), 256);
    const size_t sz_lists = pg_round_up(E * T * sizeof(int), 256), sz_counts = pg_round_up(E * sizeof(int), 256);
    const size_t sz_act = pg_round_up(P * ffn * sizeof(float), 256);
    const size_t sz_y = pg_round_up(P * d * sizeof(float), 256);
    const size_t sz_part = pg_round_up(part_floats * sizeof(float), 256);
    const size_t sz_xd = up_stream ? pg_xdigits_bytes(T, d) : pg_mmdigits_bytes(T, d);
    const size_t sz_hd = down_stream ? pg_xdigits_bytes(P, ffn) : pg_mmdigits_bytes(P, ffn);
    void *ws = nullptr;
    PG_TRY(pg_workspace(ctx, sz_idx + sz_p + sz_lists + sz_counts + 3 * sz_act + sz_y + sz_part + sz_xd + sz_hd, &ws));
    char *p = static_cast<char *>(ws);
    int *topk_idx = reinterpret_cast<int *>(p); p += sz_idx;
    float *topk_p = reinterpret_cast<float *>(p); p += sz_p;
    int *lists = reinterpret_cast<int *>(p); p += sz_lists;
    int *counts = reinterpret_cast<int *>(p); p += sz_counts;
    float *g = reinterpret_cast<float *>(p); p += sz_act;
    float *u = reinterpret_cast<float *>(p); p += sz_act;
    float *h = reinterpret_cast<float *>(p); p += sz_act;
    float *yb = reinterpret_cast<float *>(p); p += sz_y;
    float *part = sz_part ? reinterpret_cast<float *>(p) : nullptr; p += sz_part;
    char *xd_base = p; p += sz_xd;
    char *hd_base = p;

    // Expert pointer tables: [gate qs | gate d | up qs | up d | down qs | down d], E each, in a
    // device buffer kept with the context, one per distinct set of experts (a model's layers
    // alternate); uploaded (blocking: the source is this stack frame) only on a set's first use.
    // The quant planes are the tile-major copies (made on an expert's first use) for the
    // matrix-core kernel, the row-major planes for the streaming one.
    const void *host_tab[6 * MAX_EXPERTS];
    for (size_t e = 0; e < E; ++e) {
        if (!up_stream) {
            PG_TRY(pg_gguf_ensure_tiled(ctx, gate[e]));
            PG_TRY(pg_gguf_ensure_tiled(ctx, up[e]));
        }
        if (!down_stream) PG_TRY(pg_gguf_ensure_tiled(ctx, down[e]));
        host_tab[0 * E + e] = up_stream ? gate[e]->qs : gate[e]->qs_tiled; host_tab[1 * E + e] = gate[e]->d;
        host_tab[2 * E + e] = up_stream ? up[e]->qs : up[e]->qs_tiled;     host_tab[3 * E + e] = up[e]->d;
        host_tab[4 * E + e] = down_stream ? down[e]->qs : down[e]->qs_tiled; host_tab[5 * E + e] = down[e]->d;
    }
    const void **tab = nullptr;
    PG_TRY(pg_moe_cached_table(ctx, host_tab, 6 * E, &tab));

    PG_TRY(pg_launch_moe_routing(ctx, router_logits_dev, idx_dev, weight_dev, T, E, top_k, topk_idx, topk_p, lists, counts));
    auto table = [&](int which) { return reinterpret_cast<const uint8_t *const *>(tab + which * E); };
    auto dtable = [&](int which) { return reinterpret_cast<const uint16_t *const *>(tab + which * E); };
    // Each token reaches an expert at most once, so an expert owns at most T pairs.
    const int tiles = (int)((T + 31) / 32);
    if (up_stream) {  // pair p: activation row p / top_k against expert topk_idx[p]
        const pg_xdigits xd = pg_xdigits_carve(xd_base, T, d);
        PG_TRY(pg_launch_x_to_digits(ctx, x_dev, T, d, type, xd));
        const pg_gemv_batch bg = {(int)P, table(0), dtable(1), topk_idx, (int)top_k};
        PG_TRY(pg_launch_gguf_gemv(ctx, type, ffn, d, nullptr, nullptr, bg, xd, g));
        const pg_gemv_batch bu = {(int)P, table(2), dtable(3), topk_idx, (int)top_k};
        PG_TRY(pg_launch_gguf_gemv(ctx, type, ffn, d, nullptr, nullptr, bu, xd, u));
    } else {
        const pg_mmdigits xd = pg_mmdigits_carve(xd_base, T, d);
        PG_TRY(pg_launch_x_to_mm_digits(ctx, x_dev, T, d, type, xd));
        const pg_mm_group gg = {(int)E, table(0), dtable(1), lists, counts, (int)T, tiles, (int)T, (int)top_k, 0, 0, 1};
        PG_TRY(pg_launch_gguf_mm(ctx, type, ffn, d, nullptr, nullptr, gg, P, xd, g, part));
        const pg_mm_group gu = {(int)E, table(2), dtable(3), lists, counts, (int)T, tiles, (int)T, (int)top_k, 0, 0, 1};
        PG_TRY(pg_launch_gguf_mm(ctx, type, ffn, d, nullptr, nullptr, gu, P, xd, u, part));
    }
    PG_TRY(pg_launch(ctx, "moe_act_mul", act_mul_kernel, dim3(grid_for(P * ffn, 256)), dim3(256), 0, g, u, P * ffn,
                     act, h));
    if (down_stream) {
        const pg_xdigits hd = pg_xdigits_carve(hd_base, P, ffn);
        PG_TRY(pg_launch_x_to_digits(ctx, h, P, ffn, type, hd));
        const pg_gemv_batch bd = {(int)P, table(4), dtable(5), topk_idx, 1};
        PG_TRY(pg_launch_gguf_gemv(ctx, type, d, ffn, nullptr, nullptr, bd, hd, yb));
    } else {
        const pg_mmdigits hd = pg_mmdigits_carve(hd_base, P, ffn);
        PG_TRY(pg_launch_x_to_mm_digits(ctx, h, P, ffn, type, hd));
        const pg_mm_group gd = {(int)E, table(4), dtable(5), lists, counts, (int)T, tiles, (int)T, 1, 0, 0, 1};
        PG_TRY(pg_launch_gguf_mm(ctx, type, d, ffn, nullptr, nullptr, gd, P, hd, yb, part));
    }
    return pg_launch(ctx, "moe_combine", combine_kernel, dim3(grid_for(T * d, 256)), dim3(256), 0, yb, topk_p, (int)T,
                     (int)d, (int)top_k, shared_dev, out_dev);
}

PG_API pg_status pg_moe_ffn_dev(pg_ctx *ctx, const float *x_dev, size_t T,
                                const float *router_logits_dev, size_t E, size_t top_k,
                                const pg_gguf_tensor *const *gate, const pg_gguf_tensor *const *up,
                                const pg_gguf_tensor *const *down, int act, float *out_dev) {
    PG_CHECK_ARG(T == 0 || router_logits_dev, "pg_moe_ffn: null router logits");
    return moe_ffn_core(ctx, x_dev, T, router_logits_dev, nullptr, nullptr, E, top_k, gate, up, down, act, nullptr, out_dev);
}

PG_API pg_status pg_moe_ffn_routed_dev(pg_ctx *ctx, const float *x_dev, size_t T, const int32_t *expert_idx_dev,
                                       const float *weight_dev, size_t E, size_t top_k,
                                       const pg_gguf_tensor *const *gate, const pg_gguf_tensor *const *up,
                                       const pg_gguf_tensor *const *down, int act, const float *shared_dev, float *out_dev) {
    PG_CHECK_ARG(T == 0 || (expert_idx_dev && weight_dev), "pg_moe_ffn_routed: null routing");
    return moe_ffn_core(ctx, x_dev, T, nullptr, expert_idx_dev, weight_dev, E, top_k, gate, up, down, act, shared_dev, out_dev);
}

PG_API pg_status pg_moe_ffn_routed(pg_ctx *ctx, const float *x, size_t T, const int32_t *expert_idx, const float *weight,
                                   size_t E, size_t top_k, const pg_gguf_tensor *const *gate,
                                   const pg_gguf_tensor *const *up, const pg_gguf_tensor *const *down, int act,
                                   const float *shared, float *out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(gate && gate[0], "pg_moe_ffn_routed: null expert table");
    if (T == 0) return PG_OK;
    PG_CHECK_ARG(x && expert_idx && weight && out, "pg_moe_ffn_routed: null pointer");
    PG_CHECK_ARG(E >= 1 && E <= MAX_EXPERTS && top_k >= 1 && top_k <= E, "pg_moe_ffn_routed: top_k %zu of %zu experts", top_k, E);
    // the reference indexes self.experts[expert_idx] and would panic on an index out of range; a token's experts are
    // distinct in every gate on this path (the grouped products rely on it)
    for (size_t t = 0; t < T; ++t)
        for (size_t k = 0; k < top_k; ++k) {
            const int32_t e = expert_idx[t * top_k + k];
            PG_CHECK_ARG(e >= 0 && (size_t)e < E, "pg_moe_ffn_routed: token %zu names expert %d of %zu", t, (int)e, E);
            for (size_t j = 0; j < k; ++j)
                PG_CHECK_ARG(expert_idx[t * top_k + j] != e, "pg_moe_ffn_routed: token %zu names expert %d twice", t, (int)e);
        }
    const size_t d = gate[0]->k_in, P = T * top_k;
    pg_tmp dx, di, dw, dsh, dout;
    PG_TRY(dx.alloc(T * d * sizeof(float)));
    PG_TRY(di.alloc(P * sizeof(int32_t)));
    PG_TRY(dw.alloc(P * sizeof(float)));
    PG_TRY(dout.alloc(T * d * sizeof(float)));
    if (shared) PG_TRY(dsh.alloc(T * d * sizeof(float)));
    PG_HIP(hipMemcpyAsync(dx.p, x, T * d * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipMemcpyAsync(di.p, expert_idx, P * sizeof(int32_t), hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipMemcpyAsync(dw.p, weight, P * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    if (shared) PG_HIP(hipMemcpyAsync(dsh.p, shared, T * d * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_moe_ffn_routed_dev(ctx, dx.as<float>(), T, di.as<int32_t>(), dw.as<float>(), E, top_k, gate, up, down, act,
                                 shared ? dsh.as<float>() : nullptr, dout.as<float>()));
    PG_HIP(hipMemcpyAsync(out, dout.p, T * d * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

PG_API pg_status pg_moe_ffn(pg_ctx *ctx, const float *x, size_t T, const float *router_logits,
                            size_t E, size_t top_k, const pg_gguf_tensor *const *gate,
                            const pg_gguf_tensor *const *up, const pg_gguf_tensor *const *down,
                            int act, float *out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(gate && gate[0], "pg_moe_ffn: null expert table");
    if (T == 0) return PG_OK;
    PG_CHECK_ARG(x && router_logits && out, "pg_moe_ffn: null pointer");
    const size_t d = gate[0]->k_in;
    pg_tmp dx, dl, dout;
    PG_TRY(dx.alloc(T * d * sizeof(float)));
    PG_TRY(dl.alloc(T * E * sizeof(float)));
    PG_TRY(dout.alloc(T * d * sizeof(float)));
    PG_HIP(hipMemcpyAsync(dx.p, x, T * d * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipMemcpyAsync(dl.p, router_logits, T * E * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_moe_ffn_dev(ctx, dx.as<float>(), T, dl.as<float>(), E, top_k, gate, up, down, act, dout.as<float>()));
    PG_HIP(hipMemcpyAsync(out, dout.p, T * d * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}
