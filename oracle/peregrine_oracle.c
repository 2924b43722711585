/*
 * peregrine_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A scalar, single-threaded CPU restatement of the arithmetic of peregrine's
 * quantized-inference path (the non-aarch64 / non-macOS branches), written
 * from the reference's source text.  Only tests, the smoke check and the
 * CPU-baseline leg of the benchmark may load this file's shared object; the
 * HIP library never links or calls it.
 *
 * Compile WITHOUT floating-point contraction and WITHOUT fast-math
 * (see oracle/Makefile: -O2 -ffp-contract=off -fno-fast-math): Rust never
 * contracts a*b+c into an FMA and never reassociates.
 *
 * Language-semantics pins used throughout (Rust -> C):
 *   f32::round           == roundf            (half away from zero)
 *   f32::max(a, b)       == fmaxf             (returns the non-NaN operand)
 *   f32::clamp(lo, hi)   keeps NaN as NaN
 *   `as i8` from f32     saturates, NaN -> 0
 *   `as f32` from i32    round-to-nearest-even (C cast does the same)
 *
 * Parity status of each function (what pins it) is listed in
 * tests/test_oracle_*.py; every function below is pinned by at least one of:
 * the reference's own known-answer tests, its golden fixture files, a closed
 * form, or an independent brute-force restatement in NumPy.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* Rust `f32 as i8`: saturating, NaN -> 0. */
static inline int8_t sat_i8(float v) {
    if (v != v) return 0;
    if (v <= -128.0f) return (int8_t)-128;
    if (v >= 127.0f) return (int8_t)127;
    return (int8_t)v; /* truncation toward zero, value already in range */
}

/* Rust `f32::clamp(-127.0, 127.0)`: NaN stays NaN. */
static inline float clamp127(float v) {
    if (v != v) return v;
    if (v < -127.0f) return -127.0f;
    if (v > 127.0f) return 127.0f;
    return v;
}

/* ------------------------------------------------------------------------
 * quant::quantize_weights            reference: src/quant.rs:27-75
 *   w       [rows, cols] f32 row-major   (rows = K, cols = N)
 *   q       [rows, cols] i8
 *   q_t     [cols, rows] i8  (q_t[n*rows + k] = q[k*cols + n])
 *   scales  [cols]
 * ---------------------------------------------------------------------- */
ORC_API void orc_quantize_weights(const float *w, size_t rows, size_t cols,
                                  int8_t *q, int8_t *q_t, float *scales) {
    /* per-column absmax with a strict `>` compare: NaN never wins (quant.rs:31-39) */
    for (size_t n = 0; n < cols; ++n) scales[n] = 0.0f;
    for (size_t m = 0; m < rows; ++m)
        for (size_t n = 0; n < cols; ++n) {
            float v = fabsf(w[m * cols + n]);
            if (v > scales[n]) scales[n] = v;
        }
    /* scale = amax / 127, or 1.0 for an all-zero column (quant.rs:42-45) */
    for (size_t n = 0; n < cols; ++n)
        scales[n] = (scales[n] == 0.0f) ? 1.0f : scales[n] / 127.0f;
    /* q = round(w / scale) with a true divide (quant.rs:48-54) */
    for (size_t m = 0; m < rows; ++m)
        for (size_t n = 0; n < cols; ++n) {
            float v = w[m * cols + n] / scales[n];
            q[m * cols + n] = sat_i8(clamp127(roundf(v)));
        }
    /* transpose for the GEMM (quant.rs:57-62) */
    if (q_t)
        for (size_t k = 0; k < rows; ++k)
            for (size_t n = 0; n < cols; ++n) q_t[n * rows + k] = q[k * cols + n];
}

/* ------------------------------------------------------------------------
 * quant::quantize_activations        reference: src/quant.rs:79-112
 *   (the cfg(not(target_arch = "aarch64")) branch, quant.rs:97-109)
 *   a [rows, cols] f32 -> q [rows, cols] i8, row_scales [rows]
 * ---------------------------------------------------------------------- */
ORC_API void orc_quantize_activations(const float *a, size_t rows, size_t cols,
                                      int8_t *q, float *row_scales) {
    for (size_t m = 0; m < rows; ++m) {
        const float *row = a + m * cols;
        float amax = 0.0f;
        for (size_t k = 0; k < cols; ++k) amax = fmaxf(amax, fabsf(row[k]));
        float scale = (amax == 0.0f) ? 1.0f : amax / 127.0f;
        row_scales[m] = scale;
        float inv_scale = 1.0f / scale; /* multiply by reciprocal, not a divide */
        for (size_t k = 0; k < cols; ++k)
            q[m * cols + k] = sat_i8(clamp127(roundf(row[k] * inv_scale)));
    }
}

/* quant::dequantize                  reference: src/quant.rs:115-123 */
ORC_API void orc_dequantize(const int8_t *q, const float *scales, size_t rows,
                            size_t cols, float *out) {
    for (size_t m = 0; m < rows; ++m)
        for (size_t n = 0; n < cols; ++n)
            out[m * cols + n] = (float)q[m * cols + n] * scales[n];
}

/* ------------------------------------------------------------------------
 * The i8 x i8 -> i32 GEMM with f32 rescale of quant::matmul_quantized
 *                                    reference: src/quant.rs:154-166
 *   a_i8 [m, k], b_t [n, k] (the pre-transposed weights), out [m, n].
 *   acc_out (optional) receives the raw i32 accumulators.
 *   Epilogue order is ((acc as f32) * a_scale[m]) * w_scale[n].
 * ---------------------------------------------------------------------- */
ORC_API void orc_gemm_i8(const int8_t *a_i8, const float *a_scales,
                         const int8_t *b_t, const float *w_scales, size_t m,
                         size_t n, size_t k, float *out, int32_t *acc_out) {
    for (size_t mi = 0; mi < m; ++mi)
        for (size_t ni = 0; ni < n; ++ni) {
            int32_t acc = 0;
            const int8_t *ar = a_i8 + mi * k;
            const int8_t *br = b_t + ni * k;
            for (size_t ki = 0; ki < k; ++ki) acc += (int32_t)ar[ki] * (int32_t)br[ki];
            if (acc_out) acc_out[mi * n + ni] = acc;
            if (out) out[mi * n + ni] = (float)acc * a_scales[mi] * w_scales[ni];
        }
}

/* quant::matmul_quantized            reference: src/quant.rs:129-169
 *   a [m, k] f32; weights given as (q_t [n, k], w_scales [n]).
 *   Returns 0, or -1 if scratch allocation failed. */
ORC_API int orc_matmul_quantized(const float *a, size_t m, size_t k,
                                 const int8_t *q_t, const float *w_scales,
                                 size_t n, float *out, int32_t *acc_out) {
    int8_t *a_i8 = (int8_t *)malloc((m * k) > 0 ? m * k : 1);
    float *a_sc = (float *)malloc((m ? m : 1) * sizeof(float));
    if (!a_i8 || !a_sc) { free(a_i8); free(a_sc); return -1; }
    orc_quantize_activations(a, m, k, a_i8, a_sc);
    orc_gemm_i8(a_i8, a_sc, q_t, w_scales, m, n, k, out, acc_out);
    free(a_i8);
    free(a_sc);
    return 0;
}

/* Metal kernel matmul_dequant_i8     reference: src/metal/shaders.rs:2329-2375
 *   (the numerics behind quant::matmul_quantized_gpu, src/quant.rs:196-218)
 *   a [m, k] f32; q [k, n] i8 row-major; scales [n]; out [m, n].
 *   Per output: w = (float)q * scale (one rounding), sum += a * w for k ascending,
 *   multiply and add rounded separately (tiles of 16 do not change the order).
 *   Pinned by equality with orc_matmul_f32(a, orc_dequantize(q)), whose two halves
 *   are pinned on their own. */
ORC_API void orc_matmul_dequant_i8(const float *a, size_t m, size_t k, const int8_t *q,
                                   const float *scales, size_t n, float *out) {
    for (size_t mi = 0; mi < m; ++mi)
        for (size_t ni = 0; ni < n; ++ni) {
            const float w_scale = scales[ni];
            float sum = 0.0f;
            for (size_t ki = 0; ki < k; ++ki) {
                const float w = (float)q[ki * n + ni] * w_scale;
                const float prod = a[mi * k + ki] * w;
                sum = sum + prod;
            }
            out[mi * n + ni] = sum;
        }
}

/* ------------------------------------------------------------------------
 * gguf::f16_to_f32                   reference: src/gguf.rs:354-382
 *   Bit-level IEEE half -> single, including the subnormal normalise loop
 *   and NaN payload = mant << 13 (signalling NaNs are NOT quietened).
 * ---------------------------------------------------------------------- */
ORC_API uint32_t orc_f16_to_f32_bits(uint16_t bits) {
    uint32_t sign = (bits >> 15) & 1u;
    uint32_t exp = (bits >> 10) & 0x1Fu;
    uint32_t mant = bits & 0x3FFu;
    if (exp == 0) {
        if (mant == 0) return sign << 31;
        uint32_t m = mant;
        int32_t e = 0;
        while ((m & 0x400u) == 0) { m <<= 1; e -= 1; }
        m &= 0x3FFu;
        uint32_t f32_exp = (uint32_t)(127 - 15 + 1 + e);
        return (sign << 31) | (f32_exp << 23) | (m << 13);
    }
    if (exp == 31) return (sign << 31) | (0xFFu << 23) | (mant << 13);
    return (sign << 31) | ((exp + 127 - 15) << 23) | (mant << 13);
}

static inline float f16_to_f32(uint16_t bits) {
    uint32_t u = orc_f16_to_f32_bits(bits);
    float f;
    memcpy(&f, &u, 4);
    return f;
}

ORC_API float orc_f16_to_f32(uint16_t bits) { return f16_to_f32(bits); }

/* gguf::dequant_q8_0                 reference: src/gguf.rs:286-302
 *   block = [f16 d, little-endian][32 x i8]; out[32b+i] = (q as f32) * d.
 *   Returns 0, or -1 if n is not a multiple of 32 (the reference asserts). */
ORC_API int orc_dequant_q8_0(const uint8_t *data, size_t n, float *out) {
    if (n % 32) return -1;
    size_t nb = n / 32;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t *blk = data + b * 34;
        float d = f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        for (int i = 0; i < 32; ++i) out[b * 32 + i] = (float)(int8_t)blk[2 + i] * d;
    }
    return 0;
}

/* gguf::dequant_q4_0                 reference: src/gguf.rs:307-326
 *   block = [f16 d][16 bytes]; byte i -> out[32b+2i]   = ((byte & 15) - 8) * d
 *                                        out[32b+2i+1] = ((byte >> 4) - 8) * d
 *   (interleaved element order, as the reference has it). */
ORC_API int orc_dequant_q4_0(const uint8_t *data, size_t n, float *out) {
    if (n % 32) return -1;
    size_t nb = n / 32;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t *blk = data + b * 18;
        float d = f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        for (int i = 0; i < 16; ++i) {
            int32_t lo = (int32_t)(blk[2 + i] & 0x0F) - 8;
            int32_t hi = (int32_t)((blk[2 + i] >> 4) & 0x0F) - 8;
            out[b * 32 + 2 * i] = (float)lo * d;
            out[b * 32 + 2 * i + 1] = (float)hi * d;
        }
    }
    return 0;
}

/* gguf::dequant_q4_1                 reference: src/gguf.rs:331-351
 *   block = [f16 d][f16 m][16 bytes]; value = nibble * d + m (mul then add). */
ORC_API int orc_dequant_q4_1(const uint8_t *data, size_t n, float *out) {
    if (n % 32) return -1;
    size_t nb = n / 32;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t *blk = data + b * 20;
        float d = f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        float mn = f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
        for (int i = 0; i < 16; ++i) {
            float lo = (float)(blk[4 + i] & 0x0F);
            float hi = (float)((blk[4 + i] >> 4) & 0x0F);
            out[b * 32 + 2 * i] = lo * d + mn;
            out[b * 32 + 2 * i + 1] = hi * d + mn;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------
 * Tensor::matmul, non-macOS branch   reference: src/tensor.rs:1342-1353
 *   a [m, k] . b [k, n] -> out [m, n]; sum starts at 0, `sum += a*b`
 *   K-sequential, separate multiply and add.
 * ---------------------------------------------------------------------- */
ORC_API void orc_matmul_f32(const float *a, const float *b, size_t m, size_t k,
                            size_t n, float *out) {
    for (size_t i = 0; i < m; ++i)
        for (size_t j = 0; j < n; ++j) {
            float sum = 0.0f;
            for (size_t p = 0; p < k; ++p) sum += a[i * k + p] * b[p * n + j];
            out[i * n + j] = sum;
        }
}

/* Same sums as orc_matmul_f32 when b is given transposed (bt [n, k]):
 * identical operands in identical order, only the memory walk differs, so
 * results are bit-identical.  Used to make full-size checks tractable. */
static void matmul_f32_bt(const float *a, const float *bt, size_t m, size_t k,
                          size_t n, float *out) {
    for (size_t i = 0; i < m; ++i)
        for (size_t j = 0; j < n; ++j) {
            float sum = 0.0f;
            const float *ar = a + i * k, *br = bt + j * k;
            for (size_t p = 0; p < k; ++p) sum += ar[p] * br[p];
            out[i * n + j] = sum;
        }
}

/* ------------------------------------------------------------------------
 * GGUF dequant-matmul as models::llama composes it:
 *   load_tensor_f32 (gguf.rs:485-517) -> dequant_q8_0 / dequant_q4_0 of the
 *   whole [n_out, k_in] tensor, transpose to [k_in, n_out]
 *   (models/llama/model.rs:243-257), then x.matmul(w) (tensor.rs:1342-1353).
 *   ggml_type: 2 = Q4_0, 3 = Q4_1, 8 = Q8_0 (gguf.rs:30-45 numbering).
 *   y [m, n_out].  Returns 0 on success.
 * ---------------------------------------------------------------------- */
ORC_API int orc_gguf_matmul(const float *x, size_t m, const uint8_t *blocks,
                            int ggml_type, size_t n_out, size_t k_in, float *y) {
    float *wf = (float *)malloc(n_out * k_in * sizeof(float) + 4);
    if (!wf) return -1;
    int rc;
    if (ggml_type == 8) rc = orc_dequant_q8_0(blocks, n_out * k_in, wf);
    else if (ggml_type == 2) rc = orc_dequant_q4_0(blocks, n_out * k_in, wf);
    else if (ggml_type == 3) rc = orc_dequant_q4_1(blocks, n_out * k_in, wf);
    else rc = -2;
    if (rc == 0) matmul_f32_bt(x, wf, m, k_in, n_out, y); /* wf is [n_out, k_in] = b^T */
    free(wf);
    return rc;
}

/* Tensor::softmax over the last dim, non-aarch64 branch
 *                                    reference: src/tensor.rs:2833-2858 */
ORC_API void orc_softmax_rows(const float *x, size_t rows, size_t cols, float *out) {
    for (size_t r = 0; r < rows; ++r) {
        const float *xi = x + r * cols;
        float *oi = out + r * cols;
        float mx = -INFINITY;
        for (size_t d = 0; d < cols; ++d)
            if (xi[d] > mx) mx = xi[d];
        float sum = 0.0f;
        for (size_t d = 0; d < cols; ++d) {
            float e = expf(xi[d] - mx);
            oi[d] = e;
            sum += e;
        }
        for (size_t d = 0; d < cols; ++d) oi[d] /= sum;
    }
}

/* Tensor::silu, non-aarch64          reference: src/tensor.rs:6129-6133 */
static inline float silu_tensor(float x) {
    float sig = 1.0f / (1.0f + expf(-x));
    return x * sig;
}
/* Llama SwiGLU glue, non-macOS       reference: src/models/llama/decoder.rs:143-150 */
static inline float silu_llama(float g) { return g / (1.0f + expf(-g)); }
/* Tensor::gelu, non-aarch64 (tanh form) reference: src/tensor.rs:3163-3179 */
static inline float gelu_tanh(float x) {
    float c = sqrtf(2.0f / 3.14159265358979323846f);
    float inner = c * (x + 0.044715f * x * x * x);
    return 0.5f * x * (1.0f + tanhf(inner));
}

ORC_API void orc_silu(const float *x, size_t n, float *out) {
    for (size_t i = 0; i < n; ++i) out[i] = silu_tensor(x[i]);
}
ORC_API void orc_gelu_tanh(const float *x, size_t n, float *out) {
    for (size_t i = 0; i < n; ++i) out[i] = gelu_tanh(x[i]);
}
ORC_API void orc_swiglu_llama(const float *g, const float *u, size_t n, float *out) {
    for (size_t i = 0; i < n; ++i) out[i] = silu_llama(g[i]) * u[i];
}

/* ------------------------------------------------------------------------
 * MoE layer forward with block-quantised experts.
 *   Routing and accumulation: examples/grok1/moe.rs:70-109
 *     probs = softmax(logits) per token; stable sort descending by prob
 *     (ties keep the lower expert index first); for k < top_k:
 *     out[t] += prob * expert(x[t]), in k order, raw (unrenormalised) probs.
 *   Expert:  act(x.Wg) * (x.Wu) . Wd
 *     act = 0: Tensor::silu  (examples/deepseek/moe.rs:55-59)
 *     act = 1: Tensor::gelu  (examples/grok1/moe.rs:27-34)
 *   Each expert matrix is GGUF block data in [out, in] orientation and goes
 *   through the dequant -> transpose -> f32 matmul composition above.
 *     gate[e], up[e]: n_out = ffn, k_in = d;   down[e]: n_out = d, k_in = ffn
 *   x [T, d], logits [T, E], out [T, d].  Returns 0 on success.
 *   topk_idx / topk_prob (optional, [T, top_k]) receive the routing.
 * ---------------------------------------------------------------------- */
ORC_API int orc_moe_ffn(const float *x, size_t T, size_t d, size_t ffn, size_t E,
                        size_t top_k, const float *logits,
                        const uint8_t *const *gate, const uint8_t *const *up,
                        const uint8_t *const *down, int ggml_type, int act,
                        float *out, int32_t *topk_idx, float *topk_prob) {
    if (top_k > E) return -3;
    float *probs = (float *)malloc(T * E * sizeof(float) + 4);
    float *g = (float *)malloc(ffn * sizeof(float));
    float *u = (float *)malloc(ffn * sizeof(float));
    float *h = (float *)malloc(ffn * sizeof(float));
    float *y = (float *)malloc(d * sizeof(float));
    size_t *order = (size_t *)malloc((E ? E : 1) * sizeof(size_t));
    int rc = 0;
    if (!probs || !g || !u || !h || !y || !order) { rc = -1; goto done; }
    orc_softmax_rows(logits, T, E, probs);
    memset(out, 0, T * d * sizeof(float));
    for (size_t t = 0; t < T; ++t) {
        const float *p = probs + t * E;
        /* stable insertion sort, descending: equal probs keep index order */
        for (size_t e = 0; e < E; ++e) {
            size_t j = e;
            while (j > 0 && p[order[j - 1]] < p[e]) { order[j] = order[j - 1]; --j; }
            order[j] = e;
        }
        const float *xt = x + t * d;
        for (size_t k = 0; k < top_k; ++k) {
            size_t e = order[k];
            float prob = p[e];
            if (topk_idx) topk_idx[t * top_k + k] = (int32_t)e;
            if (topk_prob) topk_prob[t * top_k + k] = prob;
            if ((rc = orc_gguf_matmul(xt, 1, gate[e], ggml_type, ffn, d, g))) goto done;
            if ((rc = orc_gguf_matmul(xt, 1, up[e], ggml_type, ffn, d, u))) goto done;
            for (size_t i = 0; i < ffn; ++i)
                h[i] = (act == 1 ? gelu_tanh(g[i]) : silu_tensor(g[i])) * u[i];
            if ((rc = orc_gguf_matmul(h, 1, down[e], ggml_type, d, ffn, y))) goto done;
            for (size_t i = 0; i < d; ++i) out[t * d + i] += prob * y[i];
        }
    }
done:
    free(probs); free(g); free(u); free(h); free(y); free(order);
    return rc;
}

/* ------------------------------------------------------------------------
 * The deepseek gate: which experts a token goes to and with what weights.
 *                                    reference: examples/deepseek/moe.rs:111-215
 *   scores[e] = x[t] . w[e]  (f32, d ascending); sigmoid per score, or the softmax of the row;
 *   the weights come from these scores; the SELECTION uses scores + bias (if any), after the
 *   experts of all but the topk_groups best groups are set to 0 (group score = the sum of the
 *   group's two largest biased scores when there is a bias, else its largest; stable
 *   descending order, ties keep the lower index); sigmoid weights are divided by their sum
 *   when that is > 0; all weights are multiplied by route_scale.
 *   x [T, dim], w [E, dim], bias [E] or NULL; idx / weight [T, topk].  Returns 0 on success.
 * ---------------------------------------------------------------------- */
static void stable_order_desc(const float *v, size_t n, size_t *order) {
    for (size_t e = 0; e < n; ++e) {   /* insertion sort: an element only passes strictly smaller ones */
        size_t j = e;
        while (j > 0 && v[order[j - 1]] < v[e]) { order[j] = order[j - 1]; --j; }
        order[j] = e;
    }
}

ORC_API int orc_deepseek_gate(const float *x, size_t T, size_t dim, const float *w, const float *bias,
                              size_t E, size_t topk, size_t n_groups, size_t topk_groups, float route_scale,
                              int use_sigmoid, int32_t *idx, float *weight) {
    if (topk > E || n_groups == 0 || E % n_groups != 0 || topk_groups > n_groups) return -3;
    float *scores = (float *)malloc(E * sizeof(float)), *orig = (float *)malloc(E * sizeof(float));
    float *gs = (float *)malloc(n_groups * sizeof(float)), *gv = (float *)malloc(E * sizeof(float));
    size_t *order = (size_t *)malloc(E * sizeof(size_t)), *gorder = (size_t *)malloc(n_groups * sizeof(size_t));
    if (!scores || !orig || !gs || !gv || !order || !gorder) { free(scores); free(orig); free(gs); free(gv); free(order); free(gorder); return -1; }
    for (size_t t = 0; t < T; ++t) {
        for (size_t e = 0; e < E; ++e) {
            float dot = 0.0f;
            for (size_t d = 0; d < dim; ++d) dot += x[t * dim + d] * w[e * dim + d];
            scores[e] = use_sigmoid ? 1.0f / (1.0f + expf(-dot)) : dot;
        }
        if (!use_sigmoid) {
            float mx = -INFINITY, sum = 0.0f;
            for (size_t e = 0; e < E; ++e) mx = fmaxf(mx, scores[e]);
            for (size_t e = 0; e < E; ++e) sum += expf(scores[e] - mx);
            for (size_t e = 0; e < E; ++e) scores[e] = expf(scores[e] - mx) / sum;
        }
        memcpy(orig, scores, E * sizeof(float));
        if (bias)
            for (size_t e = 0; e < E; ++e) scores[e] += bias[e];
        if (n_groups > 1) {
            const size_t per = E / n_groups;
            for (size_t g = 0; g < n_groups; ++g) {
                const float *grp = scores + g * per;
                stable_order_desc(grp, per, order);
                gs[g] = bias ? (per >= 2 ? 0.0f + grp[order[0]] + grp[order[1]] : 0.0f + grp[order[0]]) : grp[order[0]];
            }
            stable_order_desc(gs, n_groups, gorder);
            for (size_t g = 0; g < n_groups; ++g) {
                int selected = 0;
                for (size_t s = 0; s < topk_groups; ++s) selected |= gorder[s] == g;
                if (!selected)
                    for (size_t e = g * per; e < (g + 1) * per; ++e) scores[e] = 0.0f;
            }
        }
        stable_order_desc(scores, E, order);
        float sum = 0.0f;
        for (size_t k = 0; k < topk; ++k) {
            idx[t * topk + k] = (int32_t)order[k];
            weight[t * topk + k] = orig[order[k]];
            sum += orig[order[k]];
        }
        if (use_sigmoid && sum > 0.0f)
            for (size_t k = 0; k < topk; ++k) weight[t * topk + k] /= sum;
        for (size_t k = 0; k < topk; ++k) weight[t * topk + k] *= route_scale;
    }
    free(scores); free(orig); free(gs); free(gv); free(order); free(gorder);
    return 0;
}

/* ------------------------------------------------------------------------
 * The gpt_oss router: top-k on the biased logits, then a softmax over those k.
 *                                    reference: examples/gpt_oss/moe.rs:298-330
 *   logits [T, E] (= x . gate), gate_bias [E]; idx / weight [T, topk].
 * ---------------------------------------------------------------------- */
ORC_API int orc_gpt_oss_route(const float *logits, const float *gate_bias, size_t T, size_t E, size_t topk,
                              int32_t *idx, float *weight) {
    if (topk > E) return -3;
    float *tl = (float *)malloc(E * sizeof(float));
    size_t *order = (size_t *)malloc(E * sizeof(size_t));
    if (!tl || !order) { free(tl); free(order); return -1; }
    for (size_t t = 0; t < T; ++t) {
        for (size_t e = 0; e < E; ++e) tl[e] = logits[t * E + e] + gate_bias[e];
        stable_order_desc(tl, E, order);
        float mx = -INFINITY, sum = 0.0f;
        for (size_t k = 0; k < topk; ++k) mx = fmaxf(mx, tl[order[k]]);
        for (size_t k = 0; k < topk; ++k) sum += expf(tl[order[k]] - mx);
        for (size_t k = 0; k < topk; ++k) {
            idx[t * topk + k] = (int32_t)order[k];
            weight[t * topk + k] = expf(tl[order[k]] - mx) / sum;
        }
    }
    free(tl); free(order);
    return 0;
}

/* ------------------------------------------------------------------------
 * Expert FFN over a routing that is given: out[t] = sum_k weight[t, k] * expert_{idx[t, k]}(x[t]) in k order,
 * then + shared[t] if a shared-expert output is passed.
 *                                    reference: examples/deepseek/moe.rs:271-300 (y_data += weight * out; y.add(&z)),
 *                                               examples/gpt_oss/moe.rs:334-351
 *   Expert and operand layout as orc_moe_ffn.  shared [T, d] or NULL.
 * ---------------------------------------------------------------------- */
ORC_API int orc_moe_ffn_routed(const float *x, size_t T, size_t d, size_t ffn, size_t E, size_t top_k,
                               const int32_t *idx, const float *weight,
                               const uint8_t *const *gate, const uint8_t *const *up, const uint8_t *const *down,
                               int ggml_type, int act, const float *shared, float *out) {
    float *g = (float *)malloc(ffn * sizeof(float)), *u = (float *)malloc(ffn * sizeof(float));
    float *h = (float *)malloc(ffn * sizeof(float)), *y = (float *)malloc(d * sizeof(float));
    int rc = 0;
    if (!g || !u || !h || !y) { rc = -1; goto done; }
    memset(out, 0, T * d * sizeof(float));
    for (size_t t = 0; t < T; ++t) {
        const float *xt = x + t * d;
        for (size_t k = 0; k < top_k; ++k) {
            const int32_t e = idx[t * top_k + k];
            if (e < 0 || (size_t)e >= E) { rc = -3; goto done; }
            if ((rc = orc_gguf_matmul(xt, 1, gate[e], ggml_type, ffn, d, g))) goto done;
            if ((rc = orc_gguf_matmul(xt, 1, up[e], ggml_type, ffn, d, u))) goto done;
            for (size_t i = 0; i < ffn; ++i) h[i] = (act == 1 ? gelu_tanh(g[i]) : silu_tensor(g[i])) * u[i];
            if ((rc = orc_gguf_matmul(h, 1, down[e], ggml_type, d, ffn, y))) goto done;
            for (size_t i = 0; i < d; ++i) out[t * d + i] += weight[t * top_k + k] * y[i];
        }
        if (shared)
            for (size_t i = 0; i < d; ++i) out[t * d + i] = out[t * d + i] + shared[t * d + i];
    }
done:
    free(g); free(u); free(h); free(y);
    return rc;
}

/* ------------------------------------------------------------------------
 * Input synthesis: SplitMix64-seeded Xoshiro256++ and Box-Muller normals
 *                                    reference: src/random.rs:16-53, 311-380
 *   (the sequential generator; at 200 000 elements and more the reference
 *   switches to the counter-based Philox path restated further down).
 * ---------------------------------------------------------------------- */
typedef struct { uint64_t s[4]; } orc_rng;

static inline uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

ORC_API void orc_rng_seed(orc_rng *r, uint64_t seed) {
    uint64_t sm = seed;
    for (int i = 0; i < 4; ++i) {
        sm += 0x9E3779B97F4A7C15ull;
        uint64_t z = sm;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        r->s[i] = z ^ (z >> 31);
    }
}

ORC_API uint64_t orc_rng_next_u64(orc_rng *r) {
    uint64_t *s = r->s;
    uint64_t result = rotl64(s[0] + s[3], 23) + s[0];
    uint64_t t = s[1] << 17;
    s[2] ^= s[0];
    s[3] ^= s[1];
    s[1] ^= s[2];
    s[0] ^= s[3];
    s[2] ^= t;
    s[3] = rotl64(s[3], 45);
    return result;
}

static inline float rng_next_f32(orc_rng *r) {
    return (float)(orc_rng_next_u64(r) >> 40) / (float)(1ull << 24);
}

ORC_API void orc_rng_normal(uint64_t seed, size_t n, float mean, float std, float *out) {
    orc_rng r;
    orc_rng_seed(&r, seed);
    size_t pairs = (n + 1) / 2;
    /* the reference draws all (u1, u2) pairs first, then transforms them;
     * drawing pair by pair consumes the stream in the same order */
    for (size_t i = 0; i < pairs; ++i) {
        float u1 = fmaxf(rng_next_f32(&r), 1e-10f);
        float u2 = rng_next_f32(&r);
        float rad = sqrtf(-2.0f * logf(u1));
        float theta = 2.0f * 3.14159265358979323846f * u2;
        out[2 * i] = mean + std * rad * cosf(theta);
        if (2 * i + 1 < n) out[2 * i + 1] = mean + std * rad * sinf(theta);
    }
}

/* ------------------------------------------------------------------------
 * Input synthesis, large tensors: Philox 4x32-10 counter-based generator and
 * the normal() front end that chooses between the two generators
 *                         reference: src/random.rs:72-103, 147-270, 273-380
 * ---------------------------------------------------------------------- */
#define ORC_PHILOX_THRESHOLD 200000u /* src/random.rs:79 */

/* philox_4x32_10  src/random.rs:88-103 */
ORC_API void orc_philox_4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c[4] = {counter[0], counter[1], counter[2], counter[3]};
    uint32_t k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c[0], p1 = (uint64_t)0xCD9E8D57u * c[2];
        uint32_t lo0 = (uint32_t)p0, hi0 = (uint32_t)(p0 >> 32), lo1 = (uint32_t)p1, hi1 = (uint32_t)(p1 >> 32);
        uint32_t n0 = hi1 ^ c[1] ^ k0, n2 = hi0 ^ c[3] ^ k1;
        c[0] = n0; c[1] = lo1; c[2] = n2; c[3] = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c[0]; out[1] = c[1]; out[2] = c[2]; out[3] = c[3];
}

/* random::seed + the two pieces of global state  src/random.rs:11-14, 273-278 */
typedef struct { orc_rng xo; uint64_t philox_counter; } orc_random;

ORC_API void orc_random_seed(orc_random *st, uint64_t seed) {
    orc_rng_seed(&st->xo, seed);
    st->philox_counter = seed;
}

/* philox_normal_parallel  src/random.rs:147-270 (non-macOS transform :248-258) */
static void philox_normal(orc_random *st, size_t n, float mean, float std, float *out) {
    const size_t alloc_n = n + (n & 1), pairs = alloc_n / 2, calls = (pairs + 3) / 4;
    const uint64_t base = st->philox_counter;
    st->philox_counter += (uint64_t)calls * 2;
    const uint32_t key_u1[2] = {0xDEADBEEFu, 0xCAFEBABEu}, key_u2[2] = {0xFEEDFACEu, 0xBAADF00Du};
    const float scale = 1.0f / (float)(1ull << 32), two_pi = 2.0f * 3.14159265358979323846f;
    for (size_t call = 0; call < calls; ++call) {
        const uint64_t c1 = base + call, c2 = base + calls + call;
        const uint32_t ctr1[4] = {(uint32_t)c1, (uint32_t)(c1 >> 32), 0, 0}, ctr2[4] = {(uint32_t)c2, (uint32_t)(c2 >> 32), 0, 0};
        uint32_t o1[4], o2[4];
        orc_philox_4x32_10(ctr1, key_u1, o1);
        orc_philox_4x32_10(ctr2, key_u2, o2);
        for (size_t j = 0; j < 4 && 4 * call + j < pairs; ++j) {
            const size_t i = 4 * call + j;
            const float u1 = fmaxf((float)o1[j] * scale, 1e-10f), u2 = (float)o2[j] * scale;
            const float r = sqrtf(-2.0f * logf(u1)), theta = two_pi * u2;
            if (2 * i < n) out[2 * i] = mean + std * r * cosf(theta);
            if (2 * i + 1 < n) out[2 * i + 1] = mean + std * r * sinf(theta);
        }
    }
}

/* random::normal  src/random.rs:311-380 (non-macOS branch :364-378) */
ORC_API void orc_random_normal(orc_random *st, size_t n, float mean, float std, float *out) {
    if (n >= ORC_PHILOX_THRESHOLD) {
        philox_normal(st, n, mean, std, out);
        return;
    }
    const size_t pairs = (n + 1) / 2;
    for (size_t i = 0; i < pairs; ++i) {  /* pair by pair: the stream is consumed in the reference's order */
        const float u1 = fmaxf(rng_next_f32(&st->xo), 1e-10f), u2 = rng_next_f32(&st->xo);
        const float r = sqrtf(-2.0f * logf(u1)), theta = 2.0f * 3.14159265358979323846f * u2;
        out[2 * i] = mean + std * r * cosf(theta);
        if (2 * i + 1 < n) out[2 * i + 1] = mean + std * r * sinf(theta);
    }
}
