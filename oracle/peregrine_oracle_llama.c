/*
 * peregrine_oracle_llama.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of the glue around the quantised products in peregrine's Llama
 * decoder block (the non-aarch64 / non-macOS branches), written from the reference's
 * source text: RMSNorm, RoPE, the KV cache layout, grouped-query attention and the block
 * itself.  Linked into the same shared object as peregrine_oracle.c; same compile flags
 * (no contraction, no fast-math).  Only tests and the smoke check may load it.
 *
 * Parity status (tests/test_oracle_llama_pins.py): every function is pinned by closed
 * forms, by the reference's own attention tests restated (tests/attention.rs), or by an
 * independent NumPy float64 computation.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

int orc_gguf_matmul(const float *x, size_t m, const uint8_t *blocks, int ggml_type, size_t n_out, size_t k_in, float *y);

/* nn::RMSNorm::forward, inference path, non-aarch64   reference: src/nn.rs:638-649
 *   ss = sum of x*x left to right; inv_rms = 1 / sqrt(ss * (1/dim) + eps);
 *   out = (x * inv_rms) * w. */
ORC_API void orc_rmsnorm(const float *x, size_t rows, size_t dim, const float *w, float eps, float *out) {
    const float inv_dim = 1.0f / (float)dim;
    for (size_t v = 0; v < rows; ++v) {
        const float *xs = x + v * dim;
        float ss = 0.0f;
        for (size_t i = 0; i < dim; ++i) {
            const float sq = xs[i] * xs[i];
            ss = ss + sq;
        }
        const float inv_rms = 1.0f / sqrtf(ss * inv_dim + eps);
        for (size_t i = 0; i < dim; ++i) out[v * dim + i] = xs[i] * inv_rms * w[i];
    }
}

/* nn::RoPE::new                                     reference: src/nn.rs:1258-1282
 *   cos/sin [max_seq_len][head_dim]: theta = pos / base^(2i/head_dim) for i < head_dim/2,
 *   the half-row repeated. */
ORC_API void orc_rope_tables(size_t head_dim, size_t max_seq_len, float base, float *cos_t, float *sin_t) {
    const size_t half = head_dim / 2;
    for (size_t pos = 0; pos < max_seq_len; ++pos)
        for (size_t i = 0; i < half; ++i) {
            const float theta = (float)pos / powf(base, 2.0f * (float)i / (float)head_dim);
            const float c = cosf(theta), s = sinf(theta);
            cos_t[pos * head_dim + i] = c;
            cos_t[pos * head_dim + half + i] = c;
            sin_t[pos * head_dim + i] = s;
            sin_t[pos * head_dim + half + i] = s;
        }
}

/* nn::RoPE::apply_one                               reference: src/nn.rs:1322-1338 */
static void rope_one(const float *src, float *dst, const float *c, const float *s, size_t hd) {
    const size_t half = hd / 2;
    for (size_t i = 0; i < half; ++i) {
        const float x0 = src[i], x1 = src[half + i];
        dst[i] = x0 * c[i] - x1 * s[i];
    }
    for (size_t i = 0; i < half; ++i) {
        const float x0 = src[i], x1 = src[half + i];
        dst[half + i] = x0 * s[i] + x1 * c[i];
    }
}

/* nn::RoPE::apply: x [seq_len, head_dim] at positions offset..   reference: src/nn.rs:1286-1317 */
ORC_API void orc_rope_apply(const float *x, size_t seq_len, size_t head_dim, size_t offset, const float *cos_t,
                            const float *sin_t, float *out) {
    for (size_t t = 0; t < seq_len; ++t)
        rope_one(x + t * head_dim, out + t * head_dim, cos_t + (offset + t) * head_dim, sin_t + (offset + t) * head_dim, head_dim);
}

/* attention::is_masked                              reference: src/attention.rs:269-300
 *   mask_kind 0 None, 1 Causal{offset}, 2 CausalSlidingWindow{offset, window, sink_tokens},
 *   3 LocalGlobal{offset, local_window = window, global_positions = gpos[0..ngpos)}. */
static int is_masked(int mask_kind, size_t offset, size_t window, size_t sink, const size_t *gpos, size_t ngpos,
                     size_t qt, size_t kt) {
    if (mask_kind == 0) return 0;
    const size_t query_pos = offset + qt;
    if (kt > query_pos) return 1;
    if (mask_kind == 1) return 0;
    if (mask_kind == 3) {
        if (query_pos - kt <= window) return 0; /* saturating_sub: kt <= query_pos here */
        for (size_t i = 0; i < ngpos; ++i)
            if (gpos[i] == kt) return 0;        /* global_positions.contains(&kt) */
        return 1;
    }
    if (kt < sink) return 0;
    return query_pos - kt > window;
}

/* attention::gqa_attention_cpu, non-aarch64          reference: src/attention.rs:141-265
 *   q [num_q_heads, seq_q, head_dim]; k, v caches [num_kv_heads, capacity, head_dim] with
 *   `len` valid positions; out [seq_q, num_q_heads * head_dim], ACCUMULATED INTO (the
 *   reference adds into `output`; callers pass zeros).  logit_cap > 0 applies
 *   cap * tanh(score / cap) (PostScoreTransform::LogitCap), 0 = none. */
static void attention_masked(const float *q, const float *k, const float *v, size_t len, size_t capacity,
                             size_t num_q_heads, size_t num_kv_heads, size_t seq_q, size_t head_dim, float scale,
                             int mask_kind, size_t offset, size_t window, size_t sink, const size_t *gpos, size_t ngpos,
                             float logit_cap, float *out);

ORC_API void orc_gqa_attention(const float *q, const float *k, const float *v, size_t len, size_t capacity,
                               size_t num_q_heads, size_t num_kv_heads, size_t seq_q, size_t head_dim, float scale,
                               int mask_kind, size_t offset, size_t window, size_t sink, float logit_cap, float *out) {
    attention_masked(q, k, v, len, capacity, num_q_heads, num_kv_heads, seq_q, head_dim, scale, mask_kind, offset, window,
                     sink, NULL, 0, logit_cap, out);
}

/* The same with AttentionMask::LocalGlobal { offset, local_window, global_positions }
 *                                                   reference: src/attention.rs:115-119, 287-299 */
ORC_API void orc_gqa_attention_local_global(const float *q, const float *k, const float *v, size_t len, size_t capacity,
                                            size_t num_q_heads, size_t num_kv_heads, size_t seq_q, size_t head_dim,
                                            float scale, size_t offset, size_t local_window,
                                            const size_t *global_positions, size_t num_global, float logit_cap,
                                            float *out) {
    attention_masked(q, k, v, len, capacity, num_q_heads, num_kv_heads, seq_q, head_dim, scale, 3, offset, local_window, 0,
                     global_positions, num_global, logit_cap, out);
}

static void attention_masked(const float *q, const float *k, const float *v, size_t len, size_t capacity,
                             size_t num_q_heads, size_t num_kv_heads, size_t seq_q, size_t head_dim, float scale,
                             int mask_kind, size_t offset, size_t window, size_t sink, const size_t *gpos, size_t ngpos,
                             float logit_cap, float *out) {
    const size_t group = num_q_heads / num_kv_heads, stride = capacity * head_dim;
    float *scores = (float *)malloc((len ? len : 1) * sizeof(float));
    for (size_t qh = 0; qh < num_q_heads; ++qh) {
        const size_t kvh = qh / group;
        for (size_t qt = 0; qt < seq_q; ++qt) {
            const float *qs = q + qh * seq_q * head_dim + qt * head_dim;
            for (size_t kt = 0; kt < len; ++kt) {
                if (is_masked(mask_kind, offset, window, sink, gpos, ngpos, qt, kt)) {
                    scores[kt] = -INFINITY;
                } else {
                    const float *ks = k + kvh * stride + kt * head_dim;
                    float d = 0.0f;
                    for (size_t i = 0; i < head_dim; ++i) {
                        const float p = qs[i] * ks[i];
                        d = d + p;
                    }
                    float sc = d * scale;
                    if (logit_cap > 0.0f) sc = logit_cap * tanhf(sc / logit_cap);
                    scores[kt] = sc;
                }
            }
            float mx = -INFINITY;
            for (size_t kt = 0; kt < len; ++kt) mx = fmaxf(mx, scores[kt]);
            float exp_sum = 0.0f;
            for (size_t kt = 0; kt < len; ++kt) {
                scores[kt] = expf(scores[kt] - mx);
                exp_sum = exp_sum + scores[kt];
            }
            if (exp_sum > 0.0f) {
                const float inv_sum = 1.0f / exp_sum;
                for (size_t kt = 0; kt < len; ++kt) scores[kt] *= inv_sum;
            }
            float *o = out + qt * num_q_heads * head_dim + qh * head_dim;
            for (size_t kt = 0; kt < len; ++kt) {
                const float w = scores[kt];
                if (w > 0.0f) {
                    const float *vs = v + kvh * stride + kt * head_dim;
                    for (size_t i = 0; i < head_dim; ++i) {
                        const float p = w * vs[i];
                        o[i] = o[i] + p;
                    }
                }
            }
        }
    }
    free(scores);
}

/* LlamaBlock::forward with LlamaAttention::forward, unfused projections, non-macOS
 *                              reference: src/models/llama/decoder.rs:69-155,
 *                                         src/models/llama/attention.rs:74-212
 *   h [seq, d]; weights as raw GGUF blocks [out, in] (each product is the dequantise-
 *   then-matmul of orc_gguf_matmul); norm weights [d]; k_cache / v_cache
 *   [nkv, capacity, hd] holding cache_len positions on entry, cache_len + seq on return
 *   (the caller owns capacity >= cache_len + seq).  out [seq, d].  Returns 0, or -1 on
 *   allocation failure. */
static int block_forward_types(const float *h, size_t seq, size_t d, size_t nqh, size_t nkvh, size_t hd, size_t ffn,
                               const int *ggml_types, const uint8_t *wq, const uint8_t *wk, const uint8_t *wv,
                               const uint8_t *wo, const uint8_t *wg, const uint8_t *wu, const uint8_t *wd,
                               const float *attn_norm_w, const float *ffn_norm_w, float rms_eps, const float *cos_t,
                               const float *sin_t, float *k_cache, float *v_cache, size_t cache_len, size_t capacity,
                               float *out);

ORC_API int orc_llama_block_forward(const float *h, size_t seq, size_t d, size_t nqh, size_t nkvh, size_t hd, size_t ffn,
                                    int ggml_type, const uint8_t *wq, const uint8_t *wk, const uint8_t *wv,
                                    const uint8_t *wo, const uint8_t *wg, const uint8_t *wu, const uint8_t *wd,
                                    const float *attn_norm_w, const float *ffn_norm_w, float rms_eps,
                                    const float *cos_t, const float *sin_t, float *k_cache, float *v_cache,
                                    size_t cache_len, size_t capacity, float *out) {
    const int types[7] = {ggml_type, ggml_type, ggml_type, ggml_type, ggml_type, ggml_type, ggml_type};
    return block_forward_types(h, seq, d, nqh, nkvh, hd, ffn, types, wq, wk, wv, wo, wg, wu, wd, attn_norm_w, ffn_norm_w, rms_eps,
                               cos_t, sin_t, k_cache, v_cache, cache_len, capacity, out);
}

/* The same with one GGML type per projection (q, k, v, o, gate, up, down). */
ORC_API int orc_llama_block_forward_types(const float *h, size_t seq, size_t d, size_t nqh, size_t nkvh, size_t hd,
                                          size_t ffn, const int *ggml_types, const uint8_t *wq, const uint8_t *wk,
                                          const uint8_t *wv, const uint8_t *wo, const uint8_t *wg, const uint8_t *wu,
                                          const uint8_t *wd, const float *attn_norm_w, const float *ffn_norm_w,
                                          float rms_eps, const float *cos_t, const float *sin_t, float *k_cache,
                                          float *v_cache, size_t cache_len, size_t capacity, float *out) {
    return block_forward_types(h, seq, d, nqh, nkvh, hd, ffn, ggml_types, wq, wk, wv, wo, wg, wu, wd, attn_norm_w, ffn_norm_w,
                               rms_eps, cos_t, sin_t, k_cache, v_cache, cache_len, capacity, out);
}

static int block_forward_types(const float *h, size_t seq, size_t d, size_t nqh, size_t nkvh, size_t hd, size_t ffn,
                               const int *ty, const uint8_t *wq, const uint8_t *wk, const uint8_t *wv,
                               const uint8_t *wo, const uint8_t *wg, const uint8_t *wu, const uint8_t *wd,
                               const float *attn_norm_w, const float *ffn_norm_w, float rms_eps, const float *cos_t,
                               const float *sin_t, float *k_cache, float *v_cache, size_t cache_len, size_t capacity,
                               float *out) {
    const size_t q_dim = nqh * hd, kv_dim = nkvh * hd;
    float *normed = (float *)malloc(seq * d * sizeof(float));
    float *qd = (float *)malloc(seq * q_dim * sizeof(float)), *kd = (float *)malloc(seq * kv_dim * sizeof(float));
    float *vd = (float *)malloc(seq * kv_dim * sizeof(float)), *q_rope = (float *)malloc(seq * q_dim * sizeof(float));
    float *attn = (float *)calloc(seq * q_dim, sizeof(float)), *proj = (float *)malloc(seq * d * sizeof(float));
    float *h1 = (float *)malloc(seq * d * sizeof(float)), *g = (float *)malloc(seq * ffn * sizeof(float));
    float *u = (float *)malloc(seq * ffn * sizeof(float));
    int rc = -1;
    if (normed && qd && kd && vd && q_rope && attn && proj && h1 && g && u) {
        orc_rmsnorm(h, seq, d, attn_norm_w, rms_eps, normed);
        rc = orc_gguf_matmul(normed, seq, wq, ty[0], q_dim, d, qd);
        if (!rc) rc = orc_gguf_matmul(normed, seq, wk, ty[1], kv_dim, d, kd);
        if (!rc) rc = orc_gguf_matmul(normed, seq, wv, ty[2], kv_dim, d, vd);
        if (!rc) {
            /* RoPE into head-major [heads, seq, hd]; K and V straight into the cache rows */
            for (size_t hh = 0; hh < nqh; ++hh)
                for (size_t t = 0; t < seq; ++t)
                    rope_one(qd + t * q_dim + hh * hd, q_rope + hh * seq * hd + t * hd, cos_t + (cache_len + t) * hd,
                             sin_t + (cache_len + t) * hd, hd);
            for (size_t hh = 0; hh < nkvh; ++hh)
                for (size_t t = 0; t < seq; ++t) {
                    float *kdst = k_cache + hh * capacity * hd + (cache_len + t) * hd;
                    rope_one(kd + t * kv_dim + hh * hd, kdst, cos_t + (cache_len + t) * hd, sin_t + (cache_len + t) * hd, hd);
                    memcpy(v_cache + hh * capacity * hd + (cache_len + t) * hd, vd + t * kv_dim + hh * hd, hd * sizeof(float));
                }
            orc_gqa_attention(q_rope, k_cache, v_cache, cache_len + seq, capacity, nqh, nkvh, seq, hd,
                              1.0f / sqrtf((float)hd), 1, cache_len, 0, 0, 0.0f, attn);
            rc = orc_gguf_matmul(attn, seq, wo, ty[3], d, q_dim, proj);
        }
        if (!rc) {
            for (size_t i = 0; i < seq * d; ++i) h1[i] = h[i] + proj[i];
            orc_rmsnorm(h1, seq, d, ffn_norm_w, rms_eps, normed);
            rc = orc_gguf_matmul(normed, seq, wg, ty[4], ffn, d, g);
            if (!rc) rc = orc_gguf_matmul(normed, seq, wu, ty[5], ffn, d, u);
        }
        if (!rc) {
            for (size_t i = 0; i < seq * ffn; ++i) {
                const float gi = g[i];
                const float silu = gi / (1.0f + expf(-gi));
                g[i] = silu * u[i];
            }
            rc = orc_gguf_matmul(g, seq, wd, ty[6], d, ffn, proj);
        }
        if (!rc)
            for (size_t i = 0; i < seq * d; ++i) out[i] = h1[i] + proj[i];
    }
    free(normed); free(qd); free(kd); free(vd); free(q_rope); free(attn); free(proj); free(h1); free(g); free(u);
    return rc;
}
