/*
 * peregrine_oracle_formats.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of the sibling weight formats that feed peregrine's quantised
 * products: the MXFP4 matrix-vector product and expert of the gpt_oss example.  Written
 * from the reference's source text; same compile flags as peregrine_oracle.c (no
 * contraction, no fast-math).  Only tests and the smoke check may load it.
 *
 * Parity status (tests/test_oracle_formats_pins.py): the reference holds no test or vector
 * for MXFP4; orc_mxfp4_matmul is pinned by the OCP Microscaling E2M1 / E8M0 value tables
 * (one-hot inputs read every code and every scale byte back), by the nibble order, and by a
 * float64 NumPy recomputation; orc_mxfp4_expert_forward by closed forms of its activation
 * (clamp limits, linear + 1, sigmoid(alpha * gate)) and the same float64 recomputation.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* FP4_LUT                                         reference: examples/gpt_oss/moe.rs:5-8 */
static const float FP4_LUT[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                  -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};

/* mxfp4_matmul                                    reference: examples/gpt_oss/moe.rs:16-53
 *   block_dot accumulates lo then hi per byte, left to right; row_sum += block_dot * scale
 *   with scale = f32::from_bits(scale_byte << 23). */
ORC_API void orc_mxfp4_matmul(const float *input, const uint8_t *blocks, const uint8_t *scales, size_t out_dim,
                              size_t in_dim, float *output) {
    const size_t nbr = in_dim / 32, bytes_per_row = nbr * 16;
    for (size_t r = 0; r < out_dim; ++r) {
        float row_sum = 0.0f;
        for (size_t b = 0; b < nbr; ++b) {
            const uint8_t *blk = blocks + r * bytes_per_row + b * 16;
            const uint32_t bits = (uint32_t)scales[r * nbr + b] << 23;
            float scale;
            memcpy(&scale, &bits, 4);
            const float *in = input + b * 32;
            float block_dot = 0.0f;
            for (size_t k = 0; k < 16; ++k) {
                const float p0 = FP4_LUT[blk[k] & 0x0F] * in[2 * k];
                block_dot = block_dot + p0;
                const float p1 = FP4_LUT[(blk[k] >> 4) & 0x0F] * in[2 * k + 1];
                block_dot = block_dot + p1;
            }
            const float t = block_dot * scale;
            row_sum = row_sum + t;
        }
        output[r] = row_sum;
    }
}

/* swiglu (gpt-oss)                                reference: examples/gpt_oss/moe.rs:145-154 */
static void gpt_oss_swiglu(const float *data, size_t out_dim, float alpha, float clamp, float *out) {
    for (size_t i = 0; i < out_dim; ++i) {
        const float g = data[2 * i], l = data[2 * i + 1];
        const float gate = (g != g) ? clamp : (g < clamp ? g : clamp);                         /* f32::min */
        const float linear = (l != l) ? l : (l < -clamp ? -clamp : (l > clamp ? clamp : l));   /* f32::clamp */
        const float activated = gate * (1.0f / (1.0f + expf(-alpha * gate)));
        out[i] = activated * (linear + 1.0f);
    }
}

/* Mxfp4Expert::forward, one row                   reference: examples/gpt_oss/moe.rs:84-115 */
ORC_API int orc_mxfp4_expert_forward(const float *x, size_t hidden, size_t intermediate, float alpha, float clamp,
                                     const uint8_t *mlp1_blocks, const uint8_t *mlp1_scales, const uint8_t *mlp2_blocks,
                                     const uint8_t *mlp2_scales, const float *mlp1_bias, const float *mlp2_bias,
                                     float *out) {
    const size_t inter2 = intermediate * 2;
    float *h = (float *)malloc(inter2 * sizeof(float)), *act = (float *)malloc(intermediate * sizeof(float));
    if (!h || !act) { free(h); free(act); return -1; }
    orc_mxfp4_matmul(x, mlp1_blocks, mlp1_scales, inter2, hidden, h);
    for (size_t i = 0; i < inter2; ++i) h[i] = h[i] + mlp1_bias[i];
    gpt_oss_swiglu(h, intermediate, alpha, clamp, act);
    orc_mxfp4_matmul(act, mlp2_blocks, mlp2_scales, hidden, intermediate, out);
    for (size_t i = 0; i < hidden; ++i) out[i] = out[i] + mlp2_bias[i];
    free(h);
    free(act);
    return 0;
}

/* MoELayer::forward after its router, MXFP4 experts          reference: examples/gpt_oss/moe.rs:286-352
 *   out[t] = sum over the token's k experts, in the order given, of weight * expert.forward(x[t]) (one multiply, one
 *   add per term, from 0.0).  Expert e's operands are entry e of the six arrays.  Parity status: a composition of
 *   orc_mxfp4_expert_forward (pinned above); the accumulation is pinned by recomputing it in float32 NumPy from
 *   that function's own outputs, bit for bit, on routings where the order of the terms matters. */
ORC_API int orc_mxfp4_moe_routed(const float *x, size_t T, size_t hidden, size_t intermediate, float alpha, float clamp, size_t E,
                                 size_t top_k, const int32_t *idx, const float *weight, const uint8_t *const *mlp1_blocks,
                                 const uint8_t *const *mlp1_scales, const uint8_t *const *mlp2_blocks, const uint8_t *const *mlp2_scales,
                                 const float *const *mlp1_bias, const float *const *mlp2_bias, float *out) {
    float *y = (float *)malloc(hidden * sizeof(float));
    if (!y) return -1;
    int rc = 0;
    for (size_t t = 0; t < T && rc == 0; ++t) {
        for (size_t i = 0; i < hidden; ++i) out[t * hidden + i] = 0.0f;
        for (size_t k = 0; k < top_k; ++k) {
            const int32_t e = idx[t * top_k + k];
            if (e < 0 || (size_t)e >= E) { rc = -3; break; }
            rc = orc_mxfp4_expert_forward(x + t * hidden, hidden, intermediate, alpha, clamp, mlp1_blocks[e], mlp1_scales[e],
                                          mlp2_blocks[e], mlp2_scales[e], mlp1_bias[e], mlp2_bias[e], y);
            if (rc) break;
            for (size_t i = 0; i < hidden; ++i) out[t * hidden + i] += weight[t * top_k + k] * y[i];
        }
    }
    free(y);
    return rc;
}

/* ---------------------------------------------------------------------------------------
 * Canonical Huffman over i8 symbols.  Parity status: orc_huffman_table is pinned by hand-
 * worked small cases that fix the tie-breaking (stable sort, leaf before internal node), by
 * optimality against an independent heap-based Huffman cost and by Kraft equality;
 * orc_huffman_encode / orc_huffman_decode by the reference's own tests restated
 * (src/huffman.rs:740-800: round trip on its biased generator, empty input, one symbol in
 * at most 65 bytes, two-symbol table) and by hand-packed bit strings.
 * ------------------------------------------------------------------------------------- */

#define HUF_SYMS 256
#define HUF_MAX_BITS 12 /* MAX_LUT_BITS                       reference: src/huffman.rs:30 */

/* HuffmanTable::canonical_codes                   reference: src/huffman.rs:152-186 */
ORC_API void orc_huffman_canonical_codes(const uint8_t *bl, uint32_t *codes) {
    uint32_t bl_count[256] = {0}, next_code[256] = {0};
    int max_len = 0;
    memset(codes, 0, HUF_SYMS * sizeof(uint32_t));
    for (int s = 0; s < HUF_SYMS; ++s) {
        if (bl[s] > max_len) max_len = bl[s];
        if (bl[s] > 0) bl_count[bl[s]] += 1;
    }
    if (max_len == 0) return;
    uint32_t code = 0;
    for (int bits = 1; bits <= max_len; ++bits) {
        code = (code + bl_count[bits - 1]) << 1;
        next_code[bits] = code;
    }
    for (int s = 0; s < HUF_SYMS; ++s)
        if (bl[s] > 0) {
            codes[s] = next_code[bl[s]];
            next_code[bl[s]] += 1;
        }
}

/* HuffmanTable::from_frequencies                  reference: src/huffman.rs:35-150
 *   leaves sorted by frequency (stable: equal frequencies keep symbol order); two queues;
 *   when the fronts tie the leaf is taken; depths above 12 are clamped to 12. */
ORC_API void orc_huffman_table(const uint64_t *freqs, uint8_t *bl, uint32_t *codes) {
    int symbols[HUF_SYMS], n = 0;
    uint64_t fv[HUF_SYMS];
    memset(bl, 0, HUF_SYMS);
    for (int s = 0; s < HUF_SYMS; ++s)
        if (freqs[s] > 0) { symbols[n] = s; fv[n] = freqs[s]; ++n; }
    if (n == 1) bl[symbols[0]] = 1;
    if (n >= 2) {
        int order[HUF_SYMS];
        for (int i = 0; i < n; ++i) order[i] = i;
        for (int i = 1; i < n; ++i) { /* insertion sort: stable */
            const int v = order[i];
            int j = i;
            while (j > 0 && fv[order[j - 1]] > fv[v]) { order[j] = order[j - 1]; --j; }
            order[j] = v;
        }
        uint64_t lf[HUF_SYMS], inf_[HUF_SYMS];
        int ln[HUF_SYMS], inn[HUF_SYMS], lh = 0, ih = 0, it = 0; /* queue heads / internal tail */
        for (int i = 0; i < n; ++i) { lf[i] = fv[order[i]]; ln[i] = order[i]; }
        int parent[2 * HUF_SYMS], depth[2 * HUF_SYMS], next_node = n;
        for (int step = 0; step < n - 1; ++step) {
            uint64_t f[2];
            int node[2];
            for (int k = 0; k < 2; ++k) {
                const int have_l = lh < n, have_i = ih < it;
                if (have_l && (!have_i || lf[lh] <= inf_[ih])) { f[k] = lf[lh]; node[k] = ln[lh]; ++lh; }
                else { f[k] = inf_[ih]; node[k] = inn[ih]; ++ih; }
            }
            parent[node[0]] = next_node;
            parent[node[1]] = next_node;
            inf_[it] = f[0] + f[1];
            inn[it] = next_node;
            ++it;
            ++next_node;
        }
        const int root = 2 * n - 2;
        depth[root] = 0;
        for (int i = root - 1; i >= 0; --i) depth[i] = depth[parent[i]] + 1;
        for (int i = 0; i < n; ++i) bl[symbols[i]] = (uint8_t)(depth[i] > HUF_MAX_BITS ? HUF_MAX_BITS : depth[i]);
    }
    if (codes) orc_huffman_canonical_codes(bl, codes);
}

/* HuffmanTable::encode                            reference: src/huffman.rs:216-251
 *   MSB first, the last byte padded with zero bits.  Returns the byte count (out may be
 *   NULL to size the buffer). */
ORC_API size_t orc_huffman_encode(const uint8_t *bl, const uint32_t *codes, const int8_t *data, size_t n, uint8_t *out) {
    size_t bytes = 0;
    uint8_t current = 0;
    int bits_in_byte = 0;
    for (size_t i = 0; i < n; ++i) {
        const int idx = (int)data[i] + 128;
        for (int bit_pos = (int)bl[idx] - 1; bit_pos >= 0; --bit_pos) {
            current = (uint8_t)((current << 1) | ((codes[idx] >> bit_pos) & 1u));
            if (++bits_in_byte == 8) {
                if (out) out[bytes] = current;
                ++bytes;
                current = 0;
                bits_in_byte = 0;
            }
        }
    }
    if (bits_in_byte > 0) {
        if (out) out[bytes] = (uint8_t)(current << (8 - bits_in_byte));
        ++bytes;
    }
    return bytes;
}

/* HuffmanTable::build_decode_lut + decode         reference: src/huffman.rs:189-213, 254-284
 *   12-bit window, zero-padded past the end; entry (symbol, length); a length-0 entry emits
 *   symbol 0 without advancing, as the release build does.  Returns -1 if a code does not
 *   fit the table (the reference would index out of bounds). */
ORC_API int orc_huffman_decode(const uint8_t *bl, const uint8_t *bitstream, size_t len, size_t num_symbols, int8_t *out) {
    uint32_t codes[HUF_SYMS];
    static int8_t lut_sym[1 << HUF_MAX_BITS];
    static uint8_t lut_len[1 << HUF_MAX_BITS];
    orc_huffman_canonical_codes(bl, codes);
    memset(lut_sym, 0, sizeof lut_sym);
    memset(lut_len, 0, sizeof lut_len);
    for (int s = 0; s < HUF_SYMS; ++s) {
        if (bl[s] == 0 || bl[s] > HUF_MAX_BITS) continue;
        const int shift = HUF_MAX_BITS - bl[s];
        const size_t base = (size_t)codes[s] << shift, count = (size_t)1 << shift;
        if (base + count > (size_t)(1 << HUF_MAX_BITS)) return -1;
        for (size_t j = 0; j < count; ++j) { lut_sym[base + j] = (int8_t)(s - 128); lut_len[base + j] = bl[s]; }
    }
    const size_t total_bits = len * 8;
    size_t bit_pos = 0;
    for (size_t i = 0; i < num_symbols; ++i) {
        uint32_t code = 0;
        size_t avail = total_bits > bit_pos ? total_bits - bit_pos : 0;
        if (avail > HUF_MAX_BITS) avail = HUF_MAX_BITS;
        for (size_t b = 0; b < avail; ++b) {
            const size_t byte_idx = (bit_pos + b) / 8, bit_idx = 7 - ((bit_pos + b) % 8);
            code = (code << 1) | ((bitstream[byte_idx] >> bit_idx) & 1u);
        }
        if (avail < HUF_MAX_BITS) code <<= HUF_MAX_BITS - avail;
        out[i] = lut_sym[code];
        bit_pos += lut_len[code];
    }
    return 0;
}

/* ---------------------------------------------------------------------------------------
 * HuffmanKVCache: int8 + Huffman chunks of older tokens behind an f32 window.  Parity
 * status: pinned by the reference's own tests restated (src/huffman.rs:850-905,
 * tests/huffman_parity.rs:133-186: lengths after each append, error <= scale + 1e-5), by
 * closed forms (an all-zero head has scale 1 and codes of one bit; a constant chunk is
 * ceil(n / 8) zero bytes and decodes to 127 * (c / 127); the values +-absmax become +-127),
 * by the half-step error bound |x - x'| <= scale / 2 that only round-to-nearest meets, by a
 * float32 NumPy recomputation of scales and int8 values that shares no code with this file,
 * by bitstream == orc_huffman_encode of those values under orc_huffman_table of their
 * histogram (both pinned above), and for the cache by token order: what get_kv returns is
 * decompress(compress(.)) of the tokens each chunk took, in arrival order, followed bit for
 * bit by the tokens still in the window.
 * ------------------------------------------------------------------------------------- */

/* The table a KV chunk is coded with: HuffmanTable::from_frequencies where that is a prefix code.
 * Where its depth clamp over-subscribes the code the reference panics inside from_frequencies
 * (build_decode_lut indexes past its table, src/huffman.rs:205-208), so there is nothing to
 * restate; the library then repairs the lengths and this is that rule, written independently:
 * sort the clamped lengths, hand them out shortest to most frequent (ties: lower symbol first);
 * while the Kraft sum exceeds 1 lengthen by one bit the least frequent symbol of the deepest
 * level below 12; then shorten, most frequent symbol first, whatever the slack allows.
 * Returns 1 if the repair ran. */
ORC_API int orc_huffman_table_that_decodes(const uint64_t *freqs, uint8_t *bl, uint32_t *codes) {
    orc_huffman_table(freqs, bl, NULL);
    const long full = 1L << HUF_MAX_BITS;
    long kraft = 0;
    int order[HUF_SYMS], len[HUF_SYMS], n = 0;
    for (int s = 0; s < HUF_SYMS; ++s)
        if (bl[s]) { kraft += full >> bl[s]; order[n++] = s; }
    int repaired = 0;
    if (kraft > full) {
        repaired = 1;
        for (int i = 1; i < n; ++i) { /* insertion sort: frequency descending, stable */
            const int s = order[i];
            int j = i;
            while (j > 0 && freqs[order[j - 1]] < freqs[s]) { order[j] = order[j - 1]; --j; }
            order[j] = s;
        }
        for (int i = 0; i < n; ++i) len[i] = bl[order[i]];
        for (int i = 1; i < n; ++i) { /* lengths ascending */
            const int v = len[i];
            int j = i;
            while (j > 0 && len[j - 1] > v) { len[j] = len[j - 1]; --j; }
            len[j] = v;
        }
        while (kraft > full) {
            int pick = n - 1;
            while (len[pick] >= HUF_MAX_BITS) --pick; /* exists: n symbols of 12 bits never exceed 1 */
            kraft -= full >> (len[pick] + 1);
            len[pick] += 1;
        }
        for (int i = 0; i < n; ++i)
            while (len[i] > 1 && (full >> len[i]) <= full - kraft) { kraft += full >> len[i]; len[i] -= 1; }
        for (int i = 0; i < n; ++i) bl[order[i]] = (uint8_t)len[i];
    }
    if (codes) orc_huffman_canonical_codes(bl, codes);
    return repaired;
}

static inline int8_t hkv_sat_i8(float v) { /* Rust `f32 as i8`: saturating, NaN -> 0 */
    if (v != v) return 0;
    if (v <= -128.0f) return (int8_t)-128;
    if (v >= 127.0f) return (int8_t)127;
    return (int8_t)v;
}

/* HuffmanKVCache::compress_chunk                  reference: src/huffman.rs:612-658
 *   data [num_heads][num_tokens][head_dim]; per head absmax (f32::max drops NaN), scale =
 *   absmax / 127 or 1, q = (v * (1 / scale)).round().clamp(-127, 127) as i8; one table over all
 *   heads' values (orc_huffman_table_that_decodes); codebook = the 256 bit lengths.  bitstream may be NULL to ask for the
 *   size; q_out (optional) receives the int8 values.  Returns the bitstream's bytes. */
ORC_API size_t orc_huffman_kv_compress_chunk(const float *data, size_t num_tokens, size_t num_heads, size_t head_dim,
                                             uint8_t *bitstream, float *scales, uint8_t *codebook, int8_t *q_out) {
    const size_t head_size = num_tokens * head_dim, total = num_heads * head_size;
    int8_t *q = (int8_t *)malloc(total ? total : 1);
    for (size_t h = 0; h < num_heads; ++h) {
        const float *hd = data + h * head_size;
        float absmax = 0.0f;
        for (size_t i = 0; i < head_size; ++i) {
            const float a = fabsf(hd[i]);
            if (a > absmax) absmax = a; /* a NaN compares false and is skipped, as acc.max(NaN) = acc */
        }
        const float scale = absmax == 0.0f ? 1.0f : absmax / 127.0f;
        scales[h] = scale;
        const float inv_scale = 1.0f / scale;
        for (size_t i = 0; i < head_size; ++i) {
            float r = roundf(hd[i] * inv_scale);
            if (r == r) r = r < -127.0f ? -127.0f : (r > 127.0f ? 127.0f : r);
            q[h * head_size + i] = hkv_sat_i8(r);
        }
    }
    uint64_t freqs[HUF_SYMS];
    uint32_t codes[HUF_SYMS];
    memset(freqs, 0, sizeof freqs);
    for (size_t i = 0; i < total; ++i) freqs[(int)q[i] + 128] += 1;
    orc_huffman_table_that_decodes(freqs, codebook, codes);
    const size_t bytes = orc_huffman_encode(codebook, codes, q, total, bitstream);
    if (q_out) memcpy(q_out, q, total);
    free(q);
    return bytes;
}

/* HuffmanKVCache::decompress_chunk                reference: src/huffman.rs:661-680 */
ORC_API int orc_huffman_kv_decompress_chunk(const uint8_t *bitstream, size_t bytes, const float *scales, const uint8_t *codebook,
                                            size_t num_tokens, size_t num_heads, size_t head_dim, float *out) {
    const size_t head_size = num_tokens * head_dim, total = num_heads * head_size;
    int8_t *q = (int8_t *)malloc(total ? total : 1);
    const int rc = orc_huffman_decode(codebook, bitstream, bytes, total, q);
    if (rc == 0)
        for (size_t h = 0; h < num_heads; ++h)
            for (size_t i = 0; i < head_size; ++i) out[h * head_size + i] = (float)q[h * head_size + i] * scales[h];
    free(q);
    return rc;
}

typedef struct {
    uint8_t *bitstream;
    size_t bytes;
    float *scales;
    uint8_t codebook[HUF_SYMS];
    size_t num_tokens;
} orc_hkv_chunk;

/* HuffmanKVCache over StandardKVCache             reference: src/huffman.rs:484-497, src/attention.rs:8-15 */
typedef struct {
    float *k, *v; /* [heads][capacity][head_dim] */
    size_t len, capacity, heads, head_dim;
    orc_hkv_chunk *kc, *vc;
    size_t nchunks, compressed_len, threshold, chunk_size;
} orc_hkv;

/* HuffmanKVCache::new                             reference: src/huffman.rs:524-540 */
ORC_API orc_hkv *orc_huffman_kv_new(size_t heads, size_t head_dim, size_t compress_threshold, size_t chunk_size) {
    orc_hkv *c = (orc_hkv *)calloc(1, sizeof *c);
    c->heads = heads;
    c->head_dim = head_dim;
    c->threshold = compress_threshold > chunk_size ? compress_threshold : chunk_size;
    c->chunk_size = chunk_size;
    return c;
}

ORC_API void orc_huffman_kv_free(orc_hkv *c) {
    if (!c) return;
    for (size_t i = 0; i < c->nchunks; ++i) {
        free(c->kc[i].bitstream); free(c->kc[i].scales);
        free(c->vc[i].bitstream); free(c->vc[i].scales);
    }
    free(c->kc); free(c->vc); free(c->k); free(c->v); free(c);
}

/* StandardKVCache::ensure_capacity + append       reference: src/attention.rs:31-83 */
static void hkv_hot_append(orc_hkv *c, const float *nk, const float *nv, size_t seq_len) {
    const size_t new_len = c->len + seq_len, hd = c->head_dim;
    if (new_len > c->capacity) {
        const size_t grown = (c->capacity > 16 ? c->capacity : 16) * 2, new_cap = new_len > grown ? new_len : grown;
        const size_t total = c->heads * new_cap * hd;
        float *k2 = (float *)calloc(total ? total : 1, sizeof(float)), *v2 = (float *)calloc(total ? total : 1, sizeof(float));
        for (size_t h = 0; h < c->heads && c->len > 0; ++h) {
            memcpy(k2 + h * new_cap * hd, c->k + h * c->capacity * hd, c->len * hd * sizeof(float));
            memcpy(v2 + h * new_cap * hd, c->v + h * c->capacity * hd, c->len * hd * sizeof(float));
        }
        free(c->k); free(c->v);
        c->k = k2; c->v = v2; c->capacity = new_cap;
    }
    for (size_t h = 0; h < c->heads; ++h) {
        memcpy(c->k + h * c->capacity * hd + c->len * hd, nk + h * seq_len * hd, seq_len * hd * sizeof(float));
        memcpy(c->v + h * c->capacity * hd + c->len * hd, nv + h * seq_len * hd, seq_len * hd * sizeof(float));
    }
    c->len = new_len;
}

/* extract_chunk_data + compress_chunk             reference: src/huffman.rs:579-596, 612-658 */
static void hkv_compress_side(const orc_hkv *c, const float *side, size_t tokens, orc_hkv_chunk *out) {
    const size_t hd = c->head_dim, n = c->heads * tokens * hd;
    float *flat = (float *)malloc((n ? n : 1) * sizeof(float));
    for (size_t h = 0; h < c->heads; ++h) memcpy(flat + h * tokens * hd, side + h * c->capacity * hd, tokens * hd * sizeof(float));
    out->scales = (float *)malloc((c->heads ? c->heads : 1) * sizeof(float));
    out->bitstream = (uint8_t *)malloc(2 * n + 16);
    out->bytes = orc_huffman_kv_compress_chunk(flat, tokens, c->heads, hd, out->bitstream, out->scales, out->codebook, NULL);
    out->num_tokens = tokens;
    free(flat);
}

/* HuffmanKVCache::append                          reference: src/huffman.rs:544-556
 *   compress_oldest_chunk :559-577, remove_oldest_tokens :599-610 (copy_within = memmove).
 *   chunk_size 0 never ends once the threshold is met in the reference; here it returns. */
ORC_API void orc_huffman_kv_append(orc_hkv *c, const float *nk, const float *nv, size_t seq_len) {
    hkv_hot_append(c, nk, nv, seq_len);
    while (c->len >= c->threshold) {
        const size_t tokens = c->chunk_size < c->len ? c->chunk_size : c->len, hd = c->head_dim;
        if (tokens == 0) return;
        c->kc = (orc_hkv_chunk *)realloc(c->kc, (c->nchunks + 1) * sizeof *c->kc);
        c->vc = (orc_hkv_chunk *)realloc(c->vc, (c->nchunks + 1) * sizeof *c->vc);
        hkv_compress_side(c, c->k, tokens, &c->kc[c->nchunks]);
        hkv_compress_side(c, c->v, tokens, &c->vc[c->nchunks]);
        c->nchunks += 1;
        c->compressed_len += tokens;
        const size_t new_len = c->len - tokens;
        for (size_t h = 0; h < c->heads; ++h) {
            memmove(c->k + h * c->capacity * hd, c->k + h * c->capacity * hd + tokens * hd, new_len * hd * sizeof(float));
            memmove(c->v + h * c->capacity * hd, c->v + h * c->capacity * hd + tokens * hd, new_len * hd * sizeof(float));
        }
        c->len = new_len;
    }
}

/* which: 0 len() (:683-685), 1 compressed_len, 2 hot.len, 3 hot capacity, 4 chunks, 5 compress_threshold */
ORC_API size_t orc_huffman_kv_stat(const orc_hkv *c, int which) {
    switch (which) {
    case 0: return c->compressed_len + c->len;
    case 1: return c->compressed_len;
    case 2: return c->len;
    case 3: return c->capacity;
    case 4: return c->nchunks;
    default: return c->threshold;
    }
}

ORC_API size_t orc_huffman_kv_chunk(const orc_hkv *c, int value_side, size_t index, const uint8_t **bitstream, const float **scales,
                                    const uint8_t **codebook, size_t *num_tokens) {
    const orc_hkv_chunk *ch = value_side ? &c->vc[index] : &c->kc[index];
    *bitstream = ch->bitstream; *scales = ch->scales; *codebook = ch->codebook; *num_tokens = ch->num_tokens;
    return ch->bytes;
}

/* HuffmanKVCache::get_kv                          reference: src/huffman.rs:689-724
 *   k, v [heads][len()][head_dim].  literal_hot_offsets != 0 reads head h of the window at
 *   h * hot.len * head_dim as the reference does (:707-708); 0 reads it at h * head_stride(),
 *   where append put it.  The two agree for head 0 and whenever hot.len == capacity. */
ORC_API void orc_huffman_kv_get_kv(const orc_hkv *c, int literal_hot_offsets, float *k, float *v) {
    const size_t hd = c->head_dim, total_len = c->compressed_len + c->len;
    for (int side = 0; side < 2; ++side) {
        float *dst = side ? v : k;
        const float *hot = side ? c->v : c->k;
        const orc_hkv_chunk *chunks = side ? c->vc : c->kc;
        for (size_t i = 0, off = 0; i < c->nchunks; ++i) {
            const size_t t = chunks[i].num_tokens, n = c->heads * t * hd;
            float *flat = (float *)malloc((n ? n : 1) * sizeof(float));
            orc_huffman_kv_decompress_chunk(chunks[i].bitstream, chunks[i].bytes, chunks[i].scales, chunks[i].codebook, t, c->heads, hd, flat);
            for (size_t h = 0; h < c->heads; ++h) memcpy(dst + (h * total_len + off) * hd, flat + h * t * hd, t * hd * sizeof(float));
            free(flat);
            off += t;
        }
        for (size_t h = 0; h < c->heads && c->len > 0; ++h) {
            const size_t base = literal_hot_offsets ? h * c->len * hd : h * c->capacity * hd;
            memcpy(dst + (h * total_len + c->compressed_len) * hd, hot + base, c->len * hd * sizeof(float));
        }
    }
}
