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
