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
