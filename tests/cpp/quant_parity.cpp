// C++ parity program for the host mirror (include/peregrine_hip.hpp).
// The cases follow the reference's own tests: tests/quant_parity.rs:6-77,149-173,
// src/quant.rs:225-291, tests/gguf_parity.rs:7-76, src/gguf.rs:574-631, and then
// tighten them: where the reference only bounds the error, the device result is
// compared bit-for-bit with the CPU oracle (which is test infrastructure only).
// Needs a GPU; prints one line per case and exits non-zero on the first failure.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <vector>

#include "peregrine_hip.hpp"

extern "C" {
void orc_quantize_weights(const float *, size_t, size_t, int8_t *, int8_t *, float *);
void orc_quantize_activations(const float *, size_t, size_t, int8_t *, float *);
int orc_matmul_quantized(const float *, size_t, size_t, const int8_t *, const float *, size_t, float *, int32_t *);
int orc_gguf_matmul(const float *, size_t, const uint8_t *, int, size_t, size_t, float *);
void orc_rope_tables(size_t, size_t, float, float *, float *);
void orc_gqa_attention(const float *, const float *, const float *, size_t, size_t, size_t, size_t, size_t, size_t, float,
                       int, size_t, size_t, size_t, float, float *);
int orc_llama_block_forward(const float *, size_t, size_t, size_t, size_t, size_t, size_t, int, const uint8_t *,
                            const uint8_t *, const uint8_t *, const uint8_t *, const uint8_t *, const uint8_t *,
                            const uint8_t *, const float *, const float *, float, const float *, const float *, float *,
                            float *, size_t, size_t, float *);
size_t orc_huffman_kv_compress_chunk(const float *, size_t, size_t, size_t, uint8_t *, float *, uint8_t *, int8_t *);
int orc_huffman_kv_decompress_chunk(const uint8_t *, size_t, const float *, const uint8_t *, size_t, size_t, size_t, float *);
void *orc_huffman_kv_new(size_t, size_t, size_t, size_t);
void orc_huffman_kv_free(void *);
void orc_huffman_kv_append(void *, const float *, const float *, size_t);
size_t orc_huffman_kv_stat(const void *, int);
void orc_huffman_kv_get_kv(const void *, int, float *, float *);
int orc_gpt_oss_route(const float *, const float *, size_t, size_t, size_t, int32_t *, float *);
int orc_moe_ffn_routed(const float *, size_t, size_t, size_t, size_t, size_t, const int32_t *, const float *, const uint8_t *const *,
                       const uint8_t *const *, const uint8_t *const *, int, int, const float *, float *);
int orc_mxfp4_moe_routed(const float *, size_t, size_t, size_t, float, float, size_t, size_t, const int32_t *, const float *,
                         const uint8_t *const *, const uint8_t *const *, const uint8_t *const *, const uint8_t *const *,
                         const float *const *, const float *const *, float *);
}

using namespace peregrine;

static int failures = 0;
#define EXPECT(cond, ...)                                     \
    do {                                                      \
        if (!(cond)) {                                        \
            std::printf("  FAIL %s:%d: ", __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);                         \
            std::printf("\n");                                \
            ++failures;                                       \
        }                                                     \
    } while (0)

static bool same_bits(const std::vector<float> &a, const std::vector<float> &b) {
    return a.size() == b.size() && std::memcmp(a.data(), b.data(), a.size() * sizeof(float)) == 0;
}

// tests/quant_parity.rs:6-32
static void test_quantize_dequantize_roundtrip(const GpuContext &gpu) {
    std::printf("test_quantize_dequantize_roundtrip\n");
    const size_t rows = 64, cols = 128;
    std::vector<float> data(rows * cols);
    for (size_t i = 0; i < data.size(); ++i) data[i] = (float)((i * 17 + 5) % 400) / 100.0f - 2.0f;
    auto qt = quant::quantize_weights(gpu, data, rows, cols);
    auto recovered = quant::dequantize(gpu, qt);
    EXPECT(recovered.size() == data.size(), "length");
    for (size_t i = 0; i < data.size(); ++i) {
        const float scale = qt.scales[i % cols];
        EXPECT(std::fabs(data[i] - recovered[i]) <= scale + 1e-7f, "element %zu: %g vs %g (scale %g)", i, data[i], recovered[i], scale);
    }
    // beyond the reference's bound: integers, transpose and scales equal the CPU path's exactly
    std::vector<int8_t> q(rows * cols), qt_t(rows * cols);
    std::vector<float> sc(cols);
    orc_quantize_weights(data.data(), rows, cols, q.data(), qt_t.data(), sc.data());
    EXPECT(q == qt.data_i8, "data_i8 differs from the CPU path");
    EXPECT(qt_t == qt.data_i8_t, "data_i8_t differs from the CPU path");
    EXPECT(same_bits(sc, qt.scales), "scales differ from the CPU path");
}

// tests/quant_parity.rs:35-77 and src/quant.rs:252-291
static void test_quantized_matmul_accuracy(const GpuContext &gpu, size_t m, size_t k, size_t n, int mod) {
    std::printf("test_quantized_matmul_accuracy m=%zu k=%zu n=%zu\n", m, k, n);
    std::vector<float> a(m * k), w(k * n);
    for (size_t i = 0; i < a.size(); ++i) a[i] = (float)((i * 7 + 3) % mod) / (float)mod - 0.5f;
    for (size_t i = 0; i < w.size(); ++i) w[i] = (float)((i * 13 + 7) % mod) / (float)mod - 0.5f;
    auto qt = quant::quantize_weights(gpu, w, k, n);
    auto out = quant::matmul_quantized(gpu, a, m, k, qt);
    // the reference's own check: against the f32 product, loose tolerance
    for (size_t i = 0; i < m; ++i)
        for (size_t j = 0; j < n; ++j) {
            float ref = 0.0f;
            for (size_t p = 0; p < k; ++p) ref += a[i * k + p] * w[p * n + j];
            const float diff = std::fabs(out[i * n + j] - ref);
            EXPECT(diff / std::fmax(std::fabs(ref), 1e-6f) < 0.15f || diff < 0.05f, "(%zu,%zu): %g vs f32 %g", i, j, out[i * n + j], ref);
        }
    // and bit-for-bit against the CPU path
    std::vector<float> cpu(m * n);
    orc_matmul_quantized(a.data(), m, k, qt.data_i8_t.data(), qt.scales.data(), n, cpu.data(), nullptr);
    EXPECT(same_bits(cpu, out), "matmul_quantized differs from the CPU path");
    // GPU entry point: unsynced buffer, sync, read  (tests/quant_parity.rs:95-107)
    auto buf = quant::matmul_quantized_gpu(gpu, a, m, k, qt);
    gpu.sync();
    EXPECT(same_bits(cpu, buf.read()), "matmul_quantized_gpu differs from the CPU path");
}

// quantize_activations: closed forms and CPU-path equality
static void test_quantize_activations(const GpuContext &gpu) {
    std::printf("test_quantize_activations\n");
    const size_t rows = 5, cols = 96;
    std::vector<float> x(rows * cols);
    for (size_t i = 0; i < x.size(); ++i) x[i] = std::sin(0.37f * (float)i) * (float)(1 + i % 7);
    for (size_t c = 0; c < cols; ++c) { x[1 * cols + c] = 0.0f; x[2 * cols + c] = (c % 2) ? 3.5f : -3.5f; }
    auto [q, s] = quant::quantize_activations(gpu, x, rows, cols);
    EXPECT(s[1] == 1.0f, "zero row must get scale 1.0, got %g", s[1]);
    EXPECT(s[2] == 3.5f / 127.0f, "constant row scale");
    for (size_t c = 0; c < cols; ++c) {
        EXPECT(q[1 * cols + c] == 0, "zero row");
        EXPECT(q[2 * cols + c] == ((c % 2) ? 127 : -127), "constant row -> +-127");
    }
    std::vector<int8_t> cq(rows * cols);
    std::vector<float> cs(rows);
    orc_quantize_activations(x.data(), rows, cols, cq.data(), cs.data());
    EXPECT(cq == q, "integers differ from the CPU path");
    EXPECT(same_bits(cs, s), "row scales differ from the CPU path");
}

// the reference panics on shape mismatch (src/quant.rs:28,80,135,137,208)
static void test_shape_panics(const GpuContext &gpu) {
    std::printf("test_shape_panics\n");
    std::vector<float> w(8 * 4, 0.5f), a(3 * 7, 1.0f);
    auto qt = quant::quantize_weights(gpu, w, 8, 4);
    bool threw = false;
    try { quant::matmul_quantized(gpu, a, 3, 7, qt); } catch (const Panic &) { threw = true; }
    EXPECT(threw, "k != weight rows must panic");
    threw = false;
    try { quant::quantize_weights(gpu, w, 8, 5); } catch (const Panic &) { threw = true; }
    EXPECT(threw, "data.len() != rows*cols must panic");
    threw = false;
    quant::QuantizedTensor cold = qt;  // copy shares no upload unless to_gpu ran
    try { if (!cold.on_gpu()) quant::matmul_quantized_gpu(gpu, std::vector<float>(3 * 8, 1.0f), 3, 8, cold); } catch (const Panic &) { threw = true; }
    EXPECT(threw || cold.on_gpu(), "weights not on GPU must panic");
}

// src/gguf.rs:574-631, tests/gguf_parity.rs:7-76
static void test_gguf_known_answers(const GpuContext &gpu) {
    std::printf("test_gguf_known_answers\n");
    const uint16_t bits[] = {0x0000, 0x3C00, 0xBC00, 0x3800, 0x4000, 0x4900};
    const float want[] = {0.0f, 1.0f, -1.0f, 0.5f, 2.0f, 10.0f};
    for (int i = 0; i < 6; ++i) EXPECT(gguf::f16_to_f32(gpu, bits[i]) == want[i], "f16 0x%04x", bits[i]);
    EXPECT(std::signbit(gguf::f16_to_f32(gpu, 0x8000)), "f16 -0.0 keeps its sign");
    {   // Q8_0: d = 0.5, q = 1..32  -> (i+1)/2
        std::vector<uint8_t> blk(34);
        blk[0] = 0x00; blk[1] = 0x38;
        for (int i = 0; i < 32; ++i) blk[2 + i] = (uint8_t)(int8_t)(i + 1);
        auto out = gguf::dequant_q8_0(gpu, blk, 32);
        for (int i = 0; i < 32; ++i) EXPECT(out[i] == (float)(i + 1) * 0.5f, "q8_0[%d] = %g", i, out[i]);
    }
    {   // Q4_0: d = 1.0, byte0 = 0x98 -> out[0] = 0, out[1] = 1 (interleaved order)
        std::vector<uint8_t> blk(18, 0x88);
        blk[0] = 0x00; blk[1] = 0x3C; blk[2] = 0x98;
        auto out = gguf::dequant_q4_0(gpu, blk, 32);
        EXPECT(out[0] == 0.0f && out[1] == 1.0f, "q4_0 interleave: %g %g", out[0], out[1]);
        for (int i = 2; i < 32; ++i) EXPECT(out[i] == 0.0f, "q4_0[%d] = %g", i, out[i]);
    }
    {   // Q4_1: d = 1.0, m = 10.0, byte0 = 0x53 -> 13, 15 ; rest (0x00) -> 10
        std::vector<uint8_t> blk(20, 0x00);
        blk[0] = 0x00; blk[1] = 0x3C; blk[2] = 0x00; blk[3] = 0x49; blk[4] = 0x53;
        auto out = gguf::dequant_q4_1(gpu, blk, 32);
        EXPECT(out[0] == 13.0f && out[1] == 15.0f && out[2] == 10.0f, "q4_1: %g %g %g", out[0], out[1], out[2]);
    }
    bool threw = false;
    try { gguf::dequant_q8_0(gpu, std::vector<uint8_t>(34), 33); } catch (const Panic &) { threw = true; }
    EXPECT(threw, "num_elements %% 32 != 0 must panic (src/gguf.rs:287)");
}

// dequantise-then-matmul against the CPU composition, Q4_0 and Q8_0, M = 1 and 3
static void test_block_weight_matmul(const GpuContext &gpu) {
    std::printf("test_block_weight_matmul\n");
    const size_t n_out = 48, k_in = 256, nb = n_out * k_in / 32;
    uint32_t s = 42;
    auto lcg = [&]() { s = s * 1103515245u + 12345u; return (float)s / 4294967295.0f * 2.0f - 1.0f; };  // tests/huffman_parity.rs:7-14
    for (int type : {PG_GGML_Q4_0, PG_GGML_Q8_0}) {
        const size_t bb = type == PG_GGML_Q4_0 ? 18 : 34;
        std::vector<uint8_t> blocks(nb * bb);
        for (size_t b = 0; b < nb; ++b) {
            const uint16_t d = (uint16_t)(0x2000 + (b * 37) % 0x0C00);  // positive normal halves around 1e-2
            blocks[b * bb] = (uint8_t)(d & 0xFF); blocks[b * bb + 1] = (uint8_t)(d >> 8);
            for (size_t i = 2; i < bb; ++i) { s = s * 1103515245u + 12345u; blocks[b * bb + i] = (uint8_t)(s >> 16); }
        }
        for (size_t m : {(size_t)1, (size_t)3}) {
            std::vector<float> x(m * k_in);
            for (auto &v : x) v = lcg();
            gguf::BlockWeight w(gpu, blocks, type, n_out, k_in);
            auto y = w.matmul(x, m);
            std::vector<float> ref(m * n_out);
            orc_gguf_matmul(x.data(), m, blocks.data(), type, n_out, k_in, ref.data());
            double rms = 0;
            for (float v : ref) rms += (double)v * v;
            rms = std::sqrt(rms / ref.size());
            for (size_t i = 0; i < ref.size(); ++i) {
                const double tol = 1e-3 * std::fmax(std::fabs((double)ref[i]), rms);  // the block-dequant contract
                EXPECT(std::fabs((double)y[i] - ref[i]) <= tol, "type %d m %zu [%zu]: %g vs %g", type, m, i, y[i], ref[i]);
            }
        }
    }
}

// tests/attention.rs:59-133 (MHA against the naive per-head form) with the reference's sin/cos
// inputs, then the same through a cache whose capacity exceeds its length
static void test_gqa_attention(const GpuContext &gpu) {
    std::printf("test_gqa_attention\n");
    const size_t nqh = 4, nkvh = 2, seq_q = 2, seq_kv = 3, hd = 4;
    std::vector<float> q(nqh * seq_q * hd), k(nkvh * seq_kv * hd), v(nkvh * seq_kv * hd);
    for (size_t i = 0; i < q.size(); ++i) q[i] = std::sin((float)i * 0.1f);
    for (size_t i = 0; i < k.size(); ++i) { k[i] = std::cos((float)i * 0.2f); v[i] = std::sin((float)i * 0.15f); }
    llama::StandardKVCache cache(gpu, nkvh, hd);
    cache.append(k, v, seq_kv);
    EXPECT(cache.len() == seq_kv && cache.head_stride() == 32 * hd, "len %zu stride %zu", cache.len(), cache.head_stride());
    const float scale = 1.0f / std::sqrt((float)hd);
    for (const auto &mask : {llama::AttentionMask::None(), llama::AttentionMask::Causal(1)}) {
        std::vector<float> out(seq_q * nqh * hd, 0.0f), ref(out.size(), 0.0f);
        llama::gqa_attention(gpu, q, cache, cache, nqh, nkvh, seq_q, hd, scale, mask, 0.0f, out);
        orc_gqa_attention(q.data(), k.data(), v.data(), seq_kv, seq_kv, nqh, nkvh, seq_q, hd, scale, mask.kind, mask.offset, 0, 0,
                          0.0f, ref.data());
        for (size_t i = 0; i < ref.size(); ++i)
            EXPECT(std::fabs(out[i] - ref[i]) <= 1e-5f, "mask %d [%zu]: %g vs %g", mask.kind, i, out[i], ref[i]);
    }
    bool threw = false;
    try { cache.rollback_to(4); } catch (const Panic &) { threw = true; }
    EXPECT(threw, "rollback_to beyond len must panic (src/attention.rs:88)");
}

// LlamaBlock::forward: a prefill of 3 then a decode step against the CPU composition
static void test_llama_block(const GpuContext &gpu) {
    std::printf("test_llama_block\n");
    const size_t d = 128, nqh = 4, nkvh = 2, hd = 32, ffn = 256, cap = 16;
    const size_t shp[7][2] = {{nqh * hd, d}, {nkvh * hd, d}, {nkvh * hd, d}, {d, nqh * hd}, {ffn, d}, {ffn, d}, {d, ffn}};
    uint32_t s = 7;
    auto next = [&]() { s = s * 1103515245u + 12345u; return s; };
    std::vector<std::vector<uint8_t>> raw(7);
    std::vector<std::unique_ptr<gguf::BlockWeight>> w;
    for (int i = 0; i < 7; ++i) {
        const size_t nb = shp[i][0] * shp[i][1] / 32;
        raw[i].resize(nb * 34);
        for (size_t b = 0; b < nb; ++b) {
            const uint16_t dd = (uint16_t)(0x1400 + (b * 37) % 0x0400);  // halves near 1e-3: products stay O(1)
            raw[i][b * 34] = (uint8_t)(dd & 0xFF); raw[i][b * 34 + 1] = (uint8_t)(dd >> 8);
            for (size_t j = 2; j < 34; ++j) raw[i][b * 34 + j] = (uint8_t)(next() >> 16);
        }
        w.emplace_back(new gguf::BlockWeight(gpu, raw[i], PG_GGML_Q8_0, shp[i][0], shp[i][1]));
    }
    std::vector<float> wa(d), wf(d);
    for (size_t i = 0; i < d; ++i) { wa[i] = 1.0f + 0.01f * (float)(i % 7); wf[i] = 1.0f - 0.01f * (float)(i % 5); }
    llama::LlamaBlock blk(gpu, d, nqh, nkvh, hd, ffn, cap, 10000.0f, 1e-5f);
    blk.set_weights(*w[0], *w[1], *w[2], *w[3], *w[4], *w[5], *w[6], wa, wf);
    llama::KVCache cache(gpu, nkvh, hd);
    std::vector<float> cos_t(cap * hd), sin_t(cap * hd), kc(nkvh * cap * hd, 0.0f), vc(nkvh * cap * hd, 0.0f);
    orc_rope_tables(hd, cap, 10000.0f, cos_t.data(), sin_t.data());
    size_t pos = 0;
    for (size_t seq : {(size_t)3, (size_t)1}) {
        std::vector<float> h(seq * d), ref(seq * d);
        for (auto &x : h) x = (float)next() / 4294967295.0f * 2.0f - 1.0f;
        auto out = blk.forward(h, seq, cache);
        const int rc = orc_llama_block_forward(h.data(), seq, d, nqh, nkvh, hd, ffn, PG_GGML_Q8_0, raw[0].data(), raw[1].data(),
                                               raw[2].data(), raw[3].data(), raw[4].data(), raw[5].data(), raw[6].data(),
                                               wa.data(), wf.data(), 1e-5f, cos_t.data(), sin_t.data(), kc.data(), vc.data(),
                                               pos, cap, ref.data());
        EXPECT(rc == 0, "oracle rc %d", rc);
        pos += seq;
        EXPECT(cache.len() == pos, "cache len %zu", cache.len());
        double rms = 0;
        for (float x : ref) rms += (double)x * x;
        rms = std::sqrt(rms / ref.size());
        for (size_t i = 0; i < ref.size(); ++i) {
            const double tol = 1e-3 * std::fmax(std::fabs((double)ref[i]), rms);
            EXPECT(std::fabs((double)out[i] - ref[i]) <= tol, "seq %zu [%zu]: %g vs %g", seq, i, out[i], ref[i]);
        }
    }
}

// tests/huffman_parity.rs:23-42: Huffman-coded weights give the same product as the plain
// quantised ones (here: bit for bit), through a round trip of the coded tensor
static void test_huffman_matmul(const GpuContext &gpu) {
    std::printf("test_huffman_matmul\n");
    const size_t shapes[4][3] = {{8, 32, 16}, {1, 64, 1}, {32, 128, 64}, {16, 256, 32}};
    for (const auto &sh : shapes) {
        const size_t m = sh[0], k = sh[1], n = sh[2];
        uint32_t sa = 42, sw = 123;
        auto lcg = [](uint32_t &st) { st = st * 1103515245u + 12345u; return (float)st / 4294967295.0f * 2.0f - 1.0f; };
        std::vector<float> a(m * k), w(k * n);
        for (auto &v : a) v = lcg(sa);
        for (auto &v : w) v = lcg(sw);
        auto qt = quant::quantize_weights(gpu, w, k, n);
        auto ht = huffman::HuffmanTensor::from_quantized(qt, 4);
        auto back = ht.decode_to_quantized(gpu);
        EXPECT(back.data_i8 == qt.data_i8 && back.data_i8_t == qt.data_i8_t && same_bits(back.scales, qt.scales), "round trip m=%zu", m);
        auto ref = quant::matmul_quantized(gpu, a, m, k, qt);
        auto got = huffman::matmul_huffman(gpu, a, m, k, ht);
        EXPECT(same_bits(ref, got), "matmul_huffman differs from matmul_quantized at M=%zu K=%zu N=%zu", m, k, n);
    }
    // src/huffman.rs:780-797: one symbol, 512 times, in at most 65 bytes
    std::vector<uint64_t> freqs(256, 0);
    freqs[42 + 128] = 512;
    auto table = huffman::HuffmanTable::from_frequencies(freqs);
    std::vector<int8_t> same(512, 42);
    auto enc = table.encode(same);
    EXPECT(enc.size() <= 65, "encoded %zu bytes", enc.size());
    EXPECT(table.decode(gpu, enc, 512) == same, "one-symbol round trip");
}

// src/huffman.rs:850-905 and tests/huffman_parity.rs:133-186: the compressed KV cache, checked bit
// for bit against the CPU restatement
static void test_huffman_kv_cache(const GpuContext &gpu) {
    std::printf("test_huffman_kv_cache\n");
    auto lcg = [](uint32_t &st) { st = st * 1103515245u + 12345u; return (float)st / 4294967295.0f * 2.0f - 1.0f; };
    {
        const size_t heads = 4, hd = 16, tokens = 32, n = heads * tokens * hd;
        uint32_t st = 99;
        std::vector<float> data(n);
        for (auto &v : data) v = lcg(st);
        auto chunk = huffman::HuffmanKVCache::compress_chunk(gpu, data, tokens, heads, hd);
        std::vector<uint8_t> bits(2 * n + 16), codebook(256);
        std::vector<float> scales(heads), ref(n);
        bits.resize(orc_huffman_kv_compress_chunk(data.data(), tokens, heads, hd, bits.data(), scales.data(), codebook.data(), nullptr));
        EXPECT(chunk.bitstream() == bits && chunk.codebook() == codebook && same_bits(chunk.scales(), scales), "compress_chunk differs");
        auto rec = huffman::HuffmanKVCache::decompress_chunk(gpu, chunk);
        orc_huffman_kv_decompress_chunk(bits.data(), bits.size(), scales.data(), codebook.data(), tokens, heads, hd, ref.data());
        EXPECT(same_bits(rec, ref), "decompress_chunk differs");
        for (size_t h = 0; h < heads; ++h)
            for (size_t i = 0; i < tokens * hd; ++i)
                EXPECT(std::fabs(data[h * tokens * hd + i] - rec[h * tokens * hd + i]) <= scales[h] + 1e-5f, "head %zu idx %zu", h, i);
    }
    {
        huffman::HuffmanKVCache cache(gpu, 2, 4, 8, 4);
        cache.append(std::vector<float>(32, 1.0f), std::vector<float>(32, 2.0f), 4);
        EXPECT(cache.len() == 4 && cache.compressed_len() == 0, "after 4 tokens");
        cache.append(std::vector<float>(32, 3.0f), std::vector<float>(32, 4.0f), 4);
        EXPECT(cache.len() == 8 && cache.compressed_len() == 4, "after 8 tokens");
        auto kv = cache.get_kv();
        EXPECT(kv.first.size() == 2 * 8 * 4 && kv.second.size() == 2 * 8 * 4, "get_kv sizes");
    }
    {
        const size_t heads = 2, hd = 8;
        huffman::HuffmanKVCache cache(gpu, heads, hd, 16, 8);
        void *orc = orc_huffman_kv_new(heads, hd, 16, 8);
        for (uint32_t batch = 0; batch < 4; ++batch) {
            uint32_t sk = 100 + batch, sv = 200 + batch;
            std::vector<float> k(heads * 8 * hd), v(heads * 8 * hd);
            for (auto &x : k) x = lcg(sk);
            for (auto &x : v) x = lcg(sv);
            cache.append(k, v, 8);
            orc_huffman_kv_append(orc, k.data(), v.data(), 8);
        }
        EXPECT(cache.len() == 32 && cache.compressed_len() > 0 && cache.compressed_len() == orc_huffman_kv_stat(orc, 1), "lengths");
        auto kv = cache.get_kv();
        std::vector<float> rk(heads * 32 * hd), rv(heads * 32 * hd);
        orc_huffman_kv_get_kv(orc, 0, rk.data(), rv.data());
        EXPECT(same_bits(kv.first, rk) && same_bits(kv.second, rv), "get_kv differs");
        orc_huffman_kv_free(orc);
    }
    bool threw = false;
    try { huffman::HuffmanKVCache::compress_chunk(gpu, std::vector<float>(5), 1, 2, 3); } catch (const Panic &) { threw = true; }
    EXPECT(threw, "data.len() != total must panic (src/huffman.rs:619)");
}

// The expert FFNs behind a routing the caller made (examples/deepseek/moe.rs:271-300, examples/gpt_oss/moe.rs:286-352),
// against the CPU restatement's per-token walk.
static void test_moe_routed(const GpuContext &gpu) {
    std::printf("test_moe_routed\n");
    auto lcg = [](uint32_t &st) { st = st * 1103515245u + 12345u; return (float)st / 4294967295.0f * 2.0f - 1.0f; };
    auto rel_err = [](const std::vector<float> &got, const std::vector<float> &want) {
        double num = 0, den = 0;
        for (size_t i = 0; i < got.size(); ++i) { num = std::fmax(num, std::fabs((double)got[i] - want[i])); den += (double)want[i] * want[i]; }
        return num / std::fmax(std::sqrt(den / (double)got.size()), 1e-30);
    };
    const size_t T = 9, E = 6, top_k = 2;
    uint32_t st = 7;
    std::vector<float> logits(T * E), zero_bias(E, 0.0f), w(T * top_k);
    for (auto &v : logits) v = 3.0f * lcg(st);
    std::vector<int32_t> idx(T * top_k);
    orc_gpt_oss_route(logits.data(), zero_bias.data(), T, E, top_k, idx.data(), w.data());
    std::vector<std::vector<std::pair<size_t, float>>> routing(T);
    for (size_t t = 0; t < T; ++t)
        for (size_t k = 0; k < top_k; ++k) routing[t].push_back({(size_t)idx[t * top_k + k], w[t * top_k + k]});
    {   // Q8_0 experts, SiLU, with a shared-expert term
        const size_t d = 64, ffn = 96;
        auto blocks = [&](size_t n_out, size_t k_in) {
            std::vector<uint8_t> b(n_out * k_in / 32 * 34);
            for (size_t i = 0; i < b.size(); i += 34) {
                b[i] = 0x00; b[i + 1] = 0x1E + (uint8_t)((i / 34) % 3);   // f16 scales around 2^-8
                for (size_t j = 2; j < 34; ++j) { st = st * 1103515245u + 12345u; b[i + j] = (uint8_t)(st >> 24); }
            }
            return b;
        };
        std::vector<std::vector<uint8_t>> raw[3];
        std::vector<std::unique_ptr<gguf::BlockWeight>> own;
        std::vector<const gguf::BlockWeight *> tabs[3];
        std::vector<const uint8_t *> rp[3];
        for (int which = 0; which < 3; ++which)
            for (size_t e = 0; e < E; ++e) {
                raw[which].push_back(which == 2 ? blocks(d, ffn) : blocks(ffn, d));
                own.push_back(std::make_unique<gguf::BlockWeight>(gpu, raw[which].back(), 8, which == 2 ? d : ffn, which == 2 ? ffn : d));
                tabs[which].push_back(own.back().get());
            }
        for (int which = 0; which < 3; ++which)
            for (size_t e = 0; e < E; ++e) rp[which].push_back(raw[which][e].data());
        std::vector<float> x(T * d), shared(T * d), want(T * d);
        for (auto &v : x) v = lcg(st);
        for (auto &v : shared) v = 0.1f * lcg(st);
        auto got = moe::expert_ffn_routed(gpu, x, routing, tabs[0], tabs[1], tabs[2], PG_ACT_SILU, shared);
        EXPECT(orc_moe_ffn_routed(x.data(), T, d, ffn, E, top_k, idx.data(), w.data(), rp[0].data(), rp[1].data(), rp[2].data(), 8, 0,
                                  shared.data(), want.data()) == 0, "oracle");
        EXPECT(rel_err(got, want) < 4e-4, "expert_ffn_routed: %.3g of the rms", rel_err(got, want));
        bool threw = false;
        auto bad = routing;
        bad[3][1].first = E;
        try { moe::expert_ffn_routed(gpu, x, bad, tabs[0], tabs[1], tabs[2], PG_ACT_SILU); } catch (const Panic &) { threw = true; }
        EXPECT(threw, "an expert index out of range must panic");
    }
    {   // MXFP4 experts
        const size_t hidden = 64, inter = 96;
        const float alpha = 1.702f, clamp = 7.0f;
        auto bytes = [&](size_t n, uint8_t lo, uint8_t span) {
            std::vector<uint8_t> b(n);
            for (auto &v : b) { st = st * 1103515245u + 12345u; v = (uint8_t)(lo + (st >> 24) % span); }
            return b;
        };
        std::vector<std::vector<uint8_t>> b1, s1, b2, s2;
        std::vector<std::vector<float>> bias1, bias2;
        std::vector<std::unique_ptr<mxfp4::Mxfp4Expert>> own;
        std::vector<const mxfp4::Mxfp4Expert *> tab;
        for (size_t e = 0; e < E; ++e) {
            b1.push_back(bytes(2 * inter * hidden / 2, 0, 255));
            s1.push_back(bytes(2 * inter * hidden / 32, 118, 6));     // E8M0 scales 2^-9 .. 2^-4
            b2.push_back(bytes(hidden * inter / 2, 0, 255));
            s2.push_back(bytes(hidden * inter / 32, 118, 6));
            bias1.emplace_back(2 * inter);
            bias2.emplace_back(hidden);
            for (auto &v : bias1.back()) v = 0.2f * lcg(st);
            for (auto &v : bias2.back()) v = 0.2f * lcg(st);
            own.push_back(std::make_unique<mxfp4::Mxfp4Expert>(gpu, hidden, inter, alpha, clamp, b1[e], s1[e], b2[e], s2[e], bias1[e], bias2[e]));
            tab.push_back(own.back().get());
        }
        std::vector<const uint8_t *> pb1, ps1, pb2, ps2;
        std::vector<const float *> pbi1, pbi2;
        for (size_t e = 0; e < E; ++e) {
            pb1.push_back(b1[e].data()); ps1.push_back(s1[e].data()); pb2.push_back(b2[e].data()); ps2.push_back(s2[e].data());
            pbi1.push_back(bias1[e].data()); pbi2.push_back(bias2[e].data());
        }
        std::vector<float> x(T * hidden), want(T * hidden);
        for (auto &v : x) v = lcg(st);
        auto got = mxfp4::moe_forward_routed(gpu, x, routing, tab);
        EXPECT(orc_mxfp4_moe_routed(x.data(), T, hidden, inter, alpha, clamp, E, top_k, idx.data(), w.data(), pb1.data(), ps1.data(),
                                    pb2.data(), ps2.data(), pbi1.data(), pbi2.data(), want.data()) == 0, "oracle");
        EXPECT(rel_err(got, want) < 2e-4, "mxfp4 moe_forward_routed: %.3g of the rms", rel_err(got, want));
        // one token, one expert: the layer is weight * expert.forward(x)
        std::vector<float> x0(x.begin(), x.begin() + hidden);
        auto alone = tab[2]->forward(x0);
        auto one = mxfp4::moe_forward_routed(gpu, x0, {{{2, 0.5f}}}, tab);
        double worst = 0;
        for (size_t i = 0; i < hidden; ++i) worst = std::fmax(worst, std::fabs(one[i] - 0.5f * alone[i]));
        EXPECT(worst < 1e-5, "one pair against the expert alone: %.3g", worst);
    }
}

int main() {
    try {
        GpuContext gpu(0);
        test_quantize_dequantize_roundtrip(gpu);
        test_quantized_matmul_accuracy(gpu, 32, 128, 64, 200);
        test_quantized_matmul_accuracy(gpu, 16, 64, 32, 100);
        test_quantized_matmul_accuracy(gpu, 1, 64, 1, 200);
        test_quantize_activations(gpu);
        test_shape_panics(gpu);
        test_gguf_known_answers(gpu);
        test_block_weight_matmul(gpu);
        test_gqa_attention(gpu);
        test_llama_block(gpu);
        test_huffman_matmul(gpu);
        test_huffman_kv_cache(gpu);
        test_moe_routed(gpu);
    } catch (const std::exception &e) {
        std::printf("FAIL: uncaught %s\n", e.what());
        return 2;
    }
    std::printf(failures ? "FAILED: %d check(s)\n" : "OK: all checks passed\n", failures);
    return failures ? 1 : 0;
}
