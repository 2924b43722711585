// peregrine_hip.hpp -- C++ host-side mirror of peregrine's quantized-inference API
// on top of the C ABI in peregrine_hip.h.
//
// Names, argument order and meaning follow the reference's Rust surface:
//   peregrine::quant::{QuantizedTensor, quantize_weights, quantize_activations,
//                      dequantize, matmul_quantized, matmul_quantized_gpu}   src/quant.rs:12-218
//   peregrine::gguf::{f16_to_f32, dequant_q8_0, dequant_q4_0, dequant_q4_1,
//                     load_tensor_q8_as_quantized}                           src/gguf.rs:286-401
// The reference panics (assert!/expect) on shape mismatch; here the same
// conditions throw peregrine::Panic carrying the library's message.  Outputs
// are freshly allocated vectors owned by the caller, like the reference's Vec.
// Header-only; link with -lperegrine_hip.
#ifndef PEREGRINE_HIP_HPP
#define PEREGRINE_HIP_HPP

#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "peregrine_hip.h"

namespace peregrine {

// Stands in for a Rust panic crossing the API.
struct Panic : std::runtime_error {
    pg_status status;
    Panic(pg_status st, const std::string &what) : std::runtime_error(what), status(st) {}
};

inline void check(pg_status st, const char *what) {
    if (st != PG_OK)
        throw Panic(st, std::string(what) + ": " + pg_status_string(st) + ": " + pg_last_error());
}

// GpuContext (src/metal/context.rs:2472-2510): one device, one stream.
class GpuContext {
public:
    explicit GpuContext(int device = 0, void *hip_stream = nullptr) {
        check(pg_ctx_create(device, hip_stream, &ctx_), "GpuContext::new");
    }
    ~GpuContext() { pg_ctx_destroy(ctx_); }
    GpuContext(const GpuContext &) = delete;
    GpuContext &operator=(const GpuContext &) = delete;
    void sync() const { check(pg_sync(ctx_), "GpuContext::sync"); }
    pg_ctx *raw() const { return ctx_; }

private:
    pg_ctx *ctx_ = nullptr;
};

// GpuBuffer<T> (src/metal/buffer.rs): device memory owned by the object.
template <typename T>
class GpuBuffer {
public:
    GpuBuffer(const GpuContext &gpu, size_t len) : gpu_(&gpu), len_(len) {
        check(pg_dev_alloc(gpu.raw(), len * sizeof(T), &ptr_), "GpuBuffer::alloc");
    }
    ~GpuBuffer() { if (ptr_) pg_dev_free(gpu_->raw(), ptr_); }
    GpuBuffer(GpuBuffer &&o) noexcept : gpu_(o.gpu_), ptr_(o.ptr_), len_(o.len_) { o.ptr_ = nullptr; }
    GpuBuffer(const GpuBuffer &) = delete;
    GpuBuffer &operator=(const GpuBuffer &) = delete;
    size_t len() const { return len_; }
    T *device_ptr() const { return static_cast<T *>(ptr_); }
    void upload(const T *src) { check(pg_memcpy_h2d(gpu_->raw(), ptr_, src, len_ * sizeof(T)), "GpuBuffer::upload"); }
    // GpuBuffer::read: the caller syncs first (tests/quant_parity.rs:102-107); the copy itself is synchronous.
    std::vector<T> read() const {
        std::vector<T> out(len_);
        check(pg_memcpy_d2h(gpu_->raw(), out.data(), ptr_, len_ * sizeof(T)), "GpuBuffer::read");
        return out;
    }

private:
    const GpuContext *gpu_;
    void *ptr_ = nullptr;
    size_t len_;
};

namespace quant {

// quant::QuantizedTensor  src/quant.rs:12-23
struct QuantizedTensor {
    std::vector<int8_t> data_i8;    // [rows, cols] row-major
    std::vector<int8_t> data_i8_t;  // [cols, rows]
    std::vector<float> scales;      // [cols]
    size_t rows = 0, cols = 0;

    // QuantizedTensor::to_gpu  src/quant.rs:174-181 (idempotent)
    void to_gpu(const GpuContext &gpu) {
        if (gpu_) return;
        pg_qtensor *h = nullptr;
        check(pg_qtensor_upload(gpu.raw(), data_i8.data(), scales.data(), rows, cols, &h), "QuantizedTensor::to_gpu");
        pg_ctx *c = gpu.raw();
        gpu_ = std::shared_ptr<pg_qtensor>(h, [c](pg_qtensor *t) { pg_qtensor_free(c, t); });
    }
    // QuantizedTensor::from_gpu  src/quant.rs:183-190
    void from_gpu(const GpuContext &gpu) {
        if (!gpu_) return;
        check(pg_qtensor_download(gpu.raw(), gpu_.get(), data_i8.data(), data_i8_t.data(), scales.data()),
              "QuantizedTensor::from_gpu");
    }
    bool on_gpu() const { return (bool)gpu_; }
    const pg_qtensor *gpu_handle() const { return gpu_.get(); }

private:
    std::shared_ptr<pg_qtensor> gpu_;
};

// quant::quantize_weights  src/quant.rs:27-75
inline QuantizedTensor quantize_weights(const GpuContext &gpu, const std::vector<float> &data, size_t rows, size_t cols) {
    if (data.size() != rows * cols) throw Panic(PG_EINVAL, "quantize_weights: data.len() != rows * cols");
    QuantizedTensor qt;
    qt.rows = rows; qt.cols = cols;
    qt.data_i8.resize(rows * cols); qt.data_i8_t.resize(rows * cols); qt.scales.resize(cols);
    check(pg_quantize_weights(gpu.raw(), data.data(), rows, cols, qt.data_i8.data(), qt.data_i8_t.data(), qt.scales.data()),
          "quantize_weights");
    return qt;
}

// quant::quantize_activations  src/quant.rs:79-112
inline std::pair<std::vector<int8_t>, std::vector<float>> quantize_activations(const GpuContext &gpu, const std::vector<float> &data,
                                                                                size_t rows, size_t cols) {
    if (data.size() != rows * cols) throw Panic(PG_EINVAL, "quantize_activations: data.len() != rows * cols");
    std::vector<int8_t> q(rows * cols);
    std::vector<float> s(rows);
    check(pg_quantize_activations(gpu.raw(), data.data(), rows, cols, q.data(), s.data()), "quantize_activations");
    return {std::move(q), std::move(s)};
}

// quant::dequantize  src/quant.rs:115-123
inline std::vector<float> dequantize(const GpuContext &gpu, const QuantizedTensor &qt) {
    std::vector<float> out(qt.rows * qt.cols);
    check(pg_dequantize(gpu.raw(), qt.data_i8.data(), qt.scales.data(), qt.rows, qt.cols, out.data()), "dequantize");
    return out;
}

// quant::matmul_quantized  src/quant.rs:129-169.  The reference computes this on the CPU; here the
// weights are uploaded on first use and the product runs on the device with identical results.
inline std::vector<float> matmul_quantized(const GpuContext &gpu, const std::vector<float> &a, size_t m, size_t k, QuantizedTensor &w) {
    if (w.rows != k) throw Panic(PG_EINVAL, "matmul_quantized: weight rows must equal k");
    if (a.size() != m * k) throw Panic(PG_EINVAL, "matmul_quantized: a.len() != m * k");
    w.to_gpu(gpu);
    std::vector<float> out(m * w.cols);
    check(pg_matmul_quantized(gpu.raw(), a.data(), m, k, w.gpu_handle(), out.data()), "matmul_quantized");
    return out;
}

// quant::matmul_quantized_gpu  src/quant.rs:196-218: uploads a, returns an UNSYNCED device buffer.
inline GpuBuffer<float> matmul_quantized_gpu(const GpuContext &gpu, const std::vector<float> &a, size_t m, size_t k,
                                             const QuantizedTensor &w) {
    if (w.rows != k) throw Panic(PG_EINVAL, "matmul_quantized_gpu: weight rows must equal k");
    if (a.size() != m * k) throw Panic(PG_EINVAL, "matmul_quantized_gpu: a.len() != m * k");
    if (!w.on_gpu()) throw Panic(PG_EINVAL, "weights not on GPU");  // .expect() at src/quant.rs:208-209
    GpuBuffer<float> a_buf(gpu, m * k), out(gpu, m * w.cols);
    a_buf.upload(a.data());
    check(pg_matmul_quantized_dev(gpu.raw(), a_buf.device_ptr(), m, k, w.gpu_handle(), out.device_ptr(), nullptr),
          "matmul_quantized_gpu");
    gpu.sync();  // a_buf is released on return; the product must have consumed it
    return out;
}

// The reference's GPU numerics (W8A32) for the same product: f32 activations, dequantised
// weights, f32 accumulate (dispatch_matmul_dequant_i8, src/metal/context.rs:2226-2306).
inline std::vector<float> matmul_dequant_i8(const GpuContext &gpu, const std::vector<float> &a, size_t m, size_t k, QuantizedTensor &w) {
    if (w.rows != k) throw Panic(PG_EINVAL, "matmul_dequant_i8: weight rows must equal k");
    if (a.size() != m * k) throw Panic(PG_EINVAL, "matmul_dequant_i8: a.len() != m * k");
    w.to_gpu(gpu);
    std::vector<float> out(m * w.cols);
    check(pg_matmul_dequant_i8(gpu.raw(), a.data(), m, k, w.gpu_handle(), out.data()), "matmul_dequant_i8");
    return out;
}

}  // namespace quant

namespace gguf {

// GGML block sizes  src/gguf.rs:47-55
constexpr size_t Q8_0_BLOCK_BYTES = 34, Q4_0_BLOCK_BYTES = 18, Q4_1_BLOCK_BYTES = 20, BLOCK_ELEMS = 32;

// gguf::f16_to_f32  src/gguf.rs:354-382
inline float f16_to_f32(const GpuContext &gpu, uint16_t bits) {
    float out;
    check(pg_f16_to_f32(gpu.raw(), &bits, 1, &out), "f16_to_f32");
    return out;
}

#define PEREGRINE_DEQUANT(name, bytes)                                                                        \
    inline std::vector<float> name(const GpuContext &gpu, const std::vector<uint8_t> &data, size_t n) {      \
        if (n % BLOCK_ELEMS != 0) throw Panic(PG_EINVAL, #name ": num_elements must be a multiple of 32");   \
        if (data.size() < n / BLOCK_ELEMS * (bytes)) throw Panic(PG_EINVAL, #name ": data too short");       \
        std::vector<float> out(n);                                                                            \
        check(pg_##name(gpu.raw(), data.data(), n, out.data()), #name);                                       \
        return out;                                                                                           \
    }
PEREGRINE_DEQUANT(dequant_q8_0, Q8_0_BLOCK_BYTES)  // src/gguf.rs:286-302
PEREGRINE_DEQUANT(dequant_q4_0, Q4_0_BLOCK_BYTES)  // src/gguf.rs:307-326
PEREGRINE_DEQUANT(dequant_q4_1, Q4_1_BLOCK_BYTES)  // src/gguf.rs:331-351
#undef PEREGRINE_DEQUANT

// gguf::load_tensor_q8_as_quantized  src/gguf.rs:386-401: Q8_0 -> f32 -> quantize_weights.
inline quant::QuantizedTensor load_tensor_q8_as_quantized(const GpuContext &gpu, const std::vector<uint8_t> &data, size_t rows,
                                                          size_t cols) {
    return quant::quantize_weights(gpu, dequant_q8_0(gpu, data, rows * cols), rows, cols);
}

// A GGUF weight kept block-quantised on the device; matmul() is the fused form of
// dequantise + transpose + Tensor::matmul (src/models/llama/model.rs:243-257, src/tensor.rs:1342-1353).
class BlockWeight {
public:
    BlockWeight(const GpuContext &gpu, const std::vector<uint8_t> &blocks, int ggml_type, size_t n_out, size_t k_in) : gpu_(&gpu) {
        check(pg_gguf_upload(gpu.raw(), blocks.data(), ggml_type, n_out, k_in, &h_), "BlockWeight::upload");
        n_out_ = n_out; k_in_ = k_in;
    }
    ~BlockWeight() { if (h_) pg_gguf_free(gpu_->raw(), h_); }
    BlockWeight(const BlockWeight &) = delete;
    BlockWeight &operator=(const BlockWeight &) = delete;
    std::vector<float> matmul(const std::vector<float> &x, size_t m) const {
        if (x.size() != m * k_in_) throw Panic(PG_EINVAL, "BlockWeight::matmul: x.len() != m * k_in");
        std::vector<float> y(m * n_out_);
        check(pg_gguf_matmul(gpu_->raw(), x.data(), m, h_, y.data()), "BlockWeight::matmul");
        return y;
    }
    // The load-time step: make now the derived device copies that products over up to `max_rows` rows need
    // (afterwards those products neither allocate nor wait).
    void prepare(size_t max_rows) { check(pg_gguf_prepare(gpu_->raw(), h_, max_rows), "BlockWeight::prepare"); }
    const pg_gguf_tensor *handle() const { return h_; }
    size_t n_out() const { return n_out_; }
    size_t k_in() const { return k_in_; }

private:
    const GpuContext *gpu_;
    pg_gguf_tensor *h_ = nullptr;
    size_t n_out_ = 0, k_in_ = 0;
};

// gguf::GgufFile  src/gguf.rs:166-171, 403-561.  parse() borrows the buffer; load() maps the file.
class GgufFile {
public:
    static GgufFile parse(const std::vector<uint8_t> &data) {
        pg_gguf_file *f = nullptr;
        check(pg_gguf_file_parse(data.data(), data.size(), &f), "GgufFile::parse");
        return GgufFile(f);
    }
    static GgufFile load(const std::string &path) {
        pg_gguf_file *f = nullptr;
        check(pg_gguf_file_open(path.c_str(), &f), "GgufFile::load");
        return GgufFile(f);
    }
    ~GgufFile() { pg_gguf_file_close(f_); }
    GgufFile(GgufFile &&o) noexcept : f_(o.f_) { o.f_ = nullptr; }
    GgufFile(const GgufFile &) = delete;
    GgufFile &operator=(const GgufFile &) = delete;

    std::vector<std::string> tensor_names() const {  // src/gguf.rs:559-561
        size_t n = 0;
        check(pg_gguf_file_counts(f_, &n, nullptr, nullptr, nullptr), "GgufFile::tensor_names");
        std::vector<std::string> out;
        for (size_t i = 0; i < n; ++i) {
            const char *nm = nullptr;
            check(pg_gguf_file_tensor_name(f_, i, &nm), "GgufFile::tensor_names");
            out.emplace_back(nm);
        }
        return out;
    }
    // Peregrine order: GGUF's shape reversed  src/gguf.rs:551-556
    std::vector<size_t> tensor_shape(const std::string &name) const {
        uint64_t shape[8];
        size_t nd = 0;
        check(pg_gguf_file_tensor_info(f_, name.c_str(), nullptr, &nd, shape, 8, nullptr, nullptr, nullptr), "GgufFile::tensor_shape");
        std::vector<size_t> out;
        for (size_t i = nd; i-- > 0;) out.push_back((size_t)shape[i]);
        return out;
    }
    bool get_u32(const std::string &key, uint32_t *v) const {  // src/gguf.rs:541-543
        int found = 0;
        check(pg_gguf_file_get_u32(f_, key.c_str(), v, &found), "GgufFile::get_u32");
        return found != 0;
    }
    bool get_f32(const std::string &key, float *v) const {  // src/gguf.rs:546-548
        int found = 0;
        check(pg_gguf_file_get_f32(f_, key.c_str(), v, &found), "GgufFile::get_f32");
        return found != 0;
    }
    std::vector<float> load_tensor_f32(const GpuContext &gpu, const std::string &name) const {  // src/gguf.rs:485-517
        size_t n = 1;
        for (size_t d : tensor_shape(name)) n *= d;
        std::vector<float> out(n);
        check(pg_gguf_file_load_tensor_f32(gpu.raw(), f_, name.c_str(), out.data(), n), "GgufFile::load_tensor_f32");
        return out;
    }
    quant::QuantizedTensor load_tensor_q8(const GpuContext &gpu, const std::string &name) const {  // src/gguf.rs:521-537
        const std::vector<size_t> shape = tensor_shape(name);  // [rows, cols] after the reversal
        if (shape.size() != 1 && shape.size() != 2) throw Panic(PG_EINVAL, "expected 1D or 2D tensor for q8 load");
        const size_t rows = shape.size() == 2 ? shape[0] : 1, cols = shape.back();
        return quant::quantize_weights(gpu, load_tensor_f32(gpu, name), rows, cols);
    }
    const pg_gguf_file *raw() const { return f_; }

private:
    explicit GgufFile(pg_gguf_file *f) : f_(f) {}
    pg_gguf_file *f_;
};

}  // namespace gguf

namespace moe {

// MoELayer::forward after the router matmul  examples/grok1/moe.rs:70-109.
inline std::vector<float> expert_ffn(const GpuContext &gpu, const std::vector<float> &x, size_t tokens,
                                     const std::vector<float> &router_logits, size_t top_k,
                                     const std::vector<const gguf::BlockWeight *> &gate,
                                     const std::vector<const gguf::BlockWeight *> &up,
                                     const std::vector<const gguf::BlockWeight *> &down, int act) {
    const size_t E = gate.size();
    if (E == 0 || up.size() != E || down.size() != E) throw Panic(PG_EINVAL, "expert_ffn: expert tables differ in length");
    std::vector<const pg_gguf_tensor *> g(E), u(E), d(E);
    for (size_t e = 0; e < E; ++e) { g[e] = gate[e]->handle(); u[e] = up[e]->handle(); d[e] = down[e]->handle(); }
    const size_t dm = gate[0]->k_in();
    if (x.size() != tokens * dm || router_logits.size() != tokens * E) throw Panic(PG_EINVAL, "expert_ffn: input sizes");
    std::vector<float> out(tokens * dm);
    check(pg_moe_ffn(gpu.raw(), x.data(), tokens, router_logits.data(), E, top_k, g.data(), u.data(), d.data(), act, out.data()),
          "expert_ffn");
    return out;
}

// The same expert FFN over a routing another gate made: routing[t] = the token's (expert, weight) pairs, as
// Gate::forward returns them (examples/deepseek/moe.rs:111-215, 271-297; the gpt_oss router,
// examples/gpt_oss/moe.rs:298-330, gives the same per token).  Every token names the same number of experts.
// `shared`, if not empty: the shared experts' output [tokens, d], added last (examples/deepseek/moe.rs:298-300).
inline std::vector<float> expert_ffn_routed(const GpuContext &gpu, const std::vector<float> &x,
                                            const std::vector<std::vector<std::pair<size_t, float>>> &routing,
                                            const std::vector<const gguf::BlockWeight *> &gate,
                                            const std::vector<const gguf::BlockWeight *> &up,
                                            const std::vector<const gguf::BlockWeight *> &down, int act,
                                            const std::vector<float> &shared = {}) {
    const size_t E = gate.size(), tokens = routing.size();
    if (E == 0 || up.size() != E || down.size() != E) throw Panic(PG_EINVAL, "expert_ffn_routed: expert tables differ in length");
    std::vector<const pg_gguf_tensor *> g(E), u(E), d(E);
    for (size_t e = 0; e < E; ++e) { g[e] = gate[e]->handle(); u[e] = up[e]->handle(); d[e] = down[e]->handle(); }
    const size_t dm = gate[0]->k_in(), top_k = tokens ? routing[0].size() : 1;
    if (x.size() != tokens * dm || (!shared.empty() && shared.size() != tokens * dm)) throw Panic(PG_EINVAL, "expert_ffn_routed: input sizes");
    std::vector<int32_t> idx;
    std::vector<float> w;
    for (const auto &r : routing) {
        if (r.size() != top_k) throw Panic(PG_EINVAL, "expert_ffn_routed: tokens name different numbers of experts");
        for (const auto &pr : r) { idx.push_back((int32_t)pr.first); w.push_back(pr.second); }
    }
    std::vector<float> out(tokens * dm);
    check(pg_moe_ffn_routed(gpu.raw(), x.data(), tokens, idx.data(), w.data(), E, top_k, g.data(), u.data(), d.data(), act,
                            shared.empty() ? nullptr : shared.data(), out.data()),
          "expert_ffn_routed");
    return out;
}

}  // namespace moe

namespace llama {

// nn::RMSNorm  src/nn.rs:560-652.
class RMSNorm {
public:
    RMSNorm(const GpuContext &gpu, size_t dim, float eps) : weight(dim, 1.0f), gpu_(&gpu), eps_(eps) {}
    std::vector<float> forward(const std::vector<float> &x) const {
        if (weight.empty() || x.size() % weight.size()) throw Panic(PG_EINVAL, "RMSNorm::forward: x.len() % dim != 0");
        std::vector<float> out(x.size());
        check(pg_rmsnorm(gpu_->raw(), x.data(), x.size() / weight.size(), weight.size(), weight.data(), eps_, out.data()),
              "RMSNorm::forward");
        return out;
    }
    std::vector<float> weight;

private:
    const GpuContext *gpu_;
    float eps_;
};

// nn::RoPE  src/nn.rs:1250-1345.
class RoPE {
public:
    RoPE(const GpuContext &gpu, size_t head_dim, size_t max_seq_len, float base) : gpu_(&gpu), head_dim_(head_dim) {
        check(pg_rope_create(gpu.raw(), head_dim, max_seq_len, base, &h_), "RoPE::new");
    }
    ~RoPE() { pg_rope_free(gpu_->raw(), h_); }
    RoPE(const RoPE &) = delete;
    RoPE &operator=(const RoPE &) = delete;
    std::vector<float> apply(const std::vector<float> &x, size_t seq_len, size_t offset) const {
        if (x.size() != seq_len * head_dim_) throw Panic(PG_EINVAL, "RoPE::apply: x.len() != seq_len * head_dim");
        std::vector<float> out(x.size());
        check(pg_rope_apply(gpu_->raw(), h_, x.data(), seq_len, offset, out.data()), "RoPE::apply");
        return out;
    }

private:
    const GpuContext *gpu_;
    pg_rope *h_ = nullptr;
    size_t head_dim_;
};

// attention::StandardKVCache  src/attention.rs:8-100.
class StandardKVCache {
public:
    StandardKVCache(const GpuContext &gpu, size_t num_kv_heads, size_t head_dim)
        : num_kv_heads(num_kv_heads), head_dim(head_dim), gpu_(&gpu) {
        check(pg_kv_cache_create(gpu.raw(), num_kv_heads, head_dim, &h_), "StandardKVCache::new");
    }
    ~StandardKVCache() { pg_kv_cache_free(gpu_->raw(), h_); }
    StandardKVCache(const StandardKVCache &) = delete;
    StandardKVCache &operator=(const StandardKVCache &) = delete;
    size_t len() const { return pg_kv_cache_len(h_); }
    size_t head_stride() const { return pg_kv_cache_capacity(h_) * head_dim; }
    void append(const std::vector<float> &new_k, const std::vector<float> &new_v, size_t seq_len) {
        const size_t n = num_kv_heads * seq_len * head_dim;
        if (new_k.size() != n || new_v.size() != n) throw Panic(PG_EINVAL, "StandardKVCache::append: slice lengths");
        check(pg_kv_cache_append(gpu_->raw(), h_, new_k.data(), new_v.data(), seq_len), "StandardKVCache::append");
    }
    void rollback_to(size_t new_len) { check(pg_kv_cache_rollback_to(h_, new_len), "StandardKVCache::rollback_to"); }
    pg_kv_cache *handle() const { return h_; }
    const size_t num_kv_heads, head_dim;

private:
    const GpuContext *gpu_;
    pg_kv_cache *h_ = nullptr;
};
using KVCache = StandardKVCache;  // src/models/llama/attention.rs:7

// attention::AttentionMask  src/attention.rs:102-120.
struct AttentionMask {
    int kind = PG_MASK_NONE;
    size_t offset = 0, window = 0, sink_tokens = 0;
    std::vector<size_t> global_positions;
    static AttentionMask None() { return {}; }
    static AttentionMask Causal(size_t offset) { return {PG_MASK_CAUSAL, offset, 0, 0, {}}; }
    static AttentionMask CausalSlidingWindow(size_t offset, size_t window, size_t sink_tokens) {
        return {PG_MASK_CAUSAL_SLIDING_WINDOW, offset, window, sink_tokens, {}};
    }
    static AttentionMask LocalGlobal(size_t offset, size_t local_window, std::vector<size_t> global_positions) {
        return {PG_MASK_LOCAL_GLOBAL, offset, local_window, 0, std::move(global_positions)};
    }
};

// attention::gqa_attention_cpu  src/attention.rs:141-265; `output` is added to.
inline void gqa_attention(const GpuContext &gpu, const std::vector<float> &q, const StandardKVCache &k_cache,
                          const StandardKVCache &v_cache, size_t num_q_heads, size_t num_kv_heads, size_t seq_q,
                          size_t head_dim, float scale, const AttentionMask &mask, float logit_cap,
                          std::vector<float> &output) {
    if (num_kv_heads != k_cache.num_kv_heads || head_dim != k_cache.head_dim)
        throw Panic(PG_EINVAL, "gqa_attention: num_kv_heads / head_dim differ from the cache's");
    if (q.size() != num_q_heads * seq_q * head_dim || output.size() != q.size())
        throw Panic(PG_EINVAL, "gqa_attention: q / output lengths");
    if (mask.kind == PG_MASK_LOCAL_GLOBAL) {
        check(pg_gqa_attention_local_global(gpu.raw(), q.data(), k_cache.handle(), v_cache.handle(), num_q_heads, seq_q, scale,
                                            mask.offset, mask.window, mask.global_positions.data(),
                                            mask.global_positions.size(), logit_cap, output.data()),
              "gqa_attention");
        return;
    }
    check(pg_gqa_attention(gpu.raw(), q.data(), k_cache.handle(), v_cache.handle(), num_q_heads, seq_q, scale, mask.kind,
                           mask.offset, mask.window, mask.sink_tokens, logit_cap, output.data()),
          "gqa_attention");
}

// LlamaBlock  src/models/llama/decoder.rs:7-155 over block-quantised projections.
class LlamaBlock {
public:
    LlamaBlock(const GpuContext &gpu, size_t model_dim, size_t num_q_heads, size_t num_kv_heads, size_t head_dim,
               size_t ffn_dim, size_t max_seq_len, float rope_base, float rms_eps)
        : gpu_(&gpu), model_dim_(model_dim) {
        check(pg_llama_block_create(gpu.raw(), model_dim, num_q_heads, num_kv_heads, head_dim, ffn_dim, max_seq_len,
                                    rope_base, rms_eps, &h_),
              "LlamaBlock::new");
    }
    ~LlamaBlock() { pg_llama_block_free(gpu_->raw(), h_); }
    LlamaBlock(const LlamaBlock &) = delete;
    LlamaBlock &operator=(const LlamaBlock &) = delete;
    // The block borrows the weights: they must outlive it.
    void set_weights(const gguf::BlockWeight &q_proj, const gguf::BlockWeight &k_proj, const gguf::BlockWeight &v_proj,
                     const gguf::BlockWeight &o_proj, const gguf::BlockWeight &gate_proj, const gguf::BlockWeight &up_proj,
                     const gguf::BlockWeight &down_proj, const std::vector<float> &attn_norm_w,
                     const std::vector<float> &ffn_norm_w) {
        if (attn_norm_w.size() != model_dim_ || ffn_norm_w.size() != model_dim_)
            throw Panic(PG_EINVAL, "LlamaBlock::set_weights: norm weights are not [model_dim]");
        check(pg_llama_block_set_weights(gpu_->raw(), h_, q_proj.handle(), k_proj.handle(), v_proj.handle(), o_proj.handle(),
                                         gate_proj.handle(), up_proj.handle(), down_proj.handle(), attn_norm_w.data(),
                                         ffn_norm_w.data()),
              "LlamaBlock::set_weights");
    }
    std::vector<float> forward(const std::vector<float> &h, size_t seq, KVCache &kv_cache) const {
        if (h.size() != seq * model_dim_) throw Panic(PG_EINVAL, "LlamaBlock::forward: h.len() != seq * model_dim");
        std::vector<float> out(h.size());
        check(pg_llama_block_forward(gpu_->raw(), h_, h.data(), seq, kv_cache.handle(), out.data()), "LlamaBlock::forward");
        return out;
    }

private:
    const GpuContext *gpu_;
    pg_llama_block *h_ = nullptr;
    size_t model_dim_;
};

}  // namespace llama

namespace mxfp4 {

// mxfp4_matmul  examples/gpt_oss/moe.rs:16-53.
inline std::vector<float> mxfp4_matmul(const GpuContext &gpu, const std::vector<float> &input, const std::vector<uint8_t> &blocks,
                                       const std::vector<uint8_t> &scales, size_t out_dim, size_t in_dim) {
    if (in_dim % 32 || input.size() != in_dim || blocks.size() != out_dim * in_dim / 2 || scales.size() != out_dim * in_dim / 32)
        throw Panic(PG_EINVAL, "mxfp4_matmul: slice lengths do not match [out_dim, in_dim]");
    std::vector<float> out(out_dim);
    check(pg_mxfp4_matmul(gpu.raw(), input.data(), blocks.data(), scales.data(), out_dim, in_dim, out.data()), "mxfp4_matmul");
    return out;
}

// Mxfp4Expert  examples/gpt_oss/moe.rs:55-117.
class Mxfp4Expert {
public:
    Mxfp4Expert(const GpuContext &gpu, size_t hidden, size_t intermediate, float alpha, float clamp,
                const std::vector<uint8_t> &mlp1_blocks, const std::vector<uint8_t> &mlp1_scales,
                const std::vector<uint8_t> &mlp2_blocks, const std::vector<uint8_t> &mlp2_scales,
                const std::vector<float> &mlp1_bias, const std::vector<float> &mlp2_bias)
        : gpu_(&gpu), hidden_(hidden) {
        if (hidden % 32 || intermediate % 32 || mlp1_blocks.size() != intermediate * hidden || mlp1_scales.size() != intermediate * hidden / 16 ||
            mlp2_blocks.size() != hidden * intermediate / 2 || mlp2_scales.size() != hidden * intermediate / 32 ||
            mlp1_bias.size() != 2 * intermediate || mlp2_bias.size() != hidden)
            throw Panic(PG_EINVAL, "Mxfp4Expert: slice lengths do not match (hidden, intermediate)");
        check(pg_mxfp4_expert_create(gpu.raw(), hidden, intermediate, alpha, clamp, mlp1_blocks.data(), mlp1_scales.data(),
                                     mlp2_blocks.data(), mlp2_scales.data(), mlp1_bias.data(), mlp2_bias.data(), &h_),
              "Mxfp4Expert::new");
    }
    ~Mxfp4Expert() { pg_mxfp4_expert_free(gpu_->raw(), h_); }
    Mxfp4Expert(const Mxfp4Expert &) = delete;
    Mxfp4Expert &operator=(const Mxfp4Expert &) = delete;
    std::vector<float> forward(const std::vector<float> &x) const {
        if (x.size() != hidden_) throw Panic(PG_EINVAL, "Mxfp4Expert::forward: x.len() != hidden");
        std::vector<float> out(hidden_);
        check(pg_mxfp4_expert_forward(gpu_->raw(), h_, x.data(), 1, out.data()), "Mxfp4Expert::forward");
        return out;
    }

    const pg_mxfp4_expert *handle() const { return h_; }
    size_t hidden() const { return hidden_; }

private:
    const GpuContext *gpu_;
    pg_mxfp4_expert *h_ = nullptr;
    size_t hidden_;
};

// MoELayer::forward after its router, over Mxfp4Experts  examples/gpt_oss/moe.rs:286-352: x [tokens, hidden],
// routing[t] = the token's (expert, weight) pairs in the order the router chose them; every product is one launch
// over all experts.
inline std::vector<float> moe_forward_routed(const GpuContext &gpu, const std::vector<float> &x,
                                             const std::vector<std::vector<std::pair<size_t, float>>> &routing,
                                             const std::vector<const Mxfp4Expert *> &experts) {
    if (experts.empty()) throw Panic(PG_EINVAL, "moe_forward_routed: no experts");
    const size_t tokens = routing.size(), hidden = experts[0]->hidden(), top_k = tokens ? routing[0].size() : 1;
    if (x.size() != tokens * hidden) throw Panic(PG_EINVAL, "moe_forward_routed: x.len() != tokens * hidden");
    std::vector<const pg_mxfp4_expert *> tab;
    for (const auto *e : experts) tab.push_back(e->handle());
    std::vector<int32_t> idx;
    std::vector<float> w;
    for (const auto &r : routing) {
        if (r.size() != top_k) throw Panic(PG_EINVAL, "moe_forward_routed: tokens name different numbers of experts");
        for (const auto &pr : r) { idx.push_back((int32_t)pr.first); w.push_back(pr.second); }
    }
    std::vector<float> out(tokens * hidden);
    check(pg_mxfp4_moe_ffn_routed(gpu.raw(), x.data(), tokens, idx.data(), w.data(), top_k, tab.data(), tab.size(), out.data()),
          "moe_forward_routed");
    return out;
}

}  // namespace mxfp4

namespace huffman {

// HuffmanTable  src/huffman.rs:19-306 (index = value + 128).
struct HuffmanTable {
    std::vector<uint8_t> bit_lengths = std::vector<uint8_t>(256, 0);
    std::vector<uint32_t> codes = std::vector<uint32_t>(256, 0);
    static HuffmanTable from_frequencies(const std::vector<uint64_t> &freqs) {
        if (freqs.size() != 256) throw Panic(PG_EINVAL, "HuffmanTable::from_frequencies: 256 frequencies expected");
        HuffmanTable t;
        check(pg_huffman_table_from_frequencies(freqs.data(), t.bit_lengths.data(), t.codes.data()), "HuffmanTable::from_frequencies");
        return t;
    }
    static HuffmanTable from_bytes(const std::vector<uint8_t> &data) {
        if (data.size() < 256) throw Panic(PG_EINVAL, "codebook too short");
        HuffmanTable t;
        t.bit_lengths.assign(data.begin(), data.begin() + 256);
        check(pg_huffman_canonical_codes(t.bit_lengths.data(), t.codes.data()), "HuffmanTable::from_bytes");
        return t;
    }
    std::vector<uint8_t> to_bytes() const { return bit_lengths; }
    std::vector<uint8_t> encode(const std::vector<int8_t> &data) const {
        size_t need = 0;
        check(pg_huffman_encode(bit_lengths.data(), data.data(), data.size(), nullptr, 0, &need), "HuffmanTable::encode");
        std::vector<uint8_t> out(need);
        check(pg_huffman_encode(bit_lengths.data(), data.data(), data.size(), out.data(), out.size(), &need), "HuffmanTable::encode");
        return out;
    }
    std::vector<int8_t> decode(const GpuContext &gpu, const std::vector<uint8_t> &bitstream, size_t num_symbols) const {
        std::vector<int8_t> out(num_symbols);
        check(pg_huffman_decode(gpu.raw(), bit_lengths.data(), bitstream.data(), bitstream.size(), num_symbols, out.data()),
              "HuffmanTable::decode");
        return out;
    }
};

// HuffmanTensor  src/huffman.rs:311-435.
class HuffmanTensor {
public:
    static HuffmanTensor from_quantized(const quant::QuantizedTensor &qt, size_t num_streams) {
        pg_huffman_tensor *h = nullptr;
        check(pg_huffman_tensor_from_quantized(qt.data_i8.data(), qt.scales.data(), qt.rows, qt.cols, num_streams, &h),
              "HuffmanTensor::from_quantized");
        return HuffmanTensor(h);
    }
    ~HuffmanTensor() { pg_huffman_tensor_free(h_); }
    HuffmanTensor(HuffmanTensor &&o) noexcept : h_(o.h_) { o.h_ = nullptr; }
    HuffmanTensor(const HuffmanTensor &) = delete;
    HuffmanTensor &operator=(const HuffmanTensor &) = delete;
    size_t rows() const { size_t r = 0; check(pg_huffman_tensor_info(h_, &r, nullptr, nullptr, nullptr), "HuffmanTensor"); return r; }
    size_t cols() const { size_t c = 0; check(pg_huffman_tensor_info(h_, nullptr, &c, nullptr, nullptr), "HuffmanTensor"); return c; }
    size_t compressed_size() const { size_t z = 0; check(pg_huffman_tensor_info(h_, nullptr, nullptr, nullptr, &z), "HuffmanTensor"); return z; }
    size_t uncompressed_size() const { return rows() * cols() + cols() * 4; }
    float compression_ratio() const { return (float)uncompressed_size() / (float)compressed_size(); }
    quant::QuantizedTensor decode_to_quantized(const GpuContext &gpu) const {
        quant::QuantizedTensor qt;
        qt.rows = rows(); qt.cols = cols();
        qt.data_i8.resize(qt.rows * qt.cols); qt.data_i8_t.resize(qt.rows * qt.cols); qt.scales.resize(qt.cols);
        check(pg_huffman_tensor_decode_to_quantized(gpu.raw(), h_, qt.data_i8.data(), qt.data_i8_t.data(), qt.scales.data()),
              "HuffmanTensor::decode_to_quantized");
        return qt;
    }
    const pg_huffman_tensor *handle() const { return h_; }

private:
    explicit HuffmanTensor(pg_huffman_tensor *h) : h_(h) {}
    pg_huffman_tensor *h_;
};

// matmul_huffman  src/huffman.rs:465-474.
inline std::vector<float> matmul_huffman(const GpuContext &gpu, const std::vector<float> &a, size_t m, size_t k, const HuffmanTensor &ht) {
    if (a.size() != m * k) throw Panic(PG_EINVAL, "matmul_huffman: a.len() != m * k");
    std::vector<float> out(m * ht.cols());
    check(pg_matmul_huffman(gpu.raw(), a.data(), m, k, ht.handle(), out.data()), "matmul_huffman");
    return out;
}

// CompressedChunk  src/huffman.rs:500-513; the bitstream stays in device memory.
class CompressedChunk {
public:
    CompressedChunk(const GpuContext &gpu, pg_huffman_kv_chunk *h) : gpu_(&gpu), h_(h) {}
    ~CompressedChunk() { if (h_) pg_huffman_kv_chunk_free(gpu_->raw(), h_); }
    CompressedChunk(CompressedChunk &&o) noexcept : gpu_(o.gpu_), h_(o.h_) { o.h_ = nullptr; }
    CompressedChunk(const CompressedChunk &) = delete;
    CompressedChunk &operator=(const CompressedChunk &) = delete;
    size_t num_tokens() const { size_t v = 0; check(pg_huffman_kv_chunk_info(h_, &v, nullptr, nullptr, nullptr), "CompressedChunk"); return v; }
    size_t num_heads() const { size_t v = 0; check(pg_huffman_kv_chunk_info(h_, nullptr, &v, nullptr, nullptr), "CompressedChunk"); return v; }
    size_t head_dim() const { size_t v = 0; check(pg_huffman_kv_chunk_info(h_, nullptr, nullptr, &v, nullptr), "CompressedChunk"); return v; }
    std::vector<uint8_t> bitstream() const {
        size_t n = 0;
        check(pg_huffman_kv_chunk_info(h_, nullptr, nullptr, nullptr, &n), "CompressedChunk");
        std::vector<uint8_t> out(n);
        check(pg_huffman_kv_chunk_parts(gpu_->raw(), h_, out.data(), nullptr, nullptr), "CompressedChunk::bitstream");
        return out;
    }
    std::vector<float> scales() const {
        std::vector<float> out(num_heads());
        check(pg_huffman_kv_chunk_parts(gpu_->raw(), h_, nullptr, out.data(), nullptr), "CompressedChunk::scales");
        return out;
    }
    std::vector<uint8_t> codebook() const {
        std::vector<uint8_t> out(256);
        check(pg_huffman_kv_chunk_parts(gpu_->raw(), h_, nullptr, nullptr, out.data()), "CompressedChunk::codebook");
        return out;
    }
    const pg_huffman_kv_chunk *handle() const { return h_; }

private:
    const GpuContext *gpu_;
    pg_huffman_kv_chunk *h_;
};

// HuffmanKVCache  src/huffman.rs:484-724.
class HuffmanKVCache {
public:
    HuffmanKVCache(const GpuContext &gpu, size_t num_kv_heads, size_t head_dim, size_t compress_threshold, size_t chunk_size)
        : gpu_(&gpu), heads_(num_kv_heads), head_dim_(head_dim) {
        check(pg_huffman_kv_cache_create(gpu.raw(), num_kv_heads, head_dim, compress_threshold, chunk_size, &h_), "HuffmanKVCache::new");
    }
    ~HuffmanKVCache() { if (h_) pg_huffman_kv_cache_free(gpu_->raw(), h_); }
    HuffmanKVCache(const HuffmanKVCache &) = delete;
    HuffmanKVCache &operator=(const HuffmanKVCache &) = delete;
    void append(const std::vector<float> &new_k, const std::vector<float> &new_v, size_t seq_len) {
        const size_t n = heads_ * seq_len * head_dim_;
        if (new_k.size() != n || new_v.size() != n) throw Panic(PG_EINVAL, "HuffmanKVCache::append: new_k / new_v are not [num_kv_heads, seq_len, head_dim]");
        check(pg_huffman_kv_cache_append(gpu_->raw(), h_, new_k.data(), new_v.data(), seq_len), "HuffmanKVCache::append");
    }
    static CompressedChunk compress_chunk(const GpuContext &gpu, const std::vector<float> &data, size_t num_tokens, size_t num_heads,
                                          size_t head_dim) {
        if (data.size() != num_heads * num_tokens * head_dim) throw Panic(PG_EINVAL, "compress_chunk: data.len() != total");
        pg_huffman_kv_chunk *c = nullptr;
        check(pg_huffman_kv_compress_chunk(gpu.raw(), data.data(), num_tokens, num_heads, head_dim, &c), "HuffmanKVCache::compress_chunk");
        return CompressedChunk(gpu, c);
    }
    static std::vector<float> decompress_chunk(const GpuContext &gpu, const CompressedChunk &chunk) {
        std::vector<float> out(chunk.num_heads() * chunk.num_tokens() * chunk.head_dim());
        check(pg_huffman_kv_decompress_chunk(gpu.raw(), chunk.handle(), out.data()), "HuffmanKVCache::decompress_chunk");
        return out;
    }
    size_t len() const { return pg_huffman_kv_cache_len(h_); }
    size_t compressed_len() const { return pg_huffman_kv_cache_compressed_len(h_); }
    size_t compress_threshold() const { return pg_huffman_kv_cache_compress_threshold(h_); }
    size_t num_chunks() const { return pg_huffman_kv_cache_num_chunks(h_); }
    // (k, v), each [num_kv_heads, len(), head_dim]
    std::pair<std::vector<float>, std::vector<float>> get_kv() const {
        const size_t n = heads_ * len() * head_dim_;
        std::vector<float> k(n), v(n);
        check(pg_huffman_kv_cache_get_kv(gpu_->raw(), h_, k.data(), v.data()), "HuffmanKVCache::get_kv");
        return {std::move(k), std::move(v)};
    }
    pg_huffman_kv_cache *handle() const { return h_; }

private:
    const GpuContext *gpu_;
    size_t heads_, head_dim_;
    pg_huffman_kv_cache *h_ = nullptr;
};

}  // namespace huffman
}  // namespace peregrine
#endif  // PEREGRINE_HIP_HPP
