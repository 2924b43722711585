// peregrine's HuffmanKVCache: a key/value cache whose older tokens are quantised to int8 with
// one scale per head and Huffman-coded in chunks, with a window of recent tokens kept as f32.
//
//   HuffmanKVCache::new / append / compress_oldest_chunk / remove_oldest_tokens   reference: src/huffman.rs:517-610
//   HuffmanKVCache::compress_chunk / decompress_chunk                             reference: src/huffman.rs:612-680
//   HuffmanKVCache::len / get_kv                                                  reference: src/huffman.rs:683-724
//
// Everything but the 256-entry code table is device work here: the hot window is the device
// StandardKVCache, a chunk's per-head absolute maximum, its int8 values and their histogram come
// from two kernels, the host builds the table from the histogram (2 KB down, 1 KB up), and the
// encoder is a prefix sum over the code lengths followed by one pass in which every thread packs
// 16 consecutive codes into the words of the MSB-first stream.  Coded chunks stay in device
// memory, each with its 8 KB decode table beside it; decoding is the self-synchronising decoder of
// the Huffman-coded weights over all chunks of a cache at once (every stream under its own table),
// followed by one scaling kernel that writes straight into the caller's [heads, tokens, head_dim] layout.
#include <new>
#include <vector>
#include "pg_internal.h"
#include "pg_quant_dev.h"

namespace {

constexpr int NUM_SYMBOLS = 256;
constexpr int KV_WG = 256;
constexpr int ENC_SPT = 16;                    // symbols per thread of the encoder
constexpr int ENC_PER_WG = KV_WG * ENC_SPT;    // symbols per workgroup
constexpr unsigned KV_MAX_SPLITS = 64;         // workgroups per head of the two quantising kernels

// Largest |v| of every head (NaN ignored, as f32::max does): grid (splits, heads), amax_bits zeroed.
__global__ __launch_bounds__(KV_WG) void kv_absmax_kernel(const float *__restrict__ data, size_t head_stride, size_t head_elems,
                                                          unsigned *__restrict__ amax_bits) {
    __shared__ float red[4];
    const float *p = data + (size_t)blockIdx.y * head_stride;
    float m = 0.0f;
    for (size_t i = (size_t)blockIdx.x * KV_WG + threadIdx.x; i < head_elems; i += (size_t)gridDim.x * KV_WG)
        m = fmaxf(m, fabsf(p[i]));
    m = pg_block_max_256(m, red);
    if (threadIdx.x == 0) atomicMax(amax_bits + blockIdx.y, __float_as_uint(m));  // m >= 0: the bit patterns order as the values
}

// q = round(v / scale) clamped to +-127 with scale = amax / 127 (1 for an all-zero head), the
// histogram of q, and the scales.   src/huffman.rs:624-646
__global__ __launch_bounds__(KV_WG) void kv_quant_hist_kernel(const float *__restrict__ data, size_t head_stride, size_t head_elems,
                                                              const unsigned *__restrict__ amax_bits, int8_t *__restrict__ q,
                                                              float *__restrict__ scales, unsigned long long *__restrict__ hist) {
    __shared__ unsigned lh[NUM_SYMBOLS];
    lh[threadIdx.x] = 0;
    __syncthreads();
    const float amax = __uint_as_float(amax_bits[blockIdx.y]);
    const float scale = (amax == 0.0f) ? 1.0f : amax / 127.0f;
    const float inv_scale = 1.0f / scale;
    if (blockIdx.x == 0 && threadIdx.x == 0) scales[blockIdx.y] = scale;
    const float *p = data + (size_t)blockIdx.y * head_stride;
    int8_t *o = q + (size_t)blockIdx.y * head_elems;
    for (size_t i = (size_t)blockIdx.x * KV_WG + threadIdx.x; i < head_elems; i += (size_t)gridDim.x * KV_WG) {
        const int v = pg_quant_to_i8(p[i] * inv_scale);
        o[i] = (int8_t)v;
        atomicAdd(&lh[v + 128], 1u);
    }
    __syncthreads();
    if (lh[threadIdx.x]) atomicAdd(hist + threadIdx.x, (unsigned long long)lh[threadIdx.x]);
}

// The code lengths of a thread's ENC_SPT symbols (codes[s] = length << 16 | code), and the symbols.
__device__ __forceinline__ unsigned enc_load(const int8_t *__restrict__ q, size_t n, size_t base, const unsigned *lc, int8_t *sym,
                                             int &count) {
    count = base >= n ? 0 : (int)(n - base < (size_t)ENC_SPT ? n - base : (size_t)ENC_SPT);
    if (count == ENC_SPT) {
        const uint4 v = *reinterpret_cast<const uint4 *>(q + base);  // base is a multiple of 16 and q is 256-byte aligned
        const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < ENC_SPT; ++j) sym[j] = (int8_t)(w[j >> 2] >> (8 * (j & 3)));
    } else {
#pragma unroll
        for (int j = 0; j < ENC_SPT; ++j) sym[j] = j < count ? q[base + j] : (int8_t)0;
    }
    unsigned bits = 0;
#pragma unroll
    for (int j = 0; j < ENC_SPT; ++j)
        if (j < count) bits += lc[(int)sym[j] + 128] >> 16;
    return bits;
}

// Inclusive sum over the workgroup's 256 threads; `sc` = 256 unsigned of LDS.
__device__ __forceinline__ unsigned block_inclusive_sum(unsigned v, unsigned *sc) {
    sc[threadIdx.x] = v;
    __syncthreads();
    for (int off = 1; off < KV_WG; off <<= 1) {
        const unsigned add = threadIdx.x >= (unsigned)off ? sc[threadIdx.x - off] : 0u;
        __syncthreads();
        sc[threadIdx.x] += add;
        __syncthreads();
    }
    return sc[threadIdx.x];
}

// Bits every workgroup's ENC_PER_WG symbols take.
__global__ __launch_bounds__(KV_WG) void kv_encode_bits_kernel(const int8_t *__restrict__ q, size_t n,
                                                               const unsigned *__restrict__ codes,
                                                               unsigned long long *__restrict__ wg_bits) {
    __shared__ unsigned lc[NUM_SYMBOLS], sc[KV_WG];
    lc[threadIdx.x] = codes[threadIdx.x];
    __syncthreads();
    int8_t sym[ENC_SPT];
    int count;
    const unsigned bits = enc_load(q, n, (size_t)blockIdx.x * ENC_PER_WG + (size_t)threadIdx.x * ENC_SPT, lc, sym, count);
    const unsigned incl = block_inclusive_sum(bits, sc);
    if (threadIdx.x == KV_WG - 1) wg_bits[blockIdx.x] = incl;
}

// One workgroup: wg_bits[0 .. nwg) becomes its exclusive running sum, wg_bits[nwg] the total.
__global__ __launch_bounds__(KV_WG) void kv_encode_scan_kernel(unsigned long long *__restrict__ wg_bits, size_t nwg) {
    __shared__ unsigned long long sc[KV_WG];
    unsigned long long run = 0;
    for (size_t c = 0; c < nwg; c += KV_WG) {
        const size_t i = c + threadIdx.x;
        const unsigned long long v = i < nwg ? wg_bits[i] : 0ull;
        sc[threadIdx.x] = v;
        __syncthreads();
        for (int off = 1; off < KV_WG; off <<= 1) {
            const unsigned long long add = threadIdx.x >= (unsigned)off ? sc[threadIdx.x - off] : 0ull;
            __syncthreads();
            sc[threadIdx.x] += add;
            __syncthreads();
        }
        if (i < nwg) wg_bits[i] = run + sc[threadIdx.x] - v;
        run += sc[KV_WG - 1];
        __syncthreads();
    }
    if (threadIdx.x == 0) wg_bits[nwg] = run;
}

// HuffmanTable::encode (src/huffman.rs:216-251) in parallel: every thread knows the bit its first
// code starts at, shifts its codes into a 64-bit window and ORs whole big-endian words into the
// zeroed stream (only a thread's first and last word are shared with its neighbours).
__global__ __launch_bounds__(KV_WG) void kv_encode_write_kernel(const int8_t *__restrict__ q, size_t n,
                                                                const unsigned *__restrict__ codes,
                                                                const unsigned long long *__restrict__ wg_excl,
                                                                unsigned *__restrict__ words) {
    __shared__ unsigned lc[NUM_SYMBOLS], sc[KV_WG];
    lc[threadIdx.x] = codes[threadIdx.x];
    __syncthreads();
    int8_t sym[ENC_SPT];
    int count;
    const unsigned bits = enc_load(q, n, (size_t)blockIdx.x * ENC_PER_WG + (size_t)threadIdx.x * ENC_SPT, lc, sym, count);
    const unsigned incl = block_inclusive_sum(bits, sc);
    if (bits == 0) return;
    const unsigned long long p0 = wg_excl[blockIdx.x] + (incl - bits);
    size_t word = (size_t)(p0 >> 5);
    unsigned nacc = (unsigned)(p0 & 31);  // bits of the current word that belong to earlier threads (zeros here)
    unsigned long long acc = 0;
#pragma unroll
    for (int j = 0; j < ENC_SPT; ++j) {
        if (j < count) {
            const unsigned e = lc[(int)sym[j] + 128], l = e >> 16;
            acc = (acc << l) | (e & ((1u << l) - 1u));
            nacc += l;
            if (nacc >= 32) {
                atomicOr(words + word, __builtin_bswap32((unsigned)(acc >> (nacc - 32))));
                ++word;
                nacc -= 32;
                acc &= (1ull << nacc) - 1ull;
            }
        }
    }
    if (nacc > 0) atomicOr(words + word, __builtin_bswap32((unsigned)(acc << (32 - nacc))));
}

// decoded_i8 as f32 * scale[head]   src/huffman.rs:669-677 for several chunks in one launch: grid
// (splits, heads, chunks); chunk c's values start at q + q_off and go to rows of out_stride floats per head.
struct dequant_item {
    const float *scales;
    float *out;
    size_t q_off, head_elems, out_stride;
};

__global__ __launch_bounds__(KV_WG) void kv_dequant_kernel(const int8_t *__restrict__ q, const dequant_item *__restrict__ items) {
    const dequant_item it = items[blockIdx.z];
    const float scale = it.scales[blockIdx.y];
    const int8_t *p = q + it.q_off + (size_t)blockIdx.y * it.head_elems;
    float *o = it.out + (size_t)blockIdx.y * it.out_stride;
    for (size_t i = (size_t)blockIdx.x * KV_WG + threadIdx.x; i < it.head_elems; i += (size_t)gridDim.x * KV_WG)
        o[i] = (float)p[i] * scale;
}

unsigned splits_for(size_t head_elems) {
    const size_t s = (head_elems + 4 * KV_WG - 1) / (4 * KV_WG);
    return (unsigned)std::min<size_t>(std::max<size_t>(s, 1), KV_MAX_SPLITS);
}

}  // namespace

// CompressedChunk  src/huffman.rs:500-513 with its bitstream (and a copy of the scales) in device memory.
struct pg_huffman_kv_chunk {
    uint8_t codebook[NUM_SYMBOLS];
    std::vector<float> scales;
    char *dev = nullptr;  // [scales, 256-byte rounded][decode table][bitstream, zero padded to a whole word and 16 bytes on]
    size_t bytes = 0;     // of the bitstream
    size_t num_tokens = 0, num_heads = 0, head_dim = 0;
    bool decodable = false;  // the codebook fits the decode table (always, for chunks made here)
    size_t scales_bytes() const { return pg_round_up(num_heads * sizeof(float), 256); }
    size_t head_bytes() const { return scales_bytes() + pg_huffman_lut_entries() * sizeof(uint16_t); }
    const float *scales_dev() const { return reinterpret_cast<const float *>(dev); }
    const uint16_t *lut_dev() const { return reinterpret_cast<const uint16_t *>(dev + scales_bytes()); }
    const uint8_t *bits_dev() const { return reinterpret_cast<const uint8_t *>(dev + head_bytes()); }
    size_t symbols() const { return num_heads * num_tokens * head_dim; }
    ~pg_huffman_kv_chunk() { if (dev) (void)hipFree(dev); }
};

// HuffmanKVCache  src/huffman.rs:484-497
struct pg_huffman_kv_cache {
    pg_kv_cache *hot = nullptr;
    std::vector<pg_huffman_kv_chunk *> k_chunks, v_chunks;
    size_t compressed_len = 0, compress_threshold = 0, chunk_size = 0;
};

static pg_status chunk_shape_ok(const char *who, size_t num_tokens, size_t num_heads, size_t head_dim) {
    PG_CHECK_ARG(num_heads < 65536, "%s: %zu heads (at most 65535)", who, num_heads);
    PG_CHECK_ARG(num_tokens < (1ull << 31) && head_dim < (1ull << 31) &&
                     (num_tokens == 0 || head_dim == 0 || num_heads == 0 ||
                      num_tokens * head_dim < (1ull << 31) / (num_heads ? num_heads : 1)),
                 "%s: %zu heads x %zu tokens x %zu values is beyond 2^31 symbols", who, num_heads, num_tokens, head_dim);
    return PG_OK;
}

// Allocates the chunk's device memory, zeroes it (stream ordered) and puts the decode table of c->codebook in place.
static pg_status chunk_alloc(pg_ctx *ctx, pg_huffman_kv_chunk *c, size_t bytes) {
    c->bytes = bytes;
    const size_t total = c->head_bytes() + pg_round_up(bytes, 4) + 16;
    hipError_t e = hipMalloc((void **)&c->dev, total);
    if (e != hipSuccess) {
        c->dev = nullptr;
        return pg_fail(PG_ENOMEM, "hipMalloc(%zu) failed: %s", total, hipGetErrorString(e));
    }
    PG_HIP(hipMemsetAsync(c->dev, 0, total, ctx->stream));
    std::vector<uint16_t> lut(pg_huffman_lut_entries());
    c->decodable = pg_huffman_host_lut(c->codebook, lut.data()) == PG_OK;  // else: reported when the chunk is decoded
    if (c->decodable) {
        PG_HIP(hipMemcpyAsync(c->dev + c->scales_bytes(), lut.data(), lut.size() * sizeof(uint16_t), hipMemcpyHostToDevice, ctx->stream));
        PG_HIP(hipStreamSynchronize(ctx->stream));  // lut is a local
    }
    return PG_OK;
}

// compress_chunk on device data: head h's num_tokens * head_dim values start at data + h * head_stride.
static pg_status compress_dev(pg_ctx *ctx, const float *data, size_t head_stride, size_t num_tokens, size_t num_heads,
                              size_t head_dim, pg_huffman_kv_chunk **out) {
    *out = nullptr;
    PG_TRY(chunk_shape_ok("huffman kv compress_chunk", num_tokens, num_heads, head_dim));
    pg_huffman_kv_chunk *c = new (std::nothrow) pg_huffman_kv_chunk();
    if (!c) return pg_fail(PG_ENOMEM, "host allocation failed");
    struct guard { pg_huffman_kv_chunk *c; ~guard() { delete c; } } g{c};
    c->num_tokens = num_tokens; c->num_heads = num_heads; c->head_dim = head_dim;
    std::fill(c->codebook, c->codebook + NUM_SYMBOLS, (uint8_t)0);
    c->scales.assign(num_heads, 1.0f);  // absmax == 0.0 -> 1.0
    const size_t head_elems = num_tokens * head_dim, total = num_heads * head_elems;
    if (total == 0) {  // an empty table, an empty stream
        PG_TRY(chunk_alloc(ctx, c, 0));
        if (num_heads)
            PG_HIP(hipMemcpyAsync(c->dev, c->scales.data(), num_heads * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
        PG_HIP(hipStreamSynchronize(ctx->stream));
        g.c = nullptr;
        *out = c;
        return PG_OK;
    }
    const size_t nwg = (total + ENC_PER_WG - 1) / ENC_PER_WG;
    // amax | scales | hist | codes | wg bits (+ total) | q
    const size_t o_scale = pg_round_up(num_heads * 4, 256), o_hist = o_scale + pg_round_up(num_heads * 4, 256);
    const size_t o_codes = o_hist + NUM_SYMBOLS * 8, o_wg = o_codes + NUM_SYMBOLS * 4;
    const size_t o_q = o_wg + pg_round_up((nwg + 1) * 8, 256);
    pg_tmp buf;
    PG_TRY(buf.alloc(o_q + pg_round_up(total, 16)));
    char *base = buf.as<char>();
    auto *d_amax = reinterpret_cast<unsigned *>(base);
    auto *d_scales = reinterpret_cast<float *>(base + o_scale);
    auto *d_hist = reinterpret_cast<unsigned long long *>(base + o_hist);
    auto *d_codes = reinterpret_cast<unsigned *>(base + o_codes);
    auto *d_wg = reinterpret_cast<unsigned long long *>(base + o_wg);
    auto *d_q = reinterpret_cast<int8_t *>(base + o_q);
    PG_HIP(hipMemsetAsync(base, 0, o_codes, ctx->stream));
    const dim3 grid(splits_for(head_elems), (unsigned)num_heads);
    PG_TRY(pg_launch(ctx, "huffman_kv_absmax", kv_absmax_kernel, grid, dim3(KV_WG), 0, data, head_stride, head_elems, d_amax));
    PG_TRY(pg_launch(ctx, "huffman_kv_quant", kv_quant_hist_kernel, grid, dim3(KV_WG), 0, data, head_stride, head_elems,
                     (const unsigned *)d_amax, d_q, d_scales, d_hist));
    uint64_t freqs[NUM_SYMBOLS];
    static_assert(sizeof(uint64_t) == sizeof(unsigned long long), "histogram element size");
    PG_HIP(hipMemcpyAsync(freqs, d_hist, sizeof freqs, hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipMemcpyAsync(c->scales.data(), d_scales, num_heads * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    uint32_t codes[NUM_SYMBOLS];
    (void)pg_huffman_host_table(freqs, c->codebook, codes);  // the reference's table wherever that one decodes
    for (int s = 0; s < NUM_SYMBOLS; ++s) codes[s] = (uint32_t)c->codebook[s] << 16 | (codes[s] & 0xFFFFu);
    PG_HIP(hipMemcpyAsync(d_codes, codes, sizeof codes, hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_launch(ctx, "huffman_kv_encode_bits", kv_encode_bits_kernel, dim3((unsigned)nwg), dim3(KV_WG), 0,
                     (const int8_t *)d_q, total, (const unsigned *)d_codes, d_wg));
    PG_TRY(pg_launch(ctx, "huffman_kv_encode_scan", kv_encode_scan_kernel, dim3(1), dim3(KV_WG), 0, d_wg, nwg));
    unsigned long long bits = 0;
    PG_HIP(hipMemcpyAsync(&bits, d_wg + nwg, sizeof bits, hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    PG_TRY(chunk_alloc(ctx, c, (size_t)((bits + 7) / 8)));
    PG_HIP(hipMemcpyAsync(c->dev, d_scales, num_heads * sizeof(float), hipMemcpyDeviceToDevice, ctx->stream));
    PG_TRY(pg_launch(ctx, "huffman_kv_encode_write", kv_encode_write_kernel, dim3((unsigned)nwg), dim3(KV_WG), 0,
                     (const int8_t *)d_q, total, (const unsigned *)d_codes, (const unsigned long long *)d_wg,
                     reinterpret_cast<unsigned *>(c->dev + c->head_bytes())));
    PG_HIP(hipStreamSynchronize(ctx->stream));  // buf is freed on return
    g.c = nullptr;
    *out = c;
    return PG_OK;
}

// decompress_chunk for several chunks in one pass: chunk i's head h goes to out[i] + h * out_stride[i].
static pg_status decompress_many(pg_ctx *ctx, const pg_huffman_kv_chunk *const *chunks, float *const *out, const size_t *out_stride,
                                 size_t count) {
    std::vector<pg_huffman_dev_stream> streams;
    std::vector<dequant_item> items;
    size_t total = 0, max_head_elems = 0, heads = 0;
    for (size_t i = 0; i < count; ++i) {
        const pg_huffman_kv_chunk *c = chunks[i];
        if (c->symbols() == 0) continue;
        if (!c->decodable) {  // sets the message
            std::vector<uint16_t> lut(pg_huffman_lut_entries());
            PG_TRY(pg_huffman_host_lut(c->codebook, lut.data()));
        }
        PG_CHECK_ARG(heads == 0 || heads == c->num_heads, "huffman kv: chunks of %zu and %zu heads in one pass", heads, c->num_heads);
        heads = c->num_heads;
        streams.push_back({c->bits_dev(), c->bytes, c->symbols(), c->lut_dev(), total});
        items.push_back({c->scales_dev(), out[i], total, c->num_tokens * c->head_dim, out_stride[i]});
        max_head_elems = std::max(max_head_elems, c->num_tokens * c->head_dim);
        total += pg_round_up(c->symbols(), 16);
    }
    if (items.empty()) return PG_OK;
    PG_CHECK_ARG(items.size() < 65536, "huffman kv: %zu chunks in one pass", items.size());
    const size_t o_items = pg_round_up(total, 256);
    pg_tmp buf;
    PG_TRY(buf.alloc(o_items + items.size() * sizeof(dequant_item)));
    PG_HIP(hipMemcpyAsync(buf.as<char>() + o_items, items.data(), items.size() * sizeof(dequant_item), hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_huffman_decode_device_streams(ctx, streams.data(), streams.size(), buf.as<int8_t>()));
    PG_TRY(pg_launch(ctx, "huffman_kv_dequant", kv_dequant_kernel, dim3(splits_for(max_head_elems), (unsigned)heads, (unsigned)items.size()),
                     dim3(KV_WG), 0, (const int8_t *)buf.as<int8_t>(), reinterpret_cast<const dequant_item *>(buf.as<char>() + o_items)));
    PG_HIP(hipStreamSynchronize(ctx->stream));  // buf is freed on return
    return PG_OK;
}

static pg_status decompress_dev(pg_ctx *ctx, const pg_huffman_kv_chunk *c, float *out, size_t out_stride) {
    return decompress_many(ctx, &c, &out, &out_stride, 1);
}

PG_API pg_status pg_huffman_kv_compress_chunk_dev(pg_ctx *ctx, const float *data_dev, size_t head_stride, size_t num_tokens,
                                                  size_t num_heads, size_t head_dim, pg_huffman_kv_chunk **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(out != nullptr, "pg_huffman_kv_compress_chunk_dev: out is null");
    *out = nullptr;
    PG_CHECK_ARG(data_dev || num_tokens * num_heads * head_dim == 0, "pg_huffman_kv_compress_chunk_dev: null data");
    PG_CHECK_ARG(head_stride >= num_tokens * head_dim, "pg_huffman_kv_compress_chunk_dev: head_stride %zu < %zu values per head",
                 head_stride, num_tokens * head_dim);
    return compress_dev(ctx, data_dev, head_stride, num_tokens, num_heads, head_dim, out);
}

PG_API pg_status pg_huffman_kv_compress_chunk(pg_ctx *ctx, const float *data, size_t num_tokens, size_t num_heads,
                                              size_t head_dim, pg_huffman_kv_chunk **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(out != nullptr, "pg_huffman_kv_compress_chunk: out is null");
    *out = nullptr;
    PG_TRY(chunk_shape_ok("pg_huffman_kv_compress_chunk", num_tokens, num_heads, head_dim));
    const size_t total = num_tokens * num_heads * head_dim;
    PG_CHECK_ARG(data || total == 0, "pg_huffman_kv_compress_chunk: null data");
    pg_tmp d;
    PG_TRY(d.alloc(total * sizeof(float)));
    if (total) PG_HIP(hipMemcpyAsync(d.p, data, total * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    return compress_dev(ctx, d.as<float>(), num_tokens * head_dim, num_tokens, num_heads, head_dim, out);
}

PG_API pg_status pg_huffman_kv_chunk_from_parts(pg_ctx *ctx, const uint8_t *bitstream, size_t bytes, const float *scales,
                                                const uint8_t *codebook, size_t num_tokens, size_t num_heads, size_t head_dim,
                                                pg_huffman_kv_chunk **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(out != nullptr, "pg_huffman_kv_chunk_from_parts: out is null");
    *out = nullptr;
    PG_TRY(chunk_shape_ok("pg_huffman_kv_chunk_from_parts", num_tokens, num_heads, head_dim));
    PG_CHECK_ARG(codebook && (scales || num_heads == 0) && (bitstream || bytes == 0), "pg_huffman_kv_chunk_from_parts: null pointer");
    pg_huffman_kv_chunk *c = new (std::nothrow) pg_huffman_kv_chunk();
    if (!c) return pg_fail(PG_ENOMEM, "host allocation failed");
    struct guard { pg_huffman_kv_chunk *c; ~guard() { delete c; } } g{c};
    c->num_tokens = num_tokens; c->num_heads = num_heads; c->head_dim = head_dim;
    std::copy(codebook, codebook + NUM_SYMBOLS, c->codebook);
    c->scales.assign(scales, scales + num_heads);
    PG_TRY(chunk_alloc(ctx, c, bytes));
    if (num_heads) PG_HIP(hipMemcpyAsync(c->dev, scales, num_heads * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    if (bytes) PG_HIP(hipMemcpyAsync(c->dev + c->head_bytes(), bitstream, bytes, hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    g.c = nullptr;
    *out = c;
    return PG_OK;
}

PG_API void pg_huffman_kv_chunk_free(pg_ctx *ctx, pg_huffman_kv_chunk *c) {
    if (!c) return;
    if (ctx) {
        (void)pg_use(ctx);
        (void)hipStreamSynchronize(ctx->stream);
    }
    delete c;
}

PG_API pg_status pg_huffman_kv_chunk_info(const pg_huffman_kv_chunk *c, size_t *num_tokens, size_t *num_heads, size_t *head_dim,
                                          size_t *bitstream_bytes) {
    PG_CHECK_ARG(c != nullptr, "pg_huffman_kv_chunk_info: null chunk");
    if (num_tokens) *num_tokens = c->num_tokens;
    if (num_heads) *num_heads = c->num_heads;
    if (head_dim) *head_dim = c->head_dim;
    if (bitstream_bytes) *bitstream_bytes = c->bytes;
    return PG_OK;
}

PG_API pg_status pg_huffman_kv_chunk_parts(pg_ctx *ctx, const pg_huffman_kv_chunk *c, uint8_t *bitstream, float *scales,
                                           uint8_t *codebook) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(c != nullptr, "pg_huffman_kv_chunk_parts: null chunk");
    if (codebook) std::copy(c->codebook, c->codebook + NUM_SYMBOLS, codebook);
    if (scales) std::copy(c->scales.begin(), c->scales.end(), scales);
    if (bitstream && c->bytes) {
        PG_HIP(hipMemcpyAsync(bitstream, c->bits_dev(), c->bytes, hipMemcpyDeviceToHost, ctx->stream));
        PG_HIP(hipStreamSynchronize(ctx->stream));
    }
    return PG_OK;
}

PG_API pg_status pg_huffman_kv_decompress_chunk_dev(pg_ctx *ctx, const pg_huffman_kv_chunk *c, float *out_dev, size_t head_stride) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(c != nullptr, "pg_huffman_kv_decompress_chunk_dev: null chunk");
    PG_CHECK_ARG(out_dev || c->symbols() == 0, "pg_huffman_kv_decompress_chunk_dev: null output");
    PG_CHECK_ARG(head_stride >= c->num_tokens * c->head_dim, "pg_huffman_kv_decompress_chunk_dev: head_stride %zu < %zu values per head",
                 head_stride, c->num_tokens * c->head_dim);
    return decompress_dev(ctx, c, out_dev, head_stride);
}

PG_API pg_status pg_huffman_kv_decompress_chunk(pg_ctx *ctx, const pg_huffman_kv_chunk *c, float *out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(c != nullptr, "pg_huffman_kv_decompress_chunk: null chunk");
    const size_t total = c->symbols();
    if (total == 0) return PG_OK;
    PG_CHECK_ARG(out != nullptr, "pg_huffman_kv_decompress_chunk: null output");
    pg_tmp d;
    PG_TRY(d.alloc(total * sizeof(float)));
    PG_TRY(decompress_dev(ctx, c, d.as<float>(), c->num_tokens * c->head_dim));
    PG_HIP(hipMemcpyAsync(out, d.p, total * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

// ---- the cache ---------------------------------------------------------------------------

PG_API pg_status pg_huffman_kv_cache_create(pg_ctx *ctx, size_t num_kv_heads, size_t head_dim, size_t compress_threshold,
                                            size_t chunk_size, pg_huffman_kv_cache **out) {
    PG_CHECK_ARG(out != nullptr, "pg_huffman_kv_cache_create: out is null");
    *out = nullptr;
    // with chunk_size 0 the reference's append loops forever once the threshold is reached (src/huffman.rs:545-556)
    PG_CHECK_ARG(chunk_size > 0, "pg_huffman_kv_cache_create: chunk_size is 0");
    pg_huffman_kv_cache *c = new (std::nothrow) pg_huffman_kv_cache();
    if (!c) return pg_fail(PG_ENOMEM, "host allocation failed");
    const pg_status st = pg_kv_cache_create(ctx, num_kv_heads, head_dim, &c->hot);
    if (st != PG_OK) {
        delete c;
        return st;
    }
    c->compress_threshold = std::max(compress_threshold, chunk_size);  // src/huffman.rs:535
    c->chunk_size = chunk_size;
    *out = c;
    return PG_OK;
}

PG_API void pg_huffman_kv_cache_free(pg_ctx *ctx, pg_huffman_kv_cache *c) {
    if (!c) return;
    pg_kv_cache_free(ctx, c->hot);  // waits for the stream
    for (auto *p : c->k_chunks) delete p;
    for (auto *p : c->v_chunks) delete p;
    delete c;
}

PG_API size_t pg_huffman_kv_cache_len(const pg_huffman_kv_cache *c) { return c ? c->compressed_len + c->hot->len : 0; }
PG_API size_t pg_huffman_kv_cache_compressed_len(const pg_huffman_kv_cache *c) { return c ? c->compressed_len : 0; }
PG_API size_t pg_huffman_kv_cache_num_chunks(const pg_huffman_kv_cache *c) { return c ? c->k_chunks.size() : 0; }
PG_API size_t pg_huffman_kv_cache_compress_threshold(const pg_huffman_kv_cache *c) { return c ? c->compress_threshold : 0; }
PG_API pg_status pg_huffman_kv_cache_hot(pg_huffman_kv_cache *c, pg_kv_cache **out) {
    PG_CHECK_ARG(c && out, "pg_huffman_kv_cache_hot: null pointer");
    *out = c->hot;
    return PG_OK;
}

PG_API pg_status pg_huffman_kv_cache_chunk(const pg_huffman_kv_cache *c, int value_side, size_t index,
                                           const pg_huffman_kv_chunk **out) {
    PG_CHECK_ARG(c && out, "pg_huffman_kv_cache_chunk: null pointer");
    const auto &v = value_side ? c->v_chunks : c->k_chunks;
    PG_CHECK_ARG(index < v.size(), "pg_huffman_kv_cache_chunk: chunk %zu of %zu", index, v.size());
    *out = v[index];
    return PG_OK;
}

// The reference compresses the oldest chunk_size tokens and shifts the rest to the front, once per
// chunk; here the chunks are cut at a moving token offset and the window is shifted once.
static pg_status compress_hot(pg_ctx *ctx, pg_huffman_kv_cache *c) {
    pg_kv_cache *hot = c->hot;
    const size_t hd = hot->head_dim, stride = hot->capacity * hd, heads = hot->num_kv_heads;
    size_t done = 0;
    pg_status st = PG_OK;
    while (hot->len - done >= c->compress_threshold) {
        const size_t tokens = std::min(c->chunk_size, hot->len - done);
        pg_huffman_kv_chunk *kc = nullptr, *vc = nullptr;
        st = compress_dev(ctx, hot->k + done * hd, stride, tokens, heads, hd, &kc);
        if (st == PG_OK) st = compress_dev(ctx, hot->v + done * hd, stride, tokens, heads, hd, &vc);
        if (st != PG_OK) {
            delete kc;
            break;
        }
        c->k_chunks.push_back(kc);
        c->v_chunks.push_back(vc);
        c->compressed_len += tokens;
        done += tokens;
    }
    if (done == 0) return st;
    const size_t rest = hot->len - done;
    // The rest moves to the front in slices no longer than the distance it moves, oldest first on
    // the one stream, so that no copy reads what it writes; nothing is allocated and nothing waited for.
    const size_t pitch = stride * sizeof(float);
    for (size_t at = 0; at < rest && hd * heads > 0; at += done) {
        const size_t width = std::min(done, rest - at) * hd * sizeof(float);
        PG_HIP(hipMemcpy2DAsync(hot->k + at * hd, pitch, hot->k + (done + at) * hd, pitch, width, heads, hipMemcpyDeviceToDevice, ctx->stream));
        PG_HIP(hipMemcpy2DAsync(hot->v + at * hd, pitch, hot->v + (done + at) * hd, pitch, width, heads, hipMemcpyDeviceToDevice, ctx->stream));
    }
    hot->len = rest;
    return st;
}

PG_API pg_status pg_huffman_kv_cache_append_dev(pg_ctx *ctx, pg_huffman_kv_cache *c, const float *new_k_dev,
                                                const float *new_v_dev, size_t seq_len) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(c != nullptr, "pg_huffman_kv_cache_append: null cache");
    PG_TRY(pg_kv_cache_append_dev(ctx, c->hot, new_k_dev, new_v_dev, seq_len));
    return compress_hot(ctx, c);
}

PG_API pg_status pg_huffman_kv_cache_append(pg_ctx *ctx, pg_huffman_kv_cache *c, const float *new_k, const float *new_v,
                                            size_t seq_len) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(c != nullptr, "pg_huffman_kv_cache_append: null cache");
    PG_TRY(pg_kv_cache_append(ctx, c->hot, new_k, new_v, seq_len));
    return compress_hot(ctx, c);
}

PG_API pg_status pg_huffman_kv_cache_get_kv_dev(pg_ctx *ctx, const pg_huffman_kv_cache *c, float *k_dev, float *v_dev) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(c != nullptr, "pg_huffman_kv_cache_get_kv: null cache");
    const pg_kv_cache *hot = c->hot;
    const size_t total_len = c->compressed_len + hot->len, hd = hot->head_dim, heads = hot->num_kv_heads;
    if (total_len * hd * heads == 0) return PG_OK;
    PG_CHECK_ARG(k_dev && v_dev, "pg_huffman_kv_cache_get_kv: null output");
    size_t off = 0;
    std::vector<const pg_huffman_kv_chunk *> chunks;
    std::vector<float *> outs;
    for (size_t i = 0; i < c->k_chunks.size(); ++i) {  // every chunk of both sides in one decoding pass
        chunks.push_back(c->k_chunks[i]);
        outs.push_back(k_dev + off * hd);
        chunks.push_back(c->v_chunks[i]);
        outs.push_back(v_dev + off * hd);
        off += c->k_chunks[i]->num_tokens;
    }
    const std::vector<size_t> strides(chunks.size(), total_len * hd);
    for (size_t first = 0; first < chunks.size(); first += 16384)  // (a launch takes up to 65535 chunks)
        PG_TRY(decompress_many(ctx, chunks.data() + first, outs.data() + first, strides.data() + first,
                               std::min<size_t>(16384, chunks.size() - first)));
    if (hot->len > 0) {
        const size_t width = hot->len * hd * sizeof(float);
        PG_HIP(hipMemcpy2DAsync(k_dev + off * hd, total_len * hd * sizeof(float), hot->k, hot->capacity * hd * sizeof(float), width,
                                heads, hipMemcpyDeviceToDevice, ctx->stream));
        PG_HIP(hipMemcpy2DAsync(v_dev + off * hd, total_len * hd * sizeof(float), hot->v, hot->capacity * hd * sizeof(float), width,
                                heads, hipMemcpyDeviceToDevice, ctx->stream));
    }
    return PG_OK;
}

PG_API pg_status pg_huffman_kv_cache_get_kv(pg_ctx *ctx, const pg_huffman_kv_cache *c, float *k, float *v) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(c != nullptr, "pg_huffman_kv_cache_get_kv: null cache");
    const size_t n = (c->compressed_len + c->hot->len) * c->hot->head_dim * c->hot->num_kv_heads;
    if (n == 0) return PG_OK;
    PG_CHECK_ARG(k && v, "pg_huffman_kv_cache_get_kv: null output");
    pg_tmp d;
    PG_TRY(d.alloc(2 * n * sizeof(float)));
    PG_TRY(pg_huffman_kv_cache_get_kv_dev(ctx, c, d.as<float>(), d.as<float>() + n));
    PG_HIP(hipMemcpyAsync(k, d.p, n * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipMemcpyAsync(v, d.as<float>() + n, n * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}
