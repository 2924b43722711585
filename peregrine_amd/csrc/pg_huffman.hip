// Canonical Huffman coding of int8 weights (peregrine's HuffmanTable / HuffmanTensor) in front
// of the W8A8 product: the table builder and the bit-serial encoder are host code (a format
// writer); decoding, which sits on the load path of every Huffman-coded weight, runs on the
// device.
//
//   HuffmanTable::from_frequencies / canonical_codes / build_decode_lut   reference: src/huffman.rs:35-213
//   HuffmanTable::encode / decode                                         reference: src/huffman.rs:216-284
//   HuffmanTensor::from_quantized / decode_to_quantized / to_gpu          reference: src/huffman.rs:332-435
//   matmul_huffman                                                        reference: src/huffman.rs:465-474
//
// Device decode.  A stream is a run of MSB-first variable-length codes with no markers, so the
// position of the i-th code is only known after decoding the i-1 before it.  The kernels use
// the self-synchronising property of Huffman codes instead of a serial walk: the stream is cut
// into subsequences of SUBSEQ_BITS bits, one thread each.  Every thread decodes from a guessed
// start (its subsequence's first bit) to the first code boundary past its end; a thread whose
// predecessor ended somewhere else than it started decodes again from there.  A wrong guess
// falls onto true code boundaries after a few symbols, so this settles in two or three
// rounds; it is exact when a whole round changes nothing (then start[g] == end[g-1] for every
// g, and start[0] = 0 is true by construction), and it is bounded by one round per workgroup.
// A prefix sum over the per-subsequence symbol counts then gives every thread its output
// offset and a last pass writes the symbols.
#include <algorithm>
#include <new>
#include "pg_internal.h"

namespace {

constexpr int NUM_SYMBOLS = 256;
constexpr int MAX_LUT_BITS = 12;          // src/huffman.rs:30
constexpr int LUT_SIZE = 1 << MAX_LUT_BITS;
constexpr int SUBSEQ_BITS = 256;          // bits per thread
constexpr int WG = 256;                   // subsequences per workgroup

// ---- host: table -------------------------------------------------------------------------

// src/huffman.rs:152-186
void canonical_codes(const uint8_t *bl, uint32_t *codes) {
    std::fill(codes, codes + NUM_SYMBOLS, 0u);
    int max_len = 0;
    for (int s = 0; s < NUM_SYMBOLS; ++s) max_len = std::max(max_len, (int)bl[s]);
    if (max_len == 0) return;
    std::vector<uint32_t> bl_count(max_len + 1, 0), next_code(max_len + 1, 0);
    for (int s = 0; s < NUM_SYMBOLS; ++s)
        if (bl[s] > 0) bl_count[bl[s]] += 1;
    uint32_t code = 0;
    for (int bits = 1; bits <= max_len; ++bits) {
        code = (code + bl_count[bits - 1]) << 1;
        next_code[bits] = code;
    }
    for (int s = 0; s < NUM_SYMBOLS; ++s)
        if (bl[s] > 0) codes[s] = next_code[bl[s]]++;
}

// Code lengths equal to those of src/huffman.rs:35-150 (two queues over the symbols in use,
// stably sorted by frequency; a leaf wins a tie against an internal node; depths clamped to
// MAX_LUT_BITS), computed in place in the sorted weight array without building the tree
// (Moffat & Katajainen's three passes).  Both give the same lengths because the two-queue
// construction consumes leaves in sorted order and a node consumed earlier never ends up
// shallower than one consumed later: the depth of the i-th leaf in sorted order is fixed by
// how many internal nodes each level holds, which is what the passes below count.
void table_from_frequencies(const uint64_t *freqs, uint8_t *bl) {
    std::fill(bl, bl + NUM_SYMBOLS, (uint8_t)0);
    int sym[NUM_SYMBOLS], n = 0;
    for (int s = 0; s < NUM_SYMBOLS; ++s)
        if (freqs[s] > 0) sym[n++] = s;
    if (n == 0) return;
    if (n == 1) { bl[sym[0]] = 1; return; }
    std::stable_sort(sym, sym + n, [&](int a, int b) { return freqs[a] < freqs[b]; });
    uint64_t w[NUM_SYMBOLS];  // weights, then parent indices, then depths
    for (int i = 0; i < n; ++i) w[i] = freqs[sym[i]];
    // Pass 1: w[t] becomes the weight of internal node t; a consumed internal node's slot holds
    // its parent.  `leaf` walks the unconsumed leaves, `node` the unconsumed internal nodes.
    int leaf = 0, node = 0;
    for (int t = 0; t < n - 1; ++t) {
        uint64_t sum = 0;
        for (int half = 0; half < 2; ++half) {
            const bool take_node = leaf >= n || (node < t && w[node] < w[leaf]);
            if (take_node) { sum += w[node]; w[node++] = (uint64_t)t; }
            else sum += w[leaf++];
        }
        // Leaves are consumed from the front and node t's slot is behind `leaf` by now (each
        // step consumes at least as many slots as it fills), so the write never lands on a
        // weight still to be read.
        w[t] = sum;
    }
    // Pass 2: parent indices to depths of the internal nodes, root (node n-2) first.
    w[n - 2] = 0;
    for (int t = n - 3; t >= 0; --t) w[t] = w[w[t]] + 1;
    // Pass 3: a level with `slots` places of which `inner` are internal nodes holds
    // slots - inner leaves, handed out from the most frequent symbol down.
    uint64_t depth = 0;
    int slots = 1, t = n - 2, next = n - 1;
    while (slots > 0) {
        int inner = 0;
        while (t >= 0 && w[t] == depth) { ++inner; --t; }
        for (; slots > inner; --slots) w[next--] = depth;
        slots = 2 * inner;
        ++depth;
    }
    for (int i = 0; i < n; ++i) bl[sym[i]] = (uint8_t)std::min<uint64_t>(w[i], MAX_LUT_BITS);
}

// A table for data that must decode again.  The reference's, where that is a prefix code.  Where
// its depth clamp over-subscribes the code (it then panics while filling its decode table,
// src/huffman.rs:189-213, so there is no reference result to match) the lengths are repaired:
// the deepest leaf above the limit's level is pushed down one level until the Kraft sum fits,
// any slack left is given to the most frequent symbols, and the resulting lengths are handed
// out again shortest to most frequent.  Returns whether the repair was needed.
bool table_that_decodes(const uint64_t *freqs, uint8_t *bl) {
    table_from_frequencies(freqs, bl);
    const long full = 1L << MAX_LUT_BITS;
    long kraft = 0;
    for (int s = 0; s < NUM_SYMBOLS; ++s)
        if (bl[s]) kraft += full >> bl[s];
    if (kraft <= full) return false;
    std::vector<int> by_freq;  // most frequent first, ties by symbol
    for (int s = 0; s < NUM_SYMBOLS; ++s)
        if (bl[s]) by_freq.push_back(s);
    std::stable_sort(by_freq.begin(), by_freq.end(), [&](int a, int b) { return freqs[a] > freqs[b]; });
    std::vector<int> len;
    for (int s : by_freq) len.push_back(bl[s]);
    std::sort(len.begin(), len.end());  // shortest first: position i belongs to by_freq[i]
    while (kraft > full) {              // lengthen the last (least frequent) leaf of the deepest level below the limit
        int pick = -1;
        for (int i = (int)len.size() - 1; i >= 0; --i)
            if (len[i] < MAX_LUT_BITS && (pick < 0 || len[i] > len[pick])) pick = i;
        kraft -= full >> (len[pick] + 1);
        len[pick] += 1;
        std::sort(len.begin(), len.end());
    }
    for (size_t i = 0; i < len.size(); ++i)  // spend the slack on the most frequent symbols
        while (len[i] > 1 && (full >> len[i]) <= full - kraft) {
            kraft += full >> len[i];
            len[i] -= 1;
        }
    std::sort(len.begin(), len.end());
    for (size_t i = 0; i < len.size(); ++i) bl[by_freq[i]] = (uint8_t)len[i];
    return true;
}

// src/huffman.rs:189-213 with the packing of to_gpu_lut (src/huffman.rs:727-736):
// entry = bit_length << 8 | (symbol + 128).  Codes that do not fit the table (a clamped,
// over-subscribed length set) are reported instead of indexing past it.
pg_status build_lut(const uint8_t *bl, const uint32_t *codes, uint16_t *lut) {
    std::fill(lut, lut + LUT_SIZE, (uint16_t)128);  // (symbol 0, length 0)
    for (int s = 0; s < NUM_SYMBOLS; ++s) {
        const int l = bl[s];
        if (l == 0 || l > MAX_LUT_BITS) continue;
        const int shift = MAX_LUT_BITS - l;
        const size_t base = (size_t)codes[s] << shift, count = (size_t)1 << shift;
        if (base + count > (size_t)LUT_SIZE)
            return pg_fail(PG_EINVAL, "huffman: the code of symbol %d does not fit %d bits (over-subscribed lengths)", s - 128,
                           MAX_LUT_BITS);
        for (size_t j = 0; j < count; ++j) lut[base + j] = (uint16_t)(l << 8 | s);
    }
    return PG_OK;
}

// src/huffman.rs:216-251
size_t encode_host(const uint8_t *bl, const uint32_t *codes, const int8_t *data, size_t n, uint8_t *out, size_t cap) {
    size_t bytes = 0;
    uint64_t acc = 0;  // bits not yet written, right-aligned
    int nacc = 0;
    for (size_t i = 0; i < n; ++i) {
        const int idx = (int)data[i] + 128, l = bl[idx];
        acc = (acc << l) | (codes[idx] & ((1u << l) - 1u));
        nacc += l;
        while (nacc >= 8) {
            if (bytes < cap) out[bytes] = (uint8_t)(acc >> (nacc - 8));
            ++bytes;
            nacc -= 8;
        }
    }
    if (nacc > 0) {
        if (bytes < cap) out[bytes] = (uint8_t)((acc << (8 - nacc)) & 0xFF);
        ++bytes;
    }
    return bytes;
}

// ---- device: decode ----------------------------------------------------------------------

struct stream_desc {
    const uint8_t *bytes;         // the stream, in device memory
    const uint16_t *lut;          // its decode table (LUT_SIZE entries), in device memory
    unsigned long long nbits;     // 8 * stream bytes
    unsigned long long nsym;      // symbols to produce
    unsigned long long out_off;   // into the output
    unsigned sub_base, nsub;      // subsequences of this stream
    unsigned wg_base, nwg;        // workgroups of this stream
};

// 12 bits at bit position p of an MSB-first stream of nbits bits, zero-padded past the end.
__device__ __forceinline__ unsigned peek12(const uint8_t *__restrict__ s, unsigned long long p, unsigned long long nbits) {
    const unsigned long long byte = p >> 3, nbytes = nbits >> 3;
    unsigned w = 0;
#pragma unroll
    for (int i = 0; i < 3; ++i) w = (w << 8) | (byte + i < nbytes ? s[byte + i] : 0u);
    return (w >> (12 - (unsigned)(p & 7))) & 0xFFFu;
}

// Decode from bit `start` to the first code boundary at or past `limit`.
__device__ __forceinline__ void decode_span(const uint8_t *__restrict__ s, unsigned long long nbits, const uint16_t *lut,
                                            unsigned long long start, unsigned long long limit, unsigned long long &end,
                                            unsigned &count) {
    unsigned long long p = start;
    unsigned c = 0;
    while (p < limit) {
        const unsigned l = lut[peek12(s, p, nbits)] >> 8;
        p += l ? l : 1;  // an unassigned code can only be met from a wrong guess: step on
        ++c;
    }
    end = p;
    count = c;
}

// The stream workgroup `wg` works on: the last one whose first workgroup is not past it.
__device__ __forceinline__ int find_stream(const stream_desc *__restrict__ desc, int nstreams, unsigned wg) {
    int lo = 0, hi = nstreams - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (desc[mid].wg_base <= wg) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

// One round: every workgroup settles its 256 subsequences against the end its predecessor
// workgroup reported last, and raises `changed` if anything moved.
__global__ __launch_bounds__(WG) void huff_sync_kernel(const stream_desc *__restrict__ desc, int nstreams, int first_round,
                                                       unsigned long long *__restrict__ start_g,
                                                       unsigned long long *end_g, unsigned *__restrict__ count_g,
                                                       int *__restrict__ changed) {
    __shared__ uint16_t lut[LUT_SIZE];
    __shared__ unsigned long long s_end[WG];
    const int si = find_stream(desc, nstreams, blockIdx.x);
    const stream_desc d = desc[si];
    for (int i = threadIdx.x; i < LUT_SIZE; i += WG) lut[i] = d.lut[i];
    const unsigned local = (blockIdx.x - d.wg_base) * WG + threadIdx.x;  // subsequence within the stream
    const bool live = local < d.nsub;
    const size_t g = (size_t)d.sub_base + local;
    const uint8_t *s = d.bytes;
    const unsigned long long limit = min((unsigned long long)(local + 1) * SUBSEQ_BITS, d.nbits);
    unsigned long long start = 0, end = 0;
    unsigned count = 0;
    __syncthreads();
    bool moved = false;
    if (live) {
        if (first_round) {
            start = (unsigned long long)local * SUBSEQ_BITS;
            decode_span(s, d.nbits, lut, start, limit, end, count);
            moved = true;
        } else {
            start = start_g[g];
            end = end_g[g];
            count = count_g[g];
        }
    }
    s_end[threadIdx.x] = end;
    for (int round = 0; round < WG + 1; ++round) {  // settles in at most WG rounds given the first start
        __syncthreads();
        unsigned long long want = start;
        if (live && local > 0) {
            // The neighbouring workgroup's last end is only there from the second round on.
            if (threadIdx.x > 0) want = s_end[threadIdx.x - 1];
            else if (!first_round) want = end_g[g - 1];
            // A predecessor ends on the first code boundary at or past this subsequence's first
            // bit; anything else is not an end it can have reported.
            const unsigned long long lo = (unsigned long long)local * SUBSEQ_BITS;
            if (want < lo || want >= lo + MAX_LUT_BITS) want = start;
        }
        __syncthreads();
        const bool redo = live && want != start;
        if (redo) {
            start = want;
            decode_span(s, d.nbits, lut, start, limit, end, count);
            s_end[threadIdx.x] = end;
            moved = true;
        }
        if (!__syncthreads_or(redo)) break;
    }
    if (live && moved) {
        start_g[g] = start;
        end_g[g] = end;
        count_g[g] = count;
        if (!first_round) *changed = 1;
    }
}

// Exclusive scan of the symbol counts inside each workgroup, and the workgroup totals.
__global__ __launch_bounds__(WG) void huff_scan_local_kernel(const stream_desc *__restrict__ desc, int nstreams,
                                                             const unsigned *__restrict__ count_g,
                                                             unsigned *__restrict__ excl_g,
                                                             unsigned long long *__restrict__ wg_total) {
    __shared__ unsigned sc[WG];
    const int si = find_stream(desc, nstreams, blockIdx.x);
    const stream_desc d = desc[si];
    const unsigned local = (blockIdx.x - d.wg_base) * WG + threadIdx.x;
    const bool live = local < d.nsub;
    const size_t g = (size_t)d.sub_base + local;
    const unsigned c = live ? count_g[g] : 0u;
    sc[threadIdx.x] = c;
    __syncthreads();
    for (int off = 1; off < WG; off <<= 1) {
        const unsigned add = threadIdx.x >= (unsigned)off ? sc[threadIdx.x - off] : 0u;
        __syncthreads();
        sc[threadIdx.x] += add;
        __syncthreads();
    }
    if (live) excl_g[g] = sc[threadIdx.x] - c;
    if (threadIdx.x == WG - 1) wg_total[blockIdx.x] = sc[WG - 1];
}

// One workgroup per stream: running sum of its workgroups' totals; a stream that decodes to
// fewer symbols than asked for is an error.
__global__ __launch_bounds__(64) void huff_scan_wg_kernel(const stream_desc *__restrict__ desc,
                                                          unsigned long long *__restrict__ wg_total, int *__restrict__ err) {
    if (threadIdx.x != 0) return;
    const stream_desc d = desc[blockIdx.x];
    unsigned long long run = 0;
    for (unsigned w = 0; w < d.nwg; ++w) {
        const unsigned long long t = wg_total[d.wg_base + w];
        wg_total[d.wg_base + w] = run;
        run += t;
    }
    if (run < d.nsym) *err = 1;
}

__global__ __launch_bounds__(WG) void huff_write_kernel(const stream_desc *__restrict__ desc, int nstreams,
                                                        const unsigned long long *__restrict__ start_g,
                                                        const unsigned *__restrict__ excl_g,
                                                        const unsigned long long *__restrict__ wg_excl,
                                                        int8_t *__restrict__ out, int *__restrict__ err) {
    __shared__ uint16_t lut[LUT_SIZE];
    const int si = find_stream(desc, nstreams, blockIdx.x);
    const stream_desc d = desc[si];
    for (int i = threadIdx.x; i < LUT_SIZE; i += WG) lut[i] = d.lut[i];
    __syncthreads();
    const unsigned local = (blockIdx.x - d.wg_base) * WG + threadIdx.x;
    if (local >= d.nsub) return;
    const size_t g = (size_t)d.sub_base + local;
    const uint8_t *s = d.bytes;
    const unsigned long long limit = min((unsigned long long)(local + 1) * SUBSEQ_BITS, d.nbits);
    unsigned long long p = start_g[g], idx = wg_excl[blockIdx.x] + excl_g[g];
    while (p < limit && idx < d.nsym) {
        const unsigned e = lut[peek12(s, p, d.nbits)];
        const unsigned l = e >> 8;
        if (l == 0) {  // "invalid code in bitstream" (src/huffman.rs:278)
            *err = 2;
            return;
        }
        out[d.out_off + idx] = (int8_t)((int)(e & 0xFF) - 128);
        p += l;
        ++idx;
    }
}

// Adds one stream of `bytes` bytes at bytes_dev holding `symbols` symbols, decoded through lut_dev to out + out_off.
pg_status add_stream(std::vector<stream_desc> &desc, const uint8_t *bytes_dev, const uint16_t *lut_dev, size_t bytes,
                     size_t symbols, size_t out_off, size_t &sub, size_t &wg) {
    stream_desc d;
    d.bytes = bytes_dev;
    d.lut = lut_dev;
    d.nbits = (unsigned long long)bytes * 8;
    d.nsym = symbols;
    d.out_off = out_off;
    const size_t nsub = (d.nbits + SUBSEQ_BITS - 1) / SUBSEQ_BITS, nwg = (nsub + WG - 1) / WG;
    PG_CHECK_ARG(sub + nsub < (1ull << 32) && wg + nwg < (1ull << 31), "huffman decode: stream too long");
    d.sub_base = (unsigned)sub; d.nsub = (unsigned)nsub; d.wg_base = (unsigned)wg; d.nwg = (unsigned)nwg;
    desc.push_back(d);
    sub += nsub;
    wg += nwg;
    return PG_OK;
}

// Decode the streams `desc` describes (bytes in device memory) into out_dev.  Streams without a
// table of their own (lut == nullptr) share the one built here from bit_lengths.
pg_status decode_device_streams(pg_ctx *ctx, const uint8_t *bit_lengths, std::vector<stream_desc> desc, size_t sub, size_t wg,
                                int8_t *out_dev) {
    if (desc.empty()) return PG_OK;
    // one allocation: descriptors | lut | start | end | count | excl | wg totals | flags
    const size_t o_lut = pg_round_up(desc.size() * sizeof(stream_desc), 256);
    const size_t o_start = o_lut + LUT_SIZE * sizeof(uint16_t), o_end = o_start + pg_round_up(sub * 8, 256);
    const size_t o_count = o_end + pg_round_up(sub * 8, 256), o_excl = o_count + pg_round_up(sub * 4, 256);
    const size_t o_wg = o_excl + pg_round_up(sub * 4, 256), o_flag = o_wg + pg_round_up(wg * 8, 256);
    pg_tmp buf;
    PG_TRY(buf.alloc(o_flag + 256));
    char *base = buf.as<char>();
    std::vector<uint16_t> lut;
    if (bit_lengths) {
        uint32_t codes[NUM_SYMBOLS];
        lut.resize(LUT_SIZE);
        canonical_codes(bit_lengths, codes);
        PG_TRY(build_lut(bit_lengths, codes, lut.data()));
        PG_HIP(hipMemcpyAsync(base + o_lut, lut.data(), LUT_SIZE * sizeof(uint16_t), hipMemcpyHostToDevice, ctx->stream));
    }
    for (auto &d : desc) {
        if (!d.lut) d.lut = reinterpret_cast<const uint16_t *>(base + o_lut);
        PG_CHECK_ARG(d.lut != reinterpret_cast<const uint16_t *>(base + o_lut) || bit_lengths, "huffman decode: a stream without a table");
    }
    PG_HIP(hipMemsetAsync(base + o_flag, 0, 256, ctx->stream));
    PG_HIP(hipMemcpyAsync(base, desc.data(), desc.size() * sizeof(stream_desc), hipMemcpyHostToDevice, ctx->stream));
    const stream_desc *d_desc = reinterpret_cast<const stream_desc *>(base);
    auto *d_start = reinterpret_cast<unsigned long long *>(base + o_start);
    auto *d_end = reinterpret_cast<unsigned long long *>(base + o_end);
    auto *d_count = reinterpret_cast<unsigned *>(base + o_count);
    auto *d_excl = reinterpret_cast<unsigned *>(base + o_excl);
    auto *d_wg = reinterpret_cast<unsigned long long *>(base + o_wg);
    int *d_changed = reinterpret_cast<int *>(base + o_flag), *d_err = d_changed + 1;
    const int ns = (int)desc.size();
    PG_TRY(pg_launch(ctx, "huffman_sync", huff_sync_kernel, dim3((unsigned)wg), dim3(WG), 0, d_desc, ns, 1, d_start, d_end, d_count,
                     d_changed));
    for (size_t round = 0;; ++round) {
        if (round > wg + 1) return pg_fail(PG_EDEVICE, "huffman decode: the subsequence starts did not settle");
        PG_TRY(pg_launch(ctx, "huffman_sync", huff_sync_kernel, dim3((unsigned)wg), dim3(WG), 0, d_desc, ns, 0, d_start, d_end,
                         d_count, d_changed));
        int changed = 0;
        PG_HIP(hipMemcpyAsync(&changed, d_changed, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
        PG_HIP(hipStreamSynchronize(ctx->stream));
        if (!changed) break;
        PG_HIP(hipMemsetAsync(d_changed, 0, sizeof(int), ctx->stream));
    }
    PG_TRY(pg_launch(ctx, "huffman_scan", huff_scan_local_kernel, dim3((unsigned)wg), dim3(WG), 0, d_desc, ns,
                     (const unsigned *)d_count, d_excl, d_wg));
    PG_TRY(pg_launch(ctx, "huffman_scan_wg", huff_scan_wg_kernel, dim3((unsigned)ns), dim3(64), 0, d_desc, d_wg, d_err));
    PG_TRY(pg_launch(ctx, "huffman_write", huff_write_kernel, dim3((unsigned)wg), dim3(WG), 0, d_desc, ns,
                     (const unsigned long long *)d_start, (const unsigned *)d_excl, (const unsigned long long *)d_wg, out_dev,
                     d_err));
    int err = 0;
    PG_HIP(hipMemcpyAsync(&err, d_err, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    if (err == 1) return pg_fail(PG_EINVAL, "huffman decode: a bitstream ends before its symbol count is reached");
    if (err == 2) return pg_fail(PG_EINVAL, "huffman decode: invalid code in bitstream");
    return PG_OK;
}

// Decode `nstreams` streams (host bytes) into out_dev.  streams[i] has bytes[i] bytes and
// holds symbols[i] symbols, written back to back.
pg_status decode_streams(pg_ctx *ctx, const uint8_t *bit_lengths, const uint8_t *const *streams, const size_t *bytes,
                         const size_t *symbols, size_t nstreams, int8_t *out_dev) {
    size_t total = 0;
    for (size_t i = 0; i < nstreams; ++i) {
        if (symbols[i] == 0) continue;
        PG_CHECK_ARG(bytes[i] > 0 && streams[i], "huffman decode: stream %zu holds %zu symbols in no bytes", i, symbols[i]);
        total += pg_round_up(bytes[i], 16);
    }
    if (total == 0) return PG_OK;
    pg_tmp buf;
    PG_TRY(buf.alloc(total));
    std::vector<stream_desc> desc;
    size_t byte_off = 0, out_off = 0, sub = 0, wg = 0;
    for (size_t i = 0; i < nstreams; ++i) {
        if (symbols[i] == 0) continue;
        PG_TRY(add_stream(desc, buf.as<uint8_t>() + byte_off, nullptr, bytes[i], symbols[i], out_off, sub, wg));
        PG_HIP(hipMemcpyAsync(buf.as<char>() + byte_off, streams[i], bytes[i], hipMemcpyHostToDevice, ctx->stream));
        byte_off += pg_round_up(bytes[i], 16);
        out_off += symbols[i];
    }
    return decode_device_streams(ctx, bit_lengths, desc, sub, wg, out_dev);
}

}  // namespace

// HuffmanTensor  src/huffman.rs:311-325 (host-resident, as in the reference).
struct pg_huffman_tensor {
    uint8_t bit_lengths[NUM_SYMBOLS];
    std::vector<std::vector<uint8_t>> streams;
    std::vector<size_t> stream_lengths;
    std::vector<float> scales;
    size_t rows, cols;
};

// For the other Huffman translation unit (the KV cache): the host table and one device-resident stream.
bool pg_huffman_host_table(const uint64_t *freqs, uint8_t *bit_lengths, uint32_t *codes) {
    const bool repaired = table_that_decodes(freqs, bit_lengths);
    canonical_codes(bit_lengths, codes);
    return repaired;
}

// The decode table of a code (LUT entries of 16 bits, pg_huffman_lut_entries() of them) on the host.
size_t pg_huffman_lut_entries() { return LUT_SIZE; }
pg_status pg_huffman_host_lut(const uint8_t *bit_lengths, uint16_t *lut) {
    uint32_t codes[NUM_SYMBOLS];
    canonical_codes(bit_lengths, codes);
    return build_lut(bit_lengths, codes, lut);
}

// Streams that sit in device memory, each with its own table there, decoded in one pass.
pg_status pg_huffman_decode_device_streams(pg_ctx *ctx, const pg_huffman_dev_stream *streams, size_t count, int8_t *out_dev) {
    std::vector<stream_desc> desc;
    size_t sub = 0, wg = 0;
    for (size_t i = 0; i < count; ++i) {
        const pg_huffman_dev_stream &st = streams[i];
        if (st.symbols == 0) continue;
        PG_CHECK_ARG(st.bytes > 0 && st.bytes_dev && st.lut_dev, "huffman decode: %zu symbols in no bytes or without a table", st.symbols);
        PG_TRY(add_stream(desc, st.bytes_dev, st.lut_dev, st.bytes, st.symbols, st.out_off, sub, wg));
    }
    return decode_device_streams(ctx, nullptr, desc, sub, wg, out_dev);
}

pg_status pg_qtensor_from_device_q(pg_ctx *ctx, const int8_t *q_dev, const float *scales_host, size_t rows, size_t cols,
                                   pg_qtensor **out);

PG_API pg_status pg_huffman_table_from_frequencies(const uint64_t *freqs, uint8_t *bit_lengths, uint32_t *codes) {
    PG_CHECK_ARG(freqs && bit_lengths, "pg_huffman_table_from_frequencies: null pointer");
    table_from_frequencies(freqs, bit_lengths);
    if (codes) canonical_codes(bit_lengths, codes);
    return PG_OK;
}

PG_API pg_status pg_huffman_canonical_codes(const uint8_t *bit_lengths, uint32_t *codes) {
    PG_CHECK_ARG(bit_lengths && codes, "pg_huffman_canonical_codes: null pointer");
    canonical_codes(bit_lengths, codes);
    return PG_OK;
}

PG_API pg_status pg_huffman_encode(const uint8_t *bit_lengths, const int8_t *data, size_t n, uint8_t *out, size_t cap,
                                   size_t *bytes) {
    PG_CHECK_ARG(bit_lengths && bytes, "pg_huffman_encode: null pointer");
    *bytes = 0;
    if (n == 0) return PG_OK;
    PG_CHECK_ARG(data != nullptr, "pg_huffman_encode: null data");
    uint32_t codes[NUM_SYMBOLS];
    canonical_codes(bit_lengths, codes);
    for (size_t i = 0; i < n; ++i)
        PG_CHECK_ARG(bit_lengths[(int)data[i] + 128] > 0 && bit_lengths[(int)data[i] + 128] <= MAX_LUT_BITS,
                     "pg_huffman_encode: symbol %d has no code of 1..%d bits", (int)data[i], MAX_LUT_BITS);
    *bytes = encode_host(bit_lengths, codes, data, n, out, out ? cap : 0);
    PG_CHECK_ARG(out == nullptr || *bytes <= cap, "pg_huffman_encode: %zu bytes needed, %zu given", *bytes, cap);
    return PG_OK;
}

PG_API pg_status pg_huffman_decode(pg_ctx *ctx, const uint8_t *bit_lengths, const uint8_t *bitstream, size_t len,
                                   size_t num_symbols, int8_t *out) {
    PG_TRY(pg_use(ctx));
    if (num_symbols == 0) return PG_OK;
    PG_CHECK_ARG(bit_lengths && bitstream && out, "pg_huffman_decode: null pointer");
    pg_tmp dout;
    PG_TRY(dout.alloc(num_symbols));
    PG_TRY(decode_streams(ctx, bit_lengths, &bitstream, &len, &num_symbols, 1, dout.as<int8_t>()));
    PG_HIP(hipMemcpyAsync(out, dout.p, num_symbols, hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

PG_API void pg_huffman_tensor_free(pg_huffman_tensor *t) { delete t; }

PG_API pg_status pg_huffman_tensor_from_quantized(const int8_t *q, const float *scales, size_t rows, size_t cols,
                                                  size_t num_streams, pg_huffman_tensor **out) {
    PG_CHECK_ARG(out != nullptr, "pg_huffman_tensor_from_quantized: out is null");
    *out = nullptr;
    PG_CHECK_ARG((q && scales) || rows * cols == 0, "pg_huffman_tensor_from_quantized: null pointer");
    if (num_streams < 1) num_streams = 1;
    const size_t total = rows * cols;
    pg_huffman_tensor *t = new (std::nothrow) pg_huffman_tensor();
    if (!t) return pg_fail(PG_ENOMEM, "host allocation failed");
    uint64_t freqs[NUM_SYMBOLS] = {0};
    for (size_t i = 0; i < total; ++i) freqs[(int)q[i] + 128] += 1;
    table_from_frequencies(freqs, t->bit_lengths);
    uint32_t codes[NUM_SYMBOLS];
    canonical_codes(t->bit_lengths, codes);
    const size_t chunk = (total + num_streams - 1) / num_streams;
    t->streams.resize(num_streams);
    t->stream_lengths.assign(num_streams, 0);
    for (size_t s = 0; s < num_streams; ++s) {
        const size_t start = s * chunk;
        if (start >= total) continue;
        const size_t n = std::min(chunk, total - start);
        const size_t bytes = encode_host(t->bit_lengths, codes, q + start, n, nullptr, 0);
        t->streams[s].resize(bytes);
        encode_host(t->bit_lengths, codes, q + start, n, t->streams[s].data(), bytes);
        t->stream_lengths[s] = n;
    }
    t->scales.assign(scales, scales + cols);
    t->rows = rows;
    t->cols = cols;
    *out = t;
    return PG_OK;
}

PG_API pg_status pg_huffman_tensor_from_parts(const uint8_t *bit_lengths, const uint8_t *const *streams,
                                              const size_t *stream_bytes, const size_t *stream_lengths, size_t num_streams,
                                              const float *scales, size_t rows, size_t cols, pg_huffman_tensor **out) {
    PG_CHECK_ARG(out != nullptr, "pg_huffman_tensor_from_parts: out is null");
    *out = nullptr;
    PG_CHECK_ARG(bit_lengths && streams && stream_bytes && stream_lengths && scales, "pg_huffman_tensor_from_parts: null pointer");
    size_t total = 0;
    for (size_t s = 0; s < num_streams; ++s) total += stream_lengths[s];
    PG_CHECK_ARG(total == rows * cols, "pg_huffman_tensor_from_parts: the streams hold %zu symbols, the matrix %zu", total,
                 rows * cols);
    pg_huffman_tensor *t = new (std::nothrow) pg_huffman_tensor();
    if (!t) return pg_fail(PG_ENOMEM, "host allocation failed");
    memcpy(t->bit_lengths, bit_lengths, NUM_SYMBOLS);
    t->streams.resize(num_streams);
    for (size_t s = 0; s < num_streams; ++s)
        if (stream_bytes[s]) t->streams[s].assign(streams[s], streams[s] + stream_bytes[s]);
    t->stream_lengths.assign(stream_lengths, stream_lengths + num_streams);
    t->scales.assign(scales, scales + cols);
    t->rows = rows;
    t->cols = cols;
    *out = t;
    return PG_OK;
}

PG_API pg_status pg_huffman_tensor_info(const pg_huffman_tensor *t, size_t *rows, size_t *cols, size_t *num_streams,
                                        size_t *compressed_size) {
    PG_CHECK_ARG(t != nullptr, "pg_huffman_tensor_info: null tensor");
    if (rows) *rows = t->rows;
    if (cols) *cols = t->cols;
    if (num_streams) *num_streams = t->streams.size();
    if (compressed_size) {  // src/huffman.rs:407-412: bitstreams + codebook + scales
        size_t b = NUM_SYMBOLS + t->cols * 4;
        for (const auto &s : t->streams) b += s.size();
        *compressed_size = b;
    }
    return PG_OK;
}

PG_API pg_status pg_huffman_tensor_stream(const pg_huffman_tensor *t, size_t index, const uint8_t **data, size_t *bytes,
                                          size_t *symbols) {
    PG_CHECK_ARG(t != nullptr && index < t->streams.size(), "pg_huffman_tensor_stream: no stream %zu", index);
    if (data) *data = t->streams[index].data();
    if (bytes) *bytes = t->streams[index].size();
    if (symbols) *symbols = t->stream_lengths[index];
    return PG_OK;
}

PG_API pg_status pg_huffman_tensor_table(const pg_huffman_tensor *t, const uint8_t **bit_lengths, const float **scales) {
    PG_CHECK_ARG(t != nullptr, "pg_huffman_tensor_table: null tensor");
    if (bit_lengths) *bit_lengths = t->bit_lengths;
    if (scales) *scales = t->scales.data();
    return PG_OK;
}

static pg_status huffman_decode_to_device(pg_ctx *ctx, const pg_huffman_tensor *t, int8_t *q_dev) {
    std::vector<const uint8_t *> ptrs(t->streams.size());
    std::vector<size_t> bytes(t->streams.size());
    for (size_t s = 0; s < t->streams.size(); ++s) { ptrs[s] = t->streams[s].data(); bytes[s] = t->streams[s].size(); }
    return decode_streams(ctx, t->bit_lengths, ptrs.data(), bytes.data(), t->stream_lengths.data(), t->streams.size(), q_dev);
}

PG_API pg_status pg_huffman_tensor_to_gpu(pg_ctx *ctx, const pg_huffman_tensor *t, pg_qtensor **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(t && out, "pg_huffman_tensor_to_gpu: null pointer");
    *out = nullptr;
    PG_CHECK_ARG(t->rows > 0 && t->cols > 0, "pg_huffman_tensor_to_gpu: empty tensor");
    pg_tmp dq;
    PG_TRY(dq.alloc(t->rows * t->cols));
    PG_TRY(huffman_decode_to_device(ctx, t, dq.as<int8_t>()));
    return pg_qtensor_from_device_q(ctx, dq.as<int8_t>(), t->scales.data(), t->rows, t->cols, out);
}

PG_API pg_status pg_huffman_tensor_decode_to_quantized(pg_ctx *ctx, const pg_huffman_tensor *t, int8_t *q, int8_t *q_t,
                                                       float *scales) {
    pg_qtensor *qt = nullptr;
    PG_TRY(pg_huffman_tensor_to_gpu(ctx, t, &qt));
    const pg_status st = pg_qtensor_download(ctx, qt, q, q_t, scales);
    pg_qtensor_free(ctx, qt);
    return st;
}

PG_API pg_status pg_matmul_huffman(pg_ctx *ctx, const float *a, size_t m, size_t k, const pg_huffman_tensor *t, float *out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(t != nullptr, "pg_matmul_huffman: null tensor");
    PG_CHECK_ARG(t->rows == k, "matmul_huffman: ht.rows %zu != k %zu", t->rows, k);
    pg_qtensor *qt = nullptr;
    PG_TRY(pg_huffman_tensor_to_gpu(ctx, t, &qt));
    const pg_status st = pg_matmul_quantized(ctx, a, m, k, qt, out);
    pg_qtensor_free(ctx, qt);
    return st;
}
