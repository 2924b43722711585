// The glue of peregrine's Llama decoder block around the quantised products: RMSNorm, RoPE,
// the KV cache, grouped-query attention and the block itself, all on the device so that a
// block step is one chain of stream-ordered launches with no host round trip.
//
//   nn::RMSNorm::forward            reference: src/nn.rs:577-652
//   nn::RoPE::{new, apply}          reference: src/nn.rs:1250-1345
//   attention::StandardKVCache      reference: src/attention.rs:8-100
//   attention::gqa_attention_cpu    reference: src/attention.rs:141-300
//   LlamaAttention::forward         reference: src/models/llama/attention.rs:73-212
//   LlamaBlock::forward             reference: src/models/llama/decoder.rs:69-155
//
// Layouts (all f32, row-major):
//   KV cache   k, v [num_kv_heads][capacity][head_dim], `len` positions valid per head
//   RoPE       cos, sin [max_seq_len][head_dim] (the half-row repeated, as the reference holds it)
//   q          [num_q_heads][seq_q][head_dim]; attention output [seq_q][num_q_heads * head_dim]
#include <math.h>
#include <new>
#include <vector>
#include "pg_internal.h"
#include "pg_digits.h"
#include "pg_f16_planes.h"

struct pg_rope {
    float *cos_t, *sin_t;
    size_t head_dim, max_seq_len;
};


struct pg_llama_block {
    size_t d, nqh, nkvh, hd, ffn;
    float eps;
    pg_rope *rope;
    const pg_gguf_tensor *w[7];  // q, k, v, o, gate, up, down (borrowed)
    float *attn_norm_w, *ffn_norm_w;
    float *ss_part;  // one-token step: sums of squares of the attention output row, by block of 32
    float *arena;  // activations for seq_cap tokens
    size_t seq_cap;
    void *chain;   // many-token step: digit planes of the three product inputs and the products' K-chunk planes
    size_t chain_bytes;
    // One-token step: digit buffers for the three GEMV inputs (model_dim, q_dim, ffn) and the
    // device tables that let k/v and gate/up each run as one two-item launch.
    void *dec;                        // one allocation
    pg_xdigits xd_d, xd_q, xd_f;
    const uint8_t *const *qs_qkv, *const *qs_gu;   // q cut into kv_dim-row items, then k, v; gate, up
    const uint16_t *const *d_qkv, *const *d_gu;
    const int *item_ids;              // 0, 1, 2, ...
    int qkv_items;                    // num_q_heads / num_kv_heads + 2
    int digit_kind;                   // PG_GGML_Q4_0 (nibble digits), PG_GGML_Q8_0 (byte digits), 0 = mixed: no fused step
};

namespace {

constexpr int PG_MAX_PLANES = 8;  // K chunks of a split block product (pg_gguf_mm_splitk never makes more)

__device__ __forceinline__ float block_sum(float v, float *red) {
    v = pg_wave_sum_f32(v);
    const int wave = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) t += red[i];
    return t;
}

__device__ __forceinline__ float block_max(float v, float *red) {
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m));
    const int wave = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < (int)(blockDim.x >> 6); ++i) t = fmaxf(t, red[i]);
    return t;
}

// One workgroup per row: s = a (+ b), optionally stored, then out = s / rms(s) * w.
// Generic two-pass form for any dim.
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(const float *a, const float *__restrict__ b, float *sum_out,
                                                          const float *__restrict__ w, float eps, int dim,
                                                          float *__restrict__ out) {
    __shared__ float red[4];
    const size_t row = (size_t)blockIdx.x * dim;
    float ss = 0.f;
    for (int i = threadIdx.x; i < dim; i += 256) {
        float s = a[row + i];
        if (b) {
            s = s + b[row + i];
            sum_out[row + i] = s;
        }
        ss += s * s;
    }
    ss = block_sum(ss, red);
    const float inv_rms = 1.0f / sqrtf(ss * (1.0f / (float)dim) + eps);
    const float *src = b ? sum_out : a;  // a thread re-reads only what it wrote itself
    for (int i = threadIdx.x; i < dim; i += 256) out[row + i] = src[row + i] * inv_rms * w[i];
}

// The same with the row held in registers: dim % 4 == 0 and dim <= 1024 * MAXV, so that every
// load of the row is issued before the first is needed.
// DIG: 0 = write the normalised row as f32; 1 / 2 = write it as nibble / byte digits for the
// streaming product instead (dim a multiple of 32, so that 8-lane groups hold whole blocks); 3 / 4 = as the
// two byte-digit planes of the matrix-core block product (Q4_0 / Q8_0 element order); 5 = as the two f16 planes of
// the f16 matrix-core product (pg_f16_planes.h): hi plane at `digits`, lo plane at `out`, the rows' two inverse
// scale factors at `xs`.
// The second input may come as b_planes planes, b_stride4 float4 apart (the K chunks of a split product,
// summed here in ascending order before the addition, as gguf_mm's own summing pass would).
template <int MAXV, int DIG>
__global__ __launch_bounds__(256) void add_rmsnorm_vec_kernel(const float4 *__restrict__ a, const float4 *__restrict__ b,
                                                              float4 *__restrict__ sum_out, const float4 *__restrict__ w,
                                                              float eps, int dim4, float4 *__restrict__ out,
                                                              int8_t *__restrict__ digits, float *__restrict__ xs,
                                                              int b_planes, size_t b_stride4) {
    __shared__ float red[4];
    const size_t row = (size_t)blockIdx.x * dim4;
    float4 v[MAXV], wv[MAXV];
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int i = threadIdx.x + 256 * j;
        v[j] = i < dim4 ? a[row + i] : float4{0.f, 0.f, 0.f, 0.f};
    }
    if (b) {
#pragma unroll
        for (int j = 0; j < MAXV; ++j) {
            const int i = threadIdx.x + 256 * j;
            if (i < dim4) {
                float4 tp[PG_MAX_PLANES];  // every plane requested before the first is used
#pragma unroll
                for (int pl = 0; pl < PG_MAX_PLANES; ++pl)
                    tp[pl] = pl < b_planes ? b[pl * b_stride4 + row + i] : float4{0.f, 0.f, 0.f, 0.f};
                float4 t = tp[0];
#pragma unroll
                for (int pl = 1; pl < PG_MAX_PLANES; ++pl)
                    if (pl < b_planes) { t.x += tp[pl].x; t.y += tp[pl].y; t.z += tp[pl].z; t.w += tp[pl].w; }
                v[j].x += t.x; v[j].y += t.y; v[j].z += t.z; v[j].w += t.w;
                sum_out[row + i] = v[j];
            }
        }
    }
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int i = threadIdx.x + 256 * j;
        wv[j] = i < dim4 ? w[i] : float4{0.f, 0.f, 0.f, 0.f};
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < MAXV; ++j) ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
    ss = block_sum(ss, red);
    const float inv_rms = 1.0f / sqrtf(ss * (1.0f / (float)(dim4 * 4)) + eps);
    if constexpr (DIG == 5) {
        float amax = 0.f;
#pragma unroll
        for (int j = 0; j < MAXV; ++j) {
            const int i = threadIdx.x + 256 * j;
            if (i < dim4) {
                v[j] = float4{v[j].x * inv_rms * wv[j].x, v[j].y * inv_rms * wv[j].y, v[j].z * inv_rms * wv[j].z, v[j].w * inv_rms * wv[j].w};
                amax = fmaxf(amax, fmaxf(fmaxf(pg_f16_mag(v[j].x), pg_f16_mag(v[j].y)), fmaxf(pg_f16_mag(v[j].z), pg_f16_mag(v[j].w))));
            }
        }
        const pg_f16_row_scale sc = pg_f16_row_scale_of(block_max(amax, red));
        if (threadIdx.x == 0) {
            xs[2 * blockIdx.x] = sc.i1;
            xs[2 * blockIdx.x + 1] = sc.i2;
        }
        _Float16 *hi = reinterpret_cast<_Float16 *>(digits), *lo = reinterpret_cast<_Float16 *>(out);
#pragma unroll
        for (int j = 0; j < MAXV; ++j) {
            const int i = threadIdx.x + 256 * j;
            if (i < dim4) {
                const float o[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
                pg_f16_split4(o, sc, reinterpret_cast<uint2 *>(hi + (row + i) * 4), reinterpret_cast<uint2 *>(lo + (row + i) * 4));
            }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int i = threadIdx.x + 256 * j;
        if (i < dim4) {
            const float o[4] = {v[j].x * inv_rms * wv[j].x, v[j].y * inv_rms * wv[j].y, v[j].z * inv_rms * wv[j].z,
                                v[j].w * inv_rms * wv[j].w};
            if constexpr (DIG == 0) out[row + i] = float4{o[0], o[1], o[2], o[3]};
            else if constexpr (DIG <= 2) pg_emit_digits<DIG == 1>(o, blockIdx.x, i >> 3, i & 7, dim4 >> 3, digits, xs);
            else pg_emit_mm_digits<DIG == 3>(o, blockIdx.x, i >> 3, i & 7, dim4 >> 3, ((dim4 >> 3) + 3) & ~3, digits, xs);
        }
    }
}

// Up to three [seq][heads*hd] sources re-laid head-major, rotated or copied.
struct rope_seg {
    const float *src;  // token t, head h at src + t*src_tstride + h*hd
    float *dst;        // at dst + h*dst_hstride + t*hd
    size_t src_tstride, dst_hstride;
    int heads, rotate;
    int planes = 1;          // src as the sum of this many planes (the K chunks of a split product), in ascending order
    size_t plane_stride = 0;
};
struct rope_args {
    rope_seg seg[3];
    const float *cos_t, *sin_t;
    int hd, pos0, nseg;
};

__global__ __launch_bounds__(128) void rope_kernel(rope_args ra) {
    const int t = blockIdx.x;
    int h = blockIdx.y, s = 0;
    while (s < ra.nseg - 1 && h >= ra.seg[s].heads) h -= ra.seg[s++].heads;
    const rope_seg sg = ra.seg[s];
    const float *src = sg.src + (size_t)t * sg.src_tstride + (size_t)h * ra.hd;
    float *dst = sg.dst + (size_t)h * sg.dst_hstride + (size_t)t * ra.hd;
    const int half = ra.hd / 2;
    auto at = [&](int i) {
        float xp[PG_MAX_PLANES];
#pragma unroll
        for (int pl = 0; pl < PG_MAX_PLANES; ++pl) xp[pl] = pl < sg.planes ? src[pl * sg.plane_stride + i] : 0.f;
        float x = xp[0];
#pragma unroll
        for (int pl = 1; pl < PG_MAX_PLANES; ++pl)
            if (pl < sg.planes) x += xp[pl];
        return x;
    };
    if (!sg.rotate) {
        for (int i = threadIdx.x; i < ra.hd; i += 128) dst[i] = at(i);
        return;
    }
    const float *c = ra.cos_t + (size_t)(ra.pos0 + t) * ra.hd, *sn = ra.sin_t + (size_t)(ra.pos0 + t) * ra.hd;
    for (int i = threadIdx.x; i < half; i += 128) {
        const float x0 = at(i), x1 = at(half + i);
        dst[i] = x0 * c[i] - x1 * sn[i];
        dst[half + i] = x0 * sn[i] + x1 * c[i];
    }
}

// The same for head sizes that are multiples of 8 with every pointer and stride a multiple of four floats: a
// thread takes dims 4j .. 4j+3 and their partners half + 4j .. as 128-bit loads and stores, 256 / (hd / 8)
// heads of one token to a workgroup (the operations per element are those of rope_kernel, in its order).
__global__ __launch_bounds__(256) void rope_v4_kernel(rope_args ra, int total_heads) {
    const int t = blockIdx.x, per = ra.hd >> 3;
    const int idx = blockIdx.y * 256 + threadIdx.x;
    int h = idx / per, s = 0;
    const int j = idx - h * per;
    if (h >= total_heads) return;
    while (s < ra.nseg - 1 && h >= ra.seg[s].heads) h -= ra.seg[s++].heads;
    const rope_seg sg = ra.seg[s];
    const float *src = sg.src + (size_t)t * sg.src_tstride + (size_t)h * ra.hd;
    float *dst = sg.dst + (size_t)h * sg.dst_hstride + (size_t)t * ra.hd;
    const int half = ra.hd / 2;
    auto at = [&](int i) {
        float4 xp[PG_MAX_PLANES];
#pragma unroll
        for (int pl = 0; pl < PG_MAX_PLANES; ++pl)
            xp[pl] = pl < sg.planes ? *reinterpret_cast<const float4 *>(src + pl * sg.plane_stride + i) : make_float4(0.f, 0.f, 0.f, 0.f);
        float4 x = xp[0];
#pragma unroll
        for (int pl = 1; pl < PG_MAX_PLANES; ++pl)
            if (pl < sg.planes) { x.x += xp[pl].x; x.y += xp[pl].y; x.z += xp[pl].z; x.w += xp[pl].w; }
        return x;
    };
    const float4 x0 = at(4 * j), x1 = at(half + 4 * j);
    if (!sg.rotate) {
        *reinterpret_cast<float4 *>(dst + 4 * j) = x0;
        *reinterpret_cast<float4 *>(dst + half + 4 * j) = x1;
        return;
    }
    const size_t row = (size_t)(ra.pos0 + t) * ra.hd + 4 * j;
    const float4 c = *reinterpret_cast<const float4 *>(ra.cos_t + row), sn = *reinterpret_cast<const float4 *>(ra.sin_t + row);
    float4 lo, hi;
    lo.x = x0.x * c.x - x1.x * sn.x; hi.x = x0.x * sn.x + x1.x * c.x;
    lo.y = x0.y * c.y - x1.y * sn.y; hi.y = x0.y * sn.y + x1.y * c.y;
    lo.z = x0.z * c.z - x1.z * sn.z; hi.z = x0.z * sn.z + x1.z * c.z;
    lo.w = x0.w * c.w - x1.w * sn.w; hi.w = x0.w * sn.w + x1.w * c.w;
    *reinterpret_cast<float4 *>(dst + 4 * j) = lo;
    *reinterpret_cast<float4 *>(dst + half + 4 * j) = hi;
}

// Mask kinds 0..2 as in the header; 3 = LocalGlobal (src/attention.rs:287-299): `window` is the
// local window and bit kt of `gbits` says that key position kt is a global one.
__device__ __forceinline__ bool attn_masked(int mask_kind, int offset, int window, int sink, const uint32_t *gbits, int qt,
                                            int kt) {
    if (mask_kind == 0) return false;
    const int query_pos = offset + qt;
    if (kt > query_pos) return true;
    if (mask_kind == 1) return false;
    if (mask_kind == 3) {
        if (query_pos - kt <= window) return false;
        return !((gbits[kt >> 5] >> (kt & 31)) & 1u);
    }
    if (kt < sink) return false;
    return query_pos - kt > window;
}

struct attn_args {
    const float *q, *kc, *vc;
    float *part, *out;          // part: [row][split][hd + 2] = (max, exp-sum, unnormalised P.V) when splits > 1
    size_t k_stride, v_stride;  // per kv head
    int len, nqh, group, seq_q, hd, lanes;  // lanes = power of two >= hd/4, <= 64
    int chunk, splits;                       // keys per split (the LDS score buffer holds one chunk)
    float scale, logit_cap;
    int mask_kind, offset, window, sink, accumulate;
    const uint32_t *gbits;      // mask kind 3: one bit per key position
    // One-token step with RoPE and the cache append folded in (short kernel only; null raw_q =
    // off): q, k, v as the projections left them ([heads, hd] each), the cos / sin rows of the
    // new position, and where its rotated key and its value belong in the caches.
    const float *raw_q, *raw_k, *raw_v, *rope_c, *rope_s;
    float *k_new, *v_new;       // cache rows of position new_pos, kv head 0
    int new_pos;
};

constexpr int ATT_RED = 1024;     // partial output rows: (256 / lanes) slices x (lanes * 4) dims
constexpr int ATT_CHUNK_MAX = 8192;  // keys per workgroup: 32 KB of scores in LDS

// One workgroup per (query token, query head, key split).  Scores: `lanes` lanes share one
// key, four dims each, so that a key row is one contiguous read; softmax over the split's
// scores held in LDS; then P.V with the same lane-to-dim mapping, the keys cut into
// 256/lanes slices whose partial rows are summed in a fixed order.  With one split the
// result is normalised and written (or added) here; with several, each split leaves its
// maximum, exp-sum and unnormalised row for gqa_combine_kernel.  Causal masks also cut the
// key range at the query position, so that a prefill does not visit keys it cannot see.
__global__ __launch_bounds__(256) void gqa_attention_kernel(attn_args aa) {
    extern __shared__ float lds[];
    __shared__ float red[4];
    const int tid = threadIdx.x, qt = blockIdx.x, qh = blockIdx.y, split = blockIdx.z, kvh = qh / aa.group;
    const int L = aa.lanes, hd = aa.hd;
    const int k0 = split * aa.chunk;
    int k1 = min(aa.len, k0 + aa.chunk);
    if (aa.mask_kind != 0) k1 = min(k1, aa.offset + qt + 1);
    const int n = max(k1 - k0, 0);  // keys of this split, uniform over the workgroup
    float *qs = lds, *part = lds + 256, *sc = lds + 256 + ATT_RED;
    const float *qsrc = aa.q + ((size_t)qh * aa.seq_q + qt) * hd;
    for (int i = tid; i < 4 * L; i += 256) qs[i] = i < hd ? qsrc[i] : 0.f;
    __syncthreads();
    const int sub = tid / L, within = tid % L, nsub = 256 / L, d0 = within * 4;
    const bool vec = (hd & 3) == 0;
    const float *kbase = aa.kc + (size_t)kvh * aa.k_stride + (size_t)k0 * hd;
    const float *vbase = aa.vc + (size_t)kvh * aa.v_stride + (size_t)k0 * hd;
    float q4[4];
    for (int j = 0; j < 4; ++j) q4[j] = qs[d0 + j];

    float mx = -INFINITY;
    const int rounds = (n + nsub - 1) / nsub;
    for (int r = 0; r < rounds; ++r) {  // every lane runs every round: the shuffles need the whole wave
        const int kt = r * nsub + sub;
        float dot = 0.f;
        const bool live = kt < n && !attn_masked(aa.mask_kind, aa.offset, aa.window, aa.sink, aa.gbits, qt, k0 + kt);
        if (live && d0 < hd) {
            const float *kr = kbase + (size_t)kt * hd + d0;
            if (vec) {
                const float4 kv = *reinterpret_cast<const float4 *>(kr);
                dot = q4[0] * kv.x + q4[1] * kv.y + q4[2] * kv.z + q4[3] * kv.w;
            } else {
                for (int j = 0; j < 4; ++j)
                    if (d0 + j < hd) dot += q4[j] * kr[j];
            }
        }
        for (int m = 1; m < L; m <<= 1) dot += __shfl_xor(dot, m);
        if (kt < n) {
            float s = -INFINITY;
            if (live) {
                s = dot * aa.scale;
                if (aa.logit_cap > 0.f) s = aa.logit_cap * tanhf(s / aa.logit_cap);
            }
            if (within == 0) sc[kt] = s;
            mx = fmaxf(mx, s);
        }
    }
    mx = block_max(mx, red);  // the barriers inside also publish sc[]
    float sum = 0.f;
    for (int kt = tid; kt < n; kt += 256) {
        const float s = sc[kt];
        const float e = s == -INFINITY ? 0.f : expf(s - mx);
        sc[kt] = e;
        sum += e;
    }
    sum = block_sum(sum, red);
    const bool final_pass = aa.splits == 1;
    const float inv_sum = !final_pass ? 1.0f : (sum > 0.f ? 1.0f / sum : 0.f);

    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (d0 < hd) {
        for (int kt = sub; kt < n; kt += nsub) {
            const float p = sc[kt] * inv_sum;
            if (p > 0.f) {
                const float *vr = vbase + (size_t)kt * hd + d0;
                if (vec) {
                    const float4 vv = *reinterpret_cast<const float4 *>(vr);
                    acc[0] += p * vv.x; acc[1] += p * vv.y; acc[2] += p * vv.z; acc[3] += p * vv.w;
                } else {
                    for (int j = 0; j < 4; ++j)
                        if (d0 + j < hd) acc[j] += p * vr[j];
                }
            }
        }
    }
    for (int j = 0; j < 4; ++j) part[sub * (4 * L) + d0 + j] = acc[j];
    __syncthreads();
    const size_t rowi = (size_t)qt * aa.nqh + qh;
    float *pdst = final_pass ? nullptr : aa.part + (rowi * aa.splits + split) * (size_t)(hd + 2);
    if (!final_pass && tid == 0) {
        pdst[0] = mx;
        pdst[1] = sum;
    }
    for (int i = tid; i < hd; i += 256) {
        float o = 0.f;
        for (int s = 0; s < nsub; ++s) o += part[s * (4 * L) + i];
        if (final_pass) {
            float *dst = aa.out + rowi * hd + i;
            *dst = aa.accumulate ? *dst + o : o;
        } else {
            pdst[2 + i] = o;
        }
    }
}

// The same for a split of at most 8 rounds of keys (the one-token step): q, the split's K rows
// and its V rows are all requested at once, scores stay in registers, and the only exchanges
// are the two block reductions and the sum over key slices.
constexpr int ATT_SHORT_ROUNDS = 8;
__global__ __launch_bounds__(256) void gqa_attention_short_kernel(attn_args aa) {
    __shared__ float part[ATT_RED];
    __shared__ float red[4];
    // Workgroups go to the 8 XCDs round-robin.  All query rows that read the same keys (the
    // heads of one kv group, every query token) are given to ONE XCD, one after the other, so
    // that its L2 fetches that split's K and V rows once: workgroup id = 8 * j + xcd, the
    // j-th workgroup of an XCD being member j % members of key set (j / members) * 8 + xcd.
    const int members = aa.group * aa.seq_q, nkv = aa.nqh / aa.group;
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    const int member = j % members, set = (j / members) * 8 + xcd;
    if (set >= nkv * aa.splits) return;  // the grid is rounded up to whole rounds of 8 key sets
    const int kvh = set % nkv, split = set / nkv, qh = kvh * aa.group + member % aa.group, qt = member / aa.group;
    const int tid = threadIdx.x;
    const int L = aa.lanes, hd = aa.hd;
    const int k0 = split * aa.chunk;
    int k1 = min(aa.len, k0 + aa.chunk);
    if (aa.mask_kind != 0) k1 = min(k1, aa.offset + qt + 1);
    const int n = max(k1 - k0, 0);
    const int sub = tid / L, within = tid % L, nsub = 256 / L, d0 = within * 4;
    const bool vec = (hd & 3) == 0, have = d0 < hd;
    const float *qsrc = aa.q + ((size_t)qh * aa.seq_q + qt) * hd + d0;
    const float *kbase = aa.kc + (size_t)kvh * aa.k_stride + (size_t)k0 * hd + d0;
    const float *vbase = aa.vc + (size_t)kvh * aa.v_stride + (size_t)k0 * hd + d0;
    auto load4 = [&](const float *p) {
        float4 r = {0.f, 0.f, 0.f, 0.f};
        if (vec) {
            r = *reinterpret_cast<const float4 *>(p);
        } else {
            r.x = p[0];
            if (d0 + 1 < hd) r.y = p[1];
            if (d0 + 2 < hd) r.z = p[2];
            if (d0 + 3 < hd) r.w = p[3];
        }
        return r;
    };
    // This lane's four dims of a head row after RoPE (pairs (i, i + hd/2), the operations of
    // rope_kernel in the same order); hd is a multiple of 8 on this route.
    const bool fused = aa.raw_q != nullptr;
    auto rot4 = [&](const float *row) {
        const int half = hd >> 1, i0 = d0 < half ? d0 : d0 - half;
        const float4 x0 = *reinterpret_cast<const float4 *>(row + i0), x1 = *reinterpret_cast<const float4 *>(row + half + i0);
        const float4 c = *reinterpret_cast<const float4 *>(aa.rope_c + i0), sn = *reinterpret_cast<const float4 *>(aa.rope_s + i0);
        float4 r;
        if (d0 < half) {
            r.x = x0.x * c.x - x1.x * sn.x; r.y = x0.y * c.y - x1.y * sn.y;
            r.z = x0.z * c.z - x1.z * sn.z; r.w = x0.w * c.w - x1.w * sn.w;
        } else {
            r.x = x0.x * sn.x + x1.x * c.x; r.y = x0.y * sn.y + x1.y * c.y;
            r.z = x0.z * sn.z + x1.z * c.z; r.w = x0.w * sn.w + x1.w * c.w;
        }
        return r;
    };
    float4 q4 = {0.f, 0.f, 0.f, 0.f}, kv[ATT_SHORT_ROUNDS], vv[ATT_SHORT_ROUNDS];
    bool live[ATT_SHORT_ROUNDS];
    if (have) q4 = fused ? rot4(aa.raw_q + (size_t)qh * hd) : load4(qsrc);
#pragma unroll
    for (int u = 0; u < ATT_SHORT_ROUNDS; ++u) {
        const int kt = u * nsub + sub;
        live[u] = kt < n && !attn_masked(aa.mask_kind, aa.offset, aa.window, aa.sink, aa.gbits, qt, k0 + kt);
        kv[u] = float4{0.f, 0.f, 0.f, 0.f};
        vv[u] = float4{0.f, 0.f, 0.f, 0.f};
        if (live[u] && have) {
            if (fused && k0 + kt == aa.new_pos) {
                // The new position is not in the cache yet: every workgroup that needs it makes
                // it from the projections, and the first member of the key set also stores it.
                kv[u] = rot4(aa.raw_k + (size_t)kvh * hd);
                vv[u] = *reinterpret_cast<const float4 *>(aa.raw_v + (size_t)kvh * hd + d0);
                if (member == 0) {
                    *reinterpret_cast<float4 *>(aa.k_new + (size_t)kvh * aa.k_stride + d0) = kv[u];
                    *reinterpret_cast<float4 *>(aa.v_new + (size_t)kvh * aa.v_stride + d0) = vv[u];
                }
            } else {
                kv[u] = load4(kbase + (size_t)kt * hd);
                vv[u] = load4(vbase + (size_t)kt * hd);
            }
        }
    }
    float s[ATT_SHORT_ROUNDS], mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < ATT_SHORT_ROUNDS; ++u) {
        float dot = q4.x * kv[u].x + q4.y * kv[u].y + q4.z * kv[u].z + q4.w * kv[u].w;
        for (int m = 1; m < L; m <<= 1) dot += __shfl_xor(dot, m);
        s[u] = -INFINITY;
        if (live[u]) {
            s[u] = dot * aa.scale;
            if (aa.logit_cap > 0.f) s[u] = aa.logit_cap * tanhf(s[u] / aa.logit_cap);
        }
        mx = fmaxf(mx, s[u]);
    }
    mx = block_max(mx, red);
    float sum = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < ATT_SHORT_ROUNDS; ++u) {
        const float e = s[u] == -INFINITY ? 0.f : expf(s[u] - mx);
        if (within == 0) sum += e;  // one lane per key
        s[u] = e;
    }
    sum = block_sum(sum, red);
    const bool final_pass = aa.splits == 1;
    const float inv_sum = !final_pass ? 1.0f : (sum > 0.f ? 1.0f / sum : 0.f);
#pragma unroll
    for (int u = 0; u < ATT_SHORT_ROUNDS; ++u) {
        const float p = s[u] * inv_sum;
        if (p > 0.f) { acc[0] += p * vv[u].x; acc[1] += p * vv[u].y; acc[2] += p * vv[u].z; acc[3] += p * vv[u].w; }
    }
    for (int j = 0; j < 4; ++j) part[sub * (4 * L) + d0 + j] = acc[j];
    __syncthreads();
    const size_t rowi = (size_t)qt * aa.nqh + qh;
    float *pdst = final_pass ? nullptr : aa.part + (rowi * aa.splits + split) * (size_t)(hd + 2);
    if (!final_pass && tid == 0) {
        pdst[0] = mx;
        pdst[1] = sum;
    }
    for (int i = tid; i < hd; i += 256) {
        float o = 0.f;
        for (int ss = 0; ss < nsub; ++ss) o += part[ss * (4 * L) + i];
        if (final_pass) {
            float *dst = aa.out + rowi * hd + i;
            *dst = aa.accumulate ? *dst + o : o;
        } else {
            pdst[2 + i] = o;
        }
    }
}

// ---- many query rows (prefill), head size 256: tiled, online softmax -------------------------
// (head sizes 64 and 128 run on the matrix cores, further down; the template is kept general)
// One (token, head) row per workgroup makes every row stream all of its keys and values again
// and spends most instructions on cross-lane sums.  Here a workgroup owns 32 query rows that
// read the SAME kv head (the heads of a group, then consecutive tokens), eight per wavefront,
// and walks the keys in blocks of 64 staged through LDS:
//   scores   lane = key: the lane walks its key row (LDS, row stride HD + 4 floats: conflict
//            free 128-bit reads) against the eight query rows, which are wavefront-uniform
//            and come in through scalar loads as FMA operands: no cross-lane traffic at all,
//            32 FMAs per LDS read;
//   softmax  online (running maximum and sum per row, accumulators rescaled), the only
//            cross-lane work: two wavefront reductions per row and block;
//   P.V      lane = HD/64 output dims: probabilities read back four keys at a time as
//            broadcasts, value rows as coalesced LDS reads.
// K and V share one LDS buffer (K staged, scores, V staged, P.V); the next tile is fetched into
// registers while the current one is used.  Any cache length, no key splits.
__device__ __forceinline__ float wave_max_f32(float v) {
    auto dpp_max = [](float x, auto ctrl) {
        const int y = __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xf, 0xf, false);
        return fmaxf(x, __builtin_bit_cast(float, y));
    };
    v = dpp_max(v, std::integral_constant<int, 0xB1>{});
    v = dpp_max(v, std::integral_constant<int, 0x4E>{});
    v = dpp_max(v, std::integral_constant<int, 0x141>{});
    v = dpp_max(v, std::integral_constant<int, 0x140>{});
    const int b = __builtin_bit_cast(int, v);
    return fmaxf(fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)), __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16))),
                 fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)), __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48))));
}

constexpr int ATT_T_ROWS = 32, ATT_T_RW = 8, ATT_T_KB = 64;
template <int HD> constexpr size_t att_tiled_lds() { return (size_t)(ATT_T_KB * (HD + 4) + 4 * ATT_T_RW * ATT_T_KB) * sizeof(float); }

template <int HD>
__global__ __launch_bounds__(256) void gqa_attention_tiled_kernel(attn_args aa) {
    constexpr int ROWS = ATT_T_ROWS, RW = ATT_T_RW, KB = ATT_T_KB, KS = HD + 4, DPL = HD / 64, C4 = HD / 4;
    constexpr int TPT = KB * C4 / 256;  // float4 of a staged tile per thread
    extern __shared__ float lds[];
    float *kv_l = lds, *p_l = kv_l + KB * KS;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kvh = blockIdx.y, G = aa.group, row0 = blockIdx.x * ROWS, nrows = G * aa.seq_q;  // row index = qt * G + g
    auto row_qt = [&](int row) { return min(row, nrows - 1) / G; };
    auto row_qh = [&](int row) { return kvh * G + min(row, nrows - 1) % G; };
    // The eight query rows of this wavefront are the same for all of its lanes: they are read
    // through wavefront-uniform addresses (scalar loads), not staged (rows past the end repeat
    // the last one and are not stored).
    int qt_of[RW];
    const float *qrow[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        qt_of[r] = row_qt(row0 + wave * RW + r);
        qrow[r] = aa.q + ((size_t)row_qh(row0 + wave * RW + r) * aa.seq_q + qt_of[r]) * HD;
    }
    int kend = aa.len;
    if (aa.mask_kind != 0) kend = min(kend, aa.offset + row_qt(row0 + ROWS - 1) + 1);
    const int nblocks = (kend + KB - 1) / KB;
    const float *kg = aa.kc + (size_t)kvh * aa.k_stride, *vg = aa.vc + (size_t)kvh * aa.v_stride;
    auto fetch = [&](const float *base, int k0, float4 (&reg)[TPT]) {  // tile rows k0 .. k0+63, zeros past kend
#pragma unroll
        for (int i = 0; i < TPT; ++i) {
            const int idx = tid + 256 * i, key = idx / C4, c = idx - key * C4;
            reg[i] = float4{0.f, 0.f, 0.f, 0.f};
            if (k0 + key < kend) reg[i] = *reinterpret_cast<const float4 *>(base + (size_t)(k0 + key) * HD + 4 * c);
        }
    };
    auto stage = [&](const float4 (&reg)[TPT], int stride) {
#pragma unroll
        for (int i = 0; i < TPT; ++i) {
            const int idx = tid + 256 * i, key = idx / C4, c = idx - key * C4;
            *reinterpret_cast<float4 *>(kv_l + key * stride + 4 * c) = reg[i];
        }
    };
    float m[RW], l[RW], o[RW][DPL];
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        m[r] = -INFINITY;
        l[r] = 0.f;
#pragma unroll
        for (int d = 0; d < DPL; ++d) o[r][d] = 0.f;
    }
    float4 treg[TPT];
    for (int kb = 0; kb < nblocks; ++kb) {
        const int k0 = kb * KB;
        __syncthreads();  // the previous block's P.V has finished with kv_l
        fetch(kg, k0, treg);
        stage(treg, KS);
        __syncthreads();
        // scores of key k0 + lane against this wavefront's rows
        float s[RW];
#pragma unroll
        for (int r = 0; r < RW; ++r) s[r] = 0.f;
        const float *krow = kv_l + lane * KS;
#pragma unroll 4
        for (int c = 0; c < C4; ++c) {
            const float4 k4 = *reinterpret_cast<const float4 *>(krow + 4 * c);
#pragma unroll
            for (int r = 0; r < RW; ++r) {
                const float4 q4 = *reinterpret_cast<const float4 *>(qrow[r] + 4 * c);
                s[r] = fmaf(q4.w, k4.w, fmaf(q4.z, k4.z, fmaf(q4.y, k4.y, fmaf(q4.x, k4.x, s[r]))));  // the build does not contract a*b+c
            }
        }
        __syncthreads();  // every wavefront has read K
        fetch(vg, k0, treg);
        stage(treg, HD);
        // online softmax
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            float sv = -INFINITY;
            if (k0 + lane < kend && !attn_masked(aa.mask_kind, aa.offset, aa.window, aa.sink, aa.gbits, qt_of[r], k0 + lane)) {
                sv = s[r] * aa.scale;
                if (aa.logit_cap > 0.f) sv = aa.logit_cap * tanhf(sv / aa.logit_cap);
            }
            const float m_new = fmaxf(m[r], wave_max_f32(sv));
            const float alpha = m[r] == -INFINITY ? 1.0f : expf(m[r] - m_new);  // nothing accumulated yet: any factor
            const float pv = sv == -INFINITY ? 0.f : expf(sv - m_new);
            l[r] = l[r] * alpha + pg_wave_sum_f32(pv);
#pragma unroll
            for (int d = 0; d < DPL; ++d) o[r][d] *= alpha;
            m[r] = m_new;
            p_l[(wave * RW + r) * KB + lane] = pv;
        }
        __syncthreads();  // V is staged, the probabilities are written
        const float *prow = p_l + wave * RW * KB;
#pragma unroll 2
        for (int k4 = 0; k4 < KB; k4 += 4) {
            float4 p4[RW];
#pragma unroll
            for (int r = 0; r < RW; ++r) p4[r] = *reinterpret_cast<const float4 *>(prow + r * KB + k4);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float v[DPL];
                const float *vrow = kv_l + (k4 + j) * HD + DPL * lane;
                if constexpr (DPL == 1) v[0] = vrow[0];
                else if constexpr (DPL == 2) { const float2 t = *reinterpret_cast<const float2 *>(vrow); v[0] = t.x; v[1] = t.y; }
                else { const float4 t = *reinterpret_cast<const float4 *>(vrow); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
#pragma unroll
                for (int r = 0; r < RW; ++r) {
                    const float pj = j == 0 ? p4[r].x : (j == 1 ? p4[r].y : (j == 2 ? p4[r].z : p4[r].w));
#pragma unroll
                    for (int d = 0; d < DPL; ++d) o[r][d] = fmaf(pj, v[d], o[r][d]);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        const int row = row0 + wave * RW + r;
        if (row >= nrows) continue;
        const float inv = l[r] > 0.f ? 1.0f / l[r] : 0.f;
        float *dst = aa.out + ((size_t)(row / G) * aa.nqh + kvh * G + row % G) * HD + DPL * lane;
#pragma unroll
        for (int d = 0; d < DPL; ++d) dst[d] = aa.accumulate ? dst[d] + o[r][d] * inv : o[r][d] * inv;
    }
}

// ---- many query rows on the matrix cores -------------------------------------------------------
// v_mfma_f32_32x32x2_f32 runs f32 multiply-adds at twice the rate the vector unit reaches without
// packed operations, and keeps its 32x32 tile in registers.  A wavefront owns 32 query rows of
// one kv head (row index = token * group + head in group, as above) and walks the keys 32 at a
// time, with both products transposed so that nothing has to change lanes in between:
//   S^T[key][row] = sum_d K[key][d] Q[row][d]     A = K tile (lane: key, half h), B = Q (lane: row, h)
//   O^T[d][row]  += sum_key V[key][d] P^T[key][row]   A = V tile, B = the probabilities
// The tile a lane holds after the first product (column = row l%32, register r = key
// 8(r/4) + 4h + r%4) is exactly a B operand of the second, register by register: summation
// indices may be visited in any order, so step j of the second product takes key 8(j/4) + 4h + j%4
// from half h, and the V operand is loaded in that order.  The same freedom makes every load
// 128 bits wide: step 4i+c of the first product takes d = 8i + 4h + c, and output row i of d-tile
// dt stands for d = (HD/32) i + dt.  K, V and Q go from L2 straight into operand registers; no LDS,
// no barrier inside the key loop.  Softmax is online per column; a column's two halves exchange
// only their maxima (lane ^ 32), the sums are joined at the end.
// Causal work is uneven (row block i sees i + 1 key tiles), so a workgroup of two wavefronts takes
// the pair (i, n - 1 - i) and cuts the pair's tiles in two equal parts: wavefront 0 the first part
// of the long item, wavefront 1 the short item and the rest of the long one, whose partial
// (maximum, sum, rows) it hands over through LDS.
typedef float v16f __attribute__((ext_vector_type(16)));

// SPLIT (few rows under a long cache: a chunk of a prefill, a handful of draft tokens): the keys are cut
// into aa.splits runs of aa.chunk tiles as well, workgroup = one wavefront = (kv head, item, run), no
// hand-over; every wavefront leaves (maximum, exp-sum, unnormalised rows) for gqa_combine_kernel in rows of
// HD + 4 floats, or an empty record where its rows see none of the run's keys.
template <int HD, bool SPLIT = false>
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gqa_attention_mfma_kernel(attn_args aa, int n_items, int nkvh) {
    constexpr int NDT = HD / 32, QR = HD / 2;
    typedef float vdt __attribute__((ext_vector_type(NDT)));
    __shared__ float part_l[SPLIT ? 1 : (NDT * 16 + 2) * 64];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col = lane & 31, h = lane >> 5;
    const int kvh = blockIdx.x % nkvh;
    const int pair = SPLIT ? (blockIdx.x / nkvh) % n_items : blockIdx.x / nkvh;  // SPLIT: the item itself
    const int run = SPLIT ? (blockIdx.x / nkvh) / n_items : 0;
    const int G = aa.group, nrows = G * aa.seq_q;
    const int item_a = pair, item_b = n_items - 1 - pair;  // the short and the long one (equal: one item)
    auto kend_of = [&](int item) {
        const int last_qt = min(item * 32 + 31, nrows - 1) / G;
        return aa.mask_kind != 0 ? min(aa.len, aa.offset + last_qt + 1) : aa.len;
    };
    const int tb = (kend_of(item_b) + 31) / 32, ta = item_a != item_b ? (kend_of(item_a) + 31) / 32 : 0;
    const int cut = min(tb, (ta + tb + 1) / 2);
    const float *kg = aa.kc + (size_t)kvh * aa.k_stride, *vg = aa.vc + (size_t)kvh * aa.v_stride;

    float m = -INFINITY, l = 0.f;
    v16f o[NDT];
    int row = 0, qt = 0, qh = 0;
    for (int seg = 0; seg < (SPLIT ? 1 : 2); ++seg) {
        // wavefront 0: (long item, tiles [0, cut)), nothing; wavefront 1: (short item, all), (long item, [cut, tb))
        int item = (wave == 0 || seg == 1) ? item_b : item_a;
        int t0 = wave == 0 ? 0 : (seg == 0 ? 0 : cut);
        int t1 = wave == 0 ? (seg == 0 ? cut : 0) : (seg == 0 ? ta : tb);
        if constexpr (SPLIT) {
            item = pair;
            t0 = run * aa.chunk;
            t1 = min((kend_of(item) + 31) / 32, t0 + aa.chunk);
        } else {
            if (t1 <= t0) continue;
        }
        const int kend = kend_of(item);
        row = item * 32 + col;
        const int rowc = min(row, nrows - 1);
        qt = rowc / G;
        qh = kvh * G + rowc % G;
        const int qt_min = (item * 32) / G;
        float *const rec = SPLIT ? aa.part + (((size_t)qt * aa.nqh + qh) * aa.splits + run) * (size_t)(HD + 4) : nullptr;
        if constexpr (SPLIT) {
            if (t1 <= t0) {  // none of the run's keys are before these rows
                if (row < nrows) {
                    if (h == 0) *reinterpret_cast<float2 *>(rec) = float2{-INFINITY, 0.f};
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        vdt z;
#pragma unroll
                        for (int dt = 0; dt < NDT; ++dt) z[dt] = 0.f;
                        *reinterpret_cast<vdt *>(rec + 4 + NDT * (8 * (r >> 2) + 4 * h + (r & 3))) = z;
                    }
                }
                return;
            }
        }
        m = -INFINITY;
        l = 0.f;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;
        float qreg[QR];
        {
            const float *qp = aa.q + ((size_t)qh * aa.seq_q + qt) * HD + 4 * h;
#pragma unroll
            for (int i = 0; i < HD / 8; ++i) {
                const float4 v = *reinterpret_cast<const float4 *>(qp + 8 * i);
                qreg[4 * i] = v.x; qreg[4 * i + 1] = v.y; qreg[4 * i + 2] = v.z; qreg[4 * i + 3] = v.w;
            }
        }
        float4 kreg[HD / 8];
        vdt vreg[16];
        auto load_k = [&](int t) {
            const float *kp = kg + (size_t)min(32 * t + col, kend - 1) * HD + 4 * h;
#pragma unroll
            for (int i = 0; i < HD / 8; ++i) kreg[i] = *reinterpret_cast<const float4 *>(kp + 8 * i);
        };
        auto load_v = [&](int t) {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int key = min(32 * t + 8 * (j >> 2) + 4 * h + (j & 3), kend - 1);
                vreg[j] = *reinterpret_cast<const vdt *>(vg + (size_t)key * HD + NDT * col);
            }
        };
        auto scores = [&](v16f &s) {  // S^T of the tile in kreg
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
            for (int i = 0; i < HD / 8; ++i) {
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(kreg[i].x, qreg[4 * i], s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(kreg[i].y, qreg[4 * i + 1], s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(kreg[i].z, qreg[4 * i + 2], s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(kreg[i].w, qreg[4 * i + 3], s, 0, 0, 0);
            }
        };
        // scale, cap and mask the raw scores of tile t (the branches are wavefront-uniform and kept out of
        // the straight-line part below, which the scheduler interleaves with the next tile's products)
        auto finish_scores = [&](v16f &s, int t) {
            const int k0 = 32 * t;
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] *= aa.scale;
            if (aa.logit_cap > 0.f) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = aa.logit_cap * tanhf(s[r] / aa.logit_cap);
            }
            const bool all_visible = k0 + 31 < kend && (aa.mask_kind == 0 || (aa.mask_kind == 1 && k0 + 31 <= aa.offset + qt_min));
            if (!all_visible) {
                // attn_masked() as plain bit arithmetic (selects, no lane-dependent branches); a tile's 32 keys
                // share one word of the global-position bits
                const int mk = aa.mask_kind, qp = aa.offset + qt;
                const uint32_t gw = mk == 3 ? aa.gbits[t] : 0u;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int kin = 8 * (r >> 2) + 4 * h + (r & 3), key = k0 + kin;
                    const bool far = qp - key > aa.window;
                    const bool hide = (key >= kend) | ((mk != 0) & (key > qp)) | ((mk == 2) & (key >= aa.sink) & far) |
                                      ((mk == 3) & far & !((gw >> kin) & 1u));
                    s[r] = hide ? -INFINITY : s[r];
                }
            }
        };
        // online softmax of this lane's column (16 of its 32 keys here, the rest in lane ^ 32): s becomes p
        auto softmax = [&](v16f &s) {
            float mt = s[0];
#pragma unroll
            for (int r = 1; r < 16; ++r) mt = fmaxf(mt, s[r]);
            mt = fmaxf(mt, __shfl_xor(mt, 32));
            const float m_new = fmaxf(m, mt);
            const float alpha = m == -INFINITY ? 1.0f : expf(m - m_new);
            float psum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = s[r] == -INFINITY ? 0.f : expf(s[r] - m_new);
                s[r] = p;
                psum += p;
            }
            l = l * alpha + psum;
            m = m_new;
            return alpha;
        };
        auto rescale = [&](float alpha) {
            if (__any(alpha != 1.0f)) {
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
            }
        };
        auto weighted_values = [&](const v16f &p) {
#pragma unroll
            for (int j = 0; j < 16; ++j)
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt) o[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vreg[j][dt], p[j], o[dt], 0, 0, 0);
        };
        // Software pipeline: while the vector unit turns tile t's scores into probabilities, the matrix
        // unit already forms tile t+1's scores; K is requested two tiles ahead, V one.
        v16f s_cur, s_next;
        load_k(t0);
        load_v(t0);
        scores(s_cur);
        if (t0 + 1 < t1) load_k(t0 + 1);
        for (int t = t0; t + 1 < t1; ++t) {
            finish_scores(s_cur, t);
            __builtin_amdgcn_sched_barrier(0);
            // column maximum first, then four matrix instructions of tile t+1 for every probability of tile t:
            // the order is pinned so that the vector work runs while the matrix unit is busy
            float mt = s_cur[0];
#pragma unroll
            for (int r = 1; r < 16; ++r) mt = fmaxf(mt, s_cur[r]);
            mt = fmaxf(mt, __shfl_xor(mt, 32));
            const float m_new = fmaxf(m, mt);
            const float alpha = m == -INFINITY ? 1.0f : expf(m - m_new);
            float psum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) s_next[r] = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = r * (HD / 8) / 16; i < (r + 1) * (HD / 8) / 16; ++i) {
                    s_next = __builtin_amdgcn_mfma_f32_32x32x2f32(kreg[i].x, qreg[4 * i], s_next, 0, 0, 0);
                    s_next = __builtin_amdgcn_mfma_f32_32x32x2f32(kreg[i].y, qreg[4 * i + 1], s_next, 0, 0, 0);
                    s_next = __builtin_amdgcn_mfma_f32_32x32x2f32(kreg[i].z, qreg[4 * i + 2], s_next, 0, 0, 0);
                    s_next = __builtin_amdgcn_mfma_f32_32x32x2f32(kreg[i].w, qreg[4 * i + 3], s_next, 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                const float p = s_cur[r] == -INFINITY ? 0.f : expf(s_cur[r] - m_new);
                s_cur[r] = p;
                psum += p;
            }
            l = l * alpha + psum;
            m = m_new;
            // the probabilities are pinned to this block (a use with side effects): left alone, the compiler moves
            // their computation past the matrix instructions, next to its first use
            asm volatile("" ::"v"(s_cur), "v"(l));
            __builtin_amdgcn_sched_barrier(0);
            load_k(min(t + 2, t1 - 1));  // unconditional (the last one repeats a tile): no branch splits the block
            rescale(alpha);
            weighted_values(s_cur);
            __builtin_amdgcn_sched_barrier(0);
            load_v(t + 1);
            s_cur = s_next;
        }
        finish_scores(s_cur, t1 - 1);
        rescale(softmax(s_cur));
        weighted_values(s_cur);
        if constexpr (SPLIT) {
            const float lt = l + __shfl_xor(l, 32);
            if (row < nrows) {
                if (h == 0) *reinterpret_cast<float2 *>(rec) = float2{m, lt};
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    vdt v;
#pragma unroll
                    for (int dt = 0; dt < NDT; ++dt) v[dt] = o[dt][r];
                    *reinterpret_cast<vdt *>(rec + 4 + NDT * (8 * (r >> 2) + 4 * h + (r & 3))) = v;
                }
            }
            return;
        }
        if (wave == 1 && seg == 0) {  // the short item is complete
            const float lt = l + __shfl_xor(l, 32);
            const float inv = lt > 0.f ? 1.0f / lt : 0.f;
            if (row < nrows) {
                float *dst = aa.out + ((size_t)qt * aa.nqh + qh) * HD;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    vdt v;
#pragma unroll
                    for (int dt = 0; dt < NDT; ++dt) v[dt] = o[dt][r] * inv;
                    vdt *p = reinterpret_cast<vdt *>(dst + NDT * (8 * (r >> 2) + 4 * h + (r & 3)));
                    *p = aa.accumulate ? *p + v : v;
                }
            }
        } else if (wave == 1) {  // the rest of the long item: hand it to wavefront 0
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) part_l[(dt * 16 + r) * 64 + lane] = o[dt][r];
            part_l[NDT * 16 * 64 + lane] = m;
            part_l[(NDT * 16 + 1) * 64 + lane] = l;
        }
    }
    __syncthreads();
    if (wave != 0) return;
    if (cut < tb) {  // join the two parts of the long item
        const float m1 = part_l[NDT * 16 * 64 + lane], l1 = part_l[(NDT * 16 + 1) * 64 + lane];
        const float mm = fmaxf(m, m1);
        const float w0 = m == -INFINITY ? 0.f : expf(m - mm), w1 = m1 == -INFINITY ? 0.f : expf(m1 - mm);
        l = l * w0 + l1 * w1;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[dt][r] = o[dt][r] * w0 + part_l[(dt * 16 + r) * 64 + lane] * w1;
    }
    const float lt = l + __shfl_xor(l, 32);
    const float inv = lt > 0.f ? 1.0f / lt : 0.f;
    if (row < nrows) {
        float *dst = aa.out + ((size_t)qt * aa.nqh + qh) * HD;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            vdt v;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) v[dt] = o[dt][r] * inv;
            vdt *p = reinterpret_cast<vdt *>(dst + NDT * (8 * (r >> 2) + 4 * h + (r & 3)));
            *p = aa.accumulate ? *p + v : v;
        }
    }
}

// ---- one query token, head size 64 or 128: the heads of a kv group together ----
// A workgroup owns (kv head, split of the keys) and serves every query head of the group from one read
// of the split's keys and values.  HD / 8 lanes share a key, eight dims each -- i .. i+3 and HD/2 + i ..
// HD/2 + i+3, the pairs RoPE rotates, so that the raw projections of the new position are rotated in
// registers.  A score is a sum over those lanes by DPP moves, and each such group of lanes runs its own
// online softmax (running maximum, sum and row per head) over the keys it meets: no exchange at all until
// the 64 (HD 128) or 128 (HD 64) groups of the workgroup meet once, in LDS.  Wavefront instructions, not
// bytes, bound this kernel (a wavefront instruction takes four cycles and there are one or two wavefronts
// per SIMD): fused multiply-adds, v_exp_f32 on base-2 arguments, U as a template parameter.  A split is
// `tps` tiles of U rounds of 2048 / HD keys; every workgroup leaves (maximum, exp-sum, row) per head for
// gqa_combine_kernel.
constexpr int ATT_DEC_GC = 4;  // query heads per pass over the keys

template <int LPK>
__device__ __forceinline__ float lanes_sum_f32(float v) {  // over aligned groups of LPK = 8 or 16 lanes, in every lane
    auto mv = [](float x, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xf, 0xf, false));
    };
    v += mv(v, std::integral_constant<int, 0xB1>{});
    v += mv(v, std::integral_constant<int, 0x4E>{});
    v += mv(v, std::integral_constant<int, 0x141>{});
    if constexpr (LPK == 16) v += mv(v, std::integral_constant<int, 0x140>{});
    return v;
}

// e^x for x <= 0 (or -inf -> 0) in two instructions
__device__ __forceinline__ float exp_neg(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896341f); }

template <int HD, int U>
__global__ __launch_bounds__(256) void gqa_decode_kernel(attn_args aa, int nkv, int tps) {
    constexpr int LPK = HD / 8, KPW = 64 / LPK, ROWS = 4 * KPW, GC = ATT_DEC_GC, HALF = HD / 2, TK = U * ROWS;
    __shared__ __attribute__((aligned(16))) float xch[GC][ROWS][HD];  // 32 KB: each key row's partial output rows
    __shared__ float wm[GC][ROWS], wl[GC][ROWS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kvh = blockIdx.x % nkv, split = blockIdx.x / nkv;
    const int li = lane % LPK, krow = lane / LPK;
    const int G = aa.group, splits = aa.splits;
    int kend = aa.len;
    if (aa.mask_kind != 0) kend = min(kend, aa.offset + 1);
    const bool fused = aa.raw_q != nullptr;
    const float *kbase = aa.kc + (size_t)kvh * aa.k_stride + 4 * li;
    const float *vbase = aa.vc + (size_t)kvh * aa.v_stride + 4 * li;
    // the lane's eight dims of a head row after RoPE (the operations of rope_kernel in the same order)
    auto rot = [&](const float *row, float4 &lo, float4 &hi) {
        const float4 x0 = *reinterpret_cast<const float4 *>(row + 4 * li), x1 = *reinterpret_cast<const float4 *>(row + HALF + 4 * li);
        const float4 c = *reinterpret_cast<const float4 *>(aa.rope_c + 4 * li), sn = *reinterpret_cast<const float4 *>(aa.rope_s + 4 * li);
        lo.x = x0.x * c.x - x1.x * sn.x; lo.y = x0.y * c.y - x1.y * sn.y; lo.z = x0.z * c.z - x1.z * sn.z; lo.w = x0.w * c.w - x1.w * sn.w;
        hi.x = x0.x * sn.x + x1.x * c.x; hi.y = x0.y * sn.y + x1.y * c.y; hi.z = x0.z * sn.z + x1.z * c.z; hi.w = x0.w * sn.w + x1.w * c.w;
    };
    float4 k0[U], k1[U], v0[U], v1[U];
    bool live[U];
    auto load_tile = [&](int kb, bool store_new) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            k0[u] = k1[u] = v0[u] = v1[u] = float4{0.f, 0.f, 0.f, 0.f};
            const int kt = kb + (u * 4 + wave) * KPW + krow;
            live[u] = kt < kend && !attn_masked(aa.mask_kind, aa.offset, aa.window, aa.sink, aa.gbits, 0, kt);
            if (live[u]) {
                if (fused && kt == aa.new_pos) {
                    // not in the cache yet: made from the projections, and stored by this workgroup, the only
                    // one of its kv head that meets the position
                    rot(aa.raw_k + (size_t)kvh * HD, k0[u], k1[u]);
                    v0[u] = *reinterpret_cast<const float4 *>(aa.raw_v + (size_t)kvh * HD + 4 * li);
                    v1[u] = *reinterpret_cast<const float4 *>(aa.raw_v + (size_t)kvh * HD + HALF + 4 * li);
                    if (store_new) {
                        float *kn = aa.k_new + (size_t)kvh * aa.k_stride + 4 * li, *vn = aa.v_new + (size_t)kvh * aa.v_stride + 4 * li;
                        *reinterpret_cast<float4 *>(kn) = k0[u]; *reinterpret_cast<float4 *>(kn + HALF) = k1[u];
                        *reinterpret_cast<float4 *>(vn) = v0[u]; *reinterpret_cast<float4 *>(vn + HALF) = v1[u];
                    }
                } else {
                    typedef float f4v __attribute__((ext_vector_type(4)));
                    const f4v *kr = reinterpret_cast<const f4v *>(kbase + (size_t)kt * HD);
                    const f4v *vr = reinterpret_cast<const f4v *>(vbase + (size_t)kt * HD);
                    const f4v a = __builtin_nontemporal_load(kr), b = __builtin_nontemporal_load(kr + HALF / 4);
                    const f4v c = __builtin_nontemporal_load(vr), d = __builtin_nontemporal_load(vr + HALF / 4);
                    k0[u] = float4{a.x, a.y, a.z, a.w}; k1[u] = float4{b.x, b.y, b.z, b.w};
                    v0[u] = float4{c.x, c.y, c.z, c.w}; v1[u] = float4{d.x, d.y, d.z, d.w};
                }
            }
        }
    };
    // Loads return in issue order: the query rows (from L2) are requested first and the first tile's keys and
    // values (from HBM) right behind them, all before the first use, so that the two trips overlap.
    for (int hc = 0; hc < G; hc += GC) {
        float4 q0[GC], q1[GC], qc = {0.f, 0.f, 0.f, 0.f}, qs = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int h = 0; h < GC; ++h) {
            q0[h] = q1[h] = float4{0.f, 0.f, 0.f, 0.f};
            if (hc + h < G) {
                const float *qrow = (fused ? aa.raw_q : aa.q) + ((size_t)kvh * G + hc + h) * HD;
                q0[h] = *reinterpret_cast<const float4 *>(qrow + 4 * li);
                q1[h] = *reinterpret_cast<const float4 *>(qrow + HALF + 4 * li);
            }
        }
        if (fused) {
            qc = *reinterpret_cast<const float4 *>(aa.rope_c + 4 * li);
            qs = *reinterpret_cast<const float4 *>(aa.rope_s + 4 * li);
        }
        load_tile(split * tps * TK, hc == 0);
        __builtin_amdgcn_sched_barrier(0);
        if (fused) {  // the operations of rope_kernel in the same order
#pragma unroll
            for (int h = 0; h < GC; ++h) {
                const float4 x0 = q0[h], x1 = q1[h];
                q0[h].x = x0.x * qc.x - x1.x * qs.x; q0[h].y = x0.y * qc.y - x1.y * qs.y;
                q0[h].z = x0.z * qc.z - x1.z * qs.z; q0[h].w = x0.w * qc.w - x1.w * qs.w;
                q1[h].x = x0.x * qs.x + x1.x * qc.x; q1[h].y = x0.y * qs.y + x1.y * qc.y;
                q1[h].z = x0.z * qs.z + x1.z * qc.z; q1[h].w = x0.w * qs.w + x1.w * qc.w;
            }
        }
        float m_run[GC], l_run[GC], acc[GC][8];
#pragma unroll
        for (int h = 0; h < GC; ++h) {
            m_run[h] = -INFINITY;
            l_run[h] = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[h][j] = 0.f;
        }
        for (int t = 0; t < tps; ++t) {
            if (t > 0) {
                const int kb = (split * tps + t) * TK;
                if (kb >= kend) break;
                load_tile(kb, hc == 0);
            }
#pragma unroll
            for (int h = 0; h < GC; ++h) {
                float sc[U], tmax = -INFINITY;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    float dot = q0[h].x * k0[u].x;
                    dot = fmaf(q0[h].y, k0[u].y, dot); dot = fmaf(q0[h].z, k0[u].z, dot); dot = fmaf(q0[h].w, k0[u].w, dot);
                    dot = fmaf(q1[h].x, k1[u].x, dot); dot = fmaf(q1[h].y, k1[u].y, dot);
                    dot = fmaf(q1[h].z, k1[u].z, dot); dot = fmaf(q1[h].w, k1[u].w, dot);
                    dot = lanes_sum_f32<LPK>(dot);
                    float sv = dot * aa.scale;
                    if (aa.logit_cap > 0.f) sv = aa.logit_cap * tanhf(sv / aa.logit_cap);
                    sc[u] = live[u] ? sv : -INFINITY;
                    tmax = fmaxf(tmax, sc[u]);
                }
                // this group of lanes' own running maximum: nothing crosses to the other keys' lanes
                const float m_new = fmaxf(m_run[h], tmax);
                const float m_ref = m_new == -INFINITY ? 0.f : m_new;  // (all hidden so far: every term below is e^-inf = 0)
                const float alpha = exp_neg(m_run[h] - m_ref);
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[h][j] *= alpha;
                l_run[h] *= alpha;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const float pv = exp_neg(sc[u] - m_ref);
                    l_run[h] += pv;
                    acc[h][0] = fmaf(pv, v0[u].x, acc[h][0]); acc[h][1] = fmaf(pv, v0[u].y, acc[h][1]);
                    acc[h][2] = fmaf(pv, v0[u].z, acc[h][2]); acc[h][3] = fmaf(pv, v0[u].w, acc[h][3]);
                    acc[h][4] = fmaf(pv, v1[u].x, acc[h][4]); acc[h][5] = fmaf(pv, v1[u].y, acc[h][5]);
                    acc[h][6] = fmaf(pv, v1[u].z, acc[h][6]); acc[h][7] = fmaf(pv, v1[u].w, acc[h][7]);
                }
                m_run[h] = m_new;
            }
        }
        // the groups' partial rows, maxima and sums meet in LDS
        const int row = wave * KPW + krow;
#pragma unroll
        for (int h = 0; h < GC; ++h) {
            float *dst = &xch[h][row][4 * li];
            *reinterpret_cast<float4 *>(dst) = float4{acc[h][0], acc[h][1], acc[h][2], acc[h][3]};
            *reinterpret_cast<float4 *>(dst + HALF) = float4{acc[h][4], acc[h][5], acc[h][6], acc[h][7]};
            if (li == 0) {
                wm[h][row] = m_run[h];
                wl[h][row] = l_run[h];
            }
        }
        __syncthreads();
        if (tid < GC * HD / 4) {
            const int h = tid / (HD / 4), i4 = tid % (HD / 4);
            if (hc + h < G) {
                float M = -INFINITY;
#pragma unroll
                for (int r = 0; r < ROWS; ++r) M = fmaxf(M, wm[h][r]);
                const float m_ref = M == -INFINITY ? 0.f : M;
                float L = 0.f;
                float4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    const float w = exp_neg(wm[h][r] - m_ref);
                    const float4 a = *reinterpret_cast<const float4 *>(&xch[h][r][4 * i4]);
                    L = fmaf(w, wl[h][r], L);
                    o.x = fmaf(w, a.x, o.x); o.y = fmaf(w, a.y, o.y); o.z = fmaf(w, a.z, o.z); o.w = fmaf(w, a.w, o.w);
                }
                float *dst = aa.part + (((size_t)kvh * G + hc + h) * splits + split) * (size_t)(HD + 2);
                if (i4 == 0) {
                    dst[0] = M;
                    dst[1] = L;
                }
                *reinterpret_cast<float2 *>(dst + 2 + 4 * i4) = float2{o.x, o.y};
                *reinterpret_cast<float2 *>(dst + 4 + 4 * i4) = float2{o.z, o.w};
            }
        }
        if (hc + GC < G) __syncthreads();  // the next pass of heads writes xch again
    }
}

constexpr int ATT_SPLITS_MAX = 2048;

// Merge the splits of one (query token, query head) row: with M = max of the split maxima and
// w_s = exp(m_s - M), out = sum_s w_s o_s / sum_s w_s l_s, splits in ascending order.
// DIG 1 / 2: the merged row is written as nibble / byte digits of the [seq_q, num_q_heads * hd]
// matrix that o_proj multiplies (hd a multiple of 32; workgroup = row qt * nqh + qh), not as f32.
// A record is hdr floats (maximum, exp-sum, padding) followed by the row.
template <int DIG>
__global__ __launch_bounds__(128) void gqa_combine_kernel(const float *__restrict__ part, int splits, int hd, int hdr,
                                                          float *__restrict__ out, int accumulate, int nqh,
                                                          int8_t *__restrict__ digits, float *__restrict__ xs) {
    __shared__ float wts[ATT_SPLITS_MAX];
    __shared__ float red[2];
    const size_t rec = (size_t)(hd + hdr);
    const float *p = part + (size_t)blockIdx.x * splits * rec;
    const int tid = threadIdx.x;
    float M = -INFINITY;
    for (int s = tid; s < splits; s += 128) M = fmaxf(M, p[s * rec]);
    M = block_max(M, red);
    float l = 0.f;
    for (int s = tid; s < splits; s += 128) {
        const float m = p[s * rec];
        const float w = m == -INFINITY ? 0.f : expf(m - M);
        wts[s] = w;
        l += w * p[s * rec + 1];
    }
    l = block_sum(l, red);  // its barriers publish wts[]
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    if constexpr (DIG == 0) {
        for (int i = tid; i < hd; i += 128) {
            float o = 0.f;
            for (int s = 0; s < splits; ++s) o += wts[s] * p[s * rec + hdr + i];
            float *dst = out + (size_t)blockIdx.x * hd + i;
            *dst = accumulate ? *dst + o * inv : o * inv;
        }
    } else {
        const int qt = blockIdx.x / nqh, qh = blockIdx.x - qt * nqh;
        for (int i4 = tid; i4 < hd / 4; i4 += 128) {  // whole 8-lane groups: hd / 4 is a multiple of 8
            float o[4] = {0.f, 0.f, 0.f, 0.f};
            for (int s = 0; s < splits; ++s) {
                const float wv = wts[s];
                const float *src = p + s * rec + hdr + 4 * i4;
                o[0] += wv * src[0]; o[1] += wv * src[1]; o[2] += wv * src[2]; o[3] += wv * src[3];
            }
            for (int j = 0; j < 4; ++j) o[j] *= inv;
            const int e4 = qh * (hd / 4) + i4;  // float4 index within the row
            const int nb = nqh * hd / 32;
            if constexpr (DIG <= 2) pg_emit_digits<DIG == 1>(o, qt, e4 >> 3, e4 & 7, nb, digits, xs);
            else pg_emit_mm_digits<DIG == 3>(o, qt, e4 >> 3, e4 & 7, nb, (nb + 3) & ~3, digits, xs);  // the matrix-core product's planes
        }
    }
}

// The same merge for head sizes 64 and 128 and at most MAXS (64 or 128) splits, every load in flight at once:
// thread = (float4 of the row, slice of the splits), the slices' sums meet in LDS.  Splits are still added in
// ascending order within a slice and the slices in ascending order: the result does not depend on timing.
// A record is HDR floats (maximum, exp-sum, padding) followed by the row.  DIG as in gqa_combine_kernel.
template <int HD, int DIG, int HDR, int MAXS>
__global__ __launch_bounds__(256) void gqa_combine_few_kernel(const float *__restrict__ part, int splits, float *__restrict__ out,
                                                              int accumulate, int nqh, int8_t *__restrict__ digits,
                                                              float *__restrict__ xs) {
    constexpr int UNITS = HD / 4, SLICES = 256 / UNITS, NS = MAXS / SLICES, REC = HD + HDR;
    __shared__ float sm[MAXS], sl[MAXS];
    __shared__ float ex[SLICES][UNITS][5];
    const float *p = part + (size_t)blockIdx.x * splits * REC;
    const int tid = threadIdx.x, i4 = tid % UNITS, slice = tid / UNITS;
    float2 ra[NS], rb[NS];
#pragma unroll
    for (int j = 0; j < NS; ++j) {  // this thread's splits: slice * NS + j
        const int sp = slice * NS + j;
        ra[j] = rb[j] = float2{0.f, 0.f};
        if (sp < splits) {
            ra[j] = *reinterpret_cast<const float2 *>(p + (size_t)sp * REC + HDR + 4 * i4);
            rb[j] = *reinterpret_cast<const float2 *>(p + (size_t)sp * REC + HDR + 2 + 4 * i4);
        }
    }
    if (tid < MAXS) {
        const float2 ml = tid < splits ? *reinterpret_cast<const float2 *>(p + (size_t)tid * REC) : float2{-INFINITY, 0.f};
        sm[tid] = ml.x;
        sl[tid] = ml.y;
    }
    __syncthreads();
    float mine_m = sm[tid & 63];
    if constexpr (MAXS > 64) mine_m = fmaxf(mine_m, sm[64 + (tid & 63)]);
    const float M = wave_max_f32(mine_m);
    const float m_ref = M == -INFINITY ? 0.f : M;
    float L = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int sp = slice * NS + j;
        const float w = exp_neg(sm[sp] - m_ref);  // (splits past the last: e^-inf = 0)
        L = fmaf(w, sl[sp], L);
        o[0] = fmaf(w, ra[j].x, o[0]); o[1] = fmaf(w, ra[j].y, o[1]); o[2] = fmaf(w, rb[j].x, o[2]); o[3] = fmaf(w, rb[j].y, o[3]);
    }
    float *mine = ex[slice][i4];
    mine[0] = L; mine[1] = o[0]; mine[2] = o[1]; mine[3] = o[2]; mine[4] = o[3];
    __syncthreads();
    if (tid >= UNITS) return;  // whole 8-lane groups stay: UNITS is a multiple of 8
    L = 0.f;
    o[0] = o[1] = o[2] = o[3] = 0.f;
#pragma unroll
    for (int sx = 0; sx < SLICES; ++sx) {
        const float *e = ex[sx][i4];
        L += e[0]; o[0] += e[1]; o[1] += e[2]; o[2] += e[3]; o[3] += e[4];
    }
    const float inv = L > 0.f ? 1.0f / L : 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] *= inv;
    if constexpr (DIG == 0) {
        float4 *dst = reinterpret_cast<float4 *>(out + (size_t)blockIdx.x * HD) + i4;
        float4 r = {o[0], o[1], o[2], o[3]};
        if (accumulate) {
            const float4 old = *dst;
            r.x += old.x; r.y += old.y; r.z += old.z; r.w += old.w;
        }
        *dst = r;
    } else {
        const int qt = blockIdx.x / nqh, qh = blockIdx.x - qt * nqh;
        const int e4 = qh * UNITS + i4, nb = nqh * HD / 32;  // float4 index within the row
        if constexpr (DIG <= 2) pg_emit_digits<DIG == 1>(o, qt, e4 >> 3, e4 & 7, nb, digits, xs);
        else pg_emit_mm_digits<DIG == 3>(o, qt, e4 >> 3, e4 & 7, nb, (nb + 3) & ~3, digits, xs);
    }
}

__global__ __launch_bounds__(256) void swiglu_kernel(float *__restrict__ g, const float *__restrict__ u, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        const float gi = g[i];
        g[i] = gi / (1.0f + expf(-gi)) * u[i];
    }
}

// One row: silu(g) * u written as GEMV digits (n a multiple of 32).
template <bool NIB>
__global__ __launch_bounds__(256) void swiglu_digits_kernel(const float4 *__restrict__ g, const float4 *__restrict__ u, int n4,
                                                            int8_t *__restrict__ digits, float *__restrict__ xs) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;  // whole 8-lane groups leave together
    const float4 gv = g[i], uv = u[i];
    const float o[4] = {gv.x / (1.0f + expf(-gv.x)) * uv.x, gv.y / (1.0f + expf(-gv.y)) * uv.y,
                        gv.z / (1.0f + expf(-gv.z)) * uv.z, gv.w / (1.0f + expf(-gv.w)) * uv.w};
    pg_emit_digits<NIB>(o, 0, i >> 3, i & 7, n4 >> 3, digits, xs);
}

// Rows of silu(g) * u written as the matrix-core product's digit planes (n a multiple of 32 per row); g and u
// each the sum of `planes` planes, `stride` floats apart, in ascending order.
template <bool NIB>
__global__ __launch_bounds__(256) void swiglu_mm_digits_kernel(const float *__restrict__ g, const float *__restrict__ u, int planes,
                                                               size_t stride, int nb, int nbp, int8_t *__restrict__ digits,
                                                               float *__restrict__ xs) {
    const size_t row = blockIdx.y;
    const int b = blockIdx.x * 32 + (threadIdx.x >> 3), sub = threadIdx.x & 7;
    if (b >= nb) return;  // whole 8-thread groups leave together
    const size_t at = (row * nb + b) * 8 + sub;  // float4 index
    float4 gp[PG_MAX_PLANES], up[PG_MAX_PLANES];
#pragma unroll
    for (int pl = 0; pl < PG_MAX_PLANES; ++pl) {
        const bool have = pl < planes;
        gp[pl] = have ? reinterpret_cast<const float4 *>(g + pl * stride)[at] : float4{0.f, 0.f, 0.f, 0.f};
        up[pl] = have ? reinterpret_cast<const float4 *>(u + pl * stride)[at] : float4{0.f, 0.f, 0.f, 0.f};
    }
    float4 gv = gp[0], uv = up[0];
#pragma unroll
    for (int pl = 1; pl < PG_MAX_PLANES; ++pl) {
        if (pl < planes) {
            gv.x += gp[pl].x; gv.y += gp[pl].y; gv.z += gp[pl].z; gv.w += gp[pl].w;
            uv.x += up[pl].x; uv.y += up[pl].y; uv.z += up[pl].z; uv.w += up[pl].w;
        }
    }
    const float o[4] = {gv.x / (1.0f + expf(-gv.x)) * uv.x, gv.y / (1.0f + expf(-gv.y)) * uv.y,
                        gv.z / (1.0f + expf(-gv.z)) * uv.z, gv.w / (1.0f + expf(-gv.w)) * uv.w};
    pg_emit_mm_digits<NIB>(o, row, b, sub, nb, nbp, digits, xs);
}

// Rows of silu(g) * u written as the two f16 planes of the f16 matrix-core product (pg_f16_planes.h), a workgroup per
// row with the row in registers (dim4 <= 256 * MAXV float4); g and u as the sums of `planes` planes, as above.
template <int MAXV>
__global__ __launch_bounds__(256) void swiglu_f16_planes_kernel(const float *__restrict__ g, const float *__restrict__ u, int planes,
                                                                size_t stride, int dim4, _Float16 *__restrict__ hi,
                                                                _Float16 *__restrict__ lo, float *__restrict__ inv) {
    __shared__ float red[4];
    const size_t row = (size_t)blockIdx.x * dim4;
    float4 v[MAXV];
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int i = threadIdx.x + 256 * j;
        v[j] = float4{0.f, 0.f, 0.f, 0.f};
        if (i < dim4) {
            float4 gp[PG_MAX_PLANES], up[PG_MAX_PLANES];
#pragma unroll
            for (int pl = 0; pl < PG_MAX_PLANES; ++pl) {
                const bool have = pl < planes;
                gp[pl] = have ? reinterpret_cast<const float4 *>(g + pl * stride)[row + i] : float4{0.f, 0.f, 0.f, 0.f};
                up[pl] = have ? reinterpret_cast<const float4 *>(u + pl * stride)[row + i] : float4{0.f, 0.f, 0.f, 0.f};
            }
            float4 gv = gp[0], uv = up[0];
#pragma unroll
            for (int pl = 1; pl < PG_MAX_PLANES; ++pl) {
                if (pl < planes) {
                    gv.x += gp[pl].x; gv.y += gp[pl].y; gv.z += gp[pl].z; gv.w += gp[pl].w;
                    uv.x += up[pl].x; uv.y += up[pl].y; uv.z += up[pl].z; uv.w += up[pl].w;
                }
            }
            v[j] = float4{gv.x / (1.0f + expf(-gv.x)) * uv.x, gv.y / (1.0f + expf(-gv.y)) * uv.y,
                          gv.z / (1.0f + expf(-gv.z)) * uv.z, gv.w / (1.0f + expf(-gv.w)) * uv.w};
            amax = fmaxf(amax, fmaxf(fmaxf(pg_f16_mag(v[j].x), pg_f16_mag(v[j].y)), fmaxf(pg_f16_mag(v[j].z), pg_f16_mag(v[j].w))));
        }
    }
    const pg_f16_row_scale sc = pg_f16_row_scale_of(block_max(amax, red));
    if (threadIdx.x == 0) {
        inv[2 * blockIdx.x] = sc.i1;
        inv[2 * blockIdx.x + 1] = sc.i2;
    }
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int i = threadIdx.x + 256 * j;
        if (i < dim4) {
            const float o[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
            pg_f16_split4(o, sc, reinterpret_cast<uint2 *>(hi + (row + i) * 4), reinterpret_cast<uint2 *>(lo + (row + i) * 4));
        }
    }
}

// out = a + (b as the sum of `planes` planes, in ascending order)
__global__ __launch_bounds__(256) void add_planes_kernel(const float *__restrict__ a, const float *__restrict__ b, int planes,
                                                         size_t stride, float *__restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float tp[PG_MAX_PLANES];
#pragma unroll
    for (int pl = 0; pl < PG_MAX_PLANES; ++pl) tp[pl] = pl < planes ? b[pl * stride + i] : 0.f;
    float t = tp[0];
#pragma unroll
    for (int pl = 1; pl < PG_MAX_PLANES; ++pl)
        if (pl < planes) t += tp[pl];
    out[i] = a[i] + t;
}

// (a fill kernel rather than hipMemsetAsync: a caller may capture the stream-ordered entry points in a graph)
__global__ __launch_bounds__(256) void zero_f32_kernel(float *__restrict__ p, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0.0f;
}

__global__ __launch_bounds__(256) void add_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                  float *__restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = a[i] + b[i];
}

inline unsigned blocks_for(size_t n) { return (unsigned)((n + 255) / 256); }

bool rmsnorm_vec_ok(const float *a, const float *b, float *sum_out, const float *w, float *out, size_t dim) {
    const uintptr_t align = (uintptr_t)a | (uintptr_t)b | (uintptr_t)sum_out | (uintptr_t)w | (uintptr_t)out;
    return dim % 4 == 0 && dim <= 8192 && align % 16 == 0;
}

// RMSNorm whose output goes straight to GEMV digits (kind: PG_GGML_Q4_0 nibbles, else bytes).
pg_status launch_rmsnorm_digits(pg_ctx *ctx, const float *a, const float *b, float *sum_out, const float *w, float eps,
                                size_t rows, size_t dim, int kind, const pg_xdigits &xd) {
    const bool nib = kind == PG_GGML_Q4_0;
    auto *kern = dim <= 4096 ? (nib ? add_rmsnorm_vec_kernel<4, 1> : add_rmsnorm_vec_kernel<4, 2>)
                             : (nib ? add_rmsnorm_vec_kernel<8, 1> : add_rmsnorm_vec_kernel<8, 2>);
    return pg_launch(ctx, "add_rmsnorm_digits", kern, dim3((unsigned)rows), dim3(256), 0, (const float4 *)a, (const float4 *)b,
                     (float4 *)sum_out, (const float4 *)w, eps, (int)(dim / 4), (float4 *)nullptr, xd.digits, xd.xs, 1, (size_t)0);
}

pg_status launch_rmsnorm(pg_ctx *ctx, const float *a, const float *b, float *sum_out, const float *w, float eps,
                         size_t rows, size_t dim, float *out) {
    if (rows == 0) return PG_OK;
    if (rmsnorm_vec_ok(a, b, sum_out, w, out, dim)) {
        auto *kern = dim <= 4096 ? add_rmsnorm_vec_kernel<4, 0> : add_rmsnorm_vec_kernel<8, 0>;
        return pg_launch(ctx, "add_rmsnorm", kern, dim3((unsigned)rows), dim3(256), 0, (const float4 *)a, (const float4 *)b,
                         (float4 *)sum_out, (const float4 *)w, eps, (int)(dim / 4), (float4 *)out, (int8_t *)nullptr,
                         (float *)nullptr, 1, (size_t)0);
    }
    return pg_launch(ctx, "add_rmsnorm", add_rmsnorm_kernel, dim3((unsigned)rows), dim3(256), 0, a, b, sum_out, w, eps,
                     (int)dim, out);
}

// Whether launch_attention takes the one-token kernel for `rows` (token, head) rows over `len` keys.
bool attention_is_short(const pg_ctx *ctx, size_t rows, size_t len, size_t hd) {
    size_t lanes = 1;
    while (lanes * 4 < hd) lanes <<= 1;
    const size_t keys_per_round = 256 / lanes;
    return rows < 2 * (size_t)ctx->num_cu &&
           (len + ATT_SHORT_ROUNDS * keys_per_round - 1) / (ATT_SHORT_ROUNDS * keys_per_round) <= (size_t)ATT_SPLITS_MAX;
}

// Whether a call with several query tokens should cut its keys into runs for the matrix-core kernel (its
// workgroups, one per kv head and pair of 32-row items, would leave most CUs idle while each walks a long
// cache), and how: *chunk tiles of 32 keys per run, *splits runs.
bool split_mfma_tiles(const pg_ctx *ctx, size_t group, size_t seq_q, size_t nkv, int mask_kind, size_t offset, size_t len,
                      size_t *chunk, size_t *splits) {
    const size_t n_items = (group * seq_q + 31) / 32, wgs = n_items * nkv;  // one wavefront each
    const size_t kend = mask_kind != 0 && offset + seq_q < len ? offset + seq_q : len;
    const size_t tiles = (kend + 31) / 32;
    // few wavefronts: worth it from 8 tiles on; up to three per CU (a chunk of a few hundred tokens appended to a long
    // cache): only when every wavefront would otherwise walk 64 tiles and more while SIMDs stand idle
    const bool few = wgs * 2 <= (size_t)ctx->num_cu;
    if (!(few ? tiles >= 8 : (wgs < 3 * (size_t)ctx->num_cu && tiles >= 64))) return false;
    // A tile costs a wavefront about 5 us whatever the number of live rows (128 matrix instructions of 16 passes,
    // one wavefront per SIMD), so the runs are as short as one wavefront per SIMD allows
    size_t want = 4 * (size_t)ctx->num_cu / wgs;  // (rounded down: a few wavefronts past one per SIMD would cost a second round)
    if (want < 2) return false;
    if (want > tiles) want = tiles;
    if (want > (size_t)ATT_SPLITS_MAX) want = ATT_SPLITS_MAX;
    *chunk = (tiles + want - 1) / want;
    *splits = (tiles + *chunk - 1) / *chunk;
    return *splits > 1;
}

pg_status launch_attention(pg_ctx *ctx, const float *q, const pg_kv_cache *kc, const pg_kv_cache *vc, size_t nqh,
                           size_t seq_q, float scale, int mask_kind, size_t offset, size_t window, size_t sink,
                           float logit_cap, float *out, int accumulate, const pg_xdigits *xd = nullptr, int digit_kind = 0,
                           const size_t *global_positions = nullptr, size_t num_global = 0,
                           const attn_args *rope_fusion = nullptr, const pg_mmdigits *md = nullptr, bool *md_written = nullptr) {
    // With `md` (digit_kind names the tensor type) a merge of key runs writes the rows as the matrix-core
    // product's digit planes instead of f32 and sets *md_written; a kernel that needs no merge writes `out`.
    // With `xd` (one-token step, accumulate == 0, head_dim % 32 == 0) the rows also, or only,
    // leave as GEMV digits of kind `digit_kind`; `out` must still be a valid buffer.
    const size_t len = kc->len, hd = kc->head_dim;
    if (seq_q == 0 || nqh == 0) return PG_OK;
    if (len == 0) {  // nothing to attend to: the reference adds nothing to `output`
        if (!accumulate) {
            const size_t n = seq_q * nqh * hd;
            PG_TRY(pg_launch(ctx, "zero_f32", zero_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, out, n));
        }
        return PG_OK;
    }
    attn_args aa;
    aa.q = q; aa.kc = kc->k; aa.vc = vc->v; aa.out = out; aa.part = nullptr;
    aa.k_stride = kc->capacity * hd; aa.v_stride = vc->capacity * hd;
    aa.len = (int)len; aa.nqh = (int)nqh; aa.group = (int)(nqh / kc->num_kv_heads); aa.seq_q = (int)seq_q; aa.hd = (int)hd;
    int lanes = 1;
    while ((size_t)lanes * 4 < hd) lanes <<= 1;
    aa.lanes = lanes;
    aa.scale = scale; aa.logit_cap = logit_cap;
    aa.mask_kind = mask_kind; aa.offset = (int)offset;
    aa.window = (int)(window > 0x7fffffffu ? 0x7fffffffu : window);
    aa.sink = (int)(sink > 0x7fffffffu ? 0x7fffffffu : sink);
    aa.accumulate = accumulate;
    aa.gbits = nullptr;
    aa.raw_q = aa.raw_k = aa.raw_v = aa.rope_c = aa.rope_s = nullptr;
    aa.k_new = aa.v_new = nullptr;
    aa.new_pos = -1;
    // Split the keys when the rows alone cannot fill the chip (the one-token step) or a chunk
    // would not fit the LDS score buffer.  Few rows: splits of 8 rounds of keys, which the
    // short kernel handles with every load in flight at once.
    const size_t rows = seq_q * nqh, keys_per_round = 256 / (size_t)lanes;
    size_t chunk, splits;
    bool short_kernel = false, tiled_kernel = false, decode_kernel = false, split_kernel = false;
    int dec_u = 1, dec_tps = 1;
    const uintptr_t align_all = (uintptr_t)q | (uintptr_t)out | (uintptr_t)kc->k | (uintptr_t)vc->v |
                                (rope_fusion ? (uintptr_t)rope_fusion->raw_q | (uintptr_t)rope_fusion->raw_k | (uintptr_t)rope_fusion->raw_v |
                                                   (uintptr_t)rope_fusion->rope_c | (uintptr_t)rope_fusion->rope_s
                                             : 0);
    if (seq_q == 1 && (hd == 64 || hd == 128) && align_all % 16 == 0 && rows < 2 * (size_t)ctx->num_cu) {  // (any cache length)
        // one token: the heads of a kv group share a workgroup
        const size_t nkv = kc->num_kv_heads, tile_rows = 2048 / hd;
        const size_t kend = mask_kind != 0 && offset + 1 < len ? offset + 1 : len;
        auto tiles_of = [&](size_t u) { return (kend + u * tile_rows - 1) / (u * tile_rows); };
        size_t u = 4;
        while (u > 1 && nkv * tiles_of(u) < (size_t)ctx->num_cu) u >>= 1;  // fewer rounds per tile, more workgroups
        const size_t tiles = tiles_of(u);
        size_t tps = nkv * tiles > 2 * (size_t)ctx->num_cu ? (nkv * tiles + 2 * ctx->num_cu - 1) / (2 * ctx->num_cu) : 1;
        if ((tiles + tps - 1) / tps > (size_t)ATT_SPLITS_MAX) tps = (tiles + ATT_SPLITS_MAX - 1) / ATT_SPLITS_MAX;
        splits = (tiles + tps - 1) / tps;
        chunk = tps * u * tile_rows;
        dec_u = (int)u; dec_tps = (int)tps;
        decode_kernel = true;
    } else if (seq_q > 1 && (hd == 64 || hd == 128) && align_all % 16 == 0 && split_mfma_tiles(ctx, nqh / kc->num_kv_heads, seq_q,
                                                                                                 kc->num_kv_heads, mask_kind, offset, len, &chunk, &splits)) {
        // few rows under a long cache: the matrix-core kernel over runs of key tiles, then the merge
        tiled_kernel = split_kernel = true;
    } else if (attention_is_short(ctx, rows, len, hd)) {
        chunk = ATT_SHORT_ROUNDS * keys_per_round;
        splits = (len + chunk - 1) / chunk;
        short_kernel = true;
    } else if (hd == 64 || hd == 128 || hd == 256) {
        tiled_kernel = true;  // online softmax over key blocks: any length in one pass
        splits = 1;
        chunk = len;
    } else {
        splits = (len + ATT_CHUNK_MAX - 1) / ATT_CHUNK_MAX;
        chunk = pg_round_up((len + splits - 1) / splits, keys_per_round);
        splits = (len + chunk - 1) / chunk;
    }
    if (splits > (size_t)ATT_SPLITS_MAX) return pg_fail(PG_EUNSUPPORTED, "gqa_attention: cache of %zu positions is too long", len);
    aa.chunk = (int)chunk; aa.splits = (int)splits;
    const size_t part_hdr = split_kernel ? 4 : 2;  // floats ahead of a partial row (maximum, exp-sum, padding)
    const size_t part_bytes = splits > 1 || decode_kernel ? pg_round_up(rows * splits * (hd + part_hdr) * sizeof(float), 256) : 0;
    const size_t bits_words = mask_kind == PG_MASK_LOCAL_GLOBAL ? (len + 31) / 32 : 0;
    if (part_bytes + bits_words) {
        void *ws = nullptr;
        PG_TRY(pg_workspace(ctx, part_bytes + bits_words * sizeof(uint32_t), &ws));
        if (part_bytes) aa.part = static_cast<float *>(ws);
        if (bits_words) {
            // The global positions become one bit per key position (positions past the cache
            // can never be a key).  The words are copied from this frame, hence the wait.
            std::vector<uint32_t> bits(bits_words, 0u);
            for (size_t i = 0; i < num_global; ++i)
                if (global_positions[i] < len) bits[global_positions[i] >> 5] |= 1u << (global_positions[i] & 31);
            uint32_t *dev_bits = reinterpret_cast<uint32_t *>(static_cast<char *>(ws) + part_bytes);
            PG_HIP(hipMemcpyAsync(dev_bits, bits.data(), bits_words * sizeof(uint32_t), hipMemcpyHostToDevice, ctx->stream));
            PG_HIP(hipStreamSynchronize(ctx->stream));
            aa.gbits = dev_bits;
        }
    }
    const dim3 grid((unsigned)seq_q, (unsigned)nqh, (unsigned)splits);
    if (rope_fusion) {
        if (!(short_kernel || decode_kernel) || seq_q != 1 || hd % 8 != 0)
            return pg_fail(PG_EINVAL, "gqa_attention: RoPE fusion needs a one-token kernel");
        aa.raw_q = rope_fusion->raw_q; aa.raw_k = rope_fusion->raw_k; aa.raw_v = rope_fusion->raw_v;
        aa.rope_c = rope_fusion->rope_c; aa.rope_s = rope_fusion->rope_s;
        aa.k_new = rope_fusion->k_new; aa.v_new = rope_fusion->v_new;
        aa.new_pos = rope_fusion->new_pos;
    }
    if (decode_kernel) {
        if (kc->num_kv_heads * splits >= (1ull << 31)) return pg_fail(PG_EUNSUPPORTED, "gqa_attention: grid too large");
        auto *kern = hd == 64 ? (dec_u == 4 ? gqa_decode_kernel<64, 4> : (dec_u == 2 ? gqa_decode_kernel<64, 2> : gqa_decode_kernel<64, 1>))
                              : (dec_u == 4 ? gqa_decode_kernel<128, 4> : (dec_u == 2 ? gqa_decode_kernel<128, 2> : gqa_decode_kernel<128, 1>));
        PG_TRY(pg_launch(ctx, "gqa_decode", kern, dim3((unsigned)(kc->num_kv_heads * splits)), dim3(256), 0, aa, (int)kc->num_kv_heads,
                         dec_tps));
    } else if (short_kernel) {
        const size_t sets = kc->num_kv_heads * splits, members = (nqh / kc->num_kv_heads) * seq_q;
        const size_t wgs = (sets + 7) / 8 * 8 * members;
        if (wgs >= (1ull << 31)) return pg_fail(PG_EUNSUPPORTED, "gqa_attention: grid too large");
        PG_TRY(pg_launch(ctx, "gqa_attention_short", gqa_attention_short_kernel, dim3((unsigned)wgs), dim3(256), 0, aa));
    }
    else if (tiled_kernel && (hd == 64 || hd == 128)) {
        // matrix-core kernel: one workgroup per kv head and pair of 32-row items (first with last, ...);
        // the kv head varies fastest, so with eight kv heads each XCD's L2 keeps one head's keys and values
        const size_t G = nqh / kc->num_kv_heads, n_items = (G * seq_q + 31) / 32, pairs = (n_items + 1) / 2;
        if (n_items * kc->num_kv_heads * splits >= (1ull << 31)) return pg_fail(PG_EUNSUPPORTED, "gqa_attention: grid too large");
        auto *kern = split_kernel ? (hd == 64 ? gqa_attention_mfma_kernel<64, true> : gqa_attention_mfma_kernel<128, true>)
                                  : (hd == 64 ? gqa_attention_mfma_kernel<64> : gqa_attention_mfma_kernel<128>);
        if (split_kernel)  // one wavefront per workgroup: (kv head, item, run)
            PG_TRY(pg_launch(ctx, "gqa_attention_mfma_split", kern, dim3((unsigned)(n_items * kc->num_kv_heads * splits)), dim3(64), 0, aa,
                             (int)n_items, (int)kc->num_kv_heads));
        else
            PG_TRY(pg_launch(ctx, "gqa_attention_mfma", kern, dim3((unsigned)(pairs * kc->num_kv_heads)), dim3(128), 0, aa, (int)n_items,
                             (int)kc->num_kv_heads));
    } else if (tiled_kernel) {
        const size_t G = nqh / kc->num_kv_heads, row_sets = (G * seq_q + ATT_T_ROWS - 1) / ATT_T_ROWS;
        const dim3 grid_t((unsigned)row_sets, (unsigned)kc->num_kv_heads);
        auto *kern = gqa_attention_tiled_kernel<256>;  // head sizes 64 and 128 took the matrix-core kernel above
        const size_t lds_t = att_tiled_lds<256>();
        PG_TRY(pg_allow_dynamic_lds(ctx, reinterpret_cast<const void *>(kern), lds_t));
        PG_TRY(pg_launch(ctx, "gqa_attention_tiled", kern, grid_t, dim3(256), lds_t, aa));
    } else
        PG_TRY(pg_launch(ctx, "gqa_attention", gqa_attention_kernel, grid, dim3(256), (256 + ATT_RED + chunk) * sizeof(float), aa));
    if ((decode_kernel || split_kernel) && splits <= 128) {  // (these kernels: `out` is 16-byte aligned, hd is 64 or 128)
        // what the merged rows leave as: f32, the streaming product's digits (one-token step), or -- a merge of key
        // runs under a many-token block step -- the matrix-core product's digit planes
        const bool planes = md && !xd && !accumulate;
        const int dg = xd ? (digit_kind == PG_GGML_Q4_0 ? 1 : 2) : (planes ? (digit_kind == PG_GGML_Q4_0 ? 3 : 4) : 0);
        int8_t *dig = xd ? xd->digits : (planes ? md->digits : nullptr);
        float *dxs = xd ? xd->xs : (planes ? md->xs : nullptr);
        const char *name = xd ? "gqa_combine_digits" : (planes ? "gqa_combine_mm_digits" : "gqa_combine");
#define PG_COMBINE_FEW(HD_, DG_)                                                                                                   \
    (split_kernel ? (splits <= 64 ? gqa_combine_few_kernel<HD_, DG_, 4, 64> : gqa_combine_few_kernel<HD_, DG_, 4, 128>)              \
                  : (splits <= 64 ? gqa_combine_few_kernel<HD_, DG_, 2, 64> : gqa_combine_few_kernel<HD_, DG_, 2, 128>))
#define PG_COMBINE_FEW_HD(DG_) (hd == 64 ? PG_COMBINE_FEW(64, DG_) : PG_COMBINE_FEW(128, DG_))
        auto *kern = dg == 0 ? PG_COMBINE_FEW_HD(0) : (dg == 1 ? PG_COMBINE_FEW_HD(1) : (dg == 2 ? PG_COMBINE_FEW_HD(2) : (dg == 3 ? PG_COMBINE_FEW_HD(3) : PG_COMBINE_FEW_HD(4))));
#undef PG_COMBINE_FEW_HD
#undef PG_COMBINE_FEW
        PG_TRY(pg_launch(ctx, name, kern, dim3((unsigned)rows), dim3(256), 0, (const float *)aa.part, (int)splits, out, accumulate, (int)nqh,
                         dig, dxs));
        if (planes && md_written) *md_written = true;
    } else if ((splits > 1 || decode_kernel) && md && !xd && !accumulate && hd % 32 == 0) {
        auto *kern = digit_kind == PG_GGML_Q4_0 ? gqa_combine_kernel<3> : gqa_combine_kernel<4>;
        PG_TRY(pg_launch(ctx, "gqa_combine_mm_digits", kern, dim3((unsigned)rows), dim3(128), 0, (const float *)aa.part, (int)splits,
                         (int)hd, (int)part_hdr, out, accumulate, (int)nqh, md->digits, md->xs));
        if (md_written) *md_written = true;
    } else if (splits > 1 || decode_kernel) {
        auto *kern = !xd ? gqa_combine_kernel<0> : (digit_kind == PG_GGML_Q4_0 ? gqa_combine_kernel<1> : gqa_combine_kernel<2>);
        PG_TRY(pg_launch(ctx, xd ? "gqa_combine_digits" : "gqa_combine", kern, dim3((unsigned)rows), dim3(128), 0,
                         (const float *)aa.part, (int)splits, (int)hd, (int)part_hdr, out, accumulate, (int)nqh,
                         xd ? xd->digits : nullptr, xd ? xd->xs : nullptr));
    } else if (xd) {
        PG_TRY(pg_launch_x_to_digits(ctx, out, seq_q, nqh * hd, digit_kind, *xd));
    }
    return PG_OK;
}

pg_status check_attention_args(const char *fn, const pg_kv_cache *kc, const pg_kv_cache *vc, size_t nqh, size_t seq_q,
                               int mask_kind, size_t offset) {
    PG_CHECK_ARG(kc && vc, "%s: null cache", fn);
    PG_CHECK_ARG(kc->num_kv_heads == vc->num_kv_heads && kc->head_dim == vc->head_dim && kc->len == vc->len,
                 "%s: the key and value caches differ in shape or length", fn);
    PG_CHECK_ARG(kc->num_kv_heads > 0 && nqh % kc->num_kv_heads == 0,
                 "%s: num_q_heads %zu is not a multiple of num_kv_heads %zu", fn, nqh, kc->num_kv_heads);
    PG_CHECK_ARG(mask_kind >= PG_MASK_NONE && mask_kind <= PG_MASK_CAUSAL_SLIDING_WINDOW, "%s: unknown mask kind %d", fn,
                 mask_kind);
    PG_CHECK_ARG(nqh <= 65535, "%s: more than 65535 query heads", fn);
    PG_CHECK_ARG(offset + seq_q < (1ull << 31) && kc->len < (1ull << 31), "%s: positions beyond 2^31", fn);
    return PG_OK;
}

// Room for `needed` positions per head; grows like the reference (at least double, from 16).
pg_status cache_reserve(pg_ctx *ctx, pg_kv_cache *c, size_t needed) {
    if (needed <= c->capacity) return PG_OK;
    const size_t grown = (c->capacity > 16 ? c->capacity : 16) * 2;
    const size_t new_cap = needed > grown ? needed : grown;
    const size_t hd = c->head_dim, total = c->num_kv_heads * new_cap * hd * sizeof(float);
    float *nk = nullptr, *nv = nullptr;
    PG_HIP(hipMalloc(reinterpret_cast<void **>(&nk), total));
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&nv), total);
    if (e != hipSuccess) {
        (void)hipFree(nk);
        return pg_fail(PG_ENOMEM, "hipMalloc(%zu) failed: %s", total, hipGetErrorString(e));
    }
    e = hipMemsetAsync(nk, 0, total, ctx->stream);
    if (e == hipSuccess) e = hipMemsetAsync(nv, 0, total, ctx->stream);
    if (e == hipSuccess && c->len > 0) {
        const size_t width = c->len * hd * sizeof(float);
        e = hipMemcpy2DAsync(nk, new_cap * hd * sizeof(float), c->k, c->capacity * hd * sizeof(float), width,
                             c->num_kv_heads, hipMemcpyDeviceToDevice, ctx->stream);
        if (e == hipSuccess)
            e = hipMemcpy2DAsync(nv, new_cap * hd * sizeof(float), c->v, c->capacity * hd * sizeof(float), width,
                                 c->num_kv_heads, hipMemcpyDeviceToDevice, ctx->stream);
    }
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);  // the old planes are freed next
    if (e != hipSuccess) {
        (void)hipFree(nk);
        (void)hipFree(nv);
        return pg_fail(PG_EDEVICE, "KV cache growth failed: %s", hipGetErrorString(e));
    }
    if (c->k) (void)hipFree(c->k);
    if (c->v) (void)hipFree(c->v);
    c->k = nk;
    c->v = nv;
    c->capacity = new_cap;
    return PG_OK;
}

pg_status launch_rope(pg_ctx *ctx, const rope_args &ra, size_t seq, size_t heads) {
    if (seq == 0 || heads == 0) return PG_OK;
    bool vec = ra.hd % 8 == 0 && ra.hd <= 2048 && ((uintptr_t)ra.cos_t | (uintptr_t)ra.sin_t) % 16 == 0;
    for (int i = 0; i < ra.nseg && vec; ++i) {
        const rope_seg &sg = ra.seg[i];
        vec = ((uintptr_t)sg.src | (uintptr_t)sg.dst) % 16 == 0 && sg.src_tstride % 4 == 0 && sg.dst_hstride % 4 == 0 &&
              (sg.planes <= 1 || sg.plane_stride % 4 == 0);
    }
    if (vec) {
        const size_t threads = heads * (size_t)(ra.hd / 8);
        return pg_launch(ctx, "rope", rope_v4_kernel, dim3((unsigned)seq, (unsigned)((threads + 255) / 256)), dim3(256), 0, ra, (int)heads);
    }
    return pg_launch(ctx, "rope", rope_kernel, dim3((unsigned)seq, (unsigned)heads), dim3(128), 0, ra);
}

}  // namespace

// ---- RMSNorm ----------------------------------------------------------------------------------

PG_API pg_status pg_rmsnorm_dev(pg_ctx *ctx, const float *x_dev, size_t rows, size_t dim, const float *w_dev, float eps,
                                float *out_dev) {
    PG_TRY(pg_use(ctx));
    if (rows == 0 || dim == 0) return PG_OK;
    PG_CHECK_ARG(x_dev && w_dev && out_dev, "pg_rmsnorm: null pointer");
    PG_CHECK_ARG(dim < (1ull << 31) && rows < (1ull << 31), "pg_rmsnorm: shape too large");
    return launch_rmsnorm(ctx, x_dev, nullptr, nullptr, w_dev, eps, rows, dim, out_dev);
}

PG_API pg_status pg_rmsnorm(pg_ctx *ctx, const float *x, size_t rows, size_t dim, const float *w, float eps, float *out) {
    PG_TRY(pg_use(ctx));
    if (rows == 0 || dim == 0) return PG_OK;
    PG_CHECK_ARG(x && w && out, "pg_rmsnorm: null pointer");
    pg_tmp dx, dw, dout;
    PG_TRY(dx.alloc(rows * dim * sizeof(float)));
    PG_TRY(dw.alloc(dim * sizeof(float)));
    PG_TRY(dout.alloc(rows * dim * sizeof(float)));
    PG_HIP(hipMemcpyAsync(dx.p, x, rows * dim * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipMemcpyAsync(dw.p, w, dim * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_rmsnorm_dev(ctx, dx.as<float>(), rows, dim, dw.as<float>(), eps, dout.as<float>()));
    PG_HIP(hipMemcpyAsync(out, dout.p, rows * dim * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

// ---- RoPE -------------------------------------------------------------------------------------

PG_API pg_status pg_rope_create(pg_ctx *ctx, size_t head_dim, size_t max_seq_len, float base, pg_rope **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(out != nullptr, "pg_rope_create: null output");
    *out = nullptr;
    PG_CHECK_ARG(head_dim > 0 && head_dim % 2 == 0, "pg_rope_create: head_dim %zu must be even and positive", head_dim);
    PG_CHECK_ARG(max_seq_len > 0 && max_seq_len < (1ull << 31) && head_dim < (1ull << 16), "pg_rope_create: shape out of range");
    // The tables are f32 libm values, as the reference computes them (src/nn.rs:1258-1282).
    const size_t half = head_dim / 2, n = max_seq_len * head_dim;
    std::vector<float> freq(half), c(n), s(n);
    for (size_t i = 0; i < half; ++i) freq[i] = powf(base, 2.0f * (float)i / (float)head_dim);
    for (size_t pos = 0; pos < max_seq_len; ++pos)
        for (size_t i = 0; i < half; ++i) {
            const float theta = (float)pos / freq[i];
            const float cv = cosf(theta), sv = sinf(theta);
            c[pos * head_dim + i] = cv; c[pos * head_dim + half + i] = cv;
            s[pos * head_dim + i] = sv; s[pos * head_dim + half + i] = sv;
        }
    pg_rope *r = new (std::nothrow) pg_rope{nullptr, nullptr, head_dim, max_seq_len};
    if (!r) return pg_fail(PG_ENOMEM, "pg_rope_create: out of host memory");
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&r->cos_t), n * sizeof(float));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&r->sin_t), n * sizeof(float));
    if (e == hipSuccess) e = hipMemcpyAsync(r->cos_t, c.data(), n * sizeof(float), hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipMemcpyAsync(r->sin_t, s.data(), n * sizeof(float), hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        if (r->cos_t) (void)hipFree(r->cos_t);
        if (r->sin_t) (void)hipFree(r->sin_t);
        delete r;
        return pg_fail(e == hipErrorOutOfMemory ? PG_ENOMEM : PG_EDEVICE, "pg_rope_create: %s", hipGetErrorString(e));
    }
    *out = r;
    return PG_OK;
}

PG_API void pg_rope_free(pg_ctx *ctx, pg_rope *r) {
    if (!r) return;
    if (ctx) (void)pg_use(ctx);
    if (r->cos_t) (void)hipFree(r->cos_t);
    if (r->sin_t) (void)hipFree(r->sin_t);
    delete r;
}

PG_API pg_status pg_rope_apply_dev(pg_ctx *ctx, const pg_rope *r, const float *x_dev, size_t seq_len, size_t offset,
                                   float *out_dev) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(r != nullptr, "pg_rope_apply: null table");
    if (seq_len == 0) return PG_OK;
    PG_CHECK_ARG(x_dev && out_dev, "pg_rope_apply: null pointer");
    PG_CHECK_ARG(offset + seq_len <= r->max_seq_len, "pg_rope_apply: positions %zu..%zu exceed max_seq_len %zu", offset,
                 offset + seq_len, r->max_seq_len);
    rope_args ra = {};
    ra.seg[0] = {x_dev, out_dev, r->head_dim, 0, 1, 1};
    ra.cos_t = r->cos_t; ra.sin_t = r->sin_t; ra.hd = (int)r->head_dim; ra.pos0 = (int)offset; ra.nseg = 1;
    return launch_rope(ctx, ra, seq_len, 1);
}

PG_API pg_status pg_rope_apply(pg_ctx *ctx, const pg_rope *r, const float *x, size_t seq_len, size_t offset, float *out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(r != nullptr, "pg_rope_apply: null table");
    if (seq_len == 0) return PG_OK;
    PG_CHECK_ARG(x && out, "pg_rope_apply: null pointer");
    const size_t bytes = seq_len * r->head_dim * sizeof(float);
    pg_tmp dx, dout;
    PG_TRY(dx.alloc(bytes));
    PG_TRY(dout.alloc(bytes));
    PG_HIP(hipMemcpyAsync(dx.p, x, bytes, hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_rope_apply_dev(ctx, r, dx.as<float>(), seq_len, offset, dout.as<float>()));
    PG_HIP(hipMemcpyAsync(out, dout.p, bytes, hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

// ---- KV cache ---------------------------------------------------------------------------------

PG_API pg_status pg_kv_cache_create(pg_ctx *ctx, size_t num_kv_heads, size_t head_dim, pg_kv_cache **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(out != nullptr, "pg_kv_cache_create: null output");
    *out = nullptr;
    PG_CHECK_ARG(num_kv_heads > 0 && head_dim > 0 && head_dim <= 256 && num_kv_heads < 65536,
                 "pg_kv_cache_create: num_kv_heads %zu / head_dim %zu out of range (head_dim <= 256)", num_kv_heads, head_dim);
    pg_kv_cache *c = new (std::nothrow) pg_kv_cache{nullptr, nullptr, 0, 0, num_kv_heads, head_dim};
    if (!c) return pg_fail(PG_ENOMEM, "pg_kv_cache_create: out of host memory");
    *out = c;
    return PG_OK;
}

PG_API void pg_kv_cache_free(pg_ctx *ctx, pg_kv_cache *c) {
    if (!c) return;
    if (ctx) {
        (void)pg_use(ctx);
        (void)hipStreamSynchronize(ctx->stream);
    }
    if (c->k) (void)hipFree(c->k);
    if (c->v) (void)hipFree(c->v);
    delete c;
}

PG_API size_t pg_kv_cache_len(const pg_kv_cache *c) { return c ? c->len : 0; }
PG_API size_t pg_kv_cache_capacity(const pg_kv_cache *c) { return c ? c->capacity : 0; }

PG_API pg_status pg_kv_cache_rollback_to(pg_kv_cache *c, size_t new_len) {
    PG_CHECK_ARG(c != nullptr, "pg_kv_cache_rollback_to: null cache");
    PG_CHECK_ARG(new_len <= c->len, "rollback_to: new_len %zu > current len %zu", new_len, c->len);
    c->len = new_len;
    return PG_OK;
}

PG_API pg_status pg_kv_cache_append_dev(pg_ctx *ctx, pg_kv_cache *c, const float *new_k_dev, const float *new_v_dev,
                                        size_t seq_len) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(c != nullptr, "pg_kv_cache_append: null cache");
    if (seq_len == 0) return PG_OK;
    PG_CHECK_ARG(new_k_dev && new_v_dev, "pg_kv_cache_append: null pointer");
    PG_CHECK_ARG(c->len + seq_len < (1ull << 31), "pg_kv_cache_append: length beyond 2^31");
    PG_TRY(cache_reserve(ctx, c, c->len + seq_len));
    const size_t hd = c->head_dim, width = seq_len * hd * sizeof(float);
    PG_HIP(hipMemcpy2DAsync(c->k + c->len * hd, c->capacity * hd * sizeof(float), new_k_dev, width, width,
                            c->num_kv_heads, hipMemcpyDeviceToDevice, ctx->stream));
    PG_HIP(hipMemcpy2DAsync(c->v + c->len * hd, c->capacity * hd * sizeof(float), new_v_dev, width, width,
                            c->num_kv_heads, hipMemcpyDeviceToDevice, ctx->stream));
    c->len += seq_len;
    return PG_OK;
}

PG_API pg_status pg_kv_cache_append(pg_ctx *ctx, pg_kv_cache *c, const float *new_k, const float *new_v, size_t seq_len) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(c != nullptr, "pg_kv_cache_append: null cache");
    if (seq_len == 0) return PG_OK;
    PG_CHECK_ARG(new_k && new_v, "pg_kv_cache_append: null pointer");
    const size_t bytes = c->num_kv_heads * seq_len * c->head_dim * sizeof(float);
    pg_tmp dk, dv;
    PG_TRY(dk.alloc(bytes));
    PG_TRY(dv.alloc(bytes));
    PG_HIP(hipMemcpyAsync(dk.p, new_k, bytes, hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipMemcpyAsync(dv.p, new_v, bytes, hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_kv_cache_append_dev(ctx, c, dk.as<float>(), dv.as<float>(), seq_len));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

PG_API pg_status pg_kv_cache_download(pg_ctx *ctx, const pg_kv_cache *c, float *k, float *v) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(c != nullptr, "pg_kv_cache_download: null cache");
    if (c->len == 0) return PG_OK;
    PG_CHECK_ARG(k && v, "pg_kv_cache_download: null pointer");
    const size_t hd = c->head_dim, width = c->len * hd * sizeof(float);
    PG_HIP(hipMemcpy2DAsync(k, width, c->k, c->capacity * hd * sizeof(float), width, c->num_kv_heads,
                            hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipMemcpy2DAsync(v, width, c->v, c->capacity * hd * sizeof(float), width, c->num_kv_heads,
                            hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

// ---- grouped-query attention ------------------------------------------------------------------

PG_API pg_status pg_gqa_attention_dev(pg_ctx *ctx, const float *q_dev, const pg_kv_cache *k_cache,
                                      const pg_kv_cache *v_cache, size_t num_q_heads, size_t seq_q, float scale,
                                      int mask_kind, size_t offset, size_t window, size_t sink_tokens, float logit_cap,
                                      float *out_dev) {
    PG_TRY(pg_use(ctx));
    PG_TRY(check_attention_args("pg_gqa_attention", k_cache, v_cache, num_q_heads, seq_q, mask_kind, offset));
    if (seq_q == 0 || num_q_heads == 0) return PG_OK;
    PG_CHECK_ARG(q_dev && out_dev, "pg_gqa_attention: null pointer");
    return launch_attention(ctx, q_dev, k_cache, v_cache, num_q_heads, seq_q, scale, mask_kind, offset, window,
                            sink_tokens, logit_cap, out_dev, 1);
}

PG_API pg_status pg_gqa_attention(pg_ctx *ctx, const float *q, const pg_kv_cache *k_cache, const pg_kv_cache *v_cache,
                                  size_t num_q_heads, size_t seq_q, float scale, int mask_kind, size_t offset,
                                  size_t window, size_t sink_tokens, float logit_cap, float *out) {
    PG_TRY(pg_use(ctx));
    PG_TRY(check_attention_args("pg_gqa_attention", k_cache, v_cache, num_q_heads, seq_q, mask_kind, offset));
    if (seq_q == 0 || num_q_heads == 0) return PG_OK;
    PG_CHECK_ARG(q && out, "pg_gqa_attention: null pointer");
    const size_t bytes = num_q_heads * seq_q * k_cache->head_dim * sizeof(float);
    pg_tmp dq, dout;
    PG_TRY(dq.alloc(bytes));
    PG_TRY(dout.alloc(bytes));
    PG_HIP(hipMemcpyAsync(dq.p, q, bytes, hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipMemcpyAsync(dout.p, out, bytes, hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(launch_attention(ctx, dq.as<float>(), k_cache, v_cache, num_q_heads, seq_q, scale, mask_kind, offset, window,
                            sink_tokens, logit_cap, dout.as<float>(), 1));
    PG_HIP(hipMemcpyAsync(out, dout.p, bytes, hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

PG_API pg_status pg_gqa_attention_local_global_dev(pg_ctx *ctx, const float *q_dev, const pg_kv_cache *k_cache,
                                                   const pg_kv_cache *v_cache, size_t num_q_heads, size_t seq_q,
                                                   float scale, size_t offset, size_t local_window,
                                                   const size_t *global_positions, size_t num_global, float logit_cap,
                                                   float *out_dev) {
    PG_TRY(pg_use(ctx));
    PG_TRY(check_attention_args("pg_gqa_attention_local_global", k_cache, v_cache, num_q_heads, seq_q, PG_MASK_CAUSAL, offset));
    PG_CHECK_ARG(global_positions || num_global == 0, "pg_gqa_attention_local_global: null position list");
    if (seq_q == 0 || num_q_heads == 0) return PG_OK;
    PG_CHECK_ARG(q_dev && out_dev, "pg_gqa_attention_local_global: null pointer");
    return launch_attention(ctx, q_dev, k_cache, v_cache, num_q_heads, seq_q, scale, PG_MASK_LOCAL_GLOBAL, offset,
                            local_window, 0, logit_cap, out_dev, 1, nullptr, 0, global_positions, num_global);
}

PG_API pg_status pg_gqa_attention_local_global(pg_ctx *ctx, const float *q, const pg_kv_cache *k_cache,
                                               const pg_kv_cache *v_cache, size_t num_q_heads, size_t seq_q, float scale,
                                               size_t offset, size_t local_window, const size_t *global_positions,
                                               size_t num_global, float logit_cap, float *out) {
    PG_TRY(pg_use(ctx));
    PG_TRY(check_attention_args("pg_gqa_attention_local_global", k_cache, v_cache, num_q_heads, seq_q, PG_MASK_CAUSAL, offset));
    PG_CHECK_ARG(global_positions || num_global == 0, "pg_gqa_attention_local_global: null position list");
    if (seq_q == 0 || num_q_heads == 0) return PG_OK;
    PG_CHECK_ARG(q && out, "pg_gqa_attention_local_global: null pointer");
    const size_t bytes = num_q_heads * seq_q * k_cache->head_dim * sizeof(float);
    pg_tmp dq, dout;
    PG_TRY(dq.alloc(bytes));
    PG_TRY(dout.alloc(bytes));
    PG_HIP(hipMemcpyAsync(dq.p, q, bytes, hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipMemcpyAsync(dout.p, out, bytes, hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(launch_attention(ctx, dq.as<float>(), k_cache, v_cache, num_q_heads, seq_q, scale, PG_MASK_LOCAL_GLOBAL, offset,
                            local_window, 0, logit_cap, dout.as<float>(), 1, nullptr, 0, global_positions, num_global));
    PG_HIP(hipMemcpyAsync(out, dout.p, bytes, hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}

// ---- the decoder block ------------------------------------------------------------------------

PG_API pg_status pg_llama_block_create(pg_ctx *ctx, size_t model_dim, size_t num_q_heads, size_t num_kv_heads,
                                       size_t head_dim, size_t ffn_dim, size_t max_seq_len, float rope_base,
                                       float rms_eps, pg_llama_block **out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(out != nullptr, "pg_llama_block_create: null output");
    *out = nullptr;
    PG_CHECK_ARG(model_dim > 0 && ffn_dim > 0 && num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0,
                 "pg_llama_block_create: bad shape (d %zu, ffn %zu, heads %zu/%zu)", model_dim, ffn_dim, num_q_heads,
                 num_kv_heads);
    PG_CHECK_ARG(head_dim <= 256 && num_q_heads < 65536, "pg_llama_block_create: head_dim %zu > 256 or too many heads", head_dim);
    PG_CHECK_ARG(model_dim % 32 == 0 && ffn_dim % 32 == 0 && (num_q_heads * head_dim) % 32 == 0,
                 "pg_llama_block_create: model_dim, ffn_dim and num_q_heads*head_dim must be multiples of the 32-value GGUF block");
    pg_llama_block *b = new (std::nothrow) pg_llama_block{};
    if (!b) return pg_fail(PG_ENOMEM, "pg_llama_block_create: out of host memory");
    b->d = model_dim; b->nqh = num_q_heads; b->nkvh = num_kv_heads; b->hd = head_dim; b->ffn = ffn_dim; b->eps = rms_eps;
    pg_status st = pg_rope_create(ctx, head_dim, max_seq_len, rope_base, &b->rope);
    if (st == PG_OK) {
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&b->attn_norm_w), 2 * model_dim * sizeof(float));
        if (e != hipSuccess) st = pg_fail(PG_ENOMEM, "pg_llama_block_create: %s", hipGetErrorString(e));
    }
    if (st != PG_OK) {
        pg_rope_free(ctx, b->rope);
        delete b;
        return st;
    }
    b->ffn_norm_w = b->attn_norm_w + model_dim;
    // one-token step buffers: three digit sets, then the pointer tables and the item ids
    const size_t q_dim = num_q_heads * head_dim;
    const size_t items = num_q_heads / num_kv_heads + 2;
    const size_t o_q = pg_xdigits_bytes(1, model_dim), o_f = o_q + pg_xdigits_bytes(1, q_dim);
    const size_t o_tab = o_f + pg_xdigits_bytes(1, ffn_dim);
    const size_t tab_bytes = pg_round_up((2 * items + 4) * sizeof(void *) + items * sizeof(int), 256);
    const size_t total = o_tab + tab_bytes + pg_round_up(model_dim / 32 * sizeof(float), 256);
    hipError_t e = hipMalloc(&b->dec, total);
    if (e == hipSuccess) e = hipMemsetAsync(b->dec, 0, total, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        st = pg_fail(PG_ENOMEM, "pg_llama_block_create: %s", hipGetErrorString(e));
        pg_llama_block_free(ctx, b);
        return st;
    }
    char *base = static_cast<char *>(b->dec);
    b->xd_d = pg_xdigits_carve(base, 1, model_dim);
    b->xd_q = pg_xdigits_carve(base + o_q, 1, q_dim);
    b->xd_f = pg_xdigits_carve(base + o_f, 1, ffn_dim);
    const void **tab = reinterpret_cast<const void **>(base + o_tab);
    b->qkv_items = (int)items;
    b->qs_qkv = reinterpret_cast<const uint8_t *const *>(tab);
    b->d_qkv = reinterpret_cast<const uint16_t *const *>(tab + items);
    b->qs_gu = reinterpret_cast<const uint8_t *const *>(tab + 2 * items);
    b->d_gu = reinterpret_cast<const uint16_t *const *>(tab + 2 * items + 2);
    b->item_ids = reinterpret_cast<const int *>(tab + 2 * items + 4);
    b->ss_part = reinterpret_cast<float *>(base + o_tab + tab_bytes);
    *out = b;
    return PG_OK;
}

PG_API void pg_llama_block_free(pg_ctx *ctx, pg_llama_block *b) {
    if (!b) return;
    if (ctx) {
        (void)pg_use(ctx);
        (void)hipStreamSynchronize(ctx->stream);
    }
    pg_rope_free(ctx, b->rope);
    if (b->attn_norm_w) (void)hipFree(b->attn_norm_w);
    if (b->arena) (void)hipFree(b->arena);
    if (b->chain) (void)hipFree(b->chain);
    if (b->dec) (void)hipFree(b->dec);
    delete b;
}

PG_API pg_status pg_llama_block_set_weights(pg_ctx *ctx, pg_llama_block *b, const pg_gguf_tensor *q_proj,
                                            const pg_gguf_tensor *k_proj, const pg_gguf_tensor *v_proj,
                                            const pg_gguf_tensor *o_proj, const pg_gguf_tensor *gate_proj,
                                            const pg_gguf_tensor *up_proj, const pg_gguf_tensor *down_proj,
                                            const float *attn_norm_w, const float *ffn_norm_w) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(b != nullptr, "pg_llama_block_set_weights: null block");
    const pg_gguf_tensor *w[7] = {q_proj, k_proj, v_proj, o_proj, gate_proj, up_proj, down_proj};
    const size_t q_dim = b->nqh * b->hd, kv_dim = b->nkvh * b->hd;
    const size_t want[7][2] = {{q_dim, b->d}, {kv_dim, b->d}, {kv_dim, b->d}, {b->d, q_dim},
                               {b->ffn, b->d}, {b->ffn, b->d}, {b->d, b->ffn}};
    static const char *names[7] = {"q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"};
    for (int i = 0; i < 7; ++i) {
        PG_CHECK_ARG(w[i] != nullptr, "pg_llama_block_set_weights: %s is null", names[i]);
        PG_CHECK_ARG(w[i]->n_out == want[i][0] && w[i]->k_in == want[i][1],
                     "pg_llama_block_set_weights: %s is [%zu, %zu], expected [%zu, %zu] (out, in)", names[i], w[i]->n_out,
                     w[i]->k_in, want[i][0], want[i][1]);
    }
    PG_CHECK_ARG(attn_norm_w && ffn_norm_w, "pg_llama_block_set_weights: null norm weights");
    PG_HIP(hipMemcpyAsync(b->attn_norm_w, attn_norm_w, b->d * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    PG_HIP(hipMemcpyAsync(b->ffn_norm_w, ffn_norm_w, b->d * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    // Tables for the multi-item launches.  An item is kv_dim weight rows: q contributes
    // num_q_heads / num_kv_heads of them (row offsets into its planes: 16 or 32 quant bytes and
    // one scale per block, scales in tiles of 8 rows), then k, then v; gate and up are one each.
    {
        const size_t items = (size_t)b->qkv_items, nb = b->d / 32;
        const size_t qb = w[0]->ggml_type == PG_GGML_Q4_0 ? 16 : 32;
        std::vector<const void *> ptrs(2 * items + 4);
        for (size_t i = 0; i + 2 < items; ++i) {
            ptrs[i] = w[0]->qs + i * kv_dim * nb * qb;
            ptrs[items + i] = w[0]->d + i * kv_dim * nb;  // (kv_dim / 8) tiles x nb blocks x 8 scales
        }
        ptrs[items - 2] = w[1]->qs; ptrs[items - 1] = w[2]->qs;
        ptrs[2 * items - 2] = w[1]->d; ptrs[2 * items - 1] = w[2]->d;
        ptrs[2 * items] = w[4]->qs; ptrs[2 * items + 1] = w[5]->qs;
        ptrs[2 * items + 2] = w[4]->d; ptrs[2 * items + 3] = w[5]->d;
        std::vector<int> ids(items);
        for (size_t i = 0; i < items; ++i) ids[i] = (int)i;
        PG_HIP(hipMemcpyAsync(const_cast<uint8_t **>(b->qs_qkv), ptrs.data(), ptrs.size() * sizeof(void *), hipMemcpyHostToDevice,
                              ctx->stream));
        PG_HIP(hipMemcpyAsync(const_cast<int *>(b->item_ids), ids.data(), items * sizeof(int), hipMemcpyHostToDevice, ctx->stream));
        PG_HIP(hipStreamSynchronize(ctx->stream));  // the vectors die with this scope
    }
    PG_HIP(hipStreamSynchronize(ctx->stream));
    for (int i = 0; i < 7; ++i) b->w[i] = w[i];
    // nibble digits (Q4_0) or byte digits (Q8_0); Q4_1 also needs block sums and MXFP4 its own digit
    // order, which only the separate digit kernel writes: such a block takes the product-by-product route
    auto kind = [](const pg_gguf_tensor *t) {
        return t->ggml_type == PG_GGML_Q4_0 ? PG_GGML_Q4_0 : (t->ggml_type == PG_GGML_Q8_0 ? PG_GGML_Q8_0 : -1);
    };
    b->digit_kind = kind(w[0]);
    for (int i = 1; i < 7; ++i)
        if (kind(w[i]) != b->digit_kind) b->digit_kind = 0;
    if (b->digit_kind < 0) b->digit_kind = 0;
    return PG_OK;
}

// The one-token step: every producer of a GEMV input writes digits instead of f32, and where the producer
// is a product its workgroups do so themselves (the o-projection leaves h1 * norm weights, gate|up leave
// SiLU(g) * u; the first RMSNorm rides in the q|k|v launch), q/k/v run as one multi-item launch, the
// residual adds are GEMV epilogues, RoPE and the cache append ride in the attention kernel: with Q4_0
// tensors 6 launches (q|k|v, attention, merge of its key splits, o, gate|up, down) instead of 18; Q8_0
// tensors keep the first RMSNorm as a launch (7).
static pg_status block_forward_one_token(pg_ctx *ctx, pg_llama_block *b, const float *h_dev, pg_kv_cache *cache,
                                         float *out_dev) {
    const size_t d = b->d, hd = b->hd, q_dim = b->nqh * hd, kv_dim = b->nkvh * hd, ffn = b->ffn, offset = cache->len;
    auto slot = [](size_t n) { return pg_round_up(n, 64); };
    const size_t cap = b->seq_cap;
    float *p = b->arena;
    auto take = [&](size_t n) { float *r = p; p += slot(n); return r; };
    // the arena is laid out for the many-token route (normed, h1, proj | q, q_rope, attn | k, v | g, u | q|k|v);
    // this step uses h1, q_rope, attn, g|u and the adjacent q|k|v rows
    (void)take(cap * d);
    float *h1 = take(cap * d);
    (void)take(cap * d);
    (void)take(cap * q_dim);
    float *q_rope = take(cap * q_dim), *attn = take(cap * q_dim);
    (void)take(cap * kv_dim);
    (void)take(cap * kv_dim);
    float *g = take(2 * cap * ffn), *u = g + ffn;
    // q|k|v and g|u as adjacent rows: item i of a multi-item launch writes y + i * n_out
    float *qkv = take(cap * (q_dim + 2 * kv_dim) + 128), *qd = qkv, *kd = qkv + q_dim, *vd = kd + kv_dim;
    const int kind = b->digit_kind;
    const pg_gemv_batch one = {1, nullptr, nullptr, nullptr, 1};
    const pg_gemv_batch qkv_n = {b->qkv_items, b->qs_qkv, b->d_qkv, b->item_ids, b->qkv_items};
    const pg_gemv_batch gu2 = {2, b->qs_gu, b->d_gu, b->item_ids, 2};
    const bool qkv_same = b->w[0]->ggml_type == b->w[1]->ggml_type && b->w[1]->ggml_type == b->w[2]->ggml_type && kv_dim % 8 == 0;
    const bool gu_same = b->w[4]->ggml_type == b->w[5]->ggml_type;

    if (kind == PG_GGML_Q4_0 && qkv_same && d <= 8192) {
        // the norm rides in the products' launch: digits of h * (norm weights) per workgroup, the scalar factor at the end
        PG_TRY(pg_launch_gguf_gemv_rmsnorm(ctx, kv_dim, d, nullptr, nullptr, qkv_n, h_dev, b->attn_norm_w, b->eps, qkv));
    } else if (qkv_same) {
        PG_TRY(launch_rmsnorm_digits(ctx, h_dev, nullptr, nullptr, b->attn_norm_w, b->eps, 1, d, kind, b->xd_d));
        PG_TRY(pg_launch_gguf_gemv(ctx, b->w[0]->ggml_type, kv_dim, d, nullptr, nullptr, qkv_n, b->xd_d, qkv));
    } else {
        PG_TRY(launch_rmsnorm_digits(ctx, h_dev, nullptr, nullptr, b->attn_norm_w, b->eps, 1, d, kind, b->xd_d));
        PG_TRY(pg_launch_gguf_gemv(ctx, b->w[0]->ggml_type, q_dim, d, b->w[0]->qs, b->w[0]->d, one, b->xd_d, qd));
        PG_TRY(pg_launch_gguf_gemv(ctx, b->w[1]->ggml_type, kv_dim, d, b->w[1]->qs, b->w[1]->d, one, b->xd_d, kd));
        PG_TRY(pg_launch_gguf_gemv(ctx, b->w[2]->ggml_type, kv_dim, d, b->w[2]->qs, b->w[2]->d, one, b->xd_d, vd));
    }
    PG_TRY(cache_reserve(ctx, cache, offset + 1));
    if (attention_is_short(ctx, b->nqh, offset + 1, hd)) {
        // RoPE of q and of the new key, and the append of the new key and value, happen inside
        // the attention kernel: one launch less.
        attn_args fuse = {};
        fuse.raw_q = qd; fuse.raw_k = kd; fuse.raw_v = vd;
        fuse.rope_c = b->rope->cos_t + offset * hd; fuse.rope_s = b->rope->sin_t + offset * hd;
        fuse.k_new = cache->k + offset * hd; fuse.v_new = cache->v + offset * hd;
        fuse.new_pos = (int)offset;
        cache->len = offset + 1;
        PG_TRY(launch_attention(ctx, qd, cache, cache, b->nqh, 1, 1.0f / sqrtf((float)hd), PG_MASK_CAUSAL, offset, 0, 0, 0.0f,
                                attn, 0, &b->xd_q, kind, nullptr, 0, &fuse));
    } else {
        rope_args ra = {};
        ra.seg[0] = {qd, q_rope, q_dim, hd, (int)b->nqh, 1};
        ra.seg[1] = {kd, cache->k + offset * hd, kv_dim, cache->capacity * hd, (int)b->nkvh, 1};
        ra.seg[2] = {vd, cache->v + offset * hd, kv_dim, cache->capacity * hd, (int)b->nkvh, 0};
        ra.cos_t = b->rope->cos_t; ra.sin_t = b->rope->sin_t; ra.hd = (int)hd; ra.pos0 = (int)offset; ra.nseg = 3;
        PG_TRY(launch_rope(ctx, ra, 1, b->nqh + 2 * b->nkvh));
        cache->len = offset + 1;
        PG_TRY(launch_attention(ctx, q_rope, cache, cache, b->nqh, 1, 1.0f / sqrtf((float)hd), PG_MASK_CAUSAL, offset, 0, 0, 0.0f,
                                attn, 0, &b->xd_q, kind));
    }
    if (d % 32 == 0 && ffn % 32 == 0 && d <= 8192) {  // (kind: all seven tensors Q4_0, or all Q8_0)
        // h1 = h + attn . Wo, stored, and also left as the digits of h1 * (norm weights) with its sums of
        // squares; gate and up divide by the RMS themselves and leave the digits of SiLU(g) * u: two
        // launches (RMSNorm, SiLU.up) fewer
        PG_TRY(pg_launch_gguf_gemv_norm_digits(ctx, kind, d, q_dim, b->w[3]->qs, b->w[3]->d, b->xd_q, h1, h_dev, b->ffn_norm_w, b->xd_d,
                                               b->ss_part));
        PG_TRY(pg_launch_gguf_gemv_swiglu_digits(ctx, kind, ffn, d, b->w[4]->qs, b->w[4]->d, b->w[5]->qs, b->w[5]->d, b->xd_d, b->ss_part,
                                                 d / 32, d, b->eps, b->xd_f));
        return pg_launch_gguf_gemv(ctx, kind, d, ffn, b->w[6]->qs, b->w[6]->d, one, b->xd_f, out_dev, h1);
    }
    // h1 = h + attn . Wo
    PG_TRY(pg_launch_gguf_gemv(ctx, b->w[3]->ggml_type, d, q_dim, b->w[3]->qs, b->w[3]->d, one, b->xd_q, h1, h_dev));
    PG_TRY(launch_rmsnorm_digits(ctx, h1, nullptr, nullptr, b->ffn_norm_w, b->eps, 1, d, kind, b->xd_d));
    if (gu_same) {
        PG_TRY(pg_launch_gguf_gemv(ctx, b->w[4]->ggml_type, ffn, d, nullptr, nullptr, gu2, b->xd_d, g));
    } else {
        PG_TRY(pg_launch_gguf_gemv(ctx, b->w[4]->ggml_type, ffn, d, b->w[4]->qs, b->w[4]->d, one, b->xd_d, g));
        PG_TRY(pg_launch_gguf_gemv(ctx, b->w[5]->ggml_type, ffn, d, b->w[5]->qs, b->w[5]->d, one, b->xd_d, u));
    }
    auto *sw = kind == PG_GGML_Q4_0 ? swiglu_digits_kernel<true> : swiglu_digits_kernel<false>;
    PG_TRY(pg_launch(ctx, "swiglu_digits", sw, dim3(blocks_for(ffn / 4)), dim3(256), 0, (const float4 *)g, (const float4 *)u,
                     (int)(ffn / 4), b->xd_f.digits, b->xd_f.xs));
    // out = h1 + act . Wd
    return pg_launch_gguf_gemv(ctx, b->w[6]->ggml_type, d, ffn, b->w[6]->qs, b->w[6]->d, one, b->xd_f, out_dev, h1);
}

// The many-token step with all seven tensors Q4_0 (or all Q8_0): every product's input reaches it as the two
// digit planes its producer wrote (RMSNorm, SiLU.up), and a product whose K was cut into chunks leaves the
// chunks' planes to its consumer, which adds them up as it reads (RoPE, the residual add inside the second
// RMSNorm, SiLU.up, the last residual add).  The same arithmetic in the same order as the product-by-product
// route, with q|k|v and gate|up as one launch each: 12 launches instead of 25 when every product is split (a few
// tokens: each launch is 4 us there).
static pg_status block_forward_chained(pg_ctx *ctx, pg_llama_block *b, const float *h_dev, size_t seq, pg_kv_cache *cache,
                                       float *out_dev, float *h1, float *q_rope, float *attn) {
    const size_t d = b->d, hd = b->hd, q_dim = b->nqh * hd, kv_dim = b->nkvh * hd, ffn = b->ffn, offset = cache->len;
    const int type = b->digit_kind;
    const bool nib = type == PG_GGML_Q4_0;
    const size_t tiles = (seq + 31) / 32;
    const size_t n_of[7] = {q_dim, kv_dim, kv_dim, d, ffn, ffn, d}, k_of[7] = {d, d, d, q_dim, d, d, ffn};
    // q|k|v and gate|up are one launch each (the tensors' 128-row groups one after the other): one K split for the launch
    const int first_of[7] = {0, 0, 0, 3, 4, 4, 6}, count_of[7] = {3, 3, 3, 1, 2, 2, 1};
    // Up to eight tokens: the few-rows product (one launch per tensor group, no K split between workgroups, so every
    // product leaves one plane; the weights are read in their row-major planes, no tile-major copy).
    // (Nine to sixteen tokens: only the products over fewer than 32 weight rows per CU, see pg_gguf_skinny_takes.)
    bool few[7], hm[7];
    int ks[7];
    size_t part_off[7], floats = 0;
    for (int i = 0; i < 7; ++i) {
        size_t groups = 0, rows = 0;
        for (int j = first_of[i]; j < first_of[i] + count_of[i]; ++j) {
            groups += (n_of[j] + 127) / 128;
            rows += n_of[j];
        }
        few[i] = pg_gguf_skinny_takes(ctx, type, seq, rows, k_of[i]);
        ks[i] = few[i] ? 1 : pg_gguf_mm_splitk(ctx, groups * 128, k_of[i], tiles, seq, false, nullptr);
        // Many tokens: the f16 matrix-core product where it is the faster one (its input then arrives as two f16
        // planes, not as digit planes; the down projection's producer holds a row of the FFN width in registers).
        int hks = 1;
        hm[i] = !few[i] && (i != 6 || ffn <= 32768) && count_of[i] <= PG_HMM_MAX_GROUP &&
                pg_gguf_hmm_takes(ctx, type, seq, rows, k_of[i], &hks);
        if (hm[i]) ks[i] = hks;
        if (ks[i] > PG_MAX_PLANES) return pg_fail(PG_EUNSUPPORTED, "llama block: a product in %d K chunks", ks[i]);
        part_off[i] = floats;
        floats += pg_round_up((size_t)ks[i] * seq * n_of[i], 64);
    }
    const size_t sz_d = pg_mmdigits_bytes(seq, d), sz_q = pg_mmdigits_bytes(seq, q_dim), sz_f = pg_mmdigits_bytes(seq, ffn);
    const size_t sz_hd = hm[0] || hm[4] ? pg_hmm_planes_bytes(seq, d) : 0, sz_hq = hm[3] ? pg_hmm_planes_bytes(seq, q_dim) : 0,
                 sz_hf = hm[6] ? pg_hmm_planes_bytes(seq, ffn) : 0;
    const size_t need = sz_d + sz_q + sz_f + floats * sizeof(float) + sz_hd + sz_hq + sz_hf;
    if (need > b->chain_bytes) {
        PG_HIP(hipStreamSynchronize(ctx->stream));
        if (b->chain) (void)hipFree(b->chain);
        b->chain = nullptr;
        b->chain_bytes = 0;
        const size_t want = need + need / 4;
        PG_HIP(hipMalloc(&b->chain, want));
        b->chain_bytes = want;
    }
    char *base = static_cast<char *>(b->chain);
    const pg_mmdigits md_d = pg_mmdigits_carve(base, seq, d), md_q = pg_mmdigits_carve(base + sz_d, seq, q_dim),
                      md_f = pg_mmdigits_carve(base + sz_d + sz_q, seq, ffn);
    float *parts = reinterpret_cast<float *>(base + sz_d + sz_q + sz_f);
    auto part = [&](int i) { return parts + part_off[i]; };
    char *hbase = base + sz_d + sz_q + sz_f + floats * sizeof(float);
    const pg_hmm_planes pl_d = pg_hmm_planes_carve(hbase, seq, d), pl_q = pg_hmm_planes_carve(hbase + sz_hd, seq, q_dim),
                        pl_f = pg_hmm_planes_carve(hbase + sz_hd + sz_hq, seq, ffn);  // (carved whether used or not: only those with bytes are touched)
    pg_mm_group grp = {1, nullptr, nullptr, nullptr, nullptr, 0, (int)tiles, (int)seq, 1};
    grp.tiled = 1;
    auto product = [&](int i, const pg_mmdigits &md) -> pg_status {  // tensors i .. i + count_of[i] - 1
        if (hm[i]) {
            float *ys[PG_HMM_MAX_GROUP] = {part(i), count_of[i] > 1 ? part(i + 1) : nullptr, count_of[i] > 2 ? part(i + 2) : nullptr, nullptr};
            return pg_launch_gguf_hmm_group(ctx, k_of[i], b->w + i, ys, count_of[i], seq, i == 3 ? pl_q : (i == 6 ? pl_f : pl_d), ks[i],
                                            nullptr, true);
        }
        if (few[i]) {
            float *ys[3] = {part(i), count_of[i] > 1 ? part(i + 1) : nullptr, count_of[i] > 2 ? part(i + 2) : nullptr};
            return pg_launch_gguf_skinny_group(ctx, type, k_of[i], b->w + i, ys, count_of[i], seq, md);
        }
        pg_mm_group g = grp;
        size_t groups = 0;
        g.nseg = count_of[i] > 1 ? count_of[i] : 0;
        for (int j = 0; j < count_of[i]; ++j) {
            PG_TRY(pg_gguf_ensure_tiled(ctx, b->w[i + j]));
            g.seg_first[j] = (int)groups; g.seg_n[j] = (int)n_of[i + j];
            g.seg_qs[j] = b->w[i + j]->qs_tiled; g.seg_d[j] = b->w[i + j]->d;
            g.seg_out[j] = part(i + j); g.seg_stride[j] = seq * n_of[i + j];
            groups += (n_of[i + j] + 127) / 128;
        }
        if (count_of[i] == 1)
            return pg_launch_gguf_mm(ctx, type, n_of[i], k_of[i], b->w[i]->qs_tiled, b->w[i]->d, g, seq, md, part(i), part(i), true);
        return pg_launch_gguf_mm(ctx, type, groups * 128, k_of[i], nullptr, nullptr, g, seq, md, part(i), part(i), true);
    };
    auto norm_digits = [&](const float *a, int bi, float *sum_out, const float *w, bool f16_planes) -> pg_status {
        if (f16_planes) {
            auto *kern = d <= 4096 ? add_rmsnorm_vec_kernel<4, 5> : add_rmsnorm_vec_kernel<8, 5>;
            return pg_launch(ctx, "add_rmsnorm_f16_planes", kern, dim3((unsigned)seq), dim3(256), 0, (const float4 *)a,
                             (const float4 *)(bi >= 0 ? part(bi) : nullptr), (float4 *)sum_out, (const float4 *)w, b->eps, (int)(d / 4),
                             (float4 *)pl_d.lo, (int8_t *)pl_d.hi, pl_d.inv, bi >= 0 ? ks[bi] : 1, seq * d / 4);
        }
        auto *kern = d <= 4096 ? (nib ? add_rmsnorm_vec_kernel<4, 3> : add_rmsnorm_vec_kernel<4, 4>)
                               : (nib ? add_rmsnorm_vec_kernel<8, 3> : add_rmsnorm_vec_kernel<8, 4>);
        return pg_launch(ctx, "add_rmsnorm_mm_digits", kern, dim3((unsigned)seq), dim3(256), 0, (const float4 *)a,
                         (const float4 *)(bi >= 0 ? part(bi) : nullptr), (float4 *)sum_out, (const float4 *)w, b->eps, (int)(d / 4),
                         (float4 *)nullptr, md_d.digits, md_d.xs, bi >= 0 ? ks[bi] : 1, seq * d / 4);
    };
    const int nbf = (int)(ffn / 32);

    PG_TRY(norm_digits(h_dev, -1, nullptr, b->attn_norm_w, hm[0]));
    PG_TRY(product(0, md_d));
    PG_TRY(cache_reserve(ctx, cache, offset + seq));
    rope_args ra = {};
    ra.seg[0] = {part(0), q_rope, q_dim, seq * hd, (int)b->nqh, 1, ks[0], seq * q_dim};
    ra.seg[1] = {part(1), cache->k + offset * hd, kv_dim, cache->capacity * hd, (int)b->nkvh, 1, ks[1], seq * kv_dim};
    ra.seg[2] = {part(2), cache->v + offset * hd, kv_dim, cache->capacity * hd, (int)b->nkvh, 0, ks[2], seq * kv_dim};
    ra.cos_t = b->rope->cos_t; ra.sin_t = b->rope->sin_t; ra.hd = (int)hd; ra.pos0 = (int)offset; ra.nseg = 3;
    PG_TRY(launch_rope(ctx, ra, seq, b->nqh + 2 * b->nkvh));
    cache->len = offset + seq;
    bool md_written = false;  // (a merge of key runs writes the o-projection's digit planes itself)
    PG_TRY(launch_attention(ctx, q_rope, cache, cache, b->nqh, seq, 1.0f / sqrtf((float)hd), PG_MASK_CAUSAL, offset, 0, 0,
                            0.0f, attn, 0, nullptr, type, nullptr, 0, nullptr, hd % 32 == 0 && !hm[3] ? &md_q : nullptr, &md_written));
    if (hm[3]) PG_TRY(pg_launch_rows_to_f16_planes(ctx, attn, seq, q_dim, pl_q));
    else if (!md_written) PG_TRY(pg_launch_x_to_mm_digits(ctx, attn, seq, q_dim, type, md_q));
    PG_TRY(product(3, md_q));
    PG_TRY(norm_digits(h_dev, 3, h1, b->ffn_norm_w, hm[4]));  // h1 = h + attn . Wo, and its norm as digits
    PG_TRY(product(4, md_d));
    if (hm[6]) {
        auto *kern = ffn <= 16384 ? swiglu_f16_planes_kernel<16> : swiglu_f16_planes_kernel<32>;
        PG_TRY(pg_launch(ctx, "swiglu_f16_planes", kern, dim3((unsigned)seq), dim3(256), 0, (const float *)part(4), (const float *)part(5),
                         ks[4], seq * ffn, (int)(ffn / 4), (_Float16 *)pl_f.hi, (_Float16 *)pl_f.lo, pl_f.inv));
    } else {
        auto *kern = nib ? swiglu_mm_digits_kernel<true> : swiglu_mm_digits_kernel<false>;
        PG_TRY(pg_launch(ctx, "swiglu_mm_digits", kern, dim3((unsigned)((nbf + 31) / 32), (unsigned)seq), dim3(256), 0,
                         (const float *)part(4), (const float *)part(5), ks[4], seq * ffn, nbf, (int)pg_round_up(nbf, 4),
                         md_f.digits, md_f.xs));
    }
    if (few[6]) {  // the down product adds the residual itself
        float *ys[1] = {out_dev};
        return pg_launch_gguf_skinny_group(ctx, type, k_of[6], b->w + 6, ys, 1, seq, md_f, h1);
    }
    PG_TRY(product(6, md_f));
    return pg_launch(ctx, "residual_add", add_planes_kernel, dim3(blocks_for(seq * d)), dim3(256), 0, (const float *)h1,
                     (const float *)part(6), ks[6], seq * d, out_dev, seq * d);
}

PG_API pg_status pg_llama_block_forward_dev(pg_ctx *ctx, pg_llama_block *b, const float *h_dev, size_t seq,
                                            pg_kv_cache *cache, float *out_dev) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(b && cache, "pg_llama_block_forward: null block or cache");
    PG_CHECK_ARG(b->w[0] != nullptr, "pg_llama_block_forward: weights not set");
    PG_CHECK_ARG(cache->num_kv_heads == b->nkvh && cache->head_dim == b->hd,
                 "pg_llama_block_forward: cache is %zu heads x %zu, block is %zu x %zu", cache->num_kv_heads,
                 cache->head_dim, b->nkvh, b->hd);
    if (seq == 0) return PG_OK;
    PG_CHECK_ARG(h_dev && out_dev, "pg_llama_block_forward: null pointer");
    PG_CHECK_ARG(seq < (1ull << 24), "pg_llama_block_forward: seq %zu too large", seq);
    const size_t offset = cache->len;
    PG_CHECK_ARG(offset + seq <= b->rope->max_seq_len, "pg_llama_block_forward: positions %zu..%zu exceed max_seq_len %zu",
                 offset, offset + seq, b->rope->max_seq_len);
    const size_t d = b->d, hd = b->hd, q_dim = b->nqh * hd, kv_dim = b->nkvh * hd, ffn = b->ffn;
    // activation arena: every slice a multiple of 64 floats so that each stays 256-byte aligned
    auto slot = [](size_t n) { return pg_round_up(n, 64); };
    if (seq > b->seq_cap) {
        const size_t cap = seq > 2 * b->seq_cap ? seq : 2 * b->seq_cap;
        const size_t floats = 3 * slot(cap * d) + 3 * slot(cap * q_dim) + 2 * slot(cap * kv_dim) + 2 * slot(cap * ffn) +
                              slot(cap * (q_dim + 2 * kv_dim) + 128);  // the last term: q|k|v adjacent for the one-token step
        PG_HIP(hipStreamSynchronize(ctx->stream));
        if (b->arena) (void)hipFree(b->arena);
        b->arena = nullptr;
        b->seq_cap = 0;
        PG_HIP(hipMalloc(reinterpret_cast<void **>(&b->arena), floats * sizeof(float)));
        b->seq_cap = cap;
    }
    const size_t cap = b->seq_cap;
    if (seq == 1 && b->digit_kind != 0 && hd % 32 == 0 && d <= 8192 && (uintptr_t)h_dev % 16 == 0)
        return block_forward_one_token(ctx, b, h_dev, cache, out_dev);
    float *p = b->arena;
    auto take = [&](size_t n) { float *r = p; p += slot(n); return r; };
    float *normed = take(cap * d), *h1 = take(cap * d), *proj = take(cap * d);
    float *qd = take(cap * q_dim), *q_rope = take(cap * q_dim), *attn = take(cap * q_dim);
    float *kd = take(cap * kv_dim), *vd = take(cap * kv_dim);
    float *g = take(cap * ffn), *u = take(cap * ffn);  // the one-token step relies on this order (k, v and g, u adjacent)
    const size_t min_k = PG_MM_MIN_BLOCKS * 32;
    if (b->digit_kind != 0 && seq <= 65535 && d >= min_k && q_dim >= min_k && ffn >= min_k && d <= 8192 &&
        ((uintptr_t)h_dev | (uintptr_t)out_dev) % 16 == 0)
        return block_forward_chained(ctx, b, h_dev, seq, cache, out_dev, h1, q_rope, attn);

    PG_TRY(launch_rmsnorm(ctx, h_dev, nullptr, nullptr, b->attn_norm_w, b->eps, seq, d, normed));
    float *const qkv[3] = {qd, kd, vd};
    PG_TRY(pg_gguf_matmul_rows_multi(ctx, normed, seq, b->w, qkv, 3));
    PG_TRY(cache_reserve(ctx, cache, offset + seq));
    rope_args ra = {};
    ra.seg[0] = {qd, q_rope, q_dim, seq * hd, (int)b->nqh, 1};
    ra.seg[1] = {kd, cache->k + offset * hd, kv_dim, cache->capacity * hd, (int)b->nkvh, 1};
    ra.seg[2] = {vd, cache->v + offset * hd, kv_dim, cache->capacity * hd, (int)b->nkvh, 0};
    ra.cos_t = b->rope->cos_t; ra.sin_t = b->rope->sin_t; ra.hd = (int)hd; ra.pos0 = (int)offset; ra.nseg = 3;
    PG_TRY(launch_rope(ctx, ra, seq, b->nqh + 2 * b->nkvh));
    cache->len = offset + seq;
    PG_TRY(launch_attention(ctx, q_rope, cache, cache, b->nqh, seq, 1.0f / sqrtf((float)hd), PG_MASK_CAUSAL, offset, 0, 0,
                            0.0f, attn, 0));
    PG_TRY(pg_gguf_matmul_rows(ctx, attn, seq, b->w[3], proj));
    PG_TRY(launch_rmsnorm(ctx, h_dev, proj, h1, b->ffn_norm_w, b->eps, seq, d, normed));
    float *const gu[2] = {g, u};
    PG_TRY(pg_gguf_matmul_rows_multi(ctx, normed, seq, b->w + 4, gu, 2));
    PG_TRY(pg_launch(ctx, "swiglu", swiglu_kernel, dim3(blocks_for(seq * ffn)), dim3(256), 0, g, (const float *)u, seq * ffn));
    PG_TRY(pg_gguf_matmul_rows(ctx, g, seq, b->w[6], proj));
    return pg_launch(ctx, "residual_add", add_kernel, dim3(blocks_for(seq * d)), dim3(256), 0, (const float *)h1,
                     (const float *)proj, out_dev, seq * d);
}

PG_API pg_status pg_llama_block_forward(pg_ctx *ctx, pg_llama_block *b, const float *h, size_t seq, pg_kv_cache *cache,
                                        float *out) {
    PG_TRY(pg_use(ctx));
    PG_CHECK_ARG(b != nullptr, "pg_llama_block_forward: null block");
    if (seq == 0) return PG_OK;
    PG_CHECK_ARG(h && out, "pg_llama_block_forward: null pointer");
    const size_t bytes = seq * b->d * sizeof(float);
    pg_tmp dh, dout;
    PG_TRY(dh.alloc(bytes));
    PG_TRY(dout.alloc(bytes));
    PG_HIP(hipMemcpyAsync(dh.p, h, bytes, hipMemcpyHostToDevice, ctx->stream));
    PG_TRY(pg_llama_block_forward_dev(ctx, b, dh.as<float>(), seq, cache, dout.as<float>()));
    PG_HIP(hipMemcpyAsync(out, dout.p, bytes, hipMemcpyDeviceToHost, ctx->stream));
    PG_HIP(hipStreamSynchronize(ctx->stream));
    return PG_OK;
}
