// Host-side audit of the streaming kernels' load addresses.  No kernel runs and no HIP call is made: every function
// walks the (workgroup, wavefront, lane, step) space of one launch with the index functions the kernels themselves
// use (pg_stream_addr.h) and reports, per array, the end of the furthest byte any load would touch beside the size
// of the allocation.  A test without a GPU sweeps ragged shapes over every instantiation and holds one against the
// other: an over-read of a few hundred bytes only faults on the device when the tensor happens to end a mapping.
#include <algorithm>
#include "pg_internal.h"
#include "pg_stream_addr.h"

namespace {
struct span_check {
    size_t end = 0;
    void touch(size_t offset, size_t bytes) { end = std::max(end, offset + bytes); }
};
}  // namespace

// One-row W8A8 products over a [n_pad][k_pad] weight plane (gemv_w8a8_m1_kernel: nw = 4; gemv_w8a8_m1_f32x_kernel:
// nw = 4, 8, 16).  nch = the kernel's NCH (64-lane steps over a row), rpw = rows per wavefront.  `f32_row`: the
// row arrives in f32 (k elements, k % 4 == 0) and every thread fetches float4s of it.
PG_API pg_status pg_audit_gemv_w8a8_m1(size_t k, size_t n, int nch, int rpw, int nw, int f32_row, size_t *w_end, size_t *w_bytes,
                                       size_t *x_end, size_t *x_bytes) {
    PG_CHECK_ARG(k > 0 && n > 0 && nch > 0 && rpw > 0 && nw > 0, "pg_audit_gemv_w8a8_m1: bad arguments");
    const size_t k_pad = pg_round_up(k, PG_KPAD), n_pad = pg_round_up(n, PG_NPAD);
    const int nchunk = (int)(k_pad >> 4);
    PG_CHECK_ARG((size_t)nch * 64 >= (size_t)nchunk, "pg_audit_gemv_w8a8_m1: NCH %d does not cover a row of %zu bytes", nch, k_pad);
    span_check w, x;
    const int wgs = (int)(n_pad / ((size_t)nw * rpw));
    for (int wg = 0; wg < wgs; ++wg)
        for (int wave = 0; wave < nw; ++wave) {
            const int row0 = pg_m1_row0(wg, wave, nw, rpw);
            for (int r = 0; r < rpw; ++r)
                for (int lane = 0; lane < 64; ++lane)
                    for (int j = 0; j < nch; ++j) w.touch(((size_t)(row0 + r) * k_pad) + (size_t)pg_m1_weight_chunk(lane, j, nchunk) * 16, 16);
        }
    if (f32_row) {
        const int nt = 64 * nw, nv = (nch * 256 + nt - 1) / nt, nvec = (int)(k >> 2);
        for (int t = 0; t < nt; ++t)
            for (int i = 0; i < nv; ++i) x.touch((size_t)pg_m1_x_vec(t, i, nt, nvec) * 16, 16);
    }
    if (w_end) *w_end = w.end;
    if (w_bytes) *w_bytes = n_pad * k_pad;
    if (x_end) *x_end = x.end;
    if (x_bytes) *x_bytes = k * 4;
    return PG_OK;
}

// 2 .. 64 rows in one launch over int8 weights (gemm_w8a8_skinny_kernel<MB, NB, NW, NST>): the weight plane
// [n_pad][k_pad] and the quantised activation rows [m_pad][k_pad].
PG_API pg_status pg_audit_gemm_w8a8_skinny(size_t m, size_t k, size_t n, int mb, int nb_tiles, int nw, size_t *w_end, size_t *w_bytes,
                                           size_t *a_end, size_t *a_bytes) {
    PG_CHECK_ARG(m > 0 && k > 0 && n > 0 && mb > 0 && nb_tiles > 0 && nw > 0, "pg_audit_gemm_w8a8_skinny: bad arguments");
    PG_CHECK_ARG((size_t)16 * mb >= m, "pg_audit_gemm_w8a8_skinny: %d activation tiles for %zu rows", mb, m);
    const size_t k_pad = pg_round_up(k, PG_KPAD), n_pad = pg_round_up(n, PG_NPAD), m_pad = pg_round_up(m, PG_MPAD);
    span_check w, a;
    const int wgs = (int)((n + 16 * nb_tiles - 1) / (16 * nb_tiles));
    const int units = (int)(k_pad / 128), per = (units + nw - 1) / nw;
    for (int wg = 0; wg < wgs; ++wg) {
        const int n0 = wg * 16 * nb_tiles;
        for (int wave = 0; wave < nw; ++wave) {
            const int u_begin = wave * per, u_end = std::min(u_begin + per, units), cnt = u_end - u_begin;
            if (cnt <= 0) continue;
            const int rot = (int)(((unsigned)wg * 5u) % (unsigned)cnt);
            for (int t = 0; t < cnt; ++t) {
                const int unit = pg_skinny_walk_unit(u_begin, cnt, t, rot);
                for (int lane = 0; lane < 64; ++lane)
                    for (int j = 0; j < 2; ++j) {
                        const int r = 8 * j + (lane >> 3), ch = (lane & 7) ^ ((r >> 1) & 7);
                        for (int c = 0; c < nb_tiles; ++c) w.touch(pg_skinny_fill_offset(n0 + 16 * c + r, (int)k_pad, unit, ch), 16);
                        for (int b = 0; b < mb; ++b) a.touch(pg_skinny_fill_offset(16 * b + r, (int)k_pad, unit, ch), 16);
                    }
            }
        }
    }
    if (w_end) *w_end = w.end;
    if (w_bytes) *w_bytes = n_pad * k_pad;
    if (a_end) *a_end = a.end;
    if (a_bytes) *a_bytes = m_pad * k_pad;
    return PG_OK;
}

// One-row block products (gguf_gemv_kernel<QT, BPL, RW, R, ..., NW> and the few-rows form): the payload plane
// [n_out][nh][nb][16 B] (nh = 2 for Q8_0, else 1) and the scale plane [ceil(n_out / 8)][nb][8 x f16].
// bpl = blocks per lane and K segment, rw = rows per wavefront, nw = wavefronts per workgroup.
PG_API pg_status pg_audit_gguf_gemv(size_t n_out, size_t k_in, int q8, int bpl, int rw, int nw, size_t *qs_end, size_t *qs_bytes,
                                    size_t *d_end, size_t *d_bytes) {
    PG_CHECK_ARG(n_out > 0 && k_in >= 32 && k_in % 32 == 0 && bpl >= 1 && bpl <= 4 && rw > 0 && nw > 0, "pg_audit_gguf_gemv: bad arguments");
    const int nb = (int)(k_in / 32), nh = q8 ? 2 : 1, seg = 64 * bpl;
    span_check qs, d;
    const int wgs = (int)((n_out + (size_t)rw * nw - 1) / ((size_t)rw * nw));
    for (int wg = 0; wg < wgs; ++wg)
        for (int wave = 0; wave < nw; ++wave) {
            const int row0 = (wg * nw + wave) * rw;
            const bool live = (size_t)row0 < n_out;  // the wavefronts with no row of their own load no weights
            if (!live) continue;
            for (int seg0 = 0; seg0 < nb; seg0 += seg) {
                const int seg_n = std::min(nb - seg0, seg);
                for (int lane = 0; lane < 64; ++lane)
                    for (int p = 0; p < bpl; ++p) {
                        const int blk = pg_gemv_lane_block(seg0, lane, p, seg_n);
                        d.touch(pg_gemv_scale_unit(row0, nb, blk) * 16, 16);
                        for (int r = 0; r < rw; ++r) {
                            const int row = pg_gemv_clamp_row(row0 + r, (int)n_out);
                            for (int h = 0; h < nh; ++h) qs.touch(pg_gemv_weight_unit(row, h, nh, nb, blk) * 16, 16);
                        }
                    }
            }
        }
    if (qs_end) *qs_end = qs.end;
    if (qs_bytes) *qs_bytes = n_out * (size_t)nb * nh * 16;
    if (d_end) *d_end = d.end;
    if (d_bytes) *d_bytes = (n_out + 7) / 8 * 8 * (size_t)nb * sizeof(uint16_t);
    return PG_OK;
}

// 2 .. 16 rows in one launch over a block tensor (gguf_skinny_kernel<QT, NB, MT, NW, NST>): K in units of 8 blocks
// (k_in % 256 == 0), a workgroup of nw wavefronts per `tiles` tiles of 16 weight rows.
PG_API pg_status pg_audit_gguf_skinny(size_t n_out, size_t k_in, int q8, int nw, int tiles, size_t *qs_end, size_t *qs_bytes,
                                      size_t *d_end, size_t *d_bytes) {
    PG_CHECK_ARG(n_out > 0 && k_in >= 256 && k_in % 256 == 0 && nw > 0 && (tiles == 1 || tiles == 2), "pg_audit_gguf_skinny: bad arguments");
    const int nb = (int)(k_in / 32), wf = q8 ? 4 : 2, units = nb / 8, per = (units + nw - 1) / nw, ntile = (int)((n_out + 7) / 8);
    span_check qs, d;
    const int wgs = (int)((n_out + 16 * tiles - 1) / (16 * tiles));
    for (int wg = 0; wg < wgs; ++wg) {
        const int n0 = wg * 16 * tiles;
        for (int wave = 0; wave < nw; ++wave) {
            const int u_begin = wave * per, u_end = std::min(u_begin + per, units), cnt = u_end - u_begin;
            if (cnt <= 0) continue;
            const int rot = (int)(((unsigned)wg * 5u) % (unsigned)cnt);
            for (int t = 0; t < cnt; ++t) {
                const int unit = pg_skinny_walk_unit(u_begin, cnt, t, rot);
                for (int lane = 0; lane < 64; ++lane) {
                    for (int j = 0; j < wf; ++j) {
                        const int slot = 8 * j + (lane >> 3), r = slot & 15, half = slot >> 4, ch = (lane & 7) ^ ((r >> 1) & 7);
                        for (int c = 0; c < tiles; ++c) {
                            const int row = pg_gemv_clamp_row(n0 + 16 * c + r, (int)n_out);
                            qs.touch(pg_gskinny_weight_offset(q8 ? (size_t)row * 2 + half : (size_t)row, nb, unit, ch), 16);
                        }
                    }
                    if (lane < 16 * tiles) d.touch(pg_gskinny_scale_offset(pg_gskinny_scale_tile(n0, lane, ntile), nb, unit, lane), 16);
                }
            }
        }
    }
    if (qs_end) *qs_end = qs.end;
    if (qs_bytes) *qs_bytes = n_out * (size_t)nb * (q8 ? 32 : 16);
    if (d_end) *d_end = d.end;
    if (d_bytes) *d_bytes = (n_out + 7) / 8 * 8 * (size_t)nb * sizeof(uint16_t);
    return PG_OK;
}

// Many rows on the f16 matrix cores (gguf_hmm_kernel<QT, NWM, NWN>): 256 x 256 tiles (wide = 0) or 128 x 512 (wide = 1; Q8_0 always),
// K in `ks` chunks of whole stages of 64; the planes are [m][k_in] f16, the payload [n_out][k_in / 32][16 B] (Q8_0: [n_out][2][k_in / 32][16 B]).
// (Every offset is linear in the stage: the first and the last stage of a chunk bound the rest.)
PG_API pg_status pg_audit_gguf_hmm(size_t m, size_t n_out, size_t k_in, int q8, int wide, int ks, size_t *plane_end, size_t *plane_bytes,
                                   size_t *qs_end, size_t *qs_bytes, size_t *d_end, size_t *d_bytes) {
    PG_CHECK_ARG(m > 0 && n_out >= 2 && k_in >= 64 && k_in % 64 == 0 && ks >= 1, "pg_audit_gguf_hmm: bad arguments");
    const int nb = (int)(k_in / 32), K = (int)k_in, M = (int)m, N = (int)n_out;
    PG_CHECK_ARG(!q8 || wide, "pg_audit_gguf_hmm: Q8_0 runs the 128 x 512 tiles only");
    const int nwn = wide ? 8 : 4, bm = wide ? 128 : 256, bn = 64 * nwn, lx = bm / 64, lw = (bn * (q8 ? 64 : 32) / 1024 + 7) / 8;
    const int stages = nb / 2, kt_per = (stages + ks - 1) / ks;
    const int tiles_m = (M + bm - 1) / bm, panels = (N + bn - 1) / bn;
    auto swz128 = [](int r) { return ((r >> 1) & 7) ^ ((r & 1) << 2); };
    span_check pl, qs, d;
    for (int split = 0; split * kt_per < stages; ++split) {
        const int kt0 = split * kt_per, kt_n = std::min(kt_per, stages - kt0);
        for (int tm = 0; tm < tiles_m; ++tm)
            for (int np = 0; np < panels; ++np) {
                const int m0 = tm * bm, n0 = np * bn;
                for (int wave = 0; wave < 8; ++wave)
                    for (int lane = 0; lane < 64; ++lane)
                        for (int st : {kt0, kt0 + kt_n - 1}) {
                            for (int i = 0; i < lx; ++i) {
                                const int row = 8 * (wave + 8 * i) + (lane >> 3);
                                pl.touch(pg_hmm_plane_offset(pg_hmm_clamp_row(m0 + row, M), K, st, (lane & 7) ^ swz128(row)), 16);
                            }
                            for (int i = 0; i < lw; ++i) {
                                if (q8) {
                                    const int row = 16 * (wave + 8 * i) + (lane >> 2), rc = row < bn ? row : bn - 1;
                                    const int c = (lane & 3) ^ ((row >> 2) & 3);
                                    qs.touch(pg_hmm_weight_offset_q8(pg_hmm_clamp_row(n0 + rc, N), c & 1, nb, st, c >> 1), 16);
                                } else {
                                    const int row = 32 * (wave + 8 * i) + (lane >> 1), rc = row < bn ? row : bn - 1;
                                    qs.touch(pg_hmm_weight_offset(pg_hmm_clamp_row(n0 + rc, N), nb, st, (lane & 1) ^ ((row >> 3) & 1)), 16);
                                }
                            }
                            const int row = (wave % nwn) * 64 + 2 * (lane & 31);
                            d.touch(pg_hmm_scale_offset(pg_hmm_scale_row(n0 + row, N), nb, st, lane >> 5), 4);
                        }
            }
    }
    if (plane_end) *plane_end = pl.end;
    if (plane_bytes) *plane_bytes = m * k_in * 2;
    if (qs_end) *qs_end = qs.end;
    if (qs_bytes) *qs_bytes = n_out * (size_t)nb * (q8 ? 32 : 16);
    if (d_end) *d_end = d.end;
    if (d_bytes) *d_bytes = (n_out + 7) / 8 * 8 * (size_t)nb * sizeof(uint16_t);
    return PG_OK;
}

// MXFP4 rows (mxfp4_rows_kernel<T, RG, NW>): the fragment-major code plane [row groups of 16][ncp chunks][64 lanes][16 B]
// and the scale plane [row groups][ncp / 4][64 lanes][4 B]; a wavefront = (row group, K slice), 8 chunks per batch of loads.
PG_API pg_status pg_audit_mxfp4_rows(size_t out_dim, size_t in_dim, int rg_per_wg, int nw, size_t *qs_end, size_t *qs_bytes,
                                     size_t *sc_end, size_t *sc_bytes) {
    PG_CHECK_ARG(out_dim > 0 && in_dim >= 32 && in_dim % 32 == 0 && rg_per_wg > 0 && nw >= rg_per_wg && nw % rg_per_wg == 0, "pg_audit_mxfp4_rows: bad arguments");
    const int nb = (int)(in_dim / 32), ncp = (int)((((size_t)nb + 3) / 4 + 3) & ~(size_t)3), nrg = (int)((out_dim + 15) / 16), ks = nw / rg_per_wg;
    const int mx_u = 8;
    span_check qs, sc;
    const int wgs = (nrg + rg_per_wg - 1) / rg_per_wg;
    const int cps = ((ncp + ks - 1) / ks + 3) & ~3;
    for (int wg = 0; wg < wgs; ++wg)
        for (int wave = 0; wave < nw; ++wave) {
            const int rgi = wave / ks, ksi = wave % ks;
            int rg = wg * rg_per_wg + rgi;
            rg = rg < nrg ? rg : nrg - 1;
            const int c0 = ksi * cps, c1 = std::min(c0 + cps, ncp);
            auto batch = [&](int cb) {
                for (int lane = 0; lane < 64; ++lane) {
                    for (int u = 0; u < mx_u; ++u) qs.touch((((size_t)rg * ncp + pg_mx_chunk(cb + u, ncp)) * 64 + lane) * 16, 16);
                    for (int g = 0; g < mx_u / 4; ++g) sc.touch((((size_t)rg * (ncp / 4) + pg_mx_scale_word(cb + 4 * g, ncp)) * 64 + lane) * 4, 4);
                }
            };
            batch(c0 < ncp ? c0 : 0);
            for (int cb = c0; cb < c1; cb += 2 * mx_u) {
                if (cb + mx_u < c1) batch(cb + mx_u);
                if (cb + 2 * mx_u < c1) batch(cb + 2 * mx_u);
            }
        }
    if (qs_end) *qs_end = qs.end;
    if (qs_bytes) *qs_bytes = (size_t)nrg * ncp * 64 * 16;
    if (sc_end) *sc_end = sc.end;
    if (sc_bytes) *sc_bytes = (size_t)nrg * (ncp / 4) * 64 * 4;
    return PG_OK;
}

// MXFP4 tiles (mxfp4_planes_kernel + mxfp4_tiles_kernel<RA, TB, BD>) with the plan the launcher makes for this shape on a
// part of `num_cu` CUs: the weights' code and scale planes as above, and the token records the pre-pass writes and the
// tile kernel reads ([token groups][ncp chunks][PG_MT_RECORD bytes]); rec_end covers both sides.
PG_API pg_status pg_audit_mxfp4_tiles(int num_cu, size_t out_dim, size_t in_dim, size_t m, size_t *qs_end, size_t *qs_bytes,
                                      size_t *sc_end, size_t *sc_bytes, size_t *rec_end, size_t *rec_bytes, int *ra, int *tb,
                                      int *ks) {
    PG_CHECK_ARG(num_cu > 0 && out_dim > 0 && in_dim >= 32 && in_dim % 32 == 0 && m > 0, "pg_audit_mxfp4_tiles: bad arguments");
    const int nb = (int)(in_dim / 32), ncp = (int)pg_mx_chunks((size_t)nb), nrg = (int)((out_dim + 15) / 16);
    const pg_mxfp4_tiles_plan p = pg_mxfp4_tiles_plan_for(num_cu, out_dim, m, ncp);
    PG_CHECK_ARG(p.ra <= nrg && p.cps % 4 == 0 && p.cps >= 4 && (size_t)p.ks * p.cps >= (size_t)ncp && (size_t)(p.ks - 1) * p.cps < (size_t)ncp,
                 "pg_audit_mxfp4_tiles: plan ra %d cps %d ks %d does not fit %d row groups / %d chunks", p.ra, p.cps, p.ks, nrg, ncp);
    span_check qs, sc, rec;
    // the pre-pass: a wavefront per (token group, pair of blocks)
    for (size_t tg = 0; tg < p.groups; ++tg)
        for (int b = 0; b < 4 * ncp; ++b)
            for (int col = 0; col < 16; col += 15) {
                for (int sub = 0; sub < 2; ++sub)
                    for (int j = 0; j < PG_MT_PLANES; ++j) rec.touch(pg_mt_plane_store(tg, ncp, b, sub, col, j), 16);
                rec.touch(pg_mt_scale_store(tg, ncp, b, col), 4);
            }
    // the tiles: every work item, wavefront and chunk of its run; lanes 0 and 63, threads 0 and 511
    const int units = p.tb * (PG_MT_RECORD / 16), rounds = (units + 64 * PG_MT_NW - 1) / (64 * PG_MT_NW);
    for (size_t wt = 0; wt < p.n_wt; ++wt)
        for (int split = 0; split < p.ks; ++split) {
            const int kc0 = split * p.cps, kc1 = pg_mt_run_end(split, p.cps, ncp);
            PG_CHECK_ARG(kc1 > kc0 && (kc1 - kc0) % 4 == 0, "pg_audit_mxfp4_tiles: run %d is [%d, %d)", split, kc0, kc1);
            for (int wave = 0; wave < PG_MT_NW; ++wave) {
                const int rg0 = pg_mt_first_row_group((int)(wt * PG_MT_NW + wave) * p.ra, p.ra, nrg);
                PG_CHECK_ARG(rg0 >= 0, "pg_audit_mxfp4_tiles: first row group %d", rg0);
                for (int r = 0; r < p.ra; ++r)
                    for (int c = kc0; c < kc1; ++c)
                        for (int lane = 0; lane < 64; lane += 63) {
                            qs.touch((((size_t)(rg0 + r) * ncp + c) * 64 + lane) * 16, 16);
                            sc.touch((((size_t)(rg0 + r) * (ncp / 4) + (c >> 2)) * 64 + lane) * 4, 4);
                        }
            }
            for (size_t tt = 0; tt < p.n_tt; ++tt)
                for (int i = 0; i < rounds; ++i)
                    for (int thread = 0; thread < 64 * PG_MT_NW; thread += 64 * PG_MT_NW - 1)
                        rec.touch(tt * p.tb * ncp * PG_MT_RECORD + pg_mt_unit_offset(thread + i * 64 * PG_MT_NW, units, ncp) +
                                      (size_t)(kc1 - 1) * PG_MT_RECORD, 16);
        }
    if (qs_end) *qs_end = qs.end;
    if (qs_bytes) *qs_bytes = (size_t)nrg * ncp * 64 * 16;
    if (sc_end) *sc_end = sc.end;
    if (sc_bytes) *sc_bytes = (size_t)nrg * (ncp / 4) * 64 * 4;
    if (rec_end) *rec_end = rec.end;
    if (rec_bytes) *rec_bytes = p.groups * ncp * (size_t)PG_MT_RECORD;
    if (ra) *ra = p.ra;
    if (tb) *tb = p.tb;
    if (ks) *ks = p.ks;
    return PG_OK;
}

// The read-stream probe (probe_read_kernel<U>): `total` 16-byte chunks cut into one slice per workgroup.
PG_API pg_status pg_audit_probe_read(size_t bytes, int workgroups, int threads, int loads_in_flight, size_t *end, size_t *alloc) {
    PG_CHECK_ARG(bytes >= 16 && workgroups > 0 && threads > 0 && loads_in_flight > 0, "pg_audit_probe_read: bad arguments");
    const size_t total = bytes / 16, cpw = (total + workgroups - 1) / workgroups;
    span_check s;
    for (int wg = 0; wg < workgroups; ++wg) {
        const size_t first = (size_t)wg * cpw;
        const size_t n = first >= total ? 0 : std::min(total - first, cpw);
        for (int t = 0; t < threads; ++t)
            for (size_t c = t; c < n; c += (size_t)loads_in_flight * threads)
                for (int u = 0; u < loads_in_flight; ++u) {
                    const size_t i = pg_probe_chunk(c, u, (unsigned)threads);
                    if (i < n) s.touch((first + i) * 16, 16);
                }
    }
    if (end) *end = s.end;
    if (alloc) *alloc = total * 16;
    return PG_OK;
}
