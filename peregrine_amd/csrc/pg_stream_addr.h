// Index arithmetic of the streaming kernels' loads, written once for the device and for the host.
// Lanes past the end of a row, a segment or a slice still have to name an address (or none): these
// are the expressions that decide it.  The kernels call them; pg_audit_* (pg_audit.hip) runs the same
// functions over every (workgroup, wavefront, lane, step) of a launch on the host and reports the
// largest byte offset any of them would touch, so that a test without a GPU can hold it against the
// size of the allocation.
#pragma once
#include <stddef.h>
#include <stdint.h>

#if defined(__HIPCC__)
#define PG_HD __host__ __device__ __forceinline__
#else
#define PG_HD inline
#endif

// ---- the read-stream probe: chunk `u` of the U a lane has in flight, from its position c in the slice
PG_HD size_t pg_probe_chunk(size_t c, int u, unsigned threads) { return c + (size_t)u * threads; }

// ---- one-row W8A8 products (gemv_w8a8_m1_kernel, gemv_w8a8_m1_f32x_kernel)
// chunk (16 bytes) of a weight row that lane `lane` fetches at step j of NCH: a lane past a short row fetches the
// row's first chunk again (it meets zeros of the activation row)
PG_HD int pg_m1_weight_chunk(int lane, int j, int nchunk) {
    const int c = lane + 64 * j;
    return c < nchunk ? c : 0;
}
// float4 of the f32 activation row that thread `thread` of NT fetches at step i: past the row, its last one
PG_HD int pg_m1_x_vec(int thread, int i, int nt, int nvec) {
    const int idx = thread + nt * i;
    return idx < nvec ? idx : nvec - 1;
}
// first weight row of a wavefront: workgroup `wg` of its weight, NW wavefronts of RPW rows each
PG_HD int pg_m1_row0(int wg, int wave, int nw, int rpw) { return (wg * nw + wave) * rpw; }

// ---- block-quantised one-row products (gguf_gemv_kernel and its forms)
// block of the K segment [seg0, seg0 + seg_n) that lane `lane` takes as its p-th: a lane past the segment's end
// reads the segment's first block again (with a zero scale)
PG_HD int pg_gemv_lane_block(int seg0, int lane, int p, int seg_n) {
    const int b = lane + 64 * p;
    return seg0 + (b < seg_n ? b : 0);
}
// weight row a wavefront reads for output row `row`: rows past the tensor repeat its last (masked at the store)
PG_HD int pg_gemv_clamp_row(int row, int n_out) { return row < n_out ? row : n_out - 1; }
// 16-byte unit of the payload plane: half `h` of NH (Q8_0: 2 half-blocks, else 1) of block `blk` of row `row`
PG_HD size_t pg_gemv_weight_unit(int row, int h, int nh, int nb, int blk) { return ((size_t)row * nh + h) * nb + blk; }
// 16-byte unit of the scale plane (8 rows x f16 per block): the tile of row0's eight rows, block `blk`
PG_HD size_t pg_gemv_scale_unit(int row0, int nb, int blk) { return (size_t)(row0 >> 3) * nb + blk; }
// block of the f32 activation row a digit-making thread fetches: past the row, its first
PG_HD int pg_gemv_x_block(int b, int nb) { return b < nb ? b : 0; }

// ---- few rows in one launch over int8 weights (gemm_w8a8_skinny_kernel): a wavefront walks its run of K units
// (128 bytes of K each) from a start that differs per workgroup and wraps round
PG_HD int pg_skinny_walk_unit(int u_begin, int cnt, int t, int rot) {
    const int r = t + rot;
    return u_begin + (r >= cnt ? r - cnt : r);
}
// byte offset of a 16-byte fill in a [rows][k_pad] plane: row, K unit, chunk within the unit's 128 bytes
PG_HD size_t pg_skinny_fill_offset(int row, int k_pad, int unit, int ch) { return (size_t)row * k_pad + (size_t)unit * 128 + (size_t)ch * 16; }

// ---- few rows in one launch over block tensors (gguf_skinny_kernel): units of 8 blocks
// byte offset of a 16-byte fill of the payload plane: stream row (Q8_0: 2 row + half), unit, chunk = block within the unit
PG_HD size_t pg_gskinny_weight_offset(size_t stream_row, int nb, int unit, int ch) { return stream_row * nb * 16 + (size_t)unit * 128 + (size_t)ch * 16; }
// scale tile (8 rows) a lane group fetches: past the tensor's last tile, the last
PG_HD int pg_gskinny_scale_tile(int n0, int lane, int ntile) {
    const int t = (n0 >> 3) + (lane >> 3);
    return t < ntile ? t : ntile - 1;
}
PG_HD size_t pg_gskinny_scale_offset(int tile, int nb, int unit, int lane) { return ((size_t)tile * nb + (lane & 7)) * 16 + (size_t)unit * 128; }

// ---- MXFP4 rows (mxfp4_rows_kernel): fragment chunk and scale word a wavefront fetches for chunk index c
PG_HD int pg_mx_chunk(int c, int ncp) { return c < ncp ? c : ncp - 1; }
PG_HD int pg_mx_scale_word(int c, int ncp) { return (c < ncp ? c : ncp - 4) >> 2; }

// ---- MXFP4 over many rows (mxfp4_planes_kernel writes the token records, mxfp4_tiles_kernel reads them and the weights)
// A record = one token group of 16 and one chunk of 128 k: PG_MT_PLANES operand fragments of 2 KiB, then 64 scale dwords.
constexpr int PG_MT_PLANES = 4, PG_MT_FRAG = 2048, PG_MT_RECORD = PG_MT_PLANES * PG_MT_FRAG + 256, PG_MT_NW = 8;
// chunks a row of nb blocks is padded to: whole scale dwords (4 chunks of 4 blocks)
PG_HD size_t pg_mx_chunks(size_t nb) { return ((nb + 3) / 4 + 3) & ~(size_t)3; }
// first of the `ra` row groups a wavefront reads, from the first one it owns: past the tensor's end it repeats the last ones
PG_HD int pg_mt_first_row_group(int rg_mine, int ra, int nrg) { return rg_mine + ra <= nrg ? rg_mine : nrg - ra; }
// the run of chunks a work item covers: `split` of runs of `cps` chunks
PG_HD int pg_mt_run_end(int split, int cps, int ncp) { return split * cps + cps < ncp ? split * cps + cps : ncp; }
// byte offset, from the token tile's first record of chunk 0, of 16-byte unit u of the tile's records of one chunk
// (the tile's records of a chunk lie ncp records apart; spare threads repeat the last unit)
PG_HD unsigned pg_mt_unit_offset(int u, int units, int ncp) {
    u = u < units ? u : units - 1;
    return (unsigned)(u / (PG_MT_RECORD / 16)) * (unsigned)ncp * PG_MT_RECORD + (unsigned)(u % (PG_MT_RECORD / 16)) * 16;
}
// byte offset of the 16 bytes of plane j that hold k = 32 (b % 4) + 16 sub .. + 15 of chunk b / 4 for token `col` of group tg
PG_HD size_t pg_mt_plane_store(size_t tg, int ncp, int b, int sub, int col, int j) {
    const int k0 = 32 * (b & 3) + 16 * sub, half = k0 >> 6, q = (k0 & 63) >> 4;
    return (tg * ncp + (size_t)(b >> 2)) * PG_MT_RECORD + (size_t)j * PG_MT_FRAG + half * 1024 + (col + 16 * q) * 16;
}
// byte offset of the scale dword of block b for token `col` of group tg
PG_HD size_t pg_mt_scale_store(size_t tg, int ncp, int b, int col) {
    return (tg * ncp + (size_t)(b >> 2)) * PG_MT_RECORD + (size_t)PG_MT_PLANES * PG_MT_FRAG + (size_t)(col + 16 * (b & 3)) * 4;
}

// ---- many rows on the f16 matrix cores (gguf_hmm_kernel): per stage of two blocks a wavefront fills its share
// of the two activation planes, of the packed weights and of their scales
// activation or weight row a fill lane fetches: rows past the end repeat the last (their outputs are never stored)
PG_HD int pg_hmm_clamp_row(int row, int rows) { return row < rows ? row : rows - 1; }
// byte offset in an f16 plane [rows][k]: row, stage (64 k = 128 bytes), 16-byte chunk of the stage's run
PG_HD size_t pg_hmm_plane_offset(int row, int k, int stage, int chunk) { return ((size_t)row * k + (size_t)stage * 64) * 2 + (size_t)chunk * 16; }
// byte offset of a 16-byte block in the Q4_0 payload plane [rows][nb]: block `blk` (0 or 1) of the stage
PG_HD size_t pg_hmm_weight_offset(int row, int nb, int stage, int blk) { return ((size_t)row * nb + (size_t)stage * 2 + blk) * 16; }
// the same in the Q8_0 payload plane [rows][2 halves][nb]
PG_HD size_t pg_hmm_weight_offset_q8(int row, int half, int nb, int stage, int blk) { return (((size_t)row * 2 + half) * nb + (size_t)stage * 2 + blk) * 16; }
// the scale fill takes two neighbouring rows (4 bytes): the even row it starts at; past the end, the last even row
// (the scale plane is padded to a multiple of 8 rows)
PG_HD int pg_hmm_scale_row(int row, int rows) { return row < rows ? row : (rows - 1) & ~1; }
// byte offset in the scale plane (8 rows x f16 per block and tile of 8 rows)
PG_HD size_t pg_hmm_scale_offset(int row, int nb, int stage, int blk) { return (((size_t)(row >> 3) * nb + (size_t)stage * 2 + blk) * 8 + (row & 7)) * 2; }
