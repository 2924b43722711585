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
