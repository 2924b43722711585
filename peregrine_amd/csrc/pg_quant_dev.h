// Device helpers of the activation quantisation, shared by the row kernels (pg_quant.hip) and the
// one-row product that quantises its own activations (pg_gemv_w8a8.hip).
#pragma once
#include <hip/hip_runtime.h>

// round -> clamp(-127,127) -> `as i8` (NaN -> 0), returned as int.   src/quant.rs:101-106
__device__ __forceinline__ int pg_quant_to_i8(float v) {
    float r = roundf(v);
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (r != r || v != v) ? 0 : (int)r;
}

__device__ __forceinline__ float pg_wave_max_f32(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Maximum over a 256-thread workgroup; `red` = 4 floats of LDS.  Ends with every thread past a barrier.
__device__ __forceinline__ float pg_block_max_256(float v, float *red) {
    v = pg_wave_max_f32(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    v = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    return v;
}

// The same without draining the wavefront's outstanding global loads (__syncthreads() waits for
// vmcnt(0) as well): for kernels that keep weight rows in flight across the reduction.
__device__ __forceinline__ float pg_block_max_256_keep_loads(float v, float *red) {
    v = pg_wave_max_f32(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    asm volatile("s_waitcnt lgkmcnt(0)\n s_barrier" ::: "memory");
    v = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    return v;
}
