// Device math used by the elementwise / softmax / norm kernels: the libm-level routines (rt_libm.h, shared with the host
// check), 16-bit helpers and the wave / row reductions.  Compile with -ffp-contract=off.
#ifndef RT_MATH_H
#define RT_MATH_H

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

#define RT_FN __device__ inline
#define RT_TABLE __device__ static const
#include "rt_libm.h"
#undef RT_FN
#undef RT_TABLE

// ---- 16-bit helpers -------------------------------------------------------------------------------------
__device__ __forceinline__ float h2f(half_t h) { return (float)h; }
__device__ __forceinline__ half_t f2h(float f) { return (half_t)f; }              // round to nearest even
__device__ __forceinline__ uint16_t h_bits(half_t h) { return __builtin_bit_cast(uint16_t, h); }
__device__ __forceinline__ half_t bits_h(uint16_t u) { return __builtin_bit_cast(half_t, u); }

// ---- wave64 reductions ----------------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Reduction over the LANES threads that share a row: a group of 2..64 neighbouring lanes of a wave (a butterfly over the
// group; LANES == 64 is the whole wave), or a whole 256-thread block, whose four wave results meet in LDS and are added
// in a fixed order.  Every thread of the block must call the block form.
template <int LANES> __device__ __forceinline__ float row_sum(float v) {
    if constexpr (LANES <= 64) {
#pragma unroll
        for (int off = LANES / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    } else {
        v = wave_sum(v);
        __shared__ float red[LANES / 64];
        __syncthreads();                                   // earlier readers of red are done
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
        __syncthreads();
        v = red[0];
#pragma unroll
        for (int w = 1; w < LANES / 64; w++) v += red[w];
    }
    return v;
}
template <int LANES> __device__ __forceinline__ float row_max(float v) {
    if constexpr (LANES <= 64) {
#pragma unroll
        for (int off = LANES / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    } else {
        v = wave_max(v);
        __shared__ float red[LANES / 64];
        __syncthreads();
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
        __syncthreads();
        v = red[0];
#pragma unroll
        for (int w = 1; w < LANES / 64; w++) v = fmaxf(v, red[w]);
    }
    return v;
}

#endif
