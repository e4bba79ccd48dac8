// Shared device helpers for the vkJAX gfx950 kernels (wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef float    f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float    f32x16 __attribute__((ext_vector_type(16)));

#define VKJ_WAVE 64

__device__ __forceinline__ uint32_t f2u(float x) { return __float_as_uint(x); }
__device__ __forceinline__ float    u2f(uint32_t x) { return __uint_as_float(x); }

// Butterfly reductions across the 64 lanes of a wave.
template <class T, class F>
__device__ __forceinline__ T wave_allreduce(T v, F f) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = f(v, __shfl_xor(v, off, VKJ_WAVE));
    return v;
}
