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

// Buffer-descriptor access: loads beyond `bytes` return 0 and stores there are dropped, so a lane
// that must not touch memory is given an offset of 0x80000000.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
// voff: per-lane byte offset, soff: wave-uniform byte offset; the range check covers their sum
__device__ __forceinline__ f32x4 buffer_load_x4(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff = 0) {
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
__device__ __forceinline__ float buffer_load_x1(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff = 0) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
__device__ __forceinline__ void buffer_store_x1(float v, __amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff = 0) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), r, voff, soff, 0);
}
// the same for data that is touched once (nontemporal: not kept in the caches at the expense of what is reused)
__device__ __forceinline__ float buffer_load_x1_nt(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff = 0) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 2));
}
// Bit 31 of the first word of a kernel's parameters (an element count below 2^31 in every kernel that looks at it):
// the result is stored with the nontemporal hint. The host sets it for large results that no later launch of the
// program reads (they leave for the host, or stay where they are): such an array only pushes out of the caches what
// could be reused, and the stores of a launch that reads and writes run faster past the L2 (relu on 64 M elements
// 92 -> 76 us). Results that the next launch reads are left to the caches (256 MB behind the L2s: a training step
// whose backward kernels streamed their results was 0.15 ms slower). Only for results below 4 GiB (a buffer
// addresses 32 bits); the host checks.
#define STREAM_RESULT_BIT 0x80000000u
__device__ __forceinline__ bool streams_result(uint32_t first_word) { return (first_word & STREAM_RESULT_BIT) != 0u; }
__device__ __forceinline__ uint32_t without_stream_bit(uint32_t first_word) { return first_word & ~STREAM_RESULT_BIT; }
// base[element .. element + 4) = v; `stream`: past the caches. (Through a buffer: written as two stores through one
// pointer, one of them nontemporal, the compiler merges them into one plain store.)
__device__ __forceinline__ void store_x4(uint32_t* base, uint64_t element, u32x4 v, bool stream, uint32_t result_bytes) {
    if (stream) __builtin_amdgcn_raw_buffer_store_b128(v, make_rsrc(base, result_bytes), (uint32_t)element * 4u, 0, 2);
    else *reinterpret_cast<u32x4*>(base + element) = v;
}
__device__ __forceinline__ int magic_div(int n, uint32_t magic, uint32_t shift) {
    return magic ? (int)(__umulhi((uint32_t)n, magic) >> shift) : n;
}

// Consecutive workgroup ids are handed to the 8 XCDs in turn, and every XCD has an L2 of its own.
// This renumbers the workgroups of a 1-D grid so that each XCD works through a contiguous range:
// kernels whose neighbouring workgroups read overlapping data (windows, halos) then find the
// overlap in their own L2 instead of fetching it once per XCD. A bijection on [0, gridDim.x).
__device__ __forceinline__ uint32_t xcd_contiguous_block() {
    const uint32_t b = blockIdx.x, per = gridDim.x / 8u;
    return (per > 0u && b < per * 8u) ? (b & 7u) * per + (b >> 3) : b;
}
