// Threefry-2x32, 20 rounds: the counter-based block function behind JAX's PRNG.
// out0, out1 = threefry(key0, key1, x0, x1) element by element; a scalar key is shared by all
// elements. 16 bytes per lane on each side when the length allows; pure integer ALU work,
// bandwidth-bound. Supersedes vkjax/shaders/threefry2x32.comp (reference: vkjax/ops.py:550-560,
// vkjax/shaders/threefry2x32.comp:38-91).
#include "common.h"

struct ThreefryParams { uint32_t n, key_is_scalar; };

__device__ __forceinline__ uint32_t rotl32(uint32_t v, uint32_t d) { return (v << d) | (v >> (32u - d)); }

__device__ __forceinline__ void threefry_block(uint32_t k0, uint32_t k1, uint32_t& x0, uint32_t& x1) {
    const uint32_t ks[3] = {k0, k1, k0 ^ k1 ^ 0x1BD11BDAu};
    const uint32_t rot[2][4] = {{13, 15, 26, 6}, {17, 29, 16, 24}};
    x0 += ks[0];
    x1 += ks[1];
#pragma unroll
    for (uint32_t i = 0; i < 5; ++i) {
#pragma unroll
        for (uint32_t r = 0; r < 4; ++r) {
            x0 += x1;
            x1 = rotl32(x1, rot[i & 1][r]);
            x1 ^= x0;
        }
        x0 += ks[(i + 1) % 3];
        x1 += ks[(i + 2) % 3] + (i + 1);
    }
}

template <int VEC>
__device__ __forceinline__ void threefry_body(uint32_t* __restrict__ out0, uint32_t* __restrict__ out1,
                                              const uint32_t* __restrict__ key0, const uint32_t* __restrict__ key1,
                                              const uint32_t* __restrict__ in0, const uint32_t* __restrict__ in1,
                                              const ThreefryParams& P) {
    const uint64_t e = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * VEC;
    if (e >= P.n) return;
    uint32_t a[VEC], b[VEC], ka[VEC], kb[VEC];
    if constexpr (VEC == 4) {
        const u32x4 va = *reinterpret_cast<const u32x4*>(in0 + e), vb = *reinterpret_cast<const u32x4*>(in1 + e);
        a[0] = va.x; a[1] = va.y; a[2] = va.z; a[3] = va.w;
        b[0] = vb.x; b[1] = vb.y; b[2] = vb.z; b[3] = vb.w;
    } else {
        a[0] = in0[e]; b[0] = in1[e];
    }
    if (P.key_is_scalar) {
        const uint32_t s0 = key0[0], s1 = key1[0];
#pragma unroll
        for (int j = 0; j < VEC; ++j) { ka[j] = s0; kb[j] = s1; }
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) { ka[j] = key0[e + j]; kb[j] = key1[e + j]; }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) threefry_block(ka[j], kb[j], a[j], b[j]);
    if constexpr (VEC == 4) {
        u32x4 va, vb;
        va.x = a[0]; va.y = a[1]; va.z = a[2]; va.w = a[3];
        vb.x = b[0]; vb.y = b[1]; vb.z = b[2]; vb.w = b[3];
        *reinterpret_cast<u32x4*>(out0 + e) = va;
        *reinterpret_cast<u32x4*>(out1 + e) = vb;
    } else {
        out0[e] = a[0]; out1[e] = b[0];
    }
}

extern "C" __global__ __launch_bounds__(256) void threefry2x32_v1(uint32_t* out0, uint32_t* out1, const uint32_t* key0, const uint32_t* key1,
                                                                  const uint32_t* in0, const uint32_t* in1, ThreefryParams P) {
    threefry_body<1>(out0, out1, key0, key1, in0, in1, P);
}
// requires n % 4 == 0 and 16-byte aligned data pointers
extern "C" __global__ __launch_bounds__(256) void threefry2x32_v4(uint32_t* out0, uint32_t* out1, const uint32_t* key0, const uint32_t* key1,
                                                                  const uint32_t* in0, const uint32_t* in1, ThreefryParams P) {
    threefry_body<4>(out0, out1, key0, key1, in0, in1, P);
}
