// Threefry-2x32, 20 rounds: the counter-based block function behind JAX's PRNG.
// out0, out1 = threefry(key0, key1, x0, x1) element by element; a scalar key is shared by all
// elements. 16 bytes per lane on each side when the length allows; pure integer ALU work,
// bandwidth-bound. Supersedes vkjax/shaders/threefry2x32.comp (reference: vkjax/ops.py:550-560,
// vkjax/shaders/threefry2x32.comp:38-91).
#include "ew_apply.h"

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

// SCALAR_KEY: one key for all elements (what jax.random passes), fetched through the scalar cache; else a key per
// element. Two kernels rather than a run-time switch: with both paths in one body the compiler keeps the per-element
// keys in vector registers and the scalar-key case, the usual one, ran at 4.8-5.2 TB/s instead of 5.7.
template <int VEC, bool SCALAR_KEY>
__device__ __forceinline__ void threefry_body(uint32_t* __restrict__ out0, uint32_t* __restrict__ out1,
                                              const uint32_t* __restrict__ key0, const uint32_t* __restrict__ key1,
                                              const uint32_t* __restrict__ in0, const uint32_t* __restrict__ in1,
                                              const ThreefryParams& P) {
    const uint64_t e = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * VEC;
    if (e >= P.n) return;
    uint32_t a[VEC], b[VEC], ka[VEC], kb[VEC];
    if constexpr (VEC == 4) {
        // counters in, random words out: every byte is touched once (nontemporal accesses)
        const u32x4 va = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(in0 + e)),
                    vb = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(in1 + e));
        a[0] = va.x; a[1] = va.y; a[2] = va.z; a[3] = va.w;
        b[0] = vb.x; b[1] = vb.y; b[2] = vb.z; b[3] = vb.w;
    } else {
        a[0] = in0[e]; b[0] = in1[e];
    }
    if constexpr (SCALAR_KEY) {
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
        __builtin_nontemporal_store(va, reinterpret_cast<u32x4*>(out0 + e));
        __builtin_nontemporal_store(vb, reinterpret_cast<u32x4*>(out1 + e));
    } else {
        out0[e] = a[0]; out1[e] = b[0];
    }
}

#define THREEFRY_KERNEL(name, VEC, SCALAR_KEY)                                                                                   \
    extern "C" __global__ __launch_bounds__(256) void name(uint32_t* out0, uint32_t* out1, const uint32_t* key0, const uint32_t* key1, \
                                                           const uint32_t* in0, const uint32_t* in1, ThreefryParams P) {          \
        threefry_body<VEC, SCALAR_KEY>(out0, out1, key0, key1, in0, in1, P);                                                       \
    }
THREEFRY_KERNEL(threefry2x32_v1, 1, false)
THREEFRY_KERNEL(threefry2x32_k_v1, 1, true)
// the _v4 kernels require n % 4 == 0 and 16-byte aligned data pointers
THREEFRY_KERNEL(threefry2x32_v4, 4, false)
THREEFRY_KERNEL(threefry2x32_k_v4, 4, true)

// ---------------------------------------------------------------------------------------------
// The whole random-bits pipeline in one pass. JAX (legacy counter layout) draws 2h words as
//     c = iota(2h);  a, b = threefry2x32(key, c[:h], c[h:]);  bits = concatenate(a, b)
// and then maps the bits through a chain of element-wise steps with scalar operands
// (uniform: bits >> 9 | 0x3F800000, bitcast, - 1, * (max - min), + min, max(min, .)).
// Here every thread generates its counters in registers (x0 = c0 + j, x1 = c1 + j), runs the block
// function, applies the chain to both results and writes element j and element h + j of the final
// array: 4 bytes written per element and nothing read, instead of twelve full-size passes.
#define TF_MAX_STEPS 8

struct ThreefryStreamParams {
    uint32_t h;                        // blocks to run (halves layout: the output has up to 2h elements)
    uint32_t c0, c1;                   // first counter of each word
    uint32_t nsteps;                   // element-wise steps applied to the bits (0..8)
    uint32_t op[TF_MAX_STEPS];         // opcode of step k
    uint32_t flags[TF_MAX_STEPS];      // bit0: the step has an operand (a single value); bit1: it is the LEFT argument
    uint32_t imm[TF_MAX_STEPS];        // immediate of step k (integer_pow exponent)
    uint32_t n;                        // halves layout: elements of the output (2h, or 2h - 1 for an odd-sized draw)
};

struct ThreefryStreamPtrs { const uint32_t* p[TF_MAX_STEPS]; };

// Counter layouts of the stream kernels:
//   HALVES  x0 = c0 + j, x1 = c1 + j;  out[j] = y0, out[h + j] = y1      (jax's original layout; an
//           odd-sized draw pads the counters with one zero and drops the last result, so the x1
//           counter of element n is 0 and that element is not stored)
//   XOR     x0 = c0, x1 = c1 + j;      out[j] = y0 ^ y1                   (jax's partitionable layout:
//           the 64-bit flat index of the element is the counter, 32 bits per word)
//   PAIRS   x0 = c0, x1 = c1 + j;      out[2j] = y0, out[2j + 1] = y1     (partitionable key split)
enum { TF_HALVES = 0, TF_XOR = 1, TF_PAIRS = 2 };

// Applies the element-wise steps to y. The step loop stays rolled (one copy of the opcode switch).
// Its descriptors are read from the argument block through the kernel-argument pointer: indexing
// the by-value argument with a run-time value would make the compiler copy it to scratch memory.
// Layout of the block: out, key0, key1 (24 bytes), the operand pointers (64 bytes), then
// ThreefryStreamParams.
template <int NV>
__device__ __forceinline__ void threefry_stream_steps(uint32_t (&y)[NV], uint32_t nsteps) {
    const char* const args = reinterpret_cast<const char*>(__builtin_amdgcn_kernarg_segment_ptr());
    const uint32_t* const* const op_ptr = reinterpret_cast<const uint32_t* const*>(args + 24);
    const uint32_t* const desc = reinterpret_cast<const uint32_t*>(args + 24 + 8 * TF_MAX_STEPS) + 4;
#pragma nounroll
    for (uint32_t k = 0; k < nsteps; ++k) {
        const uint32_t op = desc[k], flags = desc[TF_MAX_STEPS + k], imm = desc[2 * TF_MAX_STEPS + k];
        const uint32_t o = (flags & 1u) ? op_ptr[k][0] : 0u;                  // uniform address: a scalar load
        uint32_t v[NV];
#pragma unroll
        for (int j = 0; j < NV; ++j) v[j] = o;
        ew_apply_vec<NV>(op, y, v, (flags & 2u) != 0, imm);
    }
}

// The chain of jax.random.uniform, known at compile time: the opcode switch folds away and the six
// single-value operands are fetched before the block function runs instead of one dependent pair
// of scalar loads per step. (bits >> 9 | 0x3F800000, as float - 1, * (max - min), + min, max(min, .))
// With the operands of a draw from [0, 1) -- shift 9, exponent bits of 1.0, minus 1.0, times 1.0, plus 0.0,
// max(0.0, .) -- the first two steps are one funnel shift ((0x7F : bits) >> 9 puts 0x3F800000 above the 23
// mantissa bits) and the last three change no bit: the value after the subtraction lies in [+0, 1), where
// x * 1.0, x + 0.0 and max(0.0, x) all return x itself. Two operations per word instead of eight.
template <int NV>
__device__ __forceinline__ void threefry_uniform_steps(uint32_t (&y)[NV], const uint32_t (&o)[6]) {
    const bool unit_interval = o[0] == 9u && o[1] == 0x3F800000u && o[2] == 0x3F800000u && o[3] == 0x3F800000u && o[4] == 0u && o[5] == 0u;
    if (unit_interval) {                             // the same for every thread of the launch
#pragma unroll
        for (int j = 0; j < NV; ++j) y[j] = f2u(u2f(__builtin_amdgcn_alignbit(0x7Fu, y[j], 9u)) - 1.0f);
        return;
    }
    constexpr uint32_t ops[6] = {EW_SHR_L, EW_OR_X, EW_SUB_F, EW_MUL_F, EW_ADD_F, EW_MAX_F};
#pragma unroll
    for (int k = 0; k < 6; ++k) {
        uint32_t v[NV];
#pragma unroll
        for (int j = 0; j < NV; ++j) v[j] = o[k];
        ew_apply_vec<NV>(ops[k], y, v, k == 5, 0u);
    }
}

template <int VEC, int MODE, bool UNIFORM = false>
__device__ __forceinline__ void threefry_stream_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ key0,
                                                     const uint32_t* __restrict__ key1, const ThreefryStreamParams& P) {
    const uint32_t j0 = (blockIdx.x * 256u + threadIdx.x) * VEC;
    if (j0 >= P.h) return;
    const uint32_t k0 = key0[0], k1 = key1[0];
    uint32_t o[6] = {};
    if constexpr (UNIFORM) {
        const char* const args = reinterpret_cast<const char*>(__builtin_amdgcn_kernarg_segment_ptr());
        const uint32_t* const* const op_ptr = reinterpret_cast<const uint32_t* const*>(args + 24);
#pragma unroll
        for (int k = 0; k < 6; ++k) o[k] = op_ptr[k][0];
    }
    if constexpr (MODE == TF_HALVES) {
        uint32_t y[2 * VEC];                         // [0, VEC): first results, [VEC, 2 VEC): second results
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            y[j]       = P.c0 + j0 + j;
            y[VEC + j] = P.c1 + j0 + j;
            if (VEC == 1 && P.h + j0 >= P.n) y[VEC] = 0u;           // the padding counter of an odd-sized draw
            threefry_block(k0, k1, y[j], y[VEC + j]);
        }
        if constexpr (UNIFORM) threefry_uniform_steps<2 * VEC>(y, o);
        else threefry_stream_steps<2 * VEC>(y, P.nsteps);
        if constexpr (VEC == 4) {
            u32x4 va, vb;
            va.x = y[0]; va.y = y[1]; va.z = y[2]; va.w = y[3];
            vb.x = y[4]; vb.y = y[5]; vb.z = y[6]; vb.w = y[7];
            *reinterpret_cast<u32x4*>(out + j0) = va;
            *reinterpret_cast<u32x4*>(out + P.h + j0) = vb;
        } else {
            out[j0] = y[0];
            if (P.h + j0 < P.n) out[P.h + j0] = y[1];
        }
    } else {
        uint32_t y[VEC], z[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            y[j] = P.c0;
            z[j] = P.c1 + j0 + j;
            threefry_block(k0, k1, y[j], z[j]);
        }
        if constexpr (MODE == TF_PAIRS) {
            static_assert(VEC == 1, "pairs are written one block per thread");
            out[2 * j0] = y[0]; out[2 * j0 + 1] = z[0];
        } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) y[j] ^= z[j];
            if constexpr (UNIFORM) threefry_uniform_steps<VEC>(y, o);
            else threefry_stream_steps<VEC>(y, P.nsteps);
            if constexpr (VEC == 4) {
                u32x4 va;
                va.x = y[0]; va.y = y[1]; va.z = y[2]; va.w = y[3];
                *reinterpret_cast<u32x4*>(out + j0) = va;
            } else {
                out[j0] = y[0];
            }
        }
    }
}

#define TF_STREAM_KERNEL(name, VEC, MODE, ...)                                                                         \
    extern "C" __global__ __launch_bounds__(256) void name(uint32_t* out, const uint32_t* key0, const uint32_t* key1,  \
                                                           ThreefryStreamPtrs operands, ThreefryStreamParams P) {      \
        threefry_stream_body<VEC, MODE, ##__VA_ARGS__>(out, key0, key1, P);                                            \
    }
TF_STREAM_KERNEL(threefry2x32_stream_v1, 1, TF_HALVES)
TF_STREAM_KERNEL(threefry2x32_stream_v4, 4, TF_HALVES)          // requires h % 4 == 0, n == 2h and a 16-byte aligned output
TF_STREAM_KERNEL(threefry2x32_stream_xor_v1, 1, TF_XOR)
TF_STREAM_KERNEL(threefry2x32_stream_xor_v4, 4, TF_XOR)         // requires h % 4 == 0 and a 16-byte aligned output
TF_STREAM_KERNEL(threefry2x32_stream_pairs_v1, 1, TF_PAIRS)
// the steps are exactly jax.random.uniform's chain, every step with an operand (see threefry_uniform_steps)
TF_STREAM_KERNEL(threefry2x32_stream_uniform_v4, 4, TF_HALVES, true)
TF_STREAM_KERNEL(threefry2x32_stream_xor_uniform_v4, 4, TF_XOR, true)

