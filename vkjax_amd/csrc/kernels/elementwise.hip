// Element-wise chain kernel: one launch evaluates a linear chain of up to 8 element-wise
// steps over an output of up to 4 (collapsed) dimensions. Every step may bring one more
// operand, read through per-dimension strides so that broadcasts (stride 0), slices,
// transposes and reversals are addressed in place instead of being materialised.
//
// It supersedes the reference's one-thread-per-element GLSL kernels add/sub/mul/div/max/min/
// gt/ge/lt/le/eq/ne/and/or/rem/pow/shift_*.comp, exp/log/neg/abs/rsqrt/erf/erf_inv/unary_op.comp,
// select.comp, convert_element_type.comp, broadcast_in_dim.comp, slice.comp, transpose.comp,
// rev.comp, integer_pow.comp, nextafter.comp (reference: vkjax/ops.py:73-215, 338-347, 435-442,
// 491-502, 527-547, 563-566). Bandwidth-bound: each operand element is read once and the
// result written once, 16 bytes per lane when the layout allows.
#include "common.h"

#define EW_MAX_STEPS 8

enum EwOp : uint32_t {
#define EW_OP(name, num) EW_##name = num,
#include "ew_opcodes.h"
#undef EW_OP
};

struct EwParams {
    uint32_t n;                        // output elements
    uint32_t ndim;                     // 1..4 collapsed output dims
    uint32_t dims[4];                  // row-major, dims[ndim-1] fastest; unused = 1
    uint32_t nsteps;                   // 1..8; step 0 is the initial load
    uint32_t op[EW_MAX_STEPS];         // opcode of step k (op[0] ignored)
    uint32_t flags[EW_MAX_STEPS];      // bit0: step has an operand; bit1: operand is the LEFT argument
    uint32_t imm[EW_MAX_STEPS];        // immediate (integer_pow exponent)
    int32_t  stride[EW_MAX_STEPS][4];  // operand strides per collapsed dim, in elements
};

__device__ __forceinline__ uint32_t ipow_f(uint32_t xb, int32_t y) {
    float x = u2f(xb), acc = 1.0f;
    uint32_t e = y < 0 ? (uint32_t)(-(int64_t)y) : (uint32_t)y;
    while (e) { if (e & 1) acc *= x; x *= x; e >>= 1; }
    return f2u(y < 0 ? 1.0f / acc : acc);
}

__device__ __forceinline__ uint32_t ipow_i(uint32_t x, int32_t y) {
    uint32_t acc = 1, e = (uint32_t)y;
    while (e) { if (e & 1) acc *= x; x *= x; e >>= 1; }
    return acc;
}

// Transcendentals and other rarely used opcodes live out of line so that the unrolled
// step loop stays small.
__device__ __noinline__ uint32_t ew_apply_rare(uint32_t op, uint32_t a, uint32_t b, uint32_t imm) {
    const float x = u2f(a), y = u2f(b);
    switch (op) {
        case EW_POW_F:       return f2u(powf(x, y));
        case EW_REM_F:       return f2u(fmodf(x, y));
        case EW_NEXTAFTER_F: return f2u(nextafterf(x, y));
        case EW_LOG_F:       return f2u(logf(x));
        case EW_SQRT_F:      return f2u(sqrtf(x));
        case EW_CEIL_F:      return f2u(ceilf(x));
        case EW_FLOOR_F:     return f2u(floorf(x));
        case EW_IPOW_F:      return ipow_f(a, (int32_t)imm);
        case EW_IPOW_I:      return ipow_i(a, (int32_t)imm);
        case EW_ERF_F:       return f2u(erff(x));
        case EW_ERFINV_F:    return f2u(erfinvf(x));
        case EW_COS_F:       return f2u(cosf(x));
        case EW_SIN_F:       return f2u(sinf(x));
        case EW_TAN_F:       return f2u(tanf(x));
        case EW_COSH_F:      return f2u(coshf(x));
        case EW_SINH_F:      return f2u(sinhf(x));
        case EW_TANH_F:      return f2u(tanhf(x));
        case EW_ACOS_F:      return f2u(acosf(x));
        case EW_ASIN_F:      return f2u(asinf(x));
        case EW_ATAN_F:      return f2u(atanf(x));
        case EW_ACOSH_F:     return f2u(acoshf(x));
        case EW_ASINH_F:     return f2u(asinhf(x));
        case EW_ATANH_F:     return f2u(atanhf(x));
        case EW_DIV_I: { int32_t p = (int32_t)a, q = (int32_t)b;
                         return q == 0 ? 0xFFFFFFFFu : (p == INT32_MIN && q == -1) ? (uint32_t)INT32_MIN : (uint32_t)(p / q); }
        case EW_DIV_U:       return b == 0 ? 0xFFFFFFFFu : a / b;
        case EW_REM_I: { int32_t p = (int32_t)a, q = (int32_t)b;
                         return q == 0 ? a : (q == -1) ? 0u : (uint32_t)(p % q); }
        case EW_REM_U:       return b == 0 ? a : a % b;
        default:             return a;
    }
}

// a = left argument, b = right argument.
__device__ __forceinline__ uint32_t ew_apply(uint32_t op, uint32_t a, uint32_t b, uint32_t imm) {
    const float x = u2f(a), y = u2f(b);
    const int32_t p = (int32_t)a, q = (int32_t)b;
    switch (op) {
        case EW_NOP:     return a;
        case EW_ADD_F:   return f2u(x + y);
        case EW_SUB_F:   return f2u(x - y);
        case EW_MUL_F:   return f2u(x * y);
        case EW_DIV_F:   return f2u(x / y);
        case EW_MAX_F:   return (x > y || x != x) ? a : b;      // NaN wins, as in XLA
        case EW_MIN_F:   return (x < y || x != x) ? a : b;
        case EW_ADD_I:   return a + b;
        case EW_SUB_I:   return a - b;
        case EW_MUL_I:   return a * b;
        case EW_MAX_I:   return p > q ? a : b;
        case EW_MIN_I:   return p < q ? a : b;
        case EW_MAX_U:   return a > b ? a : b;
        case EW_MIN_U:   return a < b ? a : b;
        case EW_AND_X:   return a & b;
        case EW_OR_X:    return a | b;
        case EW_XOR_X:   return a ^ b;
        case EW_SHL_X:   return b >= 32 ? 0u : a << b;
        case EW_SHR_L:   return b >= 32 ? 0u : a >> b;
        case EW_SHR_A:   return (uint32_t)(p >> (b >= 32 ? 31u : b));
        case EW_GT_F:    return x >  y;
        case EW_GE_F:    return x >= y;
        case EW_LT_F:    return x <  y;
        case EW_LE_F:    return x <= y;
        case EW_EQ_F:    return x == y;
        case EW_NE_F:    return x != y;
        case EW_GT_I:    return p >  q;
        case EW_GE_I:    return p >= q;
        case EW_LT_I:    return p <  q;
        case EW_LE_I:    return p <= q;
        case EW_EQ_X:    return a == b;
        case EW_NE_X:    return a != b;
        case EW_GT_U:    return a >  b;
        case EW_GE_U:    return a >= b;
        case EW_LT_U:    return a <  b;
        case EW_LE_U:    return a <= b;
        case EW_NEG_F:   return a ^ 0x80000000u;
        case EW_ABS_F:   return a & 0x7FFFFFFFu;
        case EW_SIGN_F:  return x > 0.f ? f2u(1.0f) : x < 0.f ? f2u(-1.0f) : a;
        case EW_NEG_I:   return 0u - a;
        case EW_ABS_I:   return p < 0 ? 0u - a : a;
        case EW_SIGN_I:  return (uint32_t)((p > 0) - (p < 0));
        case EW_EXP_F:   return f2u(expf(x));
        case EW_RSQRT_F: return f2u(1.0f / sqrtf(x));
        case EW_CVT_F2I: return (uint32_t)(int32_t)x;           // truncates, saturates, NaN -> 0
        case EW_CVT_F2U: return (uint32_t)x;
        case EW_CVT_I2F: return f2u((float)p);
        case EW_CVT_U2F: return f2u((float)a);
        case EW_CVT_F2B: return x != 0.f;
        case EW_CVT_X2B: return a != 0u;
        default:         return ew_apply_rare(op, a, b, imm);
    }
}

template <int VEC> struct EwVec;
template <> struct EwVec<1> { uint32_t v[1]; };
template <> struct EwVec<4> { uint32_t v[4]; };

template <int VEC>
__device__ __forceinline__ void ew_load(uint32_t (&dst)[VEC], const uint32_t* __restrict__ p, int64_t idx, int32_t last_stride) {
    if constexpr (VEC == 4) {
        if (last_stride == 1) {
            const u32x4 t = *reinterpret_cast<const u32x4*>(p + idx);
            dst[0] = t.x; dst[1] = t.y; dst[2] = t.z; dst[3] = t.w;
        } else {                                   // stride 0 along the vector: one value, splat
            const uint32_t t = p[idx];
            dst[0] = dst[1] = dst[2] = dst[3] = t;
        }
    } else {
        dst[0] = p[idx];
    }
}

template <int VEC>
__device__ __forceinline__ void ew_chain_body(uint32_t* __restrict__ out, const uint32_t* const (&in)[EW_MAX_STEPS],
                                              const EwParams& P) {
    const uint32_t v = blockIdx.x * 256u + threadIdx.x;
    const uint64_t i0 = (uint64_t)v * VEC;
    if (i0 >= P.n) return;

    // coordinates of the first element of this vector in the collapsed output space
    uint32_t c[4] = {0, 0, 0, 0};
    {
        uint32_t r = (uint32_t)i0;
        if (P.ndim > 1) {
#pragma unroll
            for (int d = 3; d >= 1; --d) {
                if (d < (int)P.ndim) { const uint32_t q = r / P.dims[d]; c[d] = r - q * P.dims[d]; r = q; }
            }
        }
        c[0] = r;
    }
    const int last = (int)P.ndim - 1;

    uint32_t vals[EW_MAX_STEPS][VEC];
#pragma unroll
    for (int k = 0; k < EW_MAX_STEPS; ++k) {
        if (k < (int)P.nsteps && (P.flags[k] & 1u)) {
            int64_t idx = 0;
#pragma unroll
            for (int d = 0; d < 4; ++d) idx += (int64_t)c[d] * P.stride[k][d];
            ew_load<VEC>(vals[k], in[k], idx, P.stride[k][last]);
        } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) vals[k][j] = 0;
        }
    }

    uint32_t acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = vals[0][j];

#pragma unroll
    for (int k = 1; k < EW_MAX_STEPS; ++k) {
        if (k < (int)P.nsteps) {
            const uint32_t op = P.op[k], imm = P.imm[k];
            if (op >= EW_SEL_P && op <= EW_SEL_F) {
                // three-input select: this step's operand and the next step's operand (a NOP carrier)
                const int k2 = (k + 1 < EW_MAX_STEPS) ? k + 1 : k;
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const uint32_t s = vals[k][j], t = vals[k2][j];
                    acc[j] = op == EW_SEL_P ? (acc[j] ? s : t)       // acc is the predicate
                           : op == EW_SEL_T ? (s ? acc[j] : t)       // acc is on_true, s the predicate
                                            : (s ? t : acc[j]);      // acc is on_false, s the predicate
                }
            } else {
                const bool operand_left = (P.flags[k] & 2u) != 0;
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const uint32_t a = operand_left ? vals[k][j] : acc[j];
                    const uint32_t b = operand_left ? acc[j] : vals[k][j];
                    acc[j] = ew_apply(op, a, b, imm);
                }
            }
        }
    }

    if constexpr (VEC == 4) {
        u32x4 t; t.x = acc[0]; t.y = acc[1]; t.z = acc[2]; t.w = acc[3];
        *reinterpret_cast<u32x4*>(out + i0) = t;
    } else {
        out[i0] = acc[0];
    }
}

#define EW_KERNEL(name, VEC)                                                                          \
    extern "C" __global__ __launch_bounds__(256) void name(                                            \
        uint32_t* __restrict__ out, const uint32_t* in0, const uint32_t* in1, const uint32_t* in2,      \
        const uint32_t* in3, const uint32_t* in4, const uint32_t* in5, const uint32_t* in6,             \
        const uint32_t* in7, EwParams P) {                                                              \
        const uint32_t* const in[EW_MAX_STEPS] = {in0, in1, in2, in3, in4, in5, in6, in7};              \
        ew_chain_body<VEC>(out, in, P);                                                                 \
    }

// ew_chain_v4 requires: n % 4 == 0, dims[ndim-1] % 4 == 0, every operand's fastest stride in {0, 1},
// stride-1 operands 16-byte aligned with all slower strides % 4 == 0. The host checks this.
EW_KERNEL(ew_chain_v1, 1)
EW_KERNEL(ew_chain_v4, 4)

struct IotaParams { uint32_t n, inner, size, to_float; };

// out[i] = (i / inner) % size   (reference: vkjax/shaders/iota.comp:8-11 for the 1-D case)
extern "C" __global__ __launch_bounds__(256) void iota_nd(uint32_t* __restrict__ out, IotaParams P) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= P.n) return;
    const uint32_t v = (i / P.inner) % P.size;
    out[i] = P.to_float ? f2u((float)v) : v;
}

struct FillParams { uint32_t n, value; };

extern "C" __global__ __launch_bounds__(256) void fill_u32(uint32_t* __restrict__ out, FillParams P) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < P.n) out[i] = P.value;
}

struct ConcatParams { uint32_t n, part_inner, out_inner, out_offset; };

// One operand of a concatenation: the operand is [outer, part_inner], the output
// [outer, out_inner]; operand row r lands at out[r*out_inner + out_offset ...].
// (reference: vkjax/shaders/concatenate.comp:9-25, two operands on the last axis only)
extern "C" __global__ __launch_bounds__(256) void concat_part(uint32_t* __restrict__ out, const uint32_t* __restrict__ in,
                                                              ConcatParams P) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= P.n) return;
    const uint32_t r = i / P.part_inner, c = i - r * P.part_inner;
    out[(uint64_t)r * P.out_inner + P.out_offset + c] = in[i];
}
