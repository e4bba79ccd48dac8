// The opcode interpreter shared by the kernels that evaluate element-wise steps: one step applies
// one opcode of ew_opcodes.h to an accumulator and (for binary operations) one operand, on raw
// 32-bit words (float, int32, uint32 or a 0/1 boolean, as the opcode implies).
#pragma once
#include "common.h"

enum EwOp : uint32_t {
#define EW_OP(name, num) EW_##name = num,
#include "ew_opcodes.h"
#undef EW_OP
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
        case EW_LOGISTIC_F:  return f2u(1.0f / (1.0f + expf(-x)));
        case EW_LOG1P_F:     return f2u(log1pf(x));
        case EW_EXPM1_F:     return f2u(expm1f(x));
        case EW_EXP2_F:      return f2u(exp2f(x));
        case EW_ISFINITE_F:  return (a & 0x7F800000u) != 0x7F800000u;
        case EW_NOT_X:       return ~a;
        case EW_NOT_B:       return a == 0u;
        case EW_ROUND_AWAY_F: return f2u(roundf(x));           // halves away from zero
        case EW_ROUND_EVEN_F: return f2u(rintf(x));            // halves to even (default rounding mode)
        case EW_ATAN2_F:     return f2u(atan2f(x, y));
        case EW_CBRT_F:      return f2u(cbrtf(x));
        case EW_POPCNT_X:    return (uint32_t)__popc(a);
        case EW_CLZ_X:       return a == 0u ? 32u : (uint32_t)__clz((int)a);
        case EW_DIV_I: { int32_t p = (int32_t)a, q = (int32_t)b;
                         return q == 0 ? 0xFFFFFFFFu : (p == INT32_MIN && q == -1) ? (uint32_t)INT32_MIN : (uint32_t)(p / q); }
        case EW_DIV_U:       return b == 0 ? 0xFFFFFFFFu : a / b;
        case EW_REM_I: { int32_t p = (int32_t)a, q = (int32_t)b;
                         return q == 0 ? a : (q == -1) ? 0u : (uint32_t)(p % q); }
        case EW_REM_U:       return b == 0 ? a : a % b;
        default:             return a;
    }
}

// acc[j] = op(acc[j], v[j]) (or op(v[j], acc[j]) when `left`). The opcode is uniform: one branch
// per step, with the loop over the lanes' VEC elements inside each case.
template <int VEC>
__device__ __forceinline__ void ew_apply_vec(uint32_t op, uint32_t (&acc)[VEC], const uint32_t (&v)[VEC], bool left, uint32_t imm) {
#define EW_CASE(code, expr)                                                        \
    case code:                                                                     \
        _Pragma("unroll") for (int j = 0; j < VEC; ++j) {                          \
            const uint32_t a = left ? v[j] : acc[j], b = left ? acc[j] : v[j];     \
            const float x = u2f(a), y = u2f(b);                                    \
            const int32_t p = (int32_t)a, q = (int32_t)b;                          \
            (void)x; (void)y; (void)p; (void)q;                                    \
            acc[j] = (expr);                                                       \
        }                                                                          \
        break;
    switch (op) {
        EW_CASE(EW_NOP,     a)
        EW_CASE(EW_ADD_F,   f2u(x + y))
        EW_CASE(EW_SUB_F,   f2u(x - y))
        EW_CASE(EW_MUL_F,   f2u(x * y))
        EW_CASE(EW_DIV_F,   f2u(x / y))
        EW_CASE(EW_MAX_F,   (x > y || x != x) ? a : b)      // NaN wins, as in XLA
        EW_CASE(EW_MIN_F,   (x < y || x != x) ? a : b)
        EW_CASE(EW_ADD_I,   a + b)
        EW_CASE(EW_SUB_I,   a - b)
        EW_CASE(EW_MUL_I,   a * b)
        EW_CASE(EW_MAX_I,   p > q ? a : b)
        EW_CASE(EW_MIN_I,   p < q ? a : b)
        EW_CASE(EW_MAX_U,   a > b ? a : b)
        EW_CASE(EW_MIN_U,   a < b ? a : b)
        EW_CASE(EW_AND_X,   a & b)
        EW_CASE(EW_OR_X,    a | b)
        EW_CASE(EW_XOR_X,   a ^ b)
        EW_CASE(EW_SHL_X,   b >= 32 ? 0u : a << b)
        EW_CASE(EW_SHR_L,   b >= 32 ? 0u : a >> b)
        EW_CASE(EW_SHR_A,   (uint32_t)(p >> (b >= 32 ? 31u : b)))
        EW_CASE(EW_GT_F,    x >  y)
        EW_CASE(EW_GE_F,    x >= y)
        EW_CASE(EW_LT_F,    x <  y)
        EW_CASE(EW_LE_F,    x <= y)
        EW_CASE(EW_EQ_F,    x == y)
        EW_CASE(EW_NE_F,    x != y)
        EW_CASE(EW_GT_I,    p >  q)
        EW_CASE(EW_GE_I,    p >= q)
        EW_CASE(EW_LT_I,    p <  q)
        EW_CASE(EW_LE_I,    p <= q)
        EW_CASE(EW_EQ_X,    a == b)
        EW_CASE(EW_NE_X,    a != b)
        EW_CASE(EW_GT_U,    a >  b)
        EW_CASE(EW_GE_U,    a >= b)
        EW_CASE(EW_LT_U,    a <  b)
        EW_CASE(EW_LE_U,    a <= b)
        EW_CASE(EW_NEG_F,   a ^ 0x80000000u)
        EW_CASE(EW_ABS_F,   a & 0x7FFFFFFFu)
        EW_CASE(EW_SIGN_F,  x > 0.f ? f2u(1.0f) : x < 0.f ? f2u(-1.0f) : a)
        EW_CASE(EW_NEG_I,   0u - a)
        EW_CASE(EW_ABS_I,   p < 0 ? 0u - a : a)
        EW_CASE(EW_SIGN_I,  (uint32_t)((p > 0) - (p < 0)))
        EW_CASE(EW_EXP_F,   f2u(expf(x)))
        EW_CASE(EW_RSQRT_F, f2u(1.0f / sqrtf(x)))
        EW_CASE(EW_CVT_F2I, (uint32_t)(int32_t)x)           // truncates, saturates, NaN -> 0
        EW_CASE(EW_CVT_F2U, (uint32_t)x)
        EW_CASE(EW_CVT_I2F, f2u((float)p))
        EW_CASE(EW_CVT_U2F, f2u((float)a))
        EW_CASE(EW_CVT_F2B, x != 0.f)
        EW_CASE(EW_CVT_X2B, a != 0u)
        EW_CASE(EW_WRAP_I,  p < 0 ? a + b : a)
        default:
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                acc[j] = ew_apply_rare(op, left ? v[j] : acc[j], left ? acc[j] : v[j], imm);
            break;
    }
#undef EW_CASE
}

