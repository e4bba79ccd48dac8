// Reductions (sum / prod / max / min, argmax / argmin) and window reductions (max / sum pooling).
//
// reduce_3d views the operand as [outer, R, inner] and reduces R. A block is TI x TR threads
// (TI*TR = 256): TI consecutive `inner` positions times TR interleaved slices of R, so global
// loads are contiguous whichever of the two is the fast axis; slices are combined through LDS.
// reduce_general handles reductions whose kept and reduced dimensions interleave more than once
// (one wave per output element, butterfly combine).
// They supersede the reference's serial one-thread-per-output kernels reduce_sum/max/min/prod.comp,
// argmax/argmin.comp and reduce_window_max_2d.comp (reference: vkjax/ops.py:305-335, 505-524).
#include "common.h"

enum RedOp : uint32_t { RED_SUM = 0, RED_PROD = 1, RED_MAX = 2, RED_MIN = 3, RED_ARGMAX = 4, RED_ARGMIN = 5 };
enum RedType : uint32_t { RT_F32 = 0, RT_I32 = 1, RT_U32 = 2 };

__device__ __forceinline__ uint32_t red_identity(uint32_t op, uint32_t ty) {
    switch (op) {
        case RED_SUM:  return 0u;
        case RED_PROD: return ty == RT_F32 ? f2u(1.0f) : 1u;
        case RED_MAX:  return ty == RT_F32 ? 0xFF800000u : ty == RT_I32 ? 0x80000000u : 0u;
        default:       return ty == RT_F32 ? 0x7F800000u : ty == RT_I32 ? 0x7FFFFFFFu : 0xFFFFFFFFu;
    }
}

__device__ __forceinline__ uint32_t red_combine(uint32_t op, uint32_t ty, uint32_t a, uint32_t b) {
    if (ty == RT_F32) {
        const float x = u2f(a), y = u2f(b);
        switch (op) {
            case RED_SUM:  return f2u(x + y);
            case RED_PROD: return f2u(x * y);
            case RED_MAX:  return (x > y || x != x) ? a : b;
            default:       return (x < y || x != x) ? a : b;
        }
    }
    switch (op) {
        case RED_SUM:  return a + b;
        case RED_PROD: return a * b;
        case RED_MAX:  return ty == RT_I32 ? ((int32_t)a > (int32_t)b ? a : b) : (a > b ? a : b);
        default:       return ty == RT_I32 ? ((int32_t)a < (int32_t)b ? a : b) : (a < b ? a : b);
    }
}

// true when candidate (va, ia) should replace (vb, ib): strictly better value, a NaN over a
// number, and on equal rank the smaller index (first occurrence).
__device__ __forceinline__ bool arg_better(bool is_max, uint32_t ty, uint32_t va, uint32_t ia, uint32_t vb, uint32_t ib) {
    if (ty == RT_F32) {
        const float x = u2f(va), y = u2f(vb);
        const bool nx = x != x, ny = y != y;
        if (nx || ny) return (nx && ny) ? ia < ib : nx;
        if (x != y) return is_max ? x > y : x < y;
        return ia < ib;
    }
    if (va != vb) {
        if (ty == RT_I32) return is_max ? (int32_t)va > (int32_t)vb : (int32_t)va < (int32_t)vb;
        return is_max ? va > vb : va < vb;
    }
    return ia < ib;
}

struct Reduce3dParams { uint32_t outer, R, inner, op, type, TI, TR; };

extern "C" __global__ __launch_bounds__(256) void reduce_3d(uint32_t* __restrict__ out, const uint32_t* __restrict__ in,
                                                            Reduce3dParams P) {
    __shared__ uint32_t s_val[256];
    __shared__ uint32_t s_idx[256];
    const uint32_t tid = threadIdx.x, ti = tid % P.TI, tr = tid / P.TI;
    const uint32_t i = blockIdx.x * P.TI + ti, o = blockIdx.y;
    const bool is_arg = P.op >= RED_ARGMAX, is_max = P.op == RED_ARGMAX;
    uint32_t acc = red_identity(P.op, P.type), best_i = 0xFFFFFFFFu, best_v = 0;
    if (i < P.inner) {
        const uint32_t* p = in + ((uint64_t)o * P.R) * P.inner + i;
        for (uint32_t r = tr; r < P.R; r += P.TR) {
            const uint32_t v = p[(uint64_t)r * P.inner];
            if (is_arg) {
                if (best_i == 0xFFFFFFFFu || arg_better(is_max, P.type, v, r, best_v, best_i)) { best_v = v; best_i = r; }
            } else {
                acc = red_combine(P.op, P.type, acc, v);
            }
        }
    }
    s_val[tid] = is_arg ? best_v : acc;
    s_idx[tid] = best_i;
    __syncthreads();
    for (uint32_t s = P.TR >> 1; s >= 1; s >>= 1) {
        if (tr < s) {
            const uint32_t other = tid + s * P.TI;
            if (is_arg) {
                const uint32_t vi = s_idx[other], vv = s_val[other];
                if (vi != 0xFFFFFFFFu && (s_idx[tid] == 0xFFFFFFFFu || arg_better(is_max, P.type, vv, vi, s_val[tid], s_idx[tid]))) {
                    s_val[tid] = vv; s_idx[tid] = vi;
                }
            } else {
                s_val[tid] = red_combine(P.op, P.type, s_val[tid], s_val[other]);
            }
        }
        __syncthreads();
    }
    if (tr == 0 && i < P.inner) out[(uint64_t)o * P.inner + i] = is_arg ? (s_idx[tid] == 0xFFFFFFFFu ? 0u : s_idx[tid]) : s_val[tid];
}

struct ReduceGeneralParams {
    uint32_t n_out, n_red, op, type;
    uint32_t nk, nr;
    uint32_t kdims[4], kstrides[4];     // kept dims (row-major order of the output) and their operand strides
    uint32_t rdims[4], rstrides[4];     // reduced dims, row-major order of the linear reduce index
};

extern "C" __global__ __launch_bounds__(256) void reduce_general(uint32_t* __restrict__ out, const uint32_t* __restrict__ in,
                                                                 ReduceGeneralParams P) {
    const uint32_t lane = threadIdx.x & 63, o = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (o >= P.n_out) return;                     // whole wave leaves together
    uint64_t base = 0;
    {
        uint32_t r = o;
        for (int d = (int)P.nk - 1; d >= 0; --d) { const uint32_t q = r / P.kdims[d]; base += (uint64_t)(r - q * P.kdims[d]) * P.kstrides[d]; r = q; }
    }
    const bool is_arg = P.op >= RED_ARGMAX, is_max = P.op == RED_ARGMAX;
    uint32_t acc = red_identity(P.op, P.type), best_i = 0xFFFFFFFFu, best_v = 0;
    for (uint32_t ri = lane; ri < P.n_red; ri += 64) {
        uint64_t off = base;
        uint32_t r = ri;
        for (int d = (int)P.nr - 1; d >= 0; --d) { const uint32_t q = r / P.rdims[d]; off += (uint64_t)(r - q * P.rdims[d]) * P.rstrides[d]; r = q; }
        const uint32_t v = in[off];
        if (is_arg) {
            if (best_i == 0xFFFFFFFFu || arg_better(is_max, P.type, v, ri, best_v, best_i)) { best_v = v; best_i = ri; }
        } else {
            acc = red_combine(P.op, P.type, acc, v);
        }
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) {
        if (is_arg) {
            const uint32_t vi = __shfl_xor(best_i, s, 64), vv = __shfl_xor(best_v, s, 64);
            if (vi != 0xFFFFFFFFu && (best_i == 0xFFFFFFFFu || arg_better(is_max, P.type, vv, vi, best_v, best_i))) { best_v = vv; best_i = vi; }
        } else {
            acc = red_combine(P.op, P.type, acc, __shfl_xor(acc, s, 64));
        }
    }
    if (lane == 0) out[o] = is_arg ? (best_i == 0xFFFFFFFFu ? 0u : best_i) : acc;
}

// Window reduction over a (left-padded to) 4-D array: out[o] = combine over window taps t of
// in[o*stride + t*dilation - pad_low], taps outside the array contribute the identity
// (-inf for max, 0 for sum). VEC = 4 handles four consecutive elements of the last dimension
// per thread; it requires window = stride = dilation = 1 and no padding on that dimension and
// a last dimension divisible by 4.
struct PoolParams {
    uint32_t n_out;                 // output elements (VEC units are derived in-kernel)
    uint32_t op, type;              // RED_MAX or RED_SUM
    uint32_t in_dims[4], out_dims[4];
    uint32_t window[4], stride[4], dilation[4];
    int32_t  pad_low[4];
};

template <int VEC>
__device__ __forceinline__ void pool_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, const PoolParams& P) {
    const uint64_t e0 = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * VEC;
    if (e0 >= P.n_out) return;
    uint32_t oc[4];
    {
        uint32_t r = (uint32_t)e0;
#pragma unroll
        for (int d = 3; d >= 1; --d) { const uint32_t q = r / P.out_dims[d]; oc[d] = r - q * P.out_dims[d]; r = q; }
        oc[0] = r;
    }
    uint32_t acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = red_identity(P.op, P.type);
    const uint32_t w3 = VEC == 4 ? 1u : P.window[3];
    for (uint32_t t0 = 0; t0 < P.window[0]; ++t0) {
        const int64_t c0 = (int64_t)oc[0] * P.stride[0] + (int64_t)t0 * P.dilation[0] - P.pad_low[0];
        if (c0 < 0 || c0 >= P.in_dims[0]) continue;
        for (uint32_t t1 = 0; t1 < P.window[1]; ++t1) {
            const int64_t c1 = (int64_t)oc[1] * P.stride[1] + (int64_t)t1 * P.dilation[1] - P.pad_low[1];
            if (c1 < 0 || c1 >= P.in_dims[1]) continue;
            for (uint32_t t2 = 0; t2 < P.window[2]; ++t2) {
                const int64_t c2 = (int64_t)oc[2] * P.stride[2] + (int64_t)t2 * P.dilation[2] - P.pad_low[2];
                if (c2 < 0 || c2 >= P.in_dims[2]) continue;
                for (uint32_t t3 = 0; t3 < w3; ++t3) {
                    const int64_t c3 = VEC == 4 ? (int64_t)oc[3]
                                                : (int64_t)oc[3] * P.stride[3] + (int64_t)t3 * P.dilation[3] - P.pad_low[3];
                    if (c3 < 0 || c3 >= P.in_dims[3]) continue;
                    const uint64_t off = (((uint64_t)c0 * P.in_dims[1] + c1) * P.in_dims[2] + c2) * P.in_dims[3] + c3;
                    if constexpr (VEC == 4) {
                        const u32x4 v = *reinterpret_cast<const u32x4*>(in + off);
                        acc[0] = red_combine(P.op, P.type, acc[0], v.x);
                        acc[1] = red_combine(P.op, P.type, acc[1], v.y);
                        acc[2] = red_combine(P.op, P.type, acc[2], v.z);
                        acc[3] = red_combine(P.op, P.type, acc[3], v.w);
                    } else {
                        acc[0] = red_combine(P.op, P.type, acc[0], in[off]);
                    }
                }
            }
        }
    }
    if constexpr (VEC == 4) {
        u32x4 v; v.x = acc[0]; v.y = acc[1]; v.z = acc[2]; v.w = acc[3];
        *reinterpret_cast<u32x4*>(out + e0) = v;
    } else {
        out[e0] = acc[0];
    }
}

extern "C" __global__ __launch_bounds__(256) void pool_v1(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, PoolParams P) {
    pool_body<1>(out, in, P);
}
extern "C" __global__ __launch_bounds__(256) void pool_v4(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, PoolParams P) {
    pool_body<4>(out, in, P);
}
