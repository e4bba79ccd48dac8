// Reductions (sum / prod / max / min, argmax / argmin) and window reductions (max / sum pooling).
//
// reduce_rows / reduce_cols view the operand as [outer, R, inner] and reduce R (see below).
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

// ---------------------------------------------------------------------------------------------
// Reductions of the canonical form [outer, R, inner] -> [outer, inner].
//
// reduce_rows (inner == 1): a wave owns one (row, split) pair and streams its part of the row with
// 16-byte loads, four in flight per lane; lanes are combined with a butterfly.
// reduce_cols (inner > 1): a block owns TI*VEC consecutive `inner` positions and one split of R;
// its TR thread rows walk R interleaved, so every wave-level load is contiguous along `inner`;
// thread rows are combined through LDS.
// Splits: when outer x inner alone would not fill the GPU, R is cut into `nsplit` ranges of
// `r_chunk` rows that different waves / blocks reduce; the partial results [outer, nsplit, inner]
// are then reduced by a second launch of the same kernel. (Index-returning reductions run unsplit.)
// MODE picks the combine at compile time: 0 float sum, 1 float max (NaN wins), 2 whatever op/type say,
// 3 / 4 float argmax / argmin.
struct ReduceParams { uint32_t outer, R, inner, op, type, r_chunk, nsplit, TI; };

template <int MODE>
__device__ __forceinline__ uint32_t red_step(uint32_t op, uint32_t ty, uint32_t a, uint32_t b) {
    if constexpr (MODE == 0) return f2u(u2f(a) + u2f(b));
    else if constexpr (MODE == 1) { const float x = u2f(a), y = u2f(b); return (x > y || x != x) ? a : b; }
    else return red_combine(op, ty, a, b);
}

// POST (float sums only): the finished sum is divided (1) or multiplied (2) by the single value at `post` before it is
// stored - the step behind a mean, with the rounding of the element-wise kernel's own division / multiplication.
template <int POST>
__device__ __forceinline__ uint32_t reduce_post(uint32_t sum, const uint32_t* __restrict__ post) {
    if constexpr (POST == 1) return f2u(u2f(sum) / u2f(post[0]));
    else if constexpr (POST == 2) return f2u(u2f(sum) * u2f(post[0]));
    else return sum;
}

template <int VEC, int MODE, int POST = 0>
__device__ __forceinline__ void reduce_rows_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, const ReduceParams& P,
                                                 const uint32_t* __restrict__ post = nullptr) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint64_t unit = (uint64_t)blockIdx.x * 4u + (threadIdx.x >> 6);
    if (unit >= (uint64_t)P.outer * P.nsplit) return;                 // whole wave leaves together
    const uint32_t o = (uint32_t)(unit / P.nsplit), sp = (uint32_t)(unit - (uint64_t)o * P.nsplit);
    const uint32_t r_lo = sp * P.r_chunk, r_hi = min(P.R, r_lo + P.r_chunk);
    const uint32_t* row = in + (uint64_t)o * P.R;
    const bool is_arg = MODE >= 3 || (MODE == 2 && P.op >= RED_ARGMAX), is_max = MODE == 3 || (MODE == 2 && P.op == RED_ARGMAX);
    const uint32_t ident = MODE == 0 ? 0u : MODE == 1 ? 0xFF800000u : red_identity(P.op, P.type);
    uint32_t acc[4] = {ident, ident, ident, ident}, best_i = 0xFFFFFFFFu, best_v = 0;
    // `ok` false: position r lies beyond the row's range and v holds the identity
    auto take = [&](uint32_t v, uint32_t r, int slot, bool ok = true) {
        if constexpr (MODE >= 3) {
            // float argmax / argmin: a lane meets its elements in ascending index order, so on a tie the
            // earlier one stays; a NaN replaces any number and is never replaced
            const float x = u2f(v), y = u2f(best_v);
            const bool better = ok && ((MODE == 3 ? x > y : x < y) || (x != x && y == y) || best_i == 0xFFFFFFFFu);
            best_v = better ? v : best_v;
            best_i = better ? r : best_i;
        } else if (is_arg) {
            if (ok && (best_i == 0xFFFFFFFFu || arg_better(is_max, P.type, v, r, best_v, best_i))) { best_v = v; best_i = r; }
        } else {
            acc[slot] = red_step<MODE>(P.op, P.type, acc[slot], v);   // combining with the identity changes nothing
        }
    };
    // Every lane of the wave takes the same number of steps, four loads in flight in each; in the last step
    // the positions beyond the range are not loaded and count as the identity. (Lanes that left the
    // four-load loop one by one would each wait for their remaining loads in turn.)
    if constexpr (VEC == 4) {
        // r_lo, R and the row starts are multiples of 4 (the host checks)
        uint32_t r = r_lo + lane * 4u, base = r_lo;
        for (; base + 4u * 256u <= r_hi; base += 4u * 256u, r += 4u * 256u) {
            u32x4 v[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] = *reinterpret_cast<const u32x4*>(row + r + q * 256u);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                take(v[q].x, r + q * 256u, 0); take(v[q].y, r + q * 256u + 1u, 1); take(v[q].z, r + q * 256u + 2u, 2); take(v[q].w, r + q * 256u + 3u, 3);
            }
        }
        if (base < r_hi) {                                               // r_hi - r_lo is a multiple of 4 too
            u32x4 v[4];
            bool ok[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                ok[q] = r + q * 256u < r_hi;
                v[q] = u32x4{ident, ident, ident, ident};
                if (ok[q]) v[q] = *reinterpret_cast<const u32x4*>(row + r + q * 256u);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                take(v[q].x, r + q * 256u, 0, ok[q]); take(v[q].y, r + q * 256u + 1u, 1, ok[q]);
                take(v[q].z, r + q * 256u + 2u, 2, ok[q]); take(v[q].w, r + q * 256u + 3u, 3, ok[q]);
            }
        }
    } else {
        uint32_t r = r_lo + lane, base = r_lo;
        for (; base + 4u * 64u <= r_hi; base += 4u * 64u, r += 4u * 64u) {
            uint32_t v[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] = row[r + q * 64u];
#pragma unroll
            for (int q = 0; q < 4; ++q) take(v[q], r + q * 64u, q);
        }
        if (base < r_hi) {
            uint32_t v[4];
            bool ok[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                ok[q] = r + q * 64u < r_hi;
                v[q] = ident;
                if (ok[q]) v[q] = row[r + q * 64u];
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) take(v[q], r + q * 64u, q, ok[q]);
        }
    }
    uint32_t a = acc[0];
    if (!is_arg) {
        a = red_step<MODE>(P.op, P.type, red_step<MODE>(P.op, P.type, acc[0], acc[1]), red_step<MODE>(P.op, P.type, acc[2], acc[3]));
    }
    if constexpr (MODE >= 3) {
        // float argmax / argmin across the lanes as the maximum of one 64-bit key per lane: the value mapped to an
        // unsigned number that grows with its rank (a NaN above everything), then the complement of the index, so
        // that of two equal values the earlier one wins. Five operations per butterfly step instead of a dozen.
        // -0.0 ranks with +0.0 (the two compare equal, so the earlier of them wins)
        const uint32_t bits = best_v == 0x80000000u ? 0u : best_v, flipped = bits ^ ((bits >> 31) ? 0xFFFFFFFFu : 0x80000000u);
        const float    x    = u2f(bits);
        const uint32_t rank = x != x ? 0xFFFFFFFFu : (MODE == 3 ? flipped : ~flipped);
        uint64_t key = best_i == 0xFFFFFFFFu ? 0ull : ((uint64_t)rank << 32 | (uint32_t)~best_i);   // no rank of a value is 0
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1) {
            const uint64_t other = __shfl_xor(key, s, 64);
            key = other > key ? other : key;
        }
        if (lane == 0) out[unit] = key == 0ull ? 0u : ~(uint32_t)key;
        return;
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) {
        if (is_arg) {
            const uint32_t vi = __shfl_xor(best_i, s, 64), vv = __shfl_xor(best_v, s, 64);
            if (vi != 0xFFFFFFFFu && (best_i == 0xFFFFFFFFu || arg_better(is_max, P.type, vv, vi, best_v, best_i))) { best_v = vv; best_i = vi; }
        } else {
            a = red_step<MODE>(P.op, P.type, a, __shfl_xor(a, s, 64));
        }
    }
    if (lane == 0) out[unit] = is_arg ? (best_i == 0xFFFFFFFFu ? 0u : best_i) : reduce_post<POST>(a, post);
}

// PRO: what is reduced. 0 the operand itself; 1 its product with a second array of the same shape;
// 2 its product with a vector over `inner`; 3 its negation (float). The element-wise producer of a
// reduction's operand (the `g * x` and `-g` of a batch-norm backward pass) is applied while loading,
// with the same roundings as a separate pass, so that array never exists.
enum { PRO_NONE = 0, PRO_MUL = 1, PRO_MULV = 2, PRO_NEG = 3 };

// `block`: index of this workgroup in the reduction's own grid
template <int VEC, int MODE, int PRO = PRO_NONE, int POST = 0>
__device__ __forceinline__ void reduce_cols_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, const ReduceParams& P,
                                                 const uint32_t* __restrict__ in2 = nullptr, const uint32_t block = blockIdx.x,
                                                 const uint32_t* __restrict__ post = nullptr) {
    __shared__ uint32_t s_val[256 * VEC];
    __shared__ uint32_t s_idx[256 * VEC];
    const uint32_t TI = P.TI, TR = 256u / TI;
    const uint32_t tid = threadIdx.x, ti = tid % TI, tr = tid / TI;
    // block -> (inner tile, split, outer row)
    const uint32_t tiles_i = (P.inner + TI * VEC - 1u) / (TI * VEC);
    const uint32_t it = block % tiles_i, rest = block / tiles_i;
    const uint32_t sp = rest % P.nsplit, o = rest / P.nsplit;
    const uint32_t i = (it * TI + ti) * VEC;
    const uint32_t r_lo = sp * P.r_chunk, r_hi = min(P.R, r_lo + P.r_chunk);
    const bool is_arg = MODE >= 3 || (MODE == 2 && P.op >= RED_ARGMAX), is_max = MODE == 3 || (MODE == 2 && P.op == RED_ARGMAX);
    const uint32_t ident = MODE == 0 ? 0u : MODE == 1 ? 0xFF800000u : red_identity(P.op, P.type);
    uint32_t acc[VEC], best_i[VEC], best_v[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) { acc[j] = ident; best_i[j] = 0xFFFFFFFFu; best_v[j] = 0; }
    auto take = [&](uint32_t v, uint32_t r, int j) {
        if constexpr (MODE >= 3) {
            const float x = u2f(v), y = u2f(best_v[j]);
            const bool better = (MODE == 3 ? x > y : x < y) || (x != x && y == y) || best_i[j] == 0xFFFFFFFFu;
            best_v[j] = better ? v : best_v[j];
            best_i[j] = better ? r : best_i[j];
        } else if (is_arg) {
            if (best_i[j] == 0xFFFFFFFFu || arg_better(is_max, P.type, v, r, best_v[j], best_i[j])) { best_v[j] = v; best_i[j] = r; }
        } else {
            acc[j] = red_step<MODE>(P.op, P.type, acc[j], v);
        }
    };
    if (i < P.inner) {                                                // inner is a multiple of VEC
        const uint32_t* p  = in + (uint64_t)o * P.R * P.inner + i;
        const uint32_t* p2 = PRO == PRO_MUL ? in2 + (uint64_t)o * P.R * P.inner + i : nullptr;
        uint32_t w[VEC];                                              // PRO_MULV: this thread's part of the vector
#pragma unroll
        for (int j = 0; j < VEC; ++j) w[j] = PRO == PRO_MULV ? in2[i + j] : 0u;
        auto fetch = [&](uint32_t row, uint32_t (&v)[VEC]) {
            const uint64_t off = (uint64_t)row * P.inner;
            uint32_t b[VEC];
            if constexpr (VEC == 4) {
                const u32x4 t = *reinterpret_cast<const u32x4*>(p + off);
                v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
                if constexpr (PRO == PRO_MUL) { const u32x4 u = *reinterpret_cast<const u32x4*>(p2 + off); b[0] = u.x; b[1] = u.y; b[2] = u.z; b[3] = u.w; }
            } else {
                v[0] = p[off];
                if constexpr (PRO == PRO_MUL) b[0] = p2[off];
            }
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                if constexpr (PRO == PRO_MUL)  v[j] = f2u(u2f(v[j]) * u2f(b[j]));
                if constexpr (PRO == PRO_MULV) v[j] = f2u(u2f(v[j]) * u2f(w[j]));
                if constexpr (PRO == PRO_NEG)  v[j] ^= 0x80000000u;
            }
        };
        // all thread rows take the same number of steps, four loads in flight per thread in each; the last
        // step leaves out the rows beyond the range
        uint32_t r = r_lo + tr, first = r_lo;
        for (; first + 4u * TR <= r_hi; first += 4u * TR, r += 4u * TR) {
            uint32_t v[4][VEC];
#pragma unroll
            for (int q = 0; q < 4; ++q) fetch(r + q * TR, v[q]);
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int j = 0; j < VEC; ++j) take(v[q][j], r + q * TR, j);
        }
        if (first < r_hi) {
            uint32_t v[4][VEC];
#pragma unroll
            for (int q = 0; q < 4; ++q) if (r + q * TR < r_hi) fetch(r + q * TR, v[q]);
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (r + q * TR < r_hi) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) take(v[q][j], r + q * TR, j);
                }
        }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) { s_val[tid * VEC + j] = is_arg ? best_v[j] : acc[j]; s_idx[tid * VEC + j] = best_i[j]; }
    __syncthreads();
    for (uint32_t s = TR >> 1; s >= 1; s >>= 1) {
        if (tr < s) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const uint32_t mine = tid * VEC + j, other = (tid + s * TI) * VEC + j;
                if (is_arg) {
                    const uint32_t vi = s_idx[other], vv = s_val[other];
                    if (vi != 0xFFFFFFFFu && (s_idx[mine] == 0xFFFFFFFFu || arg_better(is_max, P.type, vv, vi, s_val[mine], s_idx[mine]))) {
                        s_val[mine] = vv; s_idx[mine] = vi;
                    }
                } else {
                    s_val[mine] = red_step<MODE>(P.op, P.type, s_val[mine], s_val[other]);
                }
            }
        }
        __syncthreads();
    }
    if (tr == 0 && i < P.inner) {
        uint32_t* dst = out + ((uint64_t)o * P.nsplit + sp) * P.inner + i;
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            dst[j] = is_arg ? (s_idx[tid * VEC + j] == 0xFFFFFFFFu ? 0u : s_idx[tid * VEC + j]) : reduce_post<POST>(s_val[tid * VEC + j], post);
    }
}

#define REDUCE_KERNELS(tag, MODE)                                                                                              \
    extern "C" __global__ __launch_bounds__(256) void reduce_rows_##tag##_v1(uint32_t* out, const uint32_t* in, ReduceParams P) { reduce_rows_body<1, MODE>(out, in, P); } \
    extern "C" __global__ __launch_bounds__(256) void reduce_rows_##tag##_v4(uint32_t* out, const uint32_t* in, ReduceParams P) { reduce_rows_body<4, MODE>(out, in, P); } \
    extern "C" __global__ __launch_bounds__(256) void reduce_cols_##tag##_v1(uint32_t* out, const uint32_t* in, ReduceParams P) { reduce_cols_body<1, MODE>(out, in, P); } \
    extern "C" __global__ __launch_bounds__(256) void reduce_cols_##tag##_v4(uint32_t* out, const uint32_t* in, ReduceParams P) { reduce_cols_body<4, MODE>(out, in, P); }
#define REDUCE_COLS_PROLOGUE_KERNELS(tag, PRO)                                                                                 \
    extern "C" __global__ __launch_bounds__(256) void reduce_cols_fsum_##tag##_v1(uint32_t* out, const uint32_t* in, const uint32_t* in2, ReduceParams P) { reduce_cols_body<1, 0, PRO>(out, in, P, in2); } \
    extern "C" __global__ __launch_bounds__(256) void reduce_cols_fsum_##tag##_v4(uint32_t* out, const uint32_t* in, const uint32_t* in2, ReduceParams P) { reduce_cols_body<4, 0, PRO>(out, in, P, in2); }
// float sums followed by a division or a multiplication by one value (a mean): unsplit reductions only
#define REDUCE_POST_KERNELS(tag, POST)                                                                                         \
    extern "C" __global__ __launch_bounds__(256) void reduce_rows_fsum_##tag##_v1(uint32_t* out, const uint32_t* in, const uint32_t* post, ReduceParams P) { reduce_rows_body<1, 0, POST>(out, in, P, post); } \
    extern "C" __global__ __launch_bounds__(256) void reduce_rows_fsum_##tag##_v4(uint32_t* out, const uint32_t* in, const uint32_t* post, ReduceParams P) { reduce_rows_body<4, 0, POST>(out, in, P, post); } \
    extern "C" __global__ __launch_bounds__(256) void reduce_cols_fsum_##tag##_v1(uint32_t* out, const uint32_t* in, const uint32_t* post, ReduceParams P) { reduce_cols_body<1, 0, PRO_NONE, POST>(out, in, P, nullptr, blockIdx.x, post); } \
    extern "C" __global__ __launch_bounds__(256) void reduce_cols_fsum_##tag##_v4(uint32_t* out, const uint32_t* in, const uint32_t* post, ReduceParams P) { reduce_cols_body<4, 0, PRO_NONE, POST>(out, in, P, nullptr, blockIdx.x, post); }
// Several small, mutually independent float column sums in ONE launch (the second stages of split sums, the
// per-channel sums of small layers): one table entry per sum, workgroup b belongs to the last entry whose
// first_block is <= b, as in ew_chain_batch.
struct ReduceBatchEntry {
    uint32_t        first_block, pad0;
    uint32_t*       out;
    const uint32_t* in;
    ReduceParams    P;
};
static_assert(sizeof(ReduceBatchEntry) == 56, "the host lays the table out with 56-byte entries");

template <int VEC>
__device__ __forceinline__ void reduce_cols_batch_body(const ReduceBatchEntry* __restrict__ table, uint32_t entries) {
    uint32_t lo = 0, hi = entries;
    while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) >> 1;
        if (table[mid].first_block <= blockIdx.x) lo = mid; else hi = mid;
    }
    lo = __builtin_amdgcn_readfirstlane(lo);
    const ReduceBatchEntry& e = table[lo];
    reduce_cols_body<VEC, 0>(e.out, e.in, e.P, nullptr, blockIdx.x - e.first_block);
}
extern "C" __global__ __launch_bounds__(256) void reduce_cols_fsum_batch_v1(const ReduceBatchEntry* __restrict__ table, uint32_t entries) {
    reduce_cols_batch_body<1>(table, entries);
}
extern "C" __global__ __launch_bounds__(256) void reduce_cols_fsum_batch_v4(const ReduceBatchEntry* __restrict__ table, uint32_t entries) {
    reduce_cols_batch_body<4>(table, entries);
}

// the _v4 variants need R % 4 == 0, r_chunk % 4 == 0 (rows) or inner % 4 == 0 (cols) and 16-byte aligned pointers
REDUCE_COLS_PROLOGUE_KERNELS(mul, PRO_MUL)
REDUCE_COLS_PROLOGUE_KERNELS(mulv, PRO_MULV)
REDUCE_COLS_PROLOGUE_KERNELS(neg, PRO_NEG)
REDUCE_POST_KERNELS(div, 1)
REDUCE_POST_KERNELS(times, 2)
REDUCE_KERNELS(fsum, 0)
REDUCE_KERNELS(fmax, 1)
// Any other combination of operation and element type. The combine is selected once per launch: every case calls the
// body with a copy of the parameters whose op and type are constants, so that the compiler folds the branches of
// red_combine out of the loops (taken per element they cost a generic reduction half its bandwidth: min over rows
// 3.4 TB/s against 5.7 for max). Index-returning reductions of integers and whatever else is left take the
// run-time path.
#define REDUCE_ANY_CASE(OP, TY, CALL) case (OP) * 4u + (TY): { ReduceParams Q = P; Q.op = (OP); Q.type = (TY); CALL; } break;
#define REDUCE_ANY_DISPATCH(CALL)                                                                              \
    switch (P.op * 4u + P.type) {                                                                              \
        REDUCE_ANY_CASE(RED_SUM, RT_I32, CALL)  REDUCE_ANY_CASE(RED_SUM, RT_U32, CALL)                          \
        REDUCE_ANY_CASE(RED_PROD, RT_F32, CALL) REDUCE_ANY_CASE(RED_PROD, RT_I32, CALL) REDUCE_ANY_CASE(RED_PROD, RT_U32, CALL) \
        REDUCE_ANY_CASE(RED_MAX, RT_I32, CALL)  REDUCE_ANY_CASE(RED_MAX, RT_U32, CALL)                          \
        REDUCE_ANY_CASE(RED_MIN, RT_F32, CALL)  REDUCE_ANY_CASE(RED_MIN, RT_I32, CALL)  REDUCE_ANY_CASE(RED_MIN, RT_U32, CALL) \
        default: { const ReduceParams& Q = P; CALL; } break;                                                    \
    }
extern "C" __global__ __launch_bounds__(256) void reduce_rows_any_v1(uint32_t* out, const uint32_t* in, ReduceParams P) { REDUCE_ANY_DISPATCH((reduce_rows_body<1, 2>(out, in, Q))) }
extern "C" __global__ __launch_bounds__(256) void reduce_rows_any_v4(uint32_t* out, const uint32_t* in, ReduceParams P) { REDUCE_ANY_DISPATCH((reduce_rows_body<4, 2>(out, in, Q))) }
extern "C" __global__ __launch_bounds__(256) void reduce_cols_any_v1(uint32_t* out, const uint32_t* in, ReduceParams P) { REDUCE_ANY_DISPATCH((reduce_cols_body<1, 2>(out, in, Q))) }
extern "C" __global__ __launch_bounds__(256) void reduce_cols_any_v4(uint32_t* out, const uint32_t* in, ReduceParams P) { REDUCE_ANY_DISPATCH((reduce_cols_body<4, 2>(out, in, Q))) }
REDUCE_KERNELS(fargmax, 3)
REDUCE_KERNELS(fargmin, 4)

// ---------------------------------------------------------------------------------------------
// Backward pass of  y = max(x * k + b, 0)  (a per-channel scale and shift followed by ReLU, k and b
// vectors over the fastest dimension) in one pass over the arrays. Autodiff spells it
//     m  = ans > t ? g : z          (t, z single values; ans the forward result, g its cotangent)
//     db = sum over rows of m       dk = sum over rows of m * x       dx = m * k
// as two element-wise launches, two more that only feed the column sums, and the two sums: nine
// passes over arrays of the activation's size. Here every element of ans, g and x is read once, dx
// written once, and both sums accumulated on the way: four passes. The sums run over exactly the
// rows, in exactly the order, of reduce_cols_body with the same ReduceParams (per-thread running
// sums over rows r_lo + tr, + TR, ..., then the same tree over tr in LDS), so sum_m and sum_mx hold
// the bits the separate launches would have produced, partial results per row range included.
// SELECT = false: m is g itself (no activation between the scale and what follows; ans, thr and alt unused).
template <int VEC, bool SELECT>
__device__ __forceinline__ void scale_relu_backward_body(float* __restrict__ dx, float* __restrict__ sum_m, float* __restrict__ sum_mx,
                                                         const float* __restrict__ ans, const float* __restrict__ thr,
                                                         const float* __restrict__ g, const float* __restrict__ alt,
                                                         const float* __restrict__ x, const float* __restrict__ kvec,
                                                         const ReduceParams& P) {
    __shared__ float s_m[256 * VEC];
    __shared__ float s_x[256 * VEC];
    const uint32_t TI = P.TI, TR = 256u / TI;
    const uint32_t tid = threadIdx.x, ti = tid % TI, tr = tid / TI;
    const uint32_t tiles_i = (P.inner + TI * VEC - 1u) / (TI * VEC);
    const uint32_t it = blockIdx.x % tiles_i, rest = blockIdx.x / tiles_i;
    const uint32_t sp = rest % P.nsplit, o = rest / P.nsplit;
    const uint32_t i = (it * TI + ti) * VEC;
    const uint32_t r_lo = sp * P.r_chunk, r_hi = min(P.R, r_lo + P.r_chunk);
    float acc_m[VEC], acc_x[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) { acc_m[j] = 0.f; acc_x[j] = 0.f; }
    if (i < P.inner) {                                                // inner is a multiple of VEC
        const float t = SELECT ? thr[0] : 0.f, z = SELECT ? alt[0] : 0.f;
        const uint64_t base = (uint64_t)o * P.R * P.inner + i;
        float kv[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) kv[j] = kvec[i + j];
        auto fetch = [&](uint32_t row, float (&a)[VEC], float (&c)[VEC], float (&v)[VEC]) {
            const uint64_t off = base + (uint64_t)row * P.inner;
            if constexpr (VEC == 4) {
                const f32x4 tc = *reinterpret_cast<const f32x4*>(g + off), tv = *reinterpret_cast<const f32x4*>(x + off);
                c[0] = tc.x; c[1] = tc.y; c[2] = tc.z; c[3] = tc.w;
                v[0] = tv.x; v[1] = tv.y; v[2] = tv.z; v[3] = tv.w;
                if constexpr (SELECT) {
                    const f32x4 ta = *reinterpret_cast<const f32x4*>(ans + off);
                    a[0] = ta.x; a[1] = ta.y; a[2] = ta.z; a[3] = ta.w;
                }
            } else {
                c[0] = g[off]; v[0] = x[off];
                if constexpr (SELECT) a[0] = ans[off];
            }
        };
        auto take = [&](uint32_t row, const float (&a)[VEC], const float (&c)[VEC], const float (&v)[VEC]) {
            float m[VEC], d[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                m[j] = SELECT ? (a[j] > t ? c[j] : z) : c[j];
                d[j] = m[j] * kv[j];
                acc_m[j] = acc_m[j] + m[j];
                acc_x[j] = acc_x[j] + m[j] * v[j];
            }
            const uint64_t off = base + (uint64_t)row * P.inner;
            if constexpr (VEC == 4) *reinterpret_cast<f32x4*>(dx + off) = f32x4{d[0], d[1], d[2], d[3]};
            else dx[off] = d[0];
        };
        // all thread rows take the same number of steps, four rows in flight per thread in each; the last
        // step leaves out the rows beyond the range
        uint32_t r = r_lo + tr, first = r_lo;
        for (; first + 4u * TR <= r_hi; first += 4u * TR, r += 4u * TR) {
            float a[4][VEC], c[4][VEC], v[4][VEC];
#pragma unroll
            for (int q = 0; q < 4; ++q) fetch(r + q * TR, a[q], c[q], v[q]);
#pragma unroll
            for (int q = 0; q < 4; ++q) take(r + q * TR, a[q], c[q], v[q]);
        }
        if (first < r_hi) {
            float a[4][VEC], c[4][VEC], v[4][VEC];
#pragma unroll
            for (int q = 0; q < 4; ++q) if (r + q * TR < r_hi) fetch(r + q * TR, a[q], c[q], v[q]);
#pragma unroll
            for (int q = 0; q < 4; ++q) if (r + q * TR < r_hi) take(r + q * TR, a[q], c[q], v[q]);
        }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) { s_m[tid * VEC + j] = acc_m[j]; s_x[tid * VEC + j] = acc_x[j]; }
    __syncthreads();
    for (uint32_t s = TR >> 1; s >= 1; s >>= 1) {
        if (tr < s) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const uint32_t mine = tid * VEC + j, other = (tid + s * TI) * VEC + j;
                s_m[mine] = s_m[mine] + s_m[other];
                s_x[mine] = s_x[mine] + s_x[other];
            }
        }
        __syncthreads();
    }
    if (tr == 0 && i < P.inner) {
        const uint64_t dst = ((uint64_t)o * P.nsplit + sp) * P.inner + i;
#pragma unroll
        for (int j = 0; j < VEC; ++j) { sum_m[dst + j] = s_m[tid * VEC + j]; sum_mx[dst + j] = s_x[tid * VEC + j]; }
    }
}

#define SCALE_RELU_BACKWARD_KERNEL(name, VEC, SELECT)                                                                       \
    extern "C" __global__ __launch_bounds__(256) void name(float* dx, float* sum_m, float* sum_mx, const float* ans,   \
                                                           const float* thr, const float* g, const float* alt,        \
                                                           const float* x, const float* kvec, ReduceParams P) {       \
        scale_relu_backward_body<VEC, SELECT>(dx, sum_m, sum_mx, ans, thr, g, alt, x, kvec, P);                              \
    }
// _v4 needs inner % 4 == 0 and 16-byte aligned arrays
SCALE_RELU_BACKWARD_KERNEL(scale_relu_backward_v1, 1, true)
SCALE_RELU_BACKWARD_KERNEL(scale_relu_backward_v4, 4, true)
SCALE_RELU_BACKWARD_KERNEL(scale_backward_v1, 1, false)
SCALE_RELU_BACKWARD_KERNEL(scale_backward_v4, 4, false)

// ---------------------------------------------------------------------------------------------
// softmax over the rows of [outer, R] in one launch: out = exp(x - max(x)) / sum(exp(x - max(x))).
// Takes the place of reduce_max -> (subtract, exp) -> reduce_sum -> divide. One wave per row; the
// sum is accumulated in exactly the order reduce_rows uses (per-lane partial sums over the same
// elements, combined pairwise, then the same butterfly), so the result has the same bits as the
// four separate launches. For rows short enough to run unsplit there (the host checks R).
struct SoftmaxParams { uint32_t outer, R; };

template <int VEC, class F>
__device__ __forceinline__ float row_sum_as_reduce_rows(F value_at, uint32_t R, uint32_t lane) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if constexpr (VEC == 4) {
        for (uint32_t r = lane * 4u; r < R; r += 256u)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] += value_at(r + j);
    } else {
        uint32_t r = lane;
        for (int q = 0; r < R; r += 64u, q = (q + 1) & 3) {
            const float v = value_at(r);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] += j == q ? v : 0.f;     // the sums are never -0, so adding 0 keeps them
        }
    }
    float a = (acc[0] + acc[1]) + (acc[2] + acc[3]);
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) a = a + __shfl_xor(a, s, 64);
    return a;
}

// `arg_out` (may be null): the index of each result row's largest value as reduce_rows_fargmax would report it
// (first occurrence, a NaN wins), for programs that take the arg-max of the probabilities right away.
template <int VEC>
__device__ __forceinline__ void softmax_rows_body(float* __restrict__ out, const float* __restrict__ in, uint32_t* __restrict__ arg_out,
                                                  const SoftmaxParams& P) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= P.outer) return;                                       // whole wave leaves together
    const float* x = in + (uint64_t)row * P.R;
    float* y = out + (uint64_t)row * P.R;
    float m = -INFINITY;                                              // the maximum does not depend on the order; a NaN wins
    for (uint32_t r = lane; r < P.R; r += 64u) { const float v = x[r]; m = (v > m || v != v) ? v : m; }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) { const float o = __shfl_xor(m, s, 64); m = (m > o || m != m) ? m : o; }
    const float total = row_sum_as_reduce_rows<VEC>([&](uint32_t r) { return expf(x[r] - m); }, P.R, lane);
    uint32_t best_v = 0, best_i = 0xFFFFFFFFu;
    for (uint32_t r = lane; r < P.R; r += 64u) {
        const float p = expf(x[r] - m) / total;
        y[r] = p;
        // a lane meets its elements in ascending order: on a tie the earlier one stays; a NaN replaces any number
        const float q = u2f(best_v);
        const bool better = p > q || (p != p && q == q) || best_i == 0xFFFFFFFFu;
        best_v = better ? f2u(p) : best_v;
        best_i = better ? r : best_i;
    }
    if (arg_out == nullptr) return;
    // across the lanes as in reduce_rows: the maximum of (rank of the value, complement of the index)
    const uint32_t zb      = best_v == 0x80000000u ? 0u : best_v;      // -0.0 ranks with +0.0
    const uint32_t flipped = zb ^ ((zb >> 31) ? 0xFFFFFFFFu : 0x80000000u);
    const float    bv      = u2f(best_v);
    uint64_t key = best_i == 0xFFFFFFFFu ? 0ull : ((uint64_t)(bv != bv ? 0xFFFFFFFFu : flipped) << 32 | (uint32_t)~best_i);
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) {
        const uint64_t other = __shfl_xor(key, s, 64);
        key = other > key ? other : key;
    }
    if (lane == 0) arg_out[row] = key == 0ull ? 0u : ~(uint32_t)key;
}

extern "C" __global__ __launch_bounds__(256) void softmax_rows_v1(float* __restrict__ out, const float* __restrict__ in, uint32_t* __restrict__ arg_out,
                                                                  SoftmaxParams P) {
    softmax_rows_body<1>(out, in, arg_out, P);
}
// R % 4 == 0: the summation order of the 16-byte reduce_rows kernel
extern "C" __global__ __launch_bounds__(256) void softmax_rows_v4(float* __restrict__ out, const float* __restrict__ in, uint32_t* __restrict__ arg_out,
                                                                  SoftmaxParams P) {
    softmax_rows_body<4>(out, in, arg_out, P);
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
    uint32_t n_out;                 // output elements (VEC units are derived in-kernel); scatter_selected: bit 31 is STREAM_RESULT_BIT
    uint32_t op, type;              // RED_MAX or RED_SUM
    uint32_t in_dims[4], out_dims[4];
    uint32_t window[4], stride[4], dilation[4];
    int32_t  pad_low[4];
    // the 2-D kernels (pool2d, select_window2d, scatter_selected2d): n / d = mulhi(n, magic) >> shift (magic 0: d = 1) for
    // the three extents a thread decodes its element number with: channels, width, height of the array the launch writes
    // (prepared on the host; three divisions by run-time values cost a thread some 120 instructions)
    uint32_t div_magic[3], div_shift[3];
};

// n / s for n >= 0 and a window stride s: 1 or 2, the usual ones, without a division
__device__ __forceinline__ int32_t div_stride(int32_t n, int32_t s) { return s == 1 ? n : s == 2 ? n >> 1 : n / s; }

template <int VEC>
__device__ __forceinline__ void pool_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, const PoolParams& P) {
    const uint64_t e0 = ((uint64_t)xcd_contiguous_block() * 256u + threadIdx.x) * VEC;
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

// The usual pooling layout, [batch, y, x, channels] with a KH x KW window over y and x only: all
// taps of a thread's four channels are requested before the first is used (the general kernel
// above walks the window with one load in flight), with 32-bit index arithmetic. Needs channels % 4 == 0
// and fewer than 2^32 bytes on either side; the host checks.
// MODE as for the reductions (0 float sum, 1 float max, 2 whatever op and type say): with the combine chosen at run
// time every one of a thread's 32 combines went through the branches of red_combine, 336 branches per wave.
template <int KH, int KW, int MODE>
__device__ __forceinline__ void pool2d_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, const PoolParams& P) {
    const uint32_t e0 = (xcd_contiguous_block() * 256u + threadIdx.x) * 4u;
    if (e0 >= P.n_out) return;
    const uint32_t C = P.out_dims[3], Wo = P.out_dims[2], Ho = P.out_dims[1];
    const uint32_t r = (uint32_t)magic_div((int)e0, P.div_magic[0], P.div_shift[0]);
    const uint32_t c = e0 - r * C;
    const uint32_t q = (uint32_t)magic_div((int)r, P.div_magic[1], P.div_shift[1]);
    const uint32_t wo = r - q * Wo;
    const uint32_t b = (uint32_t)magic_div((int)q, P.div_magic[2], P.div_shift[2]), ho = q - b * Ho;
    const int32_t y0 = (int32_t)(ho * P.stride[1]) - P.pad_low[1], x0 = (int32_t)(wo * P.stride[2]) - P.pad_low[2];
    const uint32_t ident = MODE == 0 ? 0u : MODE == 1 ? 0xFF800000u : red_identity(P.op, P.type);
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(in), 0,
        (int)(P.in_dims[0] * P.in_dims[1] * P.in_dims[2] * P.in_dims[3] * 4u), 0x00020000);
    u32x4 v[KH][KW];
#pragma unroll
    for (int ky = 0; ky < KH; ++ky)
#pragma unroll
        for (int kx = 0; kx < KW; ++kx) {
            const int32_t y = y0 + ky * (int32_t)P.dilation[1], x = x0 + kx * (int32_t)P.dilation[2];
            const bool ok = (uint32_t)y < P.in_dims[1] && (uint32_t)x < P.in_dims[2];
            const uint32_t off = ((b * P.in_dims[1] + (uint32_t)y) * P.in_dims[2] + (uint32_t)x) * C + c;
            v[ky][kx] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, ok ? off * 4u : 0x80000000u, 0, 0);   // out of range reads 0 ...
            if (!ok) v[ky][kx] = u32x4{ident, ident, ident, ident};                                         // ... and counts as the identity
        }
    u32x4 acc = v[0][0];
#pragma unroll
    for (int ky = 0; ky < KH; ++ky)
#pragma unroll
        for (int kx = 0; kx < KW; ++kx) {
            if (ky == 0 && kx == 0) continue;
            acc.x = red_step<MODE>(P.op, P.type, acc.x, v[ky][kx].x);
            acc.y = red_step<MODE>(P.op, P.type, acc.y, v[ky][kx].y);
            acc.z = red_step<MODE>(P.op, P.type, acc.z, v[ky][kx].z);
            acc.w = red_step<MODE>(P.op, P.type, acc.w, v[ky][kx].w);
        }
    *reinterpret_cast<u32x4*>(out + e0) = acc;
}
template <int KH, int KW>
__device__ __forceinline__ void pool2d_dispatch(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, const PoolParams& P) {
    if (P.type == RT_F32 && P.op == RED_MAX) pool2d_body<KH, KW, 1>(out, in, P);
    else if (P.type == RT_F32 && P.op == RED_SUM) pool2d_body<KH, KW, 0>(out, in, P);
    else pool2d_body<KH, KW, 2>(out, in, P);
}
extern "C" __global__ __launch_bounds__(256) void pool2d_3x3_v4(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, PoolParams P) {
    pool2d_dispatch<3, 3>(out, in, P);
}
extern "C" __global__ __launch_bounds__(256) void pool2d_2x2_v4(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, PoolParams P) {
    pool2d_dispatch<2, 2>(out, in, P);
}

extern "C" __global__ __launch_bounds__(256) void pool_v1(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, PoolParams P) {
    pool_body<1>(out, in, P);
}
extern "C" __global__ __launch_bounds__(256) void pool_v4(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, PoolParams P) {
    pool_body<4>(out, in, P);
}

// ---------------------------------------------------------------------------------------------
// select_and_scatter_add: the gradient of a max (or min) pooling. Every window of `operand` selects
// one of its elements (scan in row-major order over the positions inside the array, the first is
// taken, a later one replaces it when !(selected >= candidate), resp. <=); the window's `source`
// value is added at that position. Two passes, no atomics, sums in a fixed order:
//   select_window   one thread per window (four channels with VEC = 4) repeats the scan and stores
//                   the row-major number of the selected tap inside the window (0xFFFFFFFF: the
//                   window lies entirely outside the array);
//   scatter_selected one thread per operand element walks the windows that contain it in row-major
//                   order and adds the source value of those whose selected tap is this element.
// HBM sees the operand once, the result once and the two small window-sized arrays a few times.
// PoolParams: in_dims = operand, out_dims = source / selection, op = RED_MAX (ge) or RED_MIN (le);
// dilation is not used. VEC = 4 has the same conditions as for pooling.
template <int VEC>
__device__ __forceinline__ void select_window_body(uint32_t* __restrict__ sel_out, const uint32_t* __restrict__ operand, const PoolParams& P) {
    const uint64_t e0 = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * VEC;
    if (e0 >= P.n_out) return;
    int32_t o[4];
    {
        uint64_t r = e0;
#pragma unroll
        for (int d = 3; d >= 1; --d) { const uint64_t q = r / P.out_dims[d]; o[d] = (int32_t)(r - q * P.out_dims[d]); r = q; }
        o[0] = (int32_t)r;
    }
    const bool want_max = P.op == RED_MAX;
    float sel[VEC];
    uint32_t pick[VEC];
    bool have = false;
#pragma unroll
    for (int j = 0; j < VEC; ++j) { sel[j] = 0.0f; pick[j] = 0xFFFFFFFFu; }
    const uint32_t w3 = VEC == 4 ? 1u : P.window[3];
    uint32_t tap = 0;
    for (uint32_t t0 = 0; t0 < P.window[0]; ++t0)
    for (uint32_t t1 = 0; t1 < P.window[1]; ++t1)
    for (uint32_t t2 = 0; t2 < P.window[2]; ++t2)
    for (uint32_t t3 = 0; t3 < w3; ++t3, ++tap) {
        const int32_t k0 = o[0] * (int32_t)P.stride[0] - P.pad_low[0] + (int32_t)t0;
        const int32_t k1 = o[1] * (int32_t)P.stride[1] - P.pad_low[1] + (int32_t)t1;
        const int32_t k2 = o[2] * (int32_t)P.stride[2] - P.pad_low[2] + (int32_t)t2;
        const int32_t k3 = VEC == 4 ? o[3] : o[3] * (int32_t)P.stride[3] - P.pad_low[3] + (int32_t)t3;
        if ((uint32_t)k0 >= P.in_dims[0] || (uint32_t)k1 >= P.in_dims[1] || (uint32_t)k2 >= P.in_dims[2] || (uint32_t)k3 >= P.in_dims[3]) continue;
        const uint64_t off = (((uint64_t)k0 * P.in_dims[1] + k1) * P.in_dims[2] + k2) * P.in_dims[3] + k3;
        float v[VEC];
        if constexpr (VEC == 4) {
            const u32x4 q = *reinterpret_cast<const u32x4*>(operand + off);
            v[0] = u2f(q.x); v[1] = u2f(q.y); v[2] = u2f(q.z); v[3] = u2f(q.w);
        } else {
            v[0] = u2f(operand[off]);
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            const bool keep = have && (want_max ? sel[j] >= v[j] : sel[j] <= v[j]);
            if (!keep) { sel[j] = v[j]; pick[j] = tap; }
        }
        have = true;
    }
    if constexpr (VEC == 4) *reinterpret_cast<u32x4*>(sel_out + e0) = u32x4{pick[0], pick[1], pick[2], pick[3]};
    else sel_out[e0] = pick[0];
}

template <int VEC>
__device__ __forceinline__ void scatter_selected_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ source,
                                                      const uint32_t* __restrict__ selected, const PoolParams& P) {
    const uint64_t e0 = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * VEC;
    if (e0 >= without_stream_bit(P.n_out)) return;
    int32_t c[4];
    {
        uint64_t r = e0;
#pragma unroll
        for (int d = 3; d >= 1; --d) { const uint64_t q = r / P.in_dims[d]; c[d] = (int32_t)(r - q * P.in_dims[d]); r = q; }
        c[0] = (int32_t)r;
    }
    // windows that contain the element: o * stride - pad <= c < o * stride - pad + window
    int32_t lo[4], hi[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const int32_t s = (int32_t)P.stride[d], a = c[d] + P.pad_low[d];
        const int32_t first = a - (int32_t)P.window[d] + 1;
        lo[d] = first <= 0 ? 0 : div_stride(first + s - 1, s);
        hi[d] = a < 0 ? -1 : div_stride(a, s);
        if (hi[d] > (int32_t)P.out_dims[d] - 1) hi[d] = (int32_t)P.out_dims[d] - 1;
    }
    if constexpr (VEC == 4) { lo[3] = hi[3] = 0; }           // the last dimension is not windowed: handled per lane element
    const uint32_t w3 = VEC == 4 ? 1u : P.window[3];
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0.0f;
    for (int32_t o0 = lo[0]; o0 <= hi[0]; ++o0)
    for (int32_t o1 = lo[1]; o1 <= hi[1]; ++o1)
    for (int32_t o2 = lo[2]; o2 <= hi[2]; ++o2)
    for (int32_t o3 = lo[3]; o3 <= hi[3]; ++o3) {
        // this element's tap number inside the window
        const uint32_t t0 = (uint32_t)(c[0] + P.pad_low[0] - o0 * (int32_t)P.stride[0]);
        const uint32_t t1 = (uint32_t)(c[1] + P.pad_low[1] - o1 * (int32_t)P.stride[1]);
        const uint32_t t2 = (uint32_t)(c[2] + P.pad_low[2] - o2 * (int32_t)P.stride[2]);
        const uint32_t t3 = VEC == 4 ? 0u : (uint32_t)(c[3] + P.pad_low[3] - o3 * (int32_t)P.stride[3]);
        const uint32_t tap = ((t0 * P.window[1] + t1) * P.window[2] + t2) * w3 + t3;
        const uint64_t woff = (((uint64_t)o0 * P.out_dims[1] + o1) * P.out_dims[2] + o2) * P.out_dims[3] + (VEC == 4 ? c[3] : o3);
        if constexpr (VEC == 4) {
            const u32x4 s = *reinterpret_cast<const u32x4*>(selected + woff);
            const u32x4 g = *reinterpret_cast<const u32x4*>(source + woff);
            if (s.x == tap) acc[0] += u2f(g.x);
            if (s.y == tap) acc[1] += u2f(g.y);
            if (s.z == tap) acc[2] += u2f(g.z);
            if (s.w == tap) acc[3] += u2f(g.w);
        } else {
            if (selected[woff] == tap) acc[0] += u2f(source[woff]);
        }
    }
    if constexpr (VEC == 4) {
        u32x4 r; r.x = f2u(acc[0]); r.y = f2u(acc[1]); r.z = f2u(acc[2]); r.w = f2u(acc[3]);
        store_x4(out, e0, r, streams_result(P.n_out), without_stream_bit(P.n_out) * 4u);
    } else {
        out[e0] = f2u(acc[0]);
    }
}

// The usual pooling layout, [batch, y, x, channels] with a KH x KW window over y and x only and float data: the two
// passes with everything a thread reads requested before the first value is looked at, 32-bit index arithmetic and
// contiguous block ranges per XCD, like pool2d above (the general kernels walk their windows one load at a time:
// 69 + 115 us for the gradient of a 3 x 3 / 2 max pool over 64 x 112 x 112 x 64, where the pool itself takes 34).
// Same selections and the same sums in the same order as the general kernels. Needs channels % 4 == 0 and fewer than
// 2^31 bytes on either side; the host checks.
template <int KH, int KW>
__device__ __forceinline__ void select_window2d_body(uint32_t* __restrict__ sel_out, const uint32_t* __restrict__ operand, const PoolParams& P) {
    const uint32_t e0 = (xcd_contiguous_block() * 256u + threadIdx.x) * 4u;
    if (e0 >= P.n_out) return;
    const uint32_t C = P.out_dims[3], Wo = P.out_dims[2], Ho = P.out_dims[1];
    const uint32_t r = (uint32_t)magic_div((int)e0, P.div_magic[0], P.div_shift[0]);
    const uint32_t c = e0 - r * C;
    const uint32_t q = (uint32_t)magic_div((int)r, P.div_magic[1], P.div_shift[1]);
    const uint32_t wo = r - q * Wo;
    const uint32_t b = (uint32_t)magic_div((int)q, P.div_magic[2], P.div_shift[2]), ho = q - b * Ho;
    const int32_t y0 = (int32_t)(ho * P.stride[1]) - P.pad_low[1], x0 = (int32_t)(wo * P.stride[2]) - P.pad_low[2];
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(operand), 0,
        (int)(P.in_dims[0] * P.in_dims[1] * P.in_dims[2] * P.in_dims[3] * 4u), 0x00020000);
    u32x4 v[KH][KW];
    bool inside[KH][KW];
#pragma unroll
    for (int ky = 0; ky < KH; ++ky)
#pragma unroll
        for (int kx = 0; kx < KW; ++kx) {
            const int32_t y = y0 + ky, x = x0 + kx;
            inside[ky][kx] = (uint32_t)y < P.in_dims[1] && (uint32_t)x < P.in_dims[2];
            const uint32_t off = ((b * P.in_dims[1] + (uint32_t)y) * P.in_dims[2] + (uint32_t)x) * C + c;
            v[ky][kx] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, inside[ky][kx] ? off * 4u : 0x80000000u, 0, 0);
        }
    const bool want_max = P.op == RED_MAX;
    float sel[4] = {0.f, 0.f, 0.f, 0.f};
    uint32_t pick[4] = {0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu};
    bool have = false;
#pragma unroll
    for (int ky = 0; ky < KH; ++ky)
#pragma unroll
        for (int kx = 0; kx < KW; ++kx) {
            // positions outside the array are not candidates (selects, no branches: the loads stay in flight together)
            const float q[4] = {u2f(v[ky][kx].x), u2f(v[ky][kx].y), u2f(v[ky][kx].z), u2f(v[ky][kx].w)};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool keep = have && (want_max ? sel[j] >= q[j] : sel[j] <= q[j]);
                const bool take = inside[ky][kx] && !keep;
                sel[j]  = take ? q[j] : sel[j];
                pick[j] = take ? (uint32_t)(ky * KW + kx) : pick[j];
            }
            have = have || inside[ky][kx];
        }
    // a thread's four selections share one word, a byte each (0xFF: an empty window), word number e0 / 4: a quarter of the
    // bytes to write here and to read in the launch that follows
    sel_out[e0 >> 2] = (pick[0] & 255u) | (pick[1] & 255u) << 8 | (pick[2] & 255u) << 16 | (pick[3] & 255u) << 24;
}

// NY x NX: the most windows an element can lie in, ceil(window / stride) per dimension (the host picks the variant):
// loads for windows that do not exist read nothing, but nine pairs of them where four would do cost a third more time.
template <int KH, int KW, int NY, int NX>
__device__ __forceinline__ void scatter_selected2d_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ source,
                                                        const uint32_t* __restrict__ selected, const PoolParams& P) {
    const uint32_t e0 = (xcd_contiguous_block() * 256u + threadIdx.x) * 4u, n_out = without_stream_bit(P.n_out);
    if (e0 >= n_out) return;
    const uint32_t C = P.in_dims[3], W = P.in_dims[2], H = P.in_dims[1];
    const uint32_t r = (uint32_t)magic_div((int)e0, P.div_magic[0], P.div_shift[0]);
    const uint32_t c = e0 - r * C;
    const uint32_t q = (uint32_t)magic_div((int)r, P.div_magic[1], P.div_shift[1]);
    const uint32_t x = r - q * W;
    const uint32_t b = (uint32_t)magic_div((int)q, P.div_magic[2], P.div_shift[2]), y = q - b * H;
    // windows that contain the element: o * stride - pad <= coordinate < o * stride - pad + window; at most KH x KW of them
    int32_t lo[2], hi[2];
#pragma unroll
    for (int d = 0; d < 2; ++d) {
        const int32_t s = (int32_t)P.stride[d + 1], a = (int32_t)(d ? x : y) + P.pad_low[d + 1];
        const int32_t first = a - (d ? KW : KH) + 1;
        lo[d] = first <= 0 ? 0 : div_stride(first + s - 1, s);
        hi[d] = a < 0 ? -1 : div_stride(a, s);
        if (hi[d] > (int32_t)P.out_dims[d + 1] - 1) hi[d] = (int32_t)P.out_dims[d + 1] - 1;
    }
    const uint32_t nwin_bytes = P.out_dims[0] * P.out_dims[1] * P.out_dims[2] * P.out_dims[3] * 4u;
    const __amdgpu_buffer_rsrc_t r_sel = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(selected), 0, (int)nwin_bytes, 0x00020000),
                                 r_src = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(source), 0, (int)nwin_bytes, 0x00020000);
    uint32_t s[NY][NX];                  // the selections of four channels, a byte each (select_window2d_body)
    u32x4 g[NY][NX];
    uint32_t tap[NY][NX];
#pragma unroll
    for (int i = 0; i < NY; ++i)
#pragma unroll
        for (int j = 0; j < NX; ++j) {
            const int32_t oy = lo[0] + i, ox = lo[1] + j;
            const bool ok = oy <= hi[0] && ox <= hi[1];
            // this element's tap number inside that window (no window: a number no selection holds)
            tap[i][j] = ok ? (uint32_t)(((int32_t)y + P.pad_low[1] - oy * (int32_t)P.stride[1]) * KW + ((int32_t)x + P.pad_low[2] - ox * (int32_t)P.stride[2]))
                           : 0xFEu;
            const uint32_t off = ((b * P.out_dims[1] + (uint32_t)oy) * P.out_dims[2] + (uint32_t)ox) * C + c;
            s[i][j] = __builtin_amdgcn_raw_buffer_load_b32(r_sel, ok ? off : 0x80000000u, 0, 0);       // word off / 4
            g[i][j] = __builtin_amdgcn_raw_buffer_load_b128(r_src, ok ? off * 4u : 0x80000000u, 0, 0);
        }
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < NY; ++i)
#pragma unroll
        for (int j = 0; j < NX; ++j) {
            if ((s[i][j] & 255u) == tap[i][j])         acc[0] += u2f(g[i][j].x);
            if ((s[i][j] >> 8 & 255u) == tap[i][j])    acc[1] += u2f(g[i][j].y);
            if ((s[i][j] >> 16 & 255u) == tap[i][j])   acc[2] += u2f(g[i][j].z);
            if ((s[i][j] >> 24) == tap[i][j])          acc[3] += u2f(g[i][j].w);
        }
    store_x4(out, e0, u32x4{f2u(acc[0]), f2u(acc[1]), f2u(acc[2]), f2u(acc[3])}, streams_result(P.n_out), n_out * 4u);
}

// 3 x 3 windows at a stride of 2 in both directions, the usual pooling of a network's stem: a thread owns the 2 x 2
// elements (by four channels) whose padded coordinates are (2t, 2t + 1) x (2u, 2u + 1). Those four lie in the windows
// (t - 1 .. t) x (u - 1 .. u) and in no other, each at a fixed tap: four (selection, source) pairs serve four results,
// where one thread per element reads up to four pairs for one. Same sums in the same order (windows ascending).
// P.n_out counts the elements of the array of such groups, [batch, T, U, channels]; P.div_magic divides by channels, U, T.
__device__ __forceinline__ void scatter_selected2d_3x3_s2_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ source,
                                                               const uint32_t* __restrict__ selected, const PoolParams& P) {
    const uint32_t e0 = (xcd_contiguous_block() * 256u + threadIdx.x) * 4u, n_groups = without_stream_bit(P.n_out);
    if (e0 >= n_groups) return;
    const uint32_t C = P.in_dims[3], W = P.in_dims[2], H = P.in_dims[1];
    const int32_t py = P.pad_low[1], px = P.pad_low[2];
    const uint32_t t0 = (uint32_t)py >> 1, u0 = (uint32_t)px >> 1;
    const uint32_t T = ((H + (uint32_t)py - 1u) >> 1) - t0 + 1u, U = ((W + (uint32_t)px - 1u) >> 1) - u0 + 1u;
    const uint32_t r = (uint32_t)magic_div((int)e0, P.div_magic[0], P.div_shift[0]);
    const uint32_t c = e0 - r * C;
    const uint32_t q = (uint32_t)magic_div((int)r, P.div_magic[1], P.div_shift[1]);
    const uint32_t b = (uint32_t)magic_div((int)q, P.div_magic[2], P.div_shift[2]);
    const int32_t t = (int32_t)(q - b * T + t0), u = (int32_t)(r - q * U + u0);
    const uint32_t nwin_bytes = P.out_dims[0] * P.out_dims[1] * P.out_dims[2] * P.out_dims[3] * 4u;
    const __amdgpu_buffer_rsrc_t r_sel = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(selected), 0, (int)nwin_bytes, 0x00020000),
                                 r_src = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(source), 0, (int)nwin_bytes, 0x00020000);
    uint32_t s[2][2];                    // the selections of four channels, a byte each; 0xFF.. where there is no such window
    u32x4 g[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int32_t oy = t - 1 + i, ox = u - 1 + j;
            const bool ok = (uint32_t)oy < P.out_dims[1] && (uint32_t)ox < P.out_dims[2];
            const uint32_t off = ((b * P.out_dims[1] + (uint32_t)oy) * P.out_dims[2] + (uint32_t)ox) * C + c;
            const uint32_t word = __builtin_amdgcn_raw_buffer_load_b32(r_sel, ok ? off : 0x80000000u, 0, 0);       // word off / 4
            s[i][j] = ok ? word : 0xFFFFFFFFu;
            g[i][j] = __builtin_amdgcn_raw_buffer_load_b128(r_src, ok ? off * 4u : 0x80000000u, 0, 0);
        }
    // element (dy, dx) of the group holds tap (dy + 2 - 2 i, dx + 2 - 2 j) of window (i, j), where that is a tap (< 3)
    const uint32_t result_bytes = P.in_dims[0] * H * W * C * 4u;
    const bool stream = streams_result(P.n_out);
#pragma unroll
    for (int dy = 0; dy < 2; ++dy)
#pragma unroll
        for (int dx = 0; dx < 2; ++dx) {
            const int32_t y = 2 * t + dy - py, x = 2 * u + dx - px;
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int ky = dy + 2 - 2 * i, kx = dx + 2 - 2 * j;
                    if (ky > 2 || kx > 2) continue;
                    const uint32_t tap = (uint32_t)(ky * 3 + kx);
                    if ((s[i][j] & 255u) == tap)       acc[0] += u2f(g[i][j].x);
                    if ((s[i][j] >> 8 & 255u) == tap)  acc[1] += u2f(g[i][j].y);
                    if ((s[i][j] >> 16 & 255u) == tap) acc[2] += u2f(g[i][j].z);
                    if ((s[i][j] >> 24) == tap)        acc[3] += u2f(g[i][j].w);
                }
            if ((uint32_t)y < H && (uint32_t)x < W)
                store_x4(out, ((uint64_t)(b * H + (uint32_t)y) * W + (uint32_t)x) * C + c,
                         u32x4{f2u(acc[0]), f2u(acc[1]), f2u(acc[2]), f2u(acc[3])}, stream, result_bytes);
        }
}
extern "C" __global__ __launch_bounds__(256) void scatter_selected2d_3x3_s2_v4(uint32_t* __restrict__ out, const uint32_t* __restrict__ source,
                                                                              const uint32_t* __restrict__ selected, PoolParams P) {
    scatter_selected2d_3x3_s2_body(out, source, selected, P);
}

#define SELECT_WINDOW_2D(KH, KW)                                                                                                    \
    extern "C" __global__ __launch_bounds__(256) void select_window2d_##KH##x##KW##_v4(uint32_t* __restrict__ sel,                   \
                                                                                      const uint32_t* __restrict__ operand, PoolParams P) { \
        select_window2d_body<KH, KW>(sel, operand, P);                                                                              \
    }
#define SCATTER_SELECTED_2D(KH, KW, NY, NX)                                                                                         \
    extern "C" __global__ __launch_bounds__(256) void scatter_selected2d_##KH##x##KW##_n##NY##x##NX##_v4(uint32_t* __restrict__ out, \
            const uint32_t* __restrict__ source, const uint32_t* __restrict__ selected, PoolParams P) {                             \
        scatter_selected2d_body<KH, KW, NY, NX>(out, source, selected, P);                                                          \
    }
SELECT_WINDOW_2D(3, 3)
SELECT_WINDOW_2D(2, 2)
// 3 x 3 windows with strides of 1 (3 x 3 windows per element), 2 (2 x 2) and more (1 x 1); 2 x 2 windows with strides of 1 and more
SCATTER_SELECTED_2D(3, 3, 3, 3)
SCATTER_SELECTED_2D(3, 3, 2, 2)
SCATTER_SELECTED_2D(3, 3, 1, 1)
SCATTER_SELECTED_2D(2, 2, 2, 2)
SCATTER_SELECTED_2D(2, 2, 1, 1)

extern "C" __global__ __launch_bounds__(256) void select_window_v1(uint32_t* __restrict__ sel, const uint32_t* __restrict__ operand, PoolParams P) {
    select_window_body<1>(sel, operand, P);
}
extern "C" __global__ __launch_bounds__(256) void select_window_v4(uint32_t* __restrict__ sel, const uint32_t* __restrict__ operand, PoolParams P) {
    select_window_body<4>(sel, operand, P);
}
extern "C" __global__ __launch_bounds__(256) void scatter_selected_v1(uint32_t* __restrict__ out, const uint32_t* __restrict__ source,
                                                                      const uint32_t* __restrict__ selected, PoolParams P) {
    scatter_selected_body<1>(out, source, selected, P);
}
extern "C" __global__ __launch_bounds__(256) void scatter_selected_v4(uint32_t* __restrict__ out, const uint32_t* __restrict__ source,
                                                                      const uint32_t* __restrict__ selected, PoolParams P) {
    scatter_selected_body<4>(out, source, selected, P);
}
