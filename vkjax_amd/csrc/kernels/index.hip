// gather and scatter-add.
//
// gather_rows / scatter_add_rows cover the table-lookup pattern (one index per row, whole rows
// moved): consecutive lanes move consecutive 16-byte pieces of a row, so both the table side
// and the dense side are coalesced. gather_general / scatter_add_general implement the full
// XLA dimension-number rules, one thread per output / update element.
// They supersede gather.comp, scatter0.comp and scatter1.comp (reference: vkjax/ops.py:372-433;
// vkjax/shaders/gather.comp:62-103). Unlike the reference shader, gather clamps start indices
// so that the slice stays inside the operand, and scatter-add drops windows that do not fit,
// which is what XLA does.
#include "common.h"

#define IDX_MAX_RANK 6

struct GatherRowsParams { uint32_t n_idx, row_len, n_rows, idx_stride; };

// out[i, :] = table[clamp(idx[i*idx_stride]), :]
template <int VEC>
__device__ __forceinline__ void gather_rows_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ table,
                                                 const int32_t* __restrict__ idx, const GatherRowsParams& P) {
    const uint32_t vpr = P.row_len / VEC;
    const uint64_t q = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (q >= (uint64_t)P.n_idx * vpr) return;
    const uint32_t i = (uint32_t)(q / vpr), c = (uint32_t)(q - (uint64_t)i * vpr) * VEC;
    int32_t r = idx[(uint64_t)i * P.idx_stride];
    r = r < 0 ? 0 : (r > (int32_t)P.n_rows - 1 ? (int32_t)P.n_rows - 1 : r);
    const uint32_t* src = table + (uint64_t)r * P.row_len + c;
    uint32_t* dst = out + (uint64_t)i * P.row_len + c;
    if constexpr (VEC == 4) *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(src);
    else *dst = *src;
}

extern "C" __global__ __launch_bounds__(256) void gather_rows_v1(uint32_t* out, const uint32_t* table, const int32_t* idx, GatherRowsParams P) {
    gather_rows_body<1>(out, table, idx, P);
}
extern "C" __global__ __launch_bounds__(256) void gather_rows_v4(uint32_t* out, const uint32_t* table, const int32_t* idx, GatherRowsParams P) {
    gather_rows_body<4>(out, table, idx, P);
}

struct GatherGeneralParams {
    uint32_t n_out, out_rank, op_rank, n_index;       // n_index = size of the last indices dimension
    uint32_t out_dims[IDX_MAX_RANK];
    uint32_t out_is_offset[IDX_MAX_RANK];             // 1 if the output dim enumerates a slice position
    uint32_t op_dims[IDX_MAX_RANK];
    uint32_t op_strides[IDX_MAX_RANK];
    uint32_t slice_sizes[IDX_MAX_RANK];
    uint32_t op_collapsed[IDX_MAX_RANK];              // 1 if the operand dim is collapsed (slice size 1, no output dim)
    uint32_t start_index_map[IDX_MAX_RANK];           // indices component k -> operand dim
    uint32_t batch_dims[IDX_MAX_RANK];                // sizes of indices.shape[:-1] (row-major), padded with 1
    uint32_t n_batch_dims;
};

extern "C" __global__ __launch_bounds__(256) void gather_general(uint32_t* __restrict__ out, const uint32_t* __restrict__ operand,
                                                                 const int32_t* __restrict__ indices, GatherGeneralParams P) {
    const uint32_t e = blockIdx.x * 256u + threadIdx.x;
    if (e >= P.n_out) return;
    uint32_t oc[IDX_MAX_RANK];
    {
        uint32_t r = e;
        for (int d = (int)P.out_rank - 1; d >= 0; --d) { const uint32_t q = r / P.out_dims[d]; oc[d] = r - q * P.out_dims[d]; r = q; }
    }
    // batch position (row-major over the non-offset output dims) and the offsets inside the slice
    uint32_t batch = 0, offs[IDX_MAX_RANK], noffs = 0;
    for (uint32_t d = 0, b = 0; d < P.out_rank; ++d) {
        if (P.out_is_offset[d]) offs[noffs++] = oc[d];
        else { batch = batch * P.batch_dims[b] + oc[d]; ++b; }
    }
    int32_t start[IDX_MAX_RANK];
    for (uint32_t d = 0; d < P.op_rank; ++d) start[d] = 0;
    for (uint32_t k = 0; k < P.n_index; ++k) {
        const uint32_t d = P.start_index_map[k];
        int32_t s = indices[(uint64_t)batch * P.n_index + k];
        const int32_t hi = (int32_t)P.op_dims[d] - (int32_t)P.slice_sizes[d];
        start[d] = s < 0 ? 0 : (s > hi ? hi : s);
    }
    uint64_t off = 0;
    for (uint32_t d = 0, j = 0; d < P.op_rank; ++d) {
        uint32_t c = (uint32_t)start[d];
        if (!P.op_collapsed[d]) c += offs[j++];
        off += (uint64_t)c * P.op_strides[d];
    }
    out[e] = operand[off];
}

struct ScatterRowsParams { uint32_t n_idx, row_len, n_rows, idx_stride, is_float; };

// out[idx[i], :] += updates[i, :]   (out already holds the operand)
extern "C" __global__ __launch_bounds__(256) void scatter_add_rows(uint32_t* __restrict__ out, const int32_t* __restrict__ idx,
                                                                   const uint32_t* __restrict__ updates, ScatterRowsParams P) {
    const uint64_t q = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (q >= (uint64_t)P.n_idx * P.row_len) return;
    const uint32_t i = (uint32_t)(q / P.row_len), c = (uint32_t)(q - (uint64_t)i * P.row_len);
    const int32_t r = idx[(uint64_t)i * P.idx_stride];
    if (r < 0 || r >= (int32_t)P.n_rows) return;
    const uint32_t u = updates[q];
    uint32_t* dst = out + (uint64_t)r * P.row_len + c;
    if (P.is_float) unsafeAtomicAdd(reinterpret_cast<float*>(dst), u2f(u));
    else atomicAdd(dst, u);
}

// ---------------------------------------------------------------------------------------------
// scatter-add of whole rows without atomics on the data: the update rows are bucketed by target
// row with a counting sort of their indices (three small launches over the indices), then one
// wave per table row adds up its updates, in ascending update order, on top of the operand row and
// writes the result once. Every update row is read exactly once, the table is read once and
// written once, and the sum does not depend on the order in which threads happen to run (rows
// that receive more than 64 updates are summed in blocks of 64, each block in ascending order).
struct ScatterSortParams { uint32_t n_idx, row_len, n_rows, idx_stride; };

// count[r + 1] += 1 for every in-range index; count has n_rows + 1 words and starts at zero
extern "C" __global__ __launch_bounds__(256) void scatter_rows_count(uint32_t* __restrict__ count, const int32_t* __restrict__ idx,
                                                                     ScatterSortParams P) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= P.n_idx) return;
    const int32_t r = idx[(uint64_t)i * P.idx_stride];
    if (r < 0 || r >= (int32_t)P.n_rows) return;          // updates outside the operand are dropped
    atomicAdd(count + r + 1, 1u);
}

// in-place inclusive prefix sum over n words by one block: afterwards word r is the number of
// updates that go to rows before r, i.e. where row r's bucket starts. The block walks the array
// in tiles of 1024 x 16 words; a thread scans 16 consecutive words, the 1024 thread totals are
// scanned with wave shuffles and one exchange through LDS, and a running carry links the tiles.
extern "C" __global__ __launch_bounds__(1024) void scatter_rows_scan(uint32_t* __restrict__ data, uint32_t n) {
    __shared__ uint32_t wave_total[16];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint32_t carry = 0;
    for (uint32_t tile = 0; tile < n; tile += 1024u * 16u) {
        const uint32_t base = tile + threadIdx.x * 16u;
        uint32_t v[16];
        if (base + 16u <= n) {                                   // 64 aligned bytes per thread
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const u32x4 t4 = *reinterpret_cast<const u32x4*>(data + base + 4 * q);
                v[4 * q] = t4.x; v[4 * q + 1] = t4.y; v[4 * q + 2] = t4.z; v[4 * q + 3] = t4.w;
            }
        } else {
#pragma unroll
            for (int q = 0; q < 16; ++q) v[q] = base + q < n ? data[base + q] : 0u;
        }
#pragma unroll
        for (int q = 1; q < 16; ++q) v[q] += v[q - 1];
        // inclusive scan of the thread totals across the wave
        uint32_t t = v[15];
#pragma unroll
        for (uint32_t off = 1; off < 64u; off <<= 1) {
            const uint32_t up = __shfl_up(t, off, 64);
            if (lane >= off) t += up;
        }
        if (lane == 63u) wave_total[wave] = t;
        __syncthreads();
        uint32_t before = carry;                                 // everything before this thread's 16 words
        for (uint32_t w = 0; w < wave; ++w) before += wave_total[w];
        before += t - v[15];
        uint32_t tile_total = 0;
        for (uint32_t w = 0; w < 16u; ++w) tile_total += wave_total[w];
        __syncthreads();                                         // wave_total is rewritten by the next tile
        if (base + 16u <= n) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                u32x4 t4;
                t4.x = v[4 * q] + before; t4.y = v[4 * q + 1] + before; t4.z = v[4 * q + 2] + before; t4.w = v[4 * q + 3] + before;
                *reinterpret_cast<u32x4*>(data + base + 4 * q) = t4;
            }
        } else {
#pragma unroll
            for (int q = 0; q < 16; ++q)
                if (base + q < n) data[base + q] = v[q] + before;
        }
        carry += tile_total;
    }
}

// order[start[r] + k] = i for the k-th update (in order of arrival) whose index is r; cursor starts at zero
extern "C" __global__ __launch_bounds__(256) void scatter_rows_fill(uint32_t* __restrict__ order, uint32_t* __restrict__ cursor,
                                                                    const uint32_t* __restrict__ start, const int32_t* __restrict__ idx,
                                                                    ScatterSortParams P) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= P.n_idx) return;
    const int32_t r = idx[(uint64_t)i * P.idx_stride];
    if (r < 0 || r >= (int32_t)P.n_rows) return;
    order[start[r] + atomicAdd(cursor + r, 1u)] = i;
}

// ascending bitonic sort of one value per lane across the wave
__device__ __forceinline__ uint32_t wave_sort(uint32_t e, uint32_t lane) {
#pragma unroll
    for (uint32_t k = 2; k <= 64u; k <<= 1) {
#pragma unroll
        for (uint32_t j = k >> 1; j > 0; j >>= 1) {
            const uint32_t partner = __shfl_xor(e, j, 64);
            const bool keep_min = ((lane & k) == 0u) == ((lane & j) == 0u);
            e = keep_min ? min(e, partner) : max(e, partner);
        }
    }
    return e;
}

// out[r, :] = operand[r, :] + sum over the updates i in row r's bucket of updates[i, :].
// One wave takes 4 consecutive rows. Their buckets are adjacent in `order`, so one load fetches
// them all (up to 64 entries, the usual case); they are sorted together under the key
// (row, update number), and all the rows' loads of operand and update data are in flight together.
// A wave whose rows hold more than 64 entries falls back to one row at a time, 64 entries at a time.
// Update numbers are below 2^30 (the host sees to that).
#define SCATTER_ROWS_PER_WAVE 4
template <int VEC, bool IS_FLOAT>
__device__ __forceinline__ void scatter_rows_sum_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ operand,
                                                      const uint32_t* __restrict__ updates, const uint32_t* __restrict__ start,
                                                      const uint32_t* __restrict__ order, const ScatterSortParams& P) {
    constexpr int ROWS = SCATTER_ROWS_PER_WAVE;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t r0 = (blockIdx.x * 4u + (threadIdx.x >> 6)) * ROWS;
    if (r0 >= P.n_rows) return;
    auto add = [](uint32_t a, uint32_t b) -> uint32_t { return IS_FLOAT ? f2u(u2f(a) + u2f(b)) : a + b; };
    // bucket boundaries: s[j] .. s[j + 1] for row r0 + j (rows beyond the table get empty buckets)
    const uint32_t sv = start[min(r0 + lane, P.n_rows)];
    uint32_t s[ROWS + 1];
#pragma unroll
    for (int j = 0; j <= ROWS; ++j) s[j] = __builtin_amdgcn_readlane(sv, j);
    const uint32_t total = s[ROWS] - s[0];

    auto load_row = [&](const uint32_t* base, uint32_t row, uint32_t c, uint32_t (&dst)[VEC]) {
        if constexpr (VEC == 4) {
            const u32x4 t = *reinterpret_cast<const u32x4*>(base + (uint64_t)row * P.row_len + c);
            dst[0] = t.x; dst[1] = t.y; dst[2] = t.z; dst[3] = t.w;
        } else {
            dst[0] = base[(uint64_t)row * P.row_len + c];
        }
    };
    auto store_row = [&](uint32_t row, uint32_t c, const uint32_t (&src)[VEC]) {
        if constexpr (VEC == 4) {
            u32x4 t; t.x = src[0]; t.y = src[1]; t.z = src[2]; t.w = src[3];
            *reinterpret_cast<u32x4*>(out + (uint64_t)row * P.row_len + c) = t;
        } else {
            out[(uint64_t)row * P.row_len + c] = src[0];
        }
    };
    // acc += updates[e(k), c ...] for k in [k0, k1), four rows requested at a time and added in order;
    // e holds the (sorted) update numbers, one per lane
    auto accumulate = [&](uint32_t e, uint32_t k0, uint32_t k1, uint32_t c, bool live, uint32_t (&acc)[VEC]) {
        for (uint32_t k = k0; k < k1; k += 4u) {
            uint32_t t[4][VEC];
#pragma unroll
            for (uint32_t q = 0; q < 4u; ++q)
                if (k + q < k1 && live) load_row(updates, __builtin_amdgcn_readlane(e, k + q) & 0x3FFFFFFFu, c, t[q]);
#pragma unroll
            for (uint32_t q = 0; q < 4u; ++q)
                if (k + q < k1 && live) {
#pragma unroll
                    for (int v = 0; v < VEC; ++v) acc[v] = add(acc[v], t[q][v]);
                }
        }
    };

    if (total <= 64u) {
        uint32_t e = 0xFFFFFFFFu;
        if (lane < total) {
            uint32_t row = 0;
#pragma unroll
            for (int j = 1; j < ROWS; ++j) row += lane >= s[j] - s[0] ? 1u : 0u;
            e = order[s[0] + lane] | row << 30;
        }
        if (total > 1u) e = wave_sort(e, lane);
        for (uint32_t c0 = 0; c0 < P.row_len; c0 += 64u * VEC) {
            const uint32_t c = c0 + lane * VEC;
            const bool live = c < P.row_len;                   // row_len is a multiple of VEC
            uint32_t acc[ROWS][VEC];
#pragma unroll
            for (int j = 0; j < ROWS; ++j)
                if (live && r0 + j < P.n_rows) load_row(operand, r0 + j, c, acc[j]);
#pragma unroll
            for (int j = 0; j < ROWS; ++j) accumulate(e, s[j] - s[0], s[j + 1] - s[0], c, live, acc[j]);
#pragma unroll
            for (int j = 0; j < ROWS; ++j)
                if (live && r0 + j < P.n_rows) store_row(r0 + j, c, acc[j]);
        }
    } else {
        for (uint32_t j = 0; j < (uint32_t)ROWS && r0 + j < P.n_rows; ++j) {
            const uint32_t begin = __builtin_amdgcn_readlane(sv, j), end = __builtin_amdgcn_readlane(sv, j + 1);
            for (uint32_t c0 = 0; c0 < P.row_len; c0 += 64u * VEC) {
                const uint32_t c = c0 + lane * VEC;
                const bool live = c < P.row_len;
                uint32_t acc[VEC];
                if (live) load_row(operand, r0 + j, c, acc);
                for (uint32_t b0 = begin; b0 < end; b0 += 64u) {
                    const uint32_t cnt = min(64u, end - b0);
                    uint32_t e = lane < cnt ? order[b0 + lane] : 0xFFFFFFFFu;
                    if (cnt > 1u) e = wave_sort(e, lane);
                    accumulate(e, 0u, cnt, c, live, acc);
                }
                if (live) store_row(r0 + j, c, acc);
            }
        }
    }
}

#define SCATTER_SUM_KERNEL(name, VEC, IS_FLOAT)                                                                   \
    extern "C" __global__ __launch_bounds__(256) void name(uint32_t* out, const uint32_t* operand, const uint32_t* updates, \
                                                           const uint32_t* start, const uint32_t* order, ScatterSortParams P) { \
        scatter_rows_sum_body<VEC, IS_FLOAT>(out, operand, updates, start, order, P);                              \
    }
// the _v4 variants require row_len % 4 == 0 and 16-byte aligned data pointers
SCATTER_SUM_KERNEL(scatter_rows_sum_f_v1, 1, true)
SCATTER_SUM_KERNEL(scatter_rows_sum_f_v4, 4, true)
SCATTER_SUM_KERNEL(scatter_rows_sum_i_v1, 1, false)
SCATTER_SUM_KERNEL(scatter_rows_sum_i_v4, 4, false)

// ---------------------------------------------------------------------------------------------
// scatter-add of whole rows in ONE launch, no scratch memory, no atomics on the data ("owner
// computes"): a workgroup owns `rows_per_group` consecutive table rows. It reads the whole index
// array once (from L2: the array is a few hundred KB to a few MB and every workgroup reads it),
// keeps the updates that fall into its rows as keys (row within the group << 22 | update number)
// in LDS, sorts the keys, and then each wave adds up the updates of one row after the other, in
// ascending update order, on top of the operand row (or of a single value, when the operand is a
// constant filled with one value) and writes the result row once. Every update row is read exactly
// once, the table is written once, and the result does not depend on thread timing.
// A workgroup whose rows receive more keys than LDS holds works through the index array in
// several rounds, each taking as many consecutive indices as fit, adding onto what it has written.
// Needs n_idx <= 2^22 and rows_per_group <= 1024 (the host sees to that).
struct ScatterOwnerParams { uint32_t n_idx, row_len, n_rows, idx_stride, rows_per_group, operand_is_scalar; };

#define SCATTER_OWNER_CAP     4096u     // keys a workgroup holds in LDS
#define SCATTER_OWNER_THREADS 1024u
#define SCATTER_OWNER_INFLIGHT 8        // update rows a wave requests before it adds them

template <int VEC, bool IS_FLOAT>
__device__ __forceinline__ void scatter_rows_owner_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ operand,
                                                        const uint32_t* __restrict__ updates, const int32_t* __restrict__ idx,
                                                        const ScatterOwnerParams& P) {
    __shared__ uint32_t keys[SCATTER_OWNER_CAP];
    __shared__ uint32_t start[1024 + 1];
    __shared__ uint32_t n_keys, n_tile;
    constexpr uint32_t NT = SCATTER_OWNER_THREADS, NW = NT / 64u, CAP = SCATTER_OWNER_CAP;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t R0 = blockIdx.x * P.rows_per_group;
    const uint32_t nrows = min(P.rows_per_group, P.n_rows - R0);           // the grid covers n_rows exactly
    auto add = [](uint32_t a, uint32_t b) -> uint32_t { return IS_FLOAT ? f2u(u2f(a) + u2f(b)) : a + b; };
    auto take = [&](int32_t r, uint32_t i) {                               // keeps update i if its row is one of ours
        const uint32_t local = (uint32_t)r - R0;                           // negative and foreign rows wrap to >= nrows
        if (local < nrows) {
            const uint32_t p = atomicAdd(&n_keys, 1u);
            if (p < CAP) keys[p] = local << 22 | i;
        }
    };

    // keys[0 .. count) -> sorted; start[j] = first key of row j; then the sums.
    // first: the rows start from the operand and every row is written; otherwise from what `out` holds, rows with keys only
    auto process = [&](uint32_t count, bool first) {
        uint32_t n = 64u;
        while (n < count) n <<= 1;
        for (uint32_t p = count + tid; p < n; p += NT) keys[p] = 0xFFFFFFFFu;
        __syncthreads();
        for (uint32_t k = 2u; k <= n; k <<= 1) {
            for (uint32_t j = k >> 1; j > 0u; j >>= 1) {
                for (uint32_t t = tid; t < (n >> 1); t += NT) {
                    const uint32_t lo = ((t & ~(j - 1u)) << 1) | (t & (j - 1u)), hi = lo | j;
                    const uint32_t a = keys[lo], b = keys[hi];
                    if ((a > b) == ((lo & k) == 0u)) { keys[lo] = b; keys[hi] = a; }
                }
                __syncthreads();
            }
        }
        for (uint32_t j = tid; j <= nrows; j += NT) {                      // lower bound of row j's first possible key
            const uint32_t want = j << 22;
            uint32_t lo = j < nrows ? 0u : count, hi = count;              // j == nrows: 1024 << 22 does not fit a word
            while (lo < hi) {
                const uint32_t mid = (lo + hi) >> 1;
                if (keys[mid] < want) lo = mid + 1u; else hi = mid;
            }
            start[j] = lo;
        }
        __syncthreads();
        for (uint32_t j = wave; j < nrows; j += NW) {
            const uint32_t s = start[j], e = start[j + 1u];
            if (!first && s == e) continue;
            const uint64_t row = (uint64_t)(R0 + j) * P.row_len;
            for (uint32_t c0 = 0u; c0 < P.row_len; c0 += 64u * VEC) {
                const uint32_t c = c0 + lane * VEC;
                if (c >= P.row_len) continue;                              // row_len is a multiple of VEC
                uint32_t acc[VEC];
                const uint32_t* base = first ? operand : out;
                if (first && P.operand_is_scalar) {
#pragma unroll
                    for (int v = 0; v < VEC; ++v) acc[v] = operand[0];
                } else if constexpr (VEC == 4) {
                    const u32x4 t = *reinterpret_cast<const u32x4*>(base + row + c);
                    acc[0] = t.x; acc[1] = t.y; acc[2] = t.z; acc[3] = t.w;
                } else {
                    acc[0] = base[row + c];
                }
                for (uint32_t k = s; k < e; k += SCATTER_OWNER_INFLIGHT) {
                    uint32_t t[SCATTER_OWNER_INFLIGHT][VEC];
#pragma unroll
                    for (uint32_t q = 0; q < SCATTER_OWNER_INFLIGHT; ++q)
                        if (k + q < e) {
                            const uint64_t u = (uint64_t)(keys[k + q] & 0x3FFFFFu) * P.row_len + c;
                            if constexpr (VEC == 4) {
                                const u32x4 w = *reinterpret_cast<const u32x4*>(updates + u);
                                t[q][0] = w.x; t[q][1] = w.y; t[q][2] = w.z; t[q][3] = w.w;
                            } else {
                                t[q][0] = updates[u];
                            }
                        }
#pragma unroll
                    for (uint32_t q = 0; q < SCATTER_OWNER_INFLIGHT; ++q)
                        if (k + q < e) {
#pragma unroll
                            for (int v = 0; v < VEC; ++v) acc[v] = add(acc[v], t[q][v]);
                        }
                }
                if constexpr (VEC == 4) {
                    u32x4 t; t.x = acc[0]; t.y = acc[1]; t.z = acc[2]; t.w = acc[3];
                    *reinterpret_cast<u32x4*>(out + row + c) = t;
                } else {
                    out[row + c] = acc[0];
                }
            }
        }
    };

    if (tid == 0u) n_keys = 0u;
    __syncthreads();
    // the whole index array, four 16-byte loads per thread in flight where the indices are dense
    if (P.idx_stride == 1u && (reinterpret_cast<uintptr_t>(idx) & 15u) == 0u) {
        const uint32_t nvec = P.n_idx >> 2;
        const int4* idx4 = reinterpret_cast<const int4*>(idx);
        for (uint32_t v0 = tid; v0 < nvec; v0 += NT * 4u) {
            int4 t[4];
#pragma unroll
            for (uint32_t q = 0; q < 4u; ++q)
                if (v0 + q * NT < nvec) t[q] = idx4[v0 + q * NT];
#pragma unroll
            for (uint32_t q = 0; q < 4u; ++q)
                if (v0 + q * NT < nvec) {
                    const uint32_t i = (v0 + q * NT) << 2;
                    take(t[q].x, i); take(t[q].y, i + 1u); take(t[q].z, i + 2u); take(t[q].w, i + 3u);
                }
        }
        for (uint32_t i = (nvec << 2) + tid; i < P.n_idx; i += NT) take(idx[i], i);
    } else {
        for (uint32_t i = tid; i < P.n_idx; i += NT) take(idx[(uint64_t)i * P.idx_stride], i);
    }
    __syncthreads();
    const uint32_t total = n_keys;
    if (total <= CAP) {
        process(total, true);
        return;
    }
    // More keys than LDS holds: rounds over consecutive ranges of the index array. A round takes
    // tiles of NT indices while their keys still fit (a tile never holds more than NT <= CAP keys,
    // so every round advances), sums them, and the next round continues behind it.
    uint32_t pos = 0u;
    bool first = true;
    while (pos < P.n_idx) {
        __syncthreads();
        if (tid == 0u) n_keys = 0u;
        __syncthreads();
        uint32_t count = 0u;
        while (pos < P.n_idx) {
            if (tid == 0u) n_tile = 0u;
            __syncthreads();
            const uint32_t i = pos + tid;
            uint32_t local = 0xFFFFFFFFu;
            if (i < P.n_idx) local = (uint32_t)idx[(uint64_t)i * P.idx_stride] - R0;
            if (local < nrows) atomicAdd(&n_tile, 1u);
            __syncthreads();
            if (count + n_tile > CAP) break;                               // uniform: every thread reads the same two values
            if (local < nrows) keys[atomicAdd(&n_keys, 1u)] = local << 22 | i;
            count += n_tile;
            pos += NT;
            __syncthreads();                                               // n_tile is reset by the next tile
        }
        __syncthreads();
        process(count, first);
        first = false;
    }
}

#define SCATTER_OWNER_KERNEL(name, VEC, IS_FLOAT)                                                                  \
    extern "C" __global__ __launch_bounds__(SCATTER_OWNER_THREADS) void name(uint32_t* out, const uint32_t* operand, \
            const uint32_t* updates, const int32_t* idx, ScatterOwnerParams P) {                                   \
        scatter_rows_owner_body<VEC, IS_FLOAT>(out, operand, updates, idx, P);                                     \
    }
// the _v4 variants require row_len % 4 == 0 and 16-byte aligned data pointers
SCATTER_OWNER_KERNEL(scatter_rows_owner_f_v1, 1, true)
SCATTER_OWNER_KERNEL(scatter_rows_owner_f_v4, 4, true)
SCATTER_OWNER_KERNEL(scatter_rows_owner_i_v1, 1, false)
SCATTER_OWNER_KERNEL(scatter_rows_owner_i_v4, 4, false)

struct ScatterGeneralParams {
    uint32_t n_upd, upd_rank, op_rank, n_index, is_float;
    uint32_t upd_dims[IDX_MAX_RANK];
    uint32_t upd_is_window[IDX_MAX_RANK];             // 1 if the update dim runs inside the window
    uint32_t op_dims[IDX_MAX_RANK];
    uint32_t op_strides[IDX_MAX_RANK];
    uint32_t op_inserted[IDX_MAX_RANK];               // 1 if the operand dim has no window dim (window size 1)
    uint32_t window_sizes[IDX_MAX_RANK];              // per operand dim (1 where inserted)
    uint32_t sd2od[IDX_MAX_RANK];                     // indices component k -> operand dim
    uint32_t batch_dims[IDX_MAX_RANK];
};

extern "C" __global__ __launch_bounds__(256) void scatter_add_general(uint32_t* __restrict__ out, const int32_t* __restrict__ indices,
                                                                      const uint32_t* __restrict__ updates, ScatterGeneralParams P) {
    const uint32_t e = blockIdx.x * 256u + threadIdx.x;
    if (e >= P.n_upd) return;
    uint32_t uc[IDX_MAX_RANK];
    {
        uint32_t r = e;
        for (int d = (int)P.upd_rank - 1; d >= 0; --d) { const uint32_t q = r / P.upd_dims[d]; uc[d] = r - q * P.upd_dims[d]; r = q; }
    }
    uint32_t batch = 0, wc[IDX_MAX_RANK], nw = 0;
    for (uint32_t d = 0, b = 0; d < P.upd_rank; ++d) {
        if (P.upd_is_window[d]) wc[nw++] = uc[d];
        else { batch = batch * P.batch_dims[b] + uc[d]; ++b; }
    }
    int32_t start[IDX_MAX_RANK];
    for (uint32_t d = 0; d < P.op_rank; ++d) start[d] = 0;
    for (uint32_t k = 0; k < P.n_index; ++k) start[P.sd2od[k]] = indices[(uint64_t)batch * P.n_index + k];
    uint64_t off = 0;
    for (uint32_t d = 0, j = 0; d < P.op_rank; ++d) {
        // the whole window must fit, otherwise the update is dropped
        if (start[d] < 0 || (uint32_t)start[d] + P.window_sizes[d] > P.op_dims[d]) return;
        uint32_t c = (uint32_t)start[d];
        if (!P.op_inserted[d]) c += wc[j++];
        off += (uint64_t)c * P.op_strides[d];
    }
    if (P.is_float) unsafeAtomicAdd(reinterpret_cast<float*>(out + off), u2f(updates[e]));
    else atomicAdd(out + off, updates[e]);
}
