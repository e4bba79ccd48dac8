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

// wrap: added to negative indices first (0: nothing) - the normalisation `select(i < 0, i + n, i)` that tracing puts in
// front of an indexing operation, taken over from an element-wise launch of its own
struct GatherRowsParams { uint32_t n_idx, row_len, n_rows, idx_stride, fill_mode, fill_bits, wrap; };

// out[i, :] = table[clamp(idx[i*idx_stride]), :]; with fill_mode, rows outside the table read as fill_bits instead
// (jax's GatherScatterMode.FILL_OR_DROP)
template <int VEC>
__device__ __forceinline__ void gather_rows_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ table,
                                                 const int32_t* __restrict__ idx, const GatherRowsParams& P) {
    const uint32_t vpr = P.row_len / VEC;
    const uint64_t q = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (q >= (uint64_t)P.n_idx * vpr) return;
    const uint32_t i = (uint32_t)(q / vpr), c = (uint32_t)(q - (uint64_t)i * vpr) * VEC;
    int32_t r = idx[(uint64_t)i * P.idx_stride];
    r = r < 0 ? (int32_t)((uint32_t)r + P.wrap) : r;
    uint32_t* dst = out + (uint64_t)i * P.row_len + c;
    if (P.fill_mode && (r < 0 || r >= (int32_t)P.n_rows)) {
        if constexpr (VEC == 4) *reinterpret_cast<u32x4*>(dst) = u32x4{P.fill_bits, P.fill_bits, P.fill_bits, P.fill_bits};
        else *dst = P.fill_bits;
        return;
    }
    r = r < 0 ? 0 : (r > (int32_t)P.n_rows - 1 ? (int32_t)P.n_rows - 1 : r);
    const uint32_t* src = table + (uint64_t)r * P.row_len + c;
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
    uint32_t fill_mode, fill_bits;                    // fill_mode: slices that do not fit read as fill_bits instead of being moved inside
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
    bool outside = false;
    for (uint32_t d = 0; d < P.op_rank; ++d) start[d] = 0;
    for (uint32_t k = 0; k < P.n_index; ++k) {
        const uint32_t d = P.start_index_map[k];
        int32_t s = indices[(uint64_t)batch * P.n_index + k];
        const int32_t hi = (int32_t)P.op_dims[d] - (int32_t)P.slice_sizes[d];
        outside = outside || s < 0 || s > hi;
        start[d] = s < 0 ? 0 : (s > hi ? hi : s);
    }
    if (P.fill_mode && outside) { out[e] = P.fill_bits; return; }
    uint64_t off = 0;
    for (uint32_t d = 0, j = 0; d < P.op_rank; ++d) {
        uint32_t c = (uint32_t)start[d];
        if (!P.op_collapsed[d]) c += offs[j++];
        off += (uint64_t)c * P.op_strides[d];
    }
    out[e] = operand[off];
}

struct ScatterRowsParams { uint32_t n_idx, row_len, n_rows, idx_stride, is_float, clip; };   // clip: rows outside the table go to its first / last row instead of being dropped

// out[idx[i], :] += updates[i, :]   (out already holds the operand)
extern "C" __global__ __launch_bounds__(256) void scatter_add_rows(uint32_t* __restrict__ out, const int32_t* __restrict__ idx,
                                                                   const uint32_t* __restrict__ updates, ScatterRowsParams P) {
    const uint64_t q = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (q >= (uint64_t)P.n_idx * P.row_len) return;
    const uint32_t i = (uint32_t)(q / P.row_len), c = (uint32_t)(q - (uint64_t)i * P.row_len);
    int32_t r = idx[(uint64_t)i * P.idx_stride];
    if (P.clip) r = r < 0 ? 0 : (r > (int32_t)P.n_rows - 1 ? (int32_t)P.n_rows - 1 : r);
    if (r < 0 || r >= (int32_t)P.n_rows) return;
    const uint32_t u = updates[q];
    uint32_t* dst = out + (uint64_t)r * P.row_len + c;
    if (P.is_float) unsafeAtomicAdd(reinterpret_cast<float*>(dst), u2f(u));
    else atomicAdd(dst, u);
}

// ---------------------------------------------------------------------------------------------
// scatter-add of whole rows without atomics on the data: the update rows are bucketed by target
// row with a counting sort of their indices (three small launches over the indices), then one
// wave per table row adds up its updates, in ascending update order, on top of the operand row
// (or of one value, when the operand is a constant filled with it) and writes the result once.
// Every update row is read exactly once, the table is written once, and for rows that receive at
// most SCATTER_SORTED_MAX updates the sum does not depend on the order in which threads happen to
// run: it is operand + u(i0) + u(i1) + ... with i0 < i1 < ..., what a sequential loop over the
// updates computes. (A bucket of at most 64 entries is sorted across the lanes; a larger one is first
// sorted into the rank array, which nothing needs any more by then, by counting for every entry the
// entries below it - quadratic, so only up to SCATTER_SORTED_MAX. Rows with more updates are summed
// in blocks of 64, each block in ascending order; which updates share a block depends on the order
// of arrival there.)
// Scratch: count (n_rows words, all zero before and after), start (n_rows + 1), rank and order
// (n_idx each).
#define SCATTER_SORTED_MAX 4096u
struct ScatterSortParams { uint32_t n_idx, row_len, n_rows, idx_stride, operand_is_scalar, clip, wrap; };   // clip: as in ScatterRowsParams; wrap: as in GatherRowsParams

#define SCATTER_DROPPED 0xFFFFFFFFu

// rank[i] = how many updates for the same row arrived before update i (the counter's old value);
// updates outside the operand are dropped
extern "C" __global__ __launch_bounds__(256) void scatter_rows_rank(uint32_t* __restrict__ count, uint32_t* __restrict__ rank,
                                                                    const int32_t* __restrict__ idx, ScatterSortParams P) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= P.n_idx) return;
    int32_t r = idx[(uint64_t)i * P.idx_stride];
    r = r < 0 ? (int32_t)((uint32_t)r + P.wrap) : r;
    if (P.clip) r = r < 0 ? 0 : (r > (int32_t)P.n_rows - 1 ? (int32_t)P.n_rows - 1 : r);
    uint32_t k = SCATTER_DROPPED;
    if (r >= 0 && r < (int32_t)P.n_rows) k = atomicAdd(count + r, 1u);
    rank[i] = k;
}

// start[r] = number of updates for rows before r (r = 0 .. n_rows: where row r's bucket begins).
// Workgroup b produces words [b * seg, (b + 1) * seg) of start, seg a multiple of 1024: it first adds up
// all counts before its segment itself, so no workgroup waits for another (a fence between
// workgroups writes back the whole L2 on this GPU, 60 us), then scans its segment in tiles of 1024.
extern "C" __global__ __launch_bounds__(1024) void scatter_rows_starts(uint32_t* __restrict__ start, const uint32_t* __restrict__ count,
                                                                       uint32_t n_rows, uint32_t seg) {
    __shared__ uint32_t wave_total[4], wave_before[16];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t first = blockIdx.x * seg;                               // <= n_rows (the grid sees to that)
    uint32_t before = 0;
    {
        const u32x4* c4 = reinterpret_cast<const u32x4*>(count);           // first is a multiple of 1024 words
        const uint32_t nvec = first >> 2;
        uint32_t v = threadIdx.x;
        for (; v + 3072u < nvec; v += 4096u) {
            const u32x4 a = c4[v], b = c4[v + 1024u], c = c4[v + 2048u], d = c4[v + 3072u];
            before += (a.x + a.y + a.z + a.w) + (b.x + b.y + b.z + b.w) + (c.x + c.y + c.z + c.w) + (d.x + d.y + d.z + d.w);
        }
        for (; v < nvec; v += 1024u) { const u32x4 a = c4[v]; before += a.x + a.y + a.z + a.w; }
    }
    before = wave_allreduce(before, [](uint32_t a, uint32_t b) { return a + b; });
    if (lane == 0u) wave_before[wave] = before;
    __syncthreads();
    const bool scans = wave < 4u;                                          // the tiles are scanned by the first four waves
    uint32_t carry = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) carry += wave_before[w];
    for (uint32_t tile = first; tile < first + seg && tile <= n_rows; tile += 1024u) {
        const uint32_t base = tile + (threadIdx.x & 255u) * 4u;
        uint32_t v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = scans && base + q < n_rows ? count[base + q] : 0u;
        const uint32_t own = v[0] + v[1] + v[2] + v[3];
        uint32_t t = own;                                                  // inclusive scan over the wave
#pragma unroll
        for (uint32_t off = 1; off < 64u; off <<= 1) {
            const uint32_t up = __shfl_up(t, off, 64);
            if (lane >= off) t += up;
        }
        if (scans && lane == 63u) wave_total[wave] = t;
        __syncthreads();
        uint32_t x = carry + t - own;
        for (uint32_t w = 0; w < (wave & 3u); ++w) x += wave_total[w];
        const uint32_t tile_total = wave_total[0] + wave_total[1] + wave_total[2] + wave_total[3];
        __syncthreads();                                                   // wave_total is rewritten by the next tile
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (scans && base + q <= n_rows) start[base + q] = x;
            x += v[q];
        }
        carry += tile_total;
    }
}

// order[start[idx[i]] + rank[i]] = i, and the counts go back to zero for the next evaluation
extern "C" __global__ __launch_bounds__(256) void scatter_rows_order(uint32_t* __restrict__ order, uint32_t* __restrict__ count,
                                                                     const uint32_t* __restrict__ start, const uint32_t* __restrict__ rank,
                                                                     const int32_t* __restrict__ idx, ScatterSortParams P) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < P.n_rows) count[i] = 0u;
    if (i >= P.n_idx) return;
    const uint32_t k = rank[i];
    if (k == SCATTER_DROPPED) return;
    int32_t r = idx[(uint64_t)i * P.idx_stride];
    r = r < 0 ? (int32_t)((uint32_t)r + P.wrap) : r;
    if (P.clip) r = r < 0 ? 0 : (r > (int32_t)P.n_rows - 1 ? (int32_t)P.n_rows - 1 : r);
    order[start[r] + k] = i;
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

// The first n lanes hold distinct values, the others 0xFFFFFFFF: ascending order over the lanes.
// Few values (the usual bucket): every lane counts the values below its own and sends its value there.
__device__ __forceinline__ uint32_t wave_sort_first(uint32_t e, uint32_t n, uint32_t lane) {
    if (n <= 1u) return e;
    if (n > 16u) return wave_sort(e, lane);
    uint32_t below = 0;
    for (uint32_t j = 0; j < n; ++j) below += __builtin_amdgcn_readlane(e, j) < e ? 1u : 0u;
    if (lane >= n) below = lane;
    return (uint32_t)__builtin_amdgcn_ds_permute((int)(below << 2), (int)e);
}

// sorted[s .. e) = order[s .. e) in ascending order, by one wave. Entry x goes to the place given by the number of
// entries below it (they are distinct); the wave compares 64 of its entries at a time with all of them. The wave
// reads back what it has written itself: both through the L2 (relaxed device-scope accesses). Kept out of line: it
// runs for crowded rows only and must not cost the usual path registers.
__device__ __attribute__((noinline)) void sort_bucket(uint32_t* sorted, const uint32_t* __restrict__ order, uint32_t s, uint32_t e, uint32_t lane) {
    for (uint32_t p0 = s; p0 < e; p0 += 64u) {
        const uint32_t own = p0 + lane < e ? order[p0 + lane] : SCATTER_DROPPED;
        uint32_t below = 0;
        for (uint32_t c0 = s; c0 < e; c0 += 64u) {
            const uint32_t other = c0 + lane < e ? order[c0 + lane] : SCATTER_DROPPED;      // (nothing is below a dropped slot's own value)
#pragma unroll
            for (uint32_t j = 0; j < 64u; ++j) below += __builtin_amdgcn_readlane(other, j) < own ? 1u : 0u;
        }
        if (p0 + lane < e) __hip_atomic_store(sorted + s + below, own, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_s_waitcnt(0);
}

// out[r, :] = operand[r, :] + sum over the updates i in row r's bucket of updates[i, :]; one wave per row.
// Measured on 262144 updates of 1 KB into 65536 rows: the launch moves its bytes at the same rate whether a
// wave takes one row or several with all their loads in flight together, i.e. it is not bound by the chain
// start -> order -> update rows; what helped is to keep the update rows (read once) and the result
// (not read again here) out of the L2 with nontemporal accesses (65 -> 56 us).
template <int VEC, bool IS_FLOAT>
__device__ __forceinline__ void scatter_rows_sum_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ operand,
                                                      const uint32_t* __restrict__ updates, const uint32_t* __restrict__ start,
                                                      const uint32_t* __restrict__ order, uint32_t* sorted, const ScatterSortParams& P) {
    constexpr uint32_t INFLIGHT = 4;
    typedef uint32_t vec_t __attribute__((ext_vector_type(VEC)));
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t row = __builtin_amdgcn_readfirstlane(blockIdx.x * 4u + (threadIdx.x >> 6));
    if (row >= P.n_rows) return;
    const uint32_t s = start[row], e = start[row + 1u];
    auto add = [](vec_t a, vec_t b) -> vec_t {
        if constexpr (IS_FLOAT) return __builtin_bit_cast(vec_t, __builtin_bit_cast(float __attribute__((ext_vector_type(VEC))), a) +
                                                                  __builtin_bit_cast(float __attribute__((ext_vector_type(VEC))), b));
        else return a + b;
    };
    // acc += updates[ent(k), c ...] for k < n in ascending k; ent: sorted update numbers, one per lane.
    // Lanes beyond the row (live == false) ask for column 0 instead, whose values they drop.
    auto accumulate = [&](uint32_t ent, uint32_t n, uint32_t c, vec_t& acc) {
        for (uint32_t k = 0; k < n; k += INFLIGHT) {
            vec_t t[INFLIGHT];
#pragma unroll
            for (uint32_t q = 0; q < INFLIGHT; ++q) {                      // no branch around a load: the last one is repeated
                const uint32_t u = __builtin_amdgcn_readlane(ent, min(k + q, n - 1u));
                t[q] = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(updates + (uint64_t)u * P.row_len + c));
            }
#pragma unroll
            for (uint32_t q = 0; q < INFLIGHT; ++q)
                if (k + q < n) acc = add(acc, t[q]);
        }
    };
    const bool one_block = e - s <= 64u;
    uint32_t ent = SCATTER_DROPPED;
    if (one_block) {
        if (lane < e - s) ent = order[s + lane];
        ent = wave_sort_first(ent, e - s, lane);
    }
    // A crowded row: the bucket in ascending order, written to sorted[s .. e).
    const bool presorted = !one_block && e - s <= SCATTER_SORTED_MAX;
    if (presorted) sort_bucket(sorted, order, s, e, lane);
    for (uint32_t c0 = 0; c0 < P.row_len; c0 += 64u * VEC) {
        const bool live = c0 + lane * VEC < P.row_len;                     // row_len is a multiple of VEC
        const uint32_t c = live ? c0 + lane * VEC : 0u;
        vec_t acc;
        if (P.operand_is_scalar) acc = operand[0];
        else acc = *reinterpret_cast<const vec_t*>(operand + (uint64_t)row * P.row_len + c);
        if (one_block) {
            accumulate(ent, e - s, c, acc);
        } else {
            for (uint32_t b0 = s; b0 < e; b0 += 64u) {
                const uint32_t n = min(64u, e - b0);
                uint32_t block = SCATTER_DROPPED;
                if (presorted) {
                    if (lane < n) block = __hip_atomic_load(sorted + b0 + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                } else {
                    if (lane < n) block = order[b0 + lane];
                    block = wave_sort_first(block, n, lane);
                }
                accumulate(block, n, c, acc);
            }
        }
        if (live) __builtin_nontemporal_store(acc, reinterpret_cast<vec_t*>(out + (uint64_t)row * P.row_len + c));
    }
}

#define SCATTER_SUM_KERNEL(name, VEC, IS_FLOAT)                                                                   \
    extern "C" __global__ __launch_bounds__(256) void name(uint32_t* out, const uint32_t* operand, const uint32_t* updates, \
                                                           const uint32_t* start, const uint32_t* order, uint32_t* sorted,       \
                                                           ScatterSortParams P) {                                                 \
        scatter_rows_sum_body<VEC, IS_FLOAT>(out, operand, updates, start, order, sorted, P);                      \
    }
// the _v4 variants require row_len % 4 == 0 and 16-byte aligned data pointers
SCATTER_SUM_KERNEL(scatter_rows_sum_f_v1, 1, true)
SCATTER_SUM_KERNEL(scatter_rows_sum_f_v4, 4, true)
SCATTER_SUM_KERNEL(scatter_rows_sum_i_v1, 1, false)
SCATTER_SUM_KERNEL(scatter_rows_sum_i_v4, 4, false)

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
    uint32_t clip;                                    // windows that do not fit are moved inside instead of being dropped
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
        // the whole window must fit, otherwise the update is dropped (or, with clip, moved inside)
        if (P.clip) {
            const int32_t hi = (int32_t)P.op_dims[d] - (int32_t)P.window_sizes[d];
            start[d] = start[d] < 0 ? 0 : (start[d] > hi ? hi : start[d]);
        }
        if (start[d] < 0 || (uint32_t)start[d] + P.window_sizes[d] > P.op_dims[d]) return;
        uint32_t c = (uint32_t)start[d];
        if (!P.op_inserted[d]) c += wc[j++];
        off += (uint64_t)c * P.op_strides[d];
    }
    if (P.is_float) unsafeAtomicAdd(reinterpret_cast<float*>(out + off), u2f(updates[e]));
    else atomicAdd(out + off, updates[e]);
}
