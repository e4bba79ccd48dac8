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
struct GatherRowsParams { uint32_t n_idx, row_len, n_rows, idx_stride, fill_mode, fill_bits, wrap; };      // bit 31 of n_idx: STREAM_RESULT_BIT

// out[i, :] = table[clamp(idx[i*idx_stride]), :]; with fill_mode, rows outside the table read as fill_bits instead
// (jax's GatherScatterMode.FILL_OR_DROP)
template <int VEC>
__device__ __forceinline__ void gather_rows_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ table,
                                                 const int32_t* __restrict__ idx, const GatherRowsParams& P) {
    const uint32_t vpr = P.row_len / VEC, n_idx = without_stream_bit(P.n_idx);
    const uint64_t q = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (q >= (uint64_t)n_idx * vpr) return;
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
    if constexpr (VEC == 4) store_x4(out, (uint64_t)i * P.row_len + c, *reinterpret_cast<const u32x4*>(src), streams_result(P.n_idx), n_idx * P.row_len * 4u);
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
// scatter-add of whole rows without atomics on the data, in two launches: the first buckets the update
// numbers by target row, then one wave per table row adds up its updates, in ascending update order, on top
// of the operand row (or of one value, when the operand is a constant filled with it) and writes the result
// once. Every update row is read exactly once, the table is written once, and for rows that receive at
// most SCATTER_SORTED_MAX updates the sum does not depend on the order in which threads happen to
// run: it is operand + u(i0) + u(i1) + ... with i0 < i1 < ..., what a sequential loop over the
// updates computes. (A bucket of at most 64 entries is sorted across the lanes; a larger one is first
// sorted into a piece of a scratch array by counting for every entry the entries below it - quadratic,
// so only up to SCATTER_SORTED_MAX. Rows with more updates are summed in blocks of 64, each block in
// ascending order; which updates share a block depends on the order of arrival there.)
//
// Buckets. A counting sort proper needs the bucket starts - a prefix sum over all counters, i.e. a launch of
// its own between counting and placing, and a third one to place. Instead every row owns `cap` slots of a
// table `fixed` (the host picks cap a few times the average number of updates per row, at most 64; 0: no
// such table): update number i for row r takes k = count[r]++ and, if k < cap, goes to fixed[r * cap + k].
// The others go to an overflow table of at least twice as many slots as there are updates, open addressing:
// the entry (r + 1) << 32 | i is put into the first free slot from hash(r) + (k - cap) on, so that the
// overflow of one row lies in a run the row's wave later scans with coalesced loads, and entries of a row
// never collide with each other. The wave that sums row r finds count[r] - cap entries tagged with r from
// hash(r) on, empties their slots and, with the row's fixed slots, collects them in a piece of a scratch
// array (pieces are handed out by a cursor beside the counters), from where the row goes on as a bucket.
// Counters and overflow slots are zero before and after an evaluation: the wave that reads them clears them.
// Scratch: count (n_rows + 1 words: the counters, then the cursor, which the first launch resets), fixed
// (n_rows * cap), table (2 words for each of table_mask + 1 slots), gathered and sorted (n_idx words each:
// room for the buckets of rows with more than cap updates).
#define SCATTER_SORTED_MAX 4096u
struct ScatterSortParams { uint32_t n_idx, row_len, n_rows, idx_stride, operand_is_scalar, clip, wrap, cap, table_mask; };   // clip: as in ScatterRowsParams; wrap: as in GatherRowsParams

#define SCATTER_DROPPED 0xFFFFFFFFu

__device__ __forceinline__ uint32_t scatter_hash(uint32_t row) { return row * 2654435761u; }
__device__ __forceinline__ uint32_t load_word(const uint32_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_word(uint32_t* p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// update i goes to its row's next fixed slot or, when those are taken, to the overflow table; updates outside
// the operand are dropped
extern "C" __global__ __launch_bounds__(256) void scatter_rows_rank(uint32_t* __restrict__ count, uint32_t* __restrict__ fixed,
                                                                    unsigned long long* __restrict__ table, const int32_t* __restrict__ idx,
                                                                    ScatterSortParams P) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i == 0u) count[P.n_rows] = 0u;                                     // the cursor of the launch that follows
    if (i >= P.n_idx) return;
    int32_t r = idx[(uint64_t)i * P.idx_stride];
    r = r < 0 ? (int32_t)((uint32_t)r + P.wrap) : r;
    if (P.clip) r = r < 0 ? 0 : (r > (int32_t)P.n_rows - 1 ? (int32_t)P.n_rows - 1 : r);
    if (r < 0 || r >= (int32_t)P.n_rows) return;
    const uint32_t k = atomicAdd(count + r, 1u);
    if (k < P.cap) { fixed[(uint64_t)(uint32_t)r * P.cap + k] = i; return; }
    // (there are more slots than updates, so a free one is met before the table has been walked once)
    const unsigned long long entry = (unsigned long long)((uint32_t)r + 1u) << 32 | i;
    uint32_t slot = (scatter_hash((uint32_t)r) + (k - P.cap)) & P.table_mask;
    for (uint32_t probe = 0; probe <= P.table_mask; ++probe, slot = (slot + 1u) & P.table_mask)
        if (atomicCAS(table + slot, 0ull, entry) == 0ull) break;
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

// The updates of a row with more than cap of them, collected in gathered[0 .. n): the row's fixed slots, then its
// entries of the overflow table, found from hash(row) on and taken out of the table. Returns how many there are (n,
// unless the table does not hold what the counter promised). The wave later reads back what it writes here: both
// through the L2 (relaxed device-scope accesses). Out of line, like sort_bucket: crowded rows only.
__device__ __attribute__((noinline)) uint32_t gather_bucket(uint32_t* gathered, const uint32_t* fixed_row, unsigned long long* table,
                                                            uint32_t table_mask, uint32_t row, uint32_t n, uint32_t cap, uint32_t lane) {
    if (lane < cap) store_word(gathered + lane, load_word(fixed_row + lane));               // cap <= 64
    uint32_t found = cap;
    const uint32_t h0 = scatter_hash(row);
    // 64 consecutive slots a step, every slot of the table at most once (the table has at least 64 slots)
    for (uint64_t probe = 0; probe <= table_mask && found < n; probe += 64u) {
        unsigned long long* slot = table + ((h0 + (uint32_t)probe + lane) & table_mask);
        const unsigned long long v = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool mine = (uint32_t)(v >> 32) == row + 1u;
        if (mine) __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long votes = __ballot(mine);
        const uint32_t place = found + (uint32_t)__builtin_popcountll(votes & ((1ull << lane) - 1ull));
        if (mine && place < n) store_word(gathered + place, (uint32_t)v);
        found += (uint32_t)__builtin_popcountll(votes);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_s_waitcnt(0);
    return min(found, n);
}

// sorted[0 .. n) = bucket[0 .. n) in ascending order, by one wave. Entry x goes to the place given by the number of
// entries below it (they are distinct); the wave compares 64 of its entries at a time with all of them. The wave
// reads what it has written itself, here and before: through the L2 (relaxed device-scope accesses). Kept out of
// line: it runs for crowded rows only and must not cost the usual path registers.
__device__ __attribute__((noinline)) void sort_bucket(uint32_t* sorted, const uint32_t* bucket, uint32_t n, uint32_t lane) {
    for (uint32_t p0 = 0; p0 < n; p0 += 64u) {
        const uint32_t own = p0 + lane < n ? load_word(bucket + p0 + lane) : SCATTER_DROPPED;
        uint32_t below = 0;
        for (uint32_t c0 = 0; c0 < n; c0 += 64u) {
            const uint32_t other = c0 + lane < n ? load_word(bucket + c0 + lane) : SCATTER_DROPPED;      // (nothing is below a dropped slot's own value)
#pragma unroll
            for (uint32_t j = 0; j < 64u; ++j) below += __builtin_amdgcn_readlane(other, j) < own ? 1u : 0u;
        }
        if (p0 + lane < n) store_word(sorted + below, own);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_s_waitcnt(0);
}

// out[r, :] = operand[r, :] + sum over the updates i in row r's bucket of updates[i, :]; one wave per row.
// Measured on 262144 updates of 1 KB into 65536 rows: the launch moves its bytes at the same rate whether a
// wave takes one row or several with all their loads in flight together, i.e. it is not bound by the chain
// counter -> bucket -> update rows; what helped is to keep the update rows (read once) and the result
// (not read again here) out of the L2 with nontemporal accesses (65 -> 56 us).
template <int VEC, bool IS_FLOAT>
__device__ __forceinline__ void scatter_rows_sum_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ operand,
                                                      const uint32_t* __restrict__ updates, uint32_t* count, const uint32_t* fixed,
                                                      unsigned long long* table, uint32_t* gathered, uint32_t* sorted,
                                                      const ScatterSortParams& P) {
    constexpr uint32_t INFLIGHT = 4;
    typedef uint32_t vec_t __attribute__((ext_vector_type(VEC)));
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t row = __builtin_amdgcn_readfirstlane(blockIdx.x * 4u + (threadIdx.x >> 6));
    if (row >= P.n_rows) return;
    // The row's counter is read and put back to zero (for the next evaluation) by the same lane, the store behind the
    // wait for the load. (Asking for the row's fixed slots and the operand row together with the counter, one round
    // trip to memory for all three, changed nothing: 59.7 us against 59.8.)
    uint32_t n_lane0 = 0;
    if (lane == 0u) n_lane0 = count[row];
    uint32_t n = __builtin_amdgcn_readfirstlane(n_lane0);
    if (lane == 0u && n != 0u) count[row] = 0u;
    // the row's bucket: its fixed slots, or - more updates than slots - a piece of `gathered` that holds all of them
    const uint32_t* bucket = fixed + (uint64_t)row * P.cap;
    if (n > P.cap) {
        uint32_t piece_lane0 = 0;
        if (lane == 0u) piece_lane0 = atomicAdd(count + P.n_rows, n);     // (the counters add up to at most n_idx)
        const uint32_t piece = __builtin_amdgcn_readfirstlane(piece_lane0);
        n = gather_bucket(gathered + piece, bucket, table, P.table_mask, row, n, P.cap, lane);
        bucket = gathered + piece;
        sorted += piece;
    }
    auto add = [](vec_t a, vec_t b) -> vec_t {
        if constexpr (IS_FLOAT) return __builtin_bit_cast(vec_t, __builtin_bit_cast(float __attribute__((ext_vector_type(VEC))), a) +
                                                                  __builtin_bit_cast(float __attribute__((ext_vector_type(VEC))), b));
        else return a + b;
    };
    // acc += updates[ent(k), c ...] for k < m in ascending k; ent: sorted update numbers, one per lane.
    // Lanes beyond the row (live == false) ask for column 0 instead, whose values they drop. (Measured: two, four or
    // eight loads in flight, and switching the loads beyond the last update off instead of repeating the last one,
    // all give the same 59 to 60 us on 262144 updates of 1 KB; eight in flight with repeated loads 68.)
    auto accumulate = [&](uint32_t ent, uint32_t m, uint32_t c, vec_t& acc) {
        for (uint32_t k = 0; k < m; k += INFLIGHT) {
            vec_t t[INFLIGHT];
#pragma unroll
            for (uint32_t q = 0; q < INFLIGHT; ++q) {                      // no branch around a load: the last one is repeated
                const uint32_t u = __builtin_amdgcn_readlane(ent, min(k + q, m - 1u));
                t[q] = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(updates + (uint64_t)u * P.row_len + c));
            }
#pragma unroll
            for (uint32_t q = 0; q < INFLIGHT; ++q)
                if (k + q < m) acc = add(acc, t[q]);
        }
    };
    const bool one_block = n <= 64u;
    uint32_t ent = SCATTER_DROPPED;
    if (one_block) {
        if (lane < n) ent = load_word(bucket + lane);
        ent = wave_sort_first(ent, n, lane);
    }
    // A crowded row: the bucket in ascending order, written to sorted[0 .. n).
    const bool presorted = !one_block && n <= SCATTER_SORTED_MAX;
    if (presorted) sort_bucket(sorted, bucket, n, lane);
    for (uint32_t c0 = 0; c0 < P.row_len; c0 += 64u * VEC) {
        const bool live = c0 + lane * VEC < P.row_len;                     // row_len is a multiple of VEC
        const uint32_t c = live ? c0 + lane * VEC : 0u;
        vec_t acc;
        if (P.operand_is_scalar) acc = operand[0];
        else acc = *reinterpret_cast<const vec_t*>(operand + (uint64_t)row * P.row_len + c);
        if (one_block) {
            accumulate(ent, n, c, acc);
        } else {
            for (uint32_t b0 = 0; b0 < n; b0 += 64u) {
                const uint32_t m = min(64u, n - b0);
                uint32_t block = SCATTER_DROPPED;
                if (lane < m) block = load_word((presorted ? sorted : bucket) + b0 + lane);
                if (!presorted) block = wave_sort_first(block, m, lane);
                accumulate(block, m, c, acc);
            }
        }
        if (live) __builtin_nontemporal_store(acc, reinterpret_cast<vec_t*>(out + (uint64_t)row * P.row_len + c));
    }
}

#define SCATTER_SUM_KERNEL(name, VEC, IS_FLOAT)                                                                   \
    extern "C" __global__ __launch_bounds__(256) void name(uint32_t* out, const uint32_t* operand, const uint32_t* updates, \
                                                           uint32_t* count, const uint32_t* fixed, unsigned long long* table,    \
                                                           uint32_t* gathered, uint32_t* sorted, ScatterSortParams P) {          \
        scatter_rows_sum_body<VEC, IS_FLOAT>(out, operand, updates, count, fixed, table, gathered, sorted, P);     \
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
