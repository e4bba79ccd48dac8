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
