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
#include "ew_apply.h"

#define EW_MAX_STEPS 8

struct EwParams {
    uint32_t n;                        // output elements; bit 31: the result is stored past the caches (STREAM_RESULT_BIT)
    uint32_t ndim;                     // 1..4 collapsed output dims
    uint32_t dims[4];                  // row-major, dims[ndim-1] fastest; unused = 1
    uint32_t nsteps;                   // 1..8; step 0 is the initial load
    uint32_t op[EW_MAX_STEPS];         // opcode of step k (op[0] ignored)
    uint32_t flags[EW_MAX_STEPS];      // bit0: step has an operand; bit1: operand is the LEFT argument;
                                       // bit2: the operand's fastest stride is 1 (else 0: one value per vector);
                                       // bits 4-5: how the operand is addressed: 0 through its strides, 1 like the
                                       // output (element = base + linear index), 2 by the fastest dimension only
                                       // (element = base + coordinate), 3 a single element (base);
                                       // bit6: every vector of a thread reads the same elements of the operand
    uint32_t imm[EW_MAX_STEPS];        // immediate (integer_pow exponent)
    int32_t  stride[EW_MAX_STEPS][4];  // operand strides per collapsed dim, in elements
    uint32_t nbytes[EW_MAX_STEPS];     // bytes readable from each operand pointer (0 = no operand)
    uint32_t base[EW_MAX_STEPS];       // element offset of output element 0 in each operand
    uint32_t dim_magic[4], dim_shift[4];   // n / dims[d] = mulhi(n, magic) >> shift for n < 2^31; magic 0: dims[d] == 1
};

// Keeps a kernel argument in a scalar register from this point on. Used on every argument at
// the top of the kernel so that the scalar loads of the argument block are issued together and
// waited for once, instead of one round trip per operand slot further down. The 8-slot
// instantiation would run out of scalar registers and leaves its arguments to be fetched on demand.
#define EW_PIN(x) do { if constexpr (PIN && NS <= 6) asm volatile("" : "+s"(x)); } while (0)

// NS = number of step slots this instantiation looks at (the chain has at most NS steps).
// `block` is the index of this workgroup within the chain's own grid.
template <int VEC, int NS, bool PIN = true>
__device__ __forceinline__ void ew_chain_body(uint32_t* __restrict__ out, const uint32_t* const (&in)[EW_MAX_STEPS],
                                              const EwParams& P, const uint32_t block) {
    // All fields are read first and pinned afterwards: an inline-asm statement is a boundary for the instruction
    // scheduler, and loads issued behind the first pin would wait for a second round trip to the argument block.
    uint32_t n = without_stream_bit(P.n), ndim = P.ndim, nsteps = P.nsteps;
    uint32_t dims[4], op[NS], flags[NS], imm[NS], nbytes[NS], base[NS];
    int32_t  stride[NS][4];
    uint32_t dim_magic[4], dim_shift[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) { dims[d] = P.dims[d]; dim_magic[d] = P.dim_magic[d]; dim_shift[d] = P.dim_shift[d]; }
#pragma unroll
    for (int k = 0; k < NS; ++k) {
        flags[k] = P.flags[k]; nbytes[k] = P.nbytes[k]; base[k] = P.base[k];
#pragma unroll
        for (int d = 0; d < 4; ++d) stride[k][d] = P.stride[k][d];
    }
    EW_PIN(n); EW_PIN(ndim); EW_PIN(nsteps);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        EW_PIN(dims[d]);
        if (d >= 1) { EW_PIN(dim_magic[d]); EW_PIN(dim_shift[d]); }
    }
#pragma unroll
    for (int k = 0; k < NS; ++k) {
        EW_PIN(flags[k]); EW_PIN(nbytes[k]); EW_PIN(base[k]);
        if constexpr (PIN && NS <= 6) asm volatile("" :: "s"(in[k]));
#pragma unroll
        for (int d = 0; d < 4; ++d) EW_PIN(stride[k][d]);
    }

    // A thread works on U vectors, 256 vectors apart (so that a wave's loads stay contiguous). All
    // loads of all U vectors are requested before any is used: with one vector per thread the bytes a
    // CU has in flight do not cover the memory latency once a chain has several operands.
    constexpr int U = (NS == 4 || NS == 6) ? 2 : 1;
    constexpr int W = U * VEC;                                    // values per thread
    const uint32_t first = (block * U * 256u + threadIdx.x) * VEC;          // the host keeps n below 2^31
    const bool stream_out = streams_result(P.n);
    if (first >= n) return;

    // Every operand is read through a buffer descriptor with one branch-free load per slot: 16 bytes
    // (of which only the first dword is used where the operand is constant along the vector), or
    // nothing at all for an empty slot, whose descriptor has size 0.
    // (what a load returns is looked at only after all loads of all vectors have been requested: a use in between
    // would wait for the load in flight and serialise all that follow)
    u32x4 raw[NS][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t i0 = first + u * 256u * VEC;
        // coordinates of the first element of this vector in the collapsed output space (divisions by
        // multiply-high with constants from the host)
        uint32_t c[4] = {0, 0, 0, 0};
        {
            uint32_t r = i0;
            if (ndim > 1) {
#pragma unroll
                for (int d = 3; d >= 1; --d) {
                    if (d < (int)ndim) {
                        const uint32_t magic = dim_magic[d], shift = dim_shift[d];
                        const uint32_t q = magic ? __umulhi(r, magic) >> shift : r;
                        c[d] = r - q * dims[d]; r = q;
                    }
                }
            }
            c[0] = r;
        }
        // element index of this vector in operand k. Most operands are addressed in one of three simple
        // ways, told apart by a wave-uniform flag; 32-bit multiplies run at a quarter of the rate of adds.
        auto operand_index = [&](int k) -> uint32_t {
            const uint32_t how = (flags[k] >> 4) & 3u;
            if (how == 1u) return base[k] + i0;
            if (how == 3u) return base[k];
            uint32_t last = c[0];
#pragma unroll
            for (int d = 1; d < 4; ++d) last = d < (int)ndim ? c[d] : last;
            if (how == 2u) return base[k] + last;
            uint32_t idx = base[k] + c[0] * (uint32_t)stride[k][0];       // wraps correctly for negative strides
            if (ndim > 1) {
#pragma unroll
                for (int d = 1; d < 4; ++d) idx += c[d] * (uint32_t)stride[k][d];
            }
            return idx;
        };
#pragma unroll
        for (int k = 0; k < NS; ++k) {
            uint32_t byte = operand_index(k) * 4u;
            // a single value is fetched by the first lane of the wave alone and handed to the others further down: 64
            // lanes asking for the same 16 bytes are served one after the other (x * 2 + 1 on 64 M elements ran at
            // 4.9 TB/s with two such operands, x * s + b with per-column vectors at 5.9). The other lanes' offsets lie
            // beyond the descriptor's range, which returns zeros without touching memory.
            if (((flags[k] >> 4) & 3u) == 3u && (threadIdx.x & 63u) != 0u) byte = 0x80000000u;
            // a single value, or a vector over the fastest dimension whose length divides the distance between a thread's
            // vectors: what the thread's first vector loads serves the others too. Their loads go through a descriptor
            // of size 0, which returns zeros without touching memory, so that every vector issues the same instructions.
            const int readable = (u > 0 && (flags[k] & 64u)) ? 0 : (int)nbytes[k];
            const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(in[k]), 0, readable, 0x00020000);
            if constexpr (VEC == 4) raw[k][u] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte, 0, 0);
            else                    raw[k][u].x = __builtin_amdgcn_raw_buffer_load_b32(rsrc, byte, 0, 0);
        }
    }

    // opcodes and immediates are fetched while the operand loads are in flight
#pragma unroll
    for (int k = 0; k < NS; ++k) { op[k] = P.op[k]; imm[k] = P.imm[k]; EW_PIN(op[k]); EW_PIN(imm[k]); }

    uint32_t vals[NS][W];
#pragma unroll
    for (int k = 0; k < NS; ++k) {
        const bool is_vec = (flags[k] & 4u) != 0;          // else one value per vector: its first word
        const bool shared = (flags[k] & 64u) != 0;
        const bool single = ((flags[k] >> 4) & 3u) == 3u;   // what the wave's first lane has loaded is everybody's value
        const uint32_t from_first_lane = __builtin_amdgcn_readfirstlane(raw[k][0].x);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            u32x4 t = raw[k][u];
            if (u > 0) {
                t.x = shared ? raw[k][0].x : t.x; t.y = shared ? raw[k][0].y : t.y;
                t.z = shared ? raw[k][0].z : t.z; t.w = shared ? raw[k][0].w : t.w;
            }
            t.x = single ? from_first_lane : t.x;
            if constexpr (VEC == 4) {
                vals[k][u * 4 + 0] = t.x;
                vals[k][u * 4 + 1] = is_vec ? t.y : t.x;
                vals[k][u * 4 + 2] = is_vec ? t.z : t.x;
                vals[k][u * 4 + 3] = is_vec ? t.w : t.x;
            } else {
                vals[k][u] = t.x;
            }
        }
    }
    uint32_t acc[W];
#pragma unroll
    for (int j = 0; j < W; ++j) acc[j] = vals[0][j];

#pragma unroll
    for (int k = 1; k < NS; ++k) {
        if (k < (int)nsteps) {
            if (op[k] >= EW_SEL_P && op[k] <= EW_SEL_F) {
                // three-input select: this step's operand and the next step's operand (a NOP carrier)
                const int k2 = (k + 1 < NS) ? k + 1 : k;
#pragma unroll
                for (int j = 0; j < W; ++j) {
                    const uint32_t s = vals[k][j], t = vals[k2][j];
                    acc[j] = op[k] == EW_SEL_P ? (acc[j] ? s : t)       // acc is the predicate
                           : op[k] == EW_SEL_T ? (s ? acc[j] : t)       // acc is on_true, s the predicate
                                               : (s ? t : acc[j]);      // acc is on_false, s the predicate
                }
            } else {
                ew_apply_vec<W>(op[k], acc, vals[k], (flags[k] & 2u) != 0, imm[k]);
            }
        }
    }

#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t i0 = first + u * 256u * VEC;
        if (i0 < n) {
            if constexpr (VEC == 4) {
                u32x4 t; t.x = acc[u * 4]; t.y = acc[u * 4 + 1]; t.z = acc[u * 4 + 2]; t.w = acc[u * 4 + 3];
                // (a buffer store: written as two stores through the same pointer, one of them nontemporal, the compiler
                // merges them into one plain store)
                if (stream_out) __builtin_amdgcn_raw_buffer_store_b128(t, make_rsrc(out, n * 4u), i0 * 4u, 0, 2);
                else *reinterpret_cast<u32x4*>(out + i0) = t;
            } else {
                out[i0] = acc[u];
            }
        }
    }
}

// The chains that a convolution's epilogue would otherwise hold, as a launch of their own (a batch norm over an array
// that no convolution has just produced, the sum of the slices of a sliced contraction followed by scale, shift,
// residual and ReLU): on contiguous float arrays of n elements whose fastest dimension has C elements,
//     v = first + s1 + s2 + s3            (the first nsum of them, in this order)
//     v = v - vsub[c]; v = v * vmul[c]; v = v + vadd[c]; v = v + full; v = max(v, floor)      (each optional, in this order)
// No interpreter: the operands that are present are told by flags. The opcode interpreter of ew_chain
// spends 750 instructions and 170 branches per wave on such a chain, which is most of a small launch's duration and
// a quarter of the bandwidth of a large one. n and C are multiples of 4; two 16-byte vectors per thread.
struct EwAffineParams {
    uint32_t n, cq;                 // elements (bit 31: STREAM_RESULT_BIT); C / 4
    uint32_t cq_magic, cq_shift;    // v / cq = mulhi(v, magic) >> shift for v < 2^31 (magic 0: cq == 1)
    uint32_t nsum;                  // 0..3
    uint32_t flags;                 // bit0 - vsub, bit1 * vmul, bit2 + vadd, bit3 + full, bit4 max(., floor)
};

// SKIP = false: every load is issued, through a descriptor of size 0 for an absent operand (such a load returns zeros
// without touching memory), and every step is a select on its flag: no taken branch, which is what a launch of a few
// waves wants. SKIP = true: absent operands are skipped by uniform branches, which is what a large array wants (ten
// loads per vector, most of them empty, cost it a quarter of its bandwidth).
template <bool SKIP>
__device__ __forceinline__ void ew_affine_body(float* __restrict__ out, const float* first, const float* s1, const float* s2, const float* s3,
                                               const float* vsub, const float* vmul, const float* vadd, const float* full, const float* floor_,
                                               const EwAffineParams& P) {
    constexpr int U = 2;
    const uint32_t nb = without_stream_bit(P.n) * 4u, cb = P.cq * 16u, fl = P.flags;
    const __amdgpu_buffer_rsrc_t r_out = make_rsrc(out, nb), r_first = make_rsrc(first, nb),
        r_s1 = make_rsrc(s1, P.nsum >= 1u ? nb : 0u), r_s2 = make_rsrc(s2, P.nsum >= 2u ? nb : 0u), r_s3 = make_rsrc(s3, P.nsum >= 3u ? nb : 0u),
        r_sub = make_rsrc(vsub, (fl & 1u) ? cb : 0u), r_mul = make_rsrc(vmul, (fl & 2u) ? cb : 0u), r_add = make_rsrc(vadd, (fl & 4u) ? cb : 0u),
        r_full = make_rsrc(full, (fl & 8u) ? nb : 0u), r_floor = make_rsrc(floor_, (fl & 16u) ? 4u : 0u);
    f32x4 a[U], b1[U], b2[U], b3[U], fu[U], vs[U], vm[U], va[U];
    uint32_t off[U];
    float lo = 0.f;
    // every load of both vectors is requested before anything is used
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t v = (blockIdx.x * U + u) * 256u + threadIdx.x;          // vector index; beyond n / 4: every access is out of range
        const uint32_t q = P.cq_magic ? __umulhi(v, P.cq_magic) >> P.cq_shift : v;
        const uint32_t c = (P.cq == 1u ? 0u : v - q * P.cq) * 16u;
        off[u] = v * 16u;
        a[u] = buffer_load_x4(r_first, off[u]);
        if (!SKIP || P.nsum >= 1u) b1[u] = buffer_load_x4(r_s1, off[u]);
        if (!SKIP || P.nsum >= 2u) b2[u] = buffer_load_x4(r_s2, off[u]);
        if (!SKIP || P.nsum >= 3u) b3[u] = buffer_load_x4(r_s3, off[u]);
        if (!SKIP || (fl & 8u)) fu[u] = buffer_load_x4(r_full, off[u]);
        if (!SKIP || (fl & 1u)) vs[u] = buffer_load_x4(r_sub, c);
        if (!SKIP || (fl & 2u)) vm[u] = buffer_load_x4(r_mul, c);
        if (!SKIP || (fl & 4u)) va[u] = buffer_load_x4(r_add, c);
    }
    // (the floor is one value: the wave's first lane fetches it for all, see ew_chain_body)
    if (!SKIP || (fl & 16u)) lo = buffer_load_x1(r_floor, (threadIdx.x & 63u) ? 0x80000000u : 0u);
    lo = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(uint32_t, lo)));
#pragma unroll
    for (int u = 0; u < U; ++u) {
        f32x4 y = a[u];
        if constexpr (SKIP) {
            if (P.nsum >= 1u) y = y + b1[u];
            if (P.nsum >= 2u) y = y + b2[u];
            if (P.nsum >= 3u) y = y + b3[u];
            if (fl & 1u) y = y - vs[u];
            if (fl & 2u) y = y * vm[u];
            if (fl & 4u) y = y + va[u];
            if (fl & 8u) y = y + fu[u];
            if (fl & 16u) {
#pragma unroll
                for (int j = 0; j < 4; ++j) y[j] = (y[j] > lo || y[j] != y[j]) ? y[j] : lo;       // a NaN stays
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float v = y[j];
                v = P.nsum >= 1u ? v + b1[u][j] : v;
                v = P.nsum >= 2u ? v + b2[u][j] : v;
                v = P.nsum >= 3u ? v + b3[u][j] : v;
                v = (fl & 1u) ? v - vs[u][j] : v;
                v = (fl & 2u) ? v * vm[u][j] : v;
                v = (fl & 4u) ? v + va[u][j] : v;
                v = (fl & 8u) ? v + fu[u][j] : v;
                v = (fl & 16u) ? ((v > lo || v != v) ? v : lo) : v;               // a NaN stays
                y[j] = v;
            }
        }
        if (streams_result(P.n)) __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, y), r_out, off[u], 0, 2);
        else __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, y), r_out, off[u], 0, 0);
    }
}

extern "C" __global__ __launch_bounds__(256) void ew_affine_v4(
        float* __restrict__ out, const float* first, const float* s1, const float* s2, const float* s3,
        const float* vsub, const float* vmul, const float* vadd, const float* full, const float* floor_, EwAffineParams P) {
    ew_affine_body<false>(out, first, s1, s2, s3, vsub, vmul, vadd, full, floor_, P);
}
extern "C" __global__ __launch_bounds__(256) void ew_affine_big_v4(
        float* __restrict__ out, const float* first, const float* s1, const float* s2, const float* s3,
        const float* vsub, const float* vmul, const float* vadd, const float* full, const float* floor_, EwAffineParams P) {
    ew_affine_body<true>(out, first, s1, s2, s3, vsub, vmul, vadd, full, floor_, P);
}

// Requests one word of every 64-byte line of the argument block at the very start of a kernel and waits for all of
// them at once. The fields are fetched where the compiler needs them, in several dependent groups; a group that
// touches a line for the first time waits for a round trip to memory (about 1600 cycles), later ones find their
// line in the scalar cache. For a launch of a few waves those round trips are most of its duration.
template <int BYTES>
__device__ __forceinline__ void ew_touch_arguments() {
    static_assert(BYTES > 384 && BYTES <= 448, "seven lines");
    const char* args = reinterpret_cast<const char*>(__builtin_amdgcn_kernarg_segment_ptr());
    uint32_t w0, w1, w2, w3, w4, w5, w6;
    // one statement: the requests, then the wait (the compiler does not track loads issued by inline assembly)
    asm volatile("s_load_dword %0, %7, 0x0\n\ts_load_dword %1, %7, 0x40\n\ts_load_dword %2, %7, 0x80\n\t"
                 "s_load_dword %3, %7, 0xc0\n\ts_load_dword %4, %7, 0x100\n\ts_load_dword %5, %7, 0x140\n\t"
                 "s_load_dword %6, %7, 0x180\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(w0), "=&s"(w1), "=&s"(w2), "=&s"(w3), "=&s"(w4), "=&s"(w5), "=&s"(w6) : "s"(args) : "memory");
}

#define EW_KERNEL(name, VEC, NS)                                                                      \
    extern "C" __global__ __launch_bounds__(256) void name(                                            \
        uint32_t* __restrict__ out, const uint32_t* in0, const uint32_t* in1, const uint32_t* in2,      \
        const uint32_t* in3, const uint32_t* in4, const uint32_t* in5, const uint32_t* in6,             \
        const uint32_t* in7, EwParams P) {                                                              \
        const uint32_t* const in[EW_MAX_STEPS] = {in0, in1, in2, in3, in4, in5, in6, in7};              \
        ew_touch_arguments<sizeof(EwParams) + 9 * sizeof(void*)>();                                     \
        ew_chain_body<VEC, NS>(out, in, P, blockIdx.x);                                                 \
    }

// ew_chain_v4* requires: n % 4 == 0, dims[ndim-1] % 4 == 0, every operand's fastest stride in {0, 1},
// stride-1 operands 16-byte aligned with all slower strides % 4 == 0. The host checks this.
// The _sN suffix is the number of step slots the kernel handles (chains of up to N steps).
EW_KERNEL(ew_chain_v1_s2, 1, 2)
EW_KERNEL(ew_chain_v1_s4, 1, 4)
EW_KERNEL(ew_chain_v1_s6, 1, 6)
EW_KERNEL(ew_chain_v1_s8, 1, 8)
EW_KERNEL(ew_chain_v4_s2, 4, 2)
EW_KERNEL(ew_chain_v4_s4, 4, 4)
EW_KERNEL(ew_chain_v4_s6, 4, 6)
EW_KERNEL(ew_chain_v4_s8, 4, 8)

// Several small, mutually independent chains in ONE launch: a program with many little vectors
// (per-channel statistics, parameter updates) otherwise pays one launch latency for each of them.
// The host writes one entry per chain into a table in device memory; workgroup b belongs to the
// last entry whose first_block is <= b and evaluates that entry's chain as block b - first_block
// of the chain's own grid. Entries are sorted by first_block, entry 0 starts at block 0.
struct EwBatchEntry {
    uint32_t        first_block, pad0;
    uint32_t*       out;
    const uint32_t* in[EW_MAX_STEPS];
    EwParams        P;
    uint32_t        pad1;
};
static_assert(sizeof(EwBatchEntry) == 432, "the host lays the table out with 432-byte entries");

template <int VEC, int NS>
__device__ __forceinline__ void ew_batch_body(const EwBatchEntry* __restrict__ table, uint32_t entries) {
    uint32_t lo = 0, hi = entries;
    while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) >> 1;
        if (table[mid].first_block <= blockIdx.x) lo = mid; else hi = mid;
    }
    lo = __builtin_amdgcn_readfirstlane(lo);
    const EwBatchEntry& e = table[lo];
    ew_chain_body<VEC, NS, false>(e.out, e.in, e.P, blockIdx.x - e.first_block);
}

#define EW_BATCH_KERNEL(name, VEC, NS)                                                                \
    extern "C" __global__ __launch_bounds__(256) void name(const EwBatchEntry* __restrict__ table, uint32_t entries) { \
        ew_batch_body<VEC, NS>(table, entries);                                                         \
    }
EW_BATCH_KERNEL(ew_chain_batch_v1_s2, 1, 2)
EW_BATCH_KERNEL(ew_chain_batch_v1_s4, 1, 4)
EW_BATCH_KERNEL(ew_chain_batch_v4_s2, 4, 2)
EW_BATCH_KERNEL(ew_chain_batch_v4_s4, 4, 4)

struct IotaParams { uint32_t n, inner, size, to_float; };

// out[i] = (i / inner) % size   (reference: vkjax/shaders/iota.comp:8-11 for the 1-D case)
// Four consecutive elements per thread (16-byte stores); VEC = 4 needs n % 4 == 0.
template <int VEC>
__device__ __forceinline__ void iota_body(uint32_t* __restrict__ out, const IotaParams& P) {
    const uint32_t i = (blockIdx.x * 256u + threadIdx.x) * VEC;
    if (i >= P.n) return;
    // one division and one remainder per thread, then counting on (per element they made the launch ALU-bound: 57 us
    // for 64 M elements)
    uint32_t q = i / P.inner, r = i - q * P.inner, x = q % P.size;
    uint32_t v[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        v[j] = P.to_float ? f2u((float)x) : x;
        if (++r == P.inner) { r = 0; if (++x == P.size) x = 0; }
    }
    if constexpr (VEC == 4) { u32x4 t; t.x = v[0]; t.y = v[1]; t.z = v[2]; t.w = v[3]; *reinterpret_cast<u32x4*>(out + i) = t; }
    else out[i] = v[0];
}
extern "C" __global__ __launch_bounds__(256) void iota_nd_v1(uint32_t* __restrict__ out, IotaParams P) { iota_body<1>(out, P); }
extern "C" __global__ __launch_bounds__(256) void iota_nd_v4(uint32_t* __restrict__ out, IotaParams P) { iota_body<4>(out, P); }

struct FillParams { uint32_t n, value; };

// (16-byte stores for whole groups of four, single words for the tail)
extern "C" __global__ __launch_bounds__(256) void fill_u32(uint32_t* __restrict__ out, FillParams P) {
    const uint32_t i = (blockIdx.x * 256u + threadIdx.x) * 4u;
    if (i + 3u < P.n) {
        *reinterpret_cast<u32x4*>(out + i) = u32x4{P.value, P.value, P.value, P.value};
    } else {
        for (uint32_t j = i; j < P.n; ++j) out[j] = P.value;
    }
}

struct ConcatParams { uint32_t n, part_inner, out_inner, out_offset; };

// One operand of a concatenation: the operand is [outer, part_inner], the output
// [outer, out_inner]; operand row r lands at out[r*out_inner + out_offset ...].
// (reference: vkjax/shaders/concatenate.comp:9-25, two operands on the last axis only)
// VEC = 4 needs part_inner, out_inner and out_offset to be multiples of 4.
template <int VEC>
__device__ __forceinline__ void concat_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, const ConcatParams& P) {
    const uint32_t i = (blockIdx.x * 256u + threadIdx.x) * VEC, n = without_stream_bit(P.n);
    if (i >= n) return;
    const uint32_t r = i / P.part_inner, c = i - r * P.part_inner;
    const uint64_t at = (uint64_t)r * P.out_inner + P.out_offset + c;
    // (the rows of the result this part reaches into: n / part_inner of them; below 4 GiB when the host asks for streaming)
    const uint64_t reach = ((uint64_t)(n / P.part_inner) * P.out_inner + P.out_offset) * 4u;
    if constexpr (VEC == 4) store_x4(out, at, *reinterpret_cast<const u32x4*>(in + i), streams_result(P.n), (uint32_t)reach);
    else out[at] = in[i];
}
extern "C" __global__ __launch_bounds__(256) void concat_part_v1(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, ConcatParams P) {
    concat_body<1>(out, in, P);
}
extern "C" __global__ __launch_bounds__(256) void concat_part_v4(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, ConcatParams P) {
    concat_body<4>(out, in, P);
}

// XLA pad: out = value everywhere except at low + i * (interior + 1) along every dimension, where it
// is in[i]; negative low / high crop. One output element per thread (four with VEC = 4, which needs
// the last dimension untouched by the padding and divisible by 4). Up to 6 dimensions (unused = 1).
#define PAD_MAX_RANK 6
struct PadParams {
    uint32_t n;                           // output elements
    uint32_t out_dims[PAD_MAX_RANK], in_dims[PAD_MAX_RANK];
    int32_t  low[PAD_MAX_RANK];
    uint32_t step[PAD_MAX_RANK];          // interior + 1
};

// 32-bit index arithmetic (the host keeps both arrays below 2^32 - 2^12 elements); dimensions of extent 1 and
// steps of 1 cost no division: those branches are the same for the whole launch.
template <int VEC>
__device__ __forceinline__ void pad_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ in,
                                         const uint32_t* __restrict__ value, const PadParams& P) {
    const uint32_t e0 = (blockIdx.x * 256u + threadIdx.x) * VEC, n = without_stream_bit(P.n);
    if (e0 >= n) return;
    uint32_t r = e0, off = 0, mul = 1;
    bool inside = true;
#pragma unroll
    for (int d = PAD_MAX_RANK - 1; d >= 0; --d) {
        const uint32_t od = P.out_dims[d], step = P.step[d];
        if (od == 1u && P.low[d] == 0 && P.in_dims[d] == 1u) continue;
        uint32_t c = r;
        if (d > 0) { const uint32_t q = r / od; c = r - q * od; r = q; }   // the slowest dimension needs no split
        const int32_t p = (int32_t)c - P.low[d];
        uint32_t i = (uint32_t)p;
        bool on_grid = true;
        if (step != 1u) { i = (uint32_t)p / step; on_grid = i * step == (uint32_t)p; }
        inside = inside && p >= 0 && on_grid && i < P.in_dims[d];
        off += i * mul;
        mul *= P.in_dims[d];
    }
    const uint32_t v = value[0];
    if constexpr (VEC == 4) {
        u32x4 q = u32x4{v, v, v, v};
        if (inside) q = *reinterpret_cast<const u32x4*>(in + off);
        store_x4(out, e0, q, streams_result(P.n), n * 4u);
    } else {
        out[e0] = inside ? in[off] : v;
    }
}
extern "C" __global__ __launch_bounds__(256) void pad_nd_v1(uint32_t* __restrict__ out, const uint32_t* __restrict__ in,
                                                            const uint32_t* __restrict__ value, PadParams P) {
    pad_body<1>(out, in, value, P);
}
extern "C" __global__ __launch_bounds__(256) void pad_nd_v4(uint32_t* __restrict__ out, const uint32_t* __restrict__ in,
                                                            const uint32_t* __restrict__ value, PadParams P) {
    pad_body<4>(out, in, value, P);
}

// Copy that swaps the two fastest dimensions: out[b, i, j] = in[b * sb + j * sj + i], out dense
// [B, I, J]. The strided gather of the element-wise kernel touches a new cache line per element on
// one side; here a 64 x 64 tile goes through LDS, read along i (contiguous in `in`) and written
// along j (contiguous in `out`). Covers 2-D transposes and NHWC <-> NCHW style permutations.
struct TransposeParams { uint32_t B, I, J; int32_t sb; uint32_t sj; };      // sb may be negative (a reversed leading dimension); bit 31 of B: STREAM_RESULT_BIT

extern "C" __global__ __launch_bounds__(256) void transpose_tiled(uint32_t* __restrict__ out, const uint32_t* __restrict__ in,
                                                                  TransposeParams P) {
    __shared__ uint32_t tile[64][65];
    const uint32_t ti = threadIdx.x & 63u, tr = threadIdx.x >> 6;
    // Tiles are taken along diagonals: with a row pitch that is a large power of two, the tiles of one row or one
    // column of tiles all start in the same memory channel, and workgroups that run together would queue there.
    const uint32_t j0 = blockIdx.x * 64u, i0 = ((blockIdx.y + blockIdx.x) % gridDim.y) * 64u, b = blockIdx.z;
    const uint32_t* src = in + (int64_t)b * P.sb;
    uint32_t* dst = out + (uint64_t)b * P.I * P.J;
#pragma unroll
    for (uint32_t p = 0; p < 16; ++p) {
        const uint32_t j = j0 + tr + 4u * p, i = i0 + ti;
        if (i < P.I && j < P.J) tile[tr + 4u * p][ti] = src[(uint64_t)j * P.sj + i];
    }
    __syncthreads();
#pragma unroll
    for (uint32_t p = 0; p < 16; ++p) {
        const uint32_t i = i0 + tr + 4u * p, j = j0 + ti;
        if (i < P.I && j < P.J) dst[(uint64_t)i * P.J + j] = tile[ti][tr + 4u * p];
    }
}

// The same with 16-byte global accesses on both sides: needs I, J, sj, sb and the source offset to be
// multiples of 4. A thread reads four consecutive i of one j and, after the exchange through LDS,
// writes four consecutive j of one i.
// (bx, by, bz): the workgroup's place in the copy's own grid of (gx, gy, B) workgroups
__device__ __forceinline__ void transpose_v4_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, const TransposeParams& P,
                                                  const uint32_t bx, const uint32_t by, const uint32_t bz, const uint32_t gy) {
    __shared__ uint32_t tile[64][65];
    const uint32_t t16 = threadIdx.x & 15u, tr = threadIdx.x >> 4;        // 16 vectors per tile row, 16 rows per pass
    // Tiles are taken along diagonals: with a row pitch that is a large power of two, the tiles of one row or one
    // column of tiles all start in the same memory channel, and workgroups that run together would queue there.
    const uint32_t j0 = bx * 64u, i0 = ((by + bx) % gy) * 64u, b = bz;
    const uint32_t* src = in + (int64_t)b * P.sb;
    const uint64_t total = (uint64_t)without_stream_bit(P.B) * P.I * P.J * 4u;      // (below 4 GiB when the host asks for streaming)
    const bool stream = streams_result(P.B);
#pragma unroll
    for (uint32_t p = 0; p < 4; ++p) {
        const uint32_t j = j0 + tr + 16u * p, i = i0 + 4u * t16;
        if (i < P.I && j < P.J) {                                         // I % 4 == 0: a vector is inside or outside as a whole
            const u32x4 v = *reinterpret_cast<const u32x4*>(src + (uint64_t)j * P.sj + i);
            tile[tr + 16u * p][4u * t16] = v.x; tile[tr + 16u * p][4u * t16 + 1u] = v.y;
            tile[tr + 16u * p][4u * t16 + 2u] = v.z; tile[tr + 16u * p][4u * t16 + 3u] = v.w;
        }
    }
    __syncthreads();
#pragma unroll
    for (uint32_t p = 0; p < 4; ++p) {
        const uint32_t i = i0 + tr + 16u * p, j = j0 + 4u * t16;
        if (i < P.I && j < P.J) {
            u32x4 v;
            v.x = tile[4u * t16][tr + 16u * p]; v.y = tile[4u * t16 + 1u][tr + 16u * p];
            v.z = tile[4u * t16 + 2u][tr + 16u * p]; v.w = tile[4u * t16 + 3u][tr + 16u * p];
            store_x4(out, (uint64_t)b * P.I * P.J + (uint64_t)i * P.J + j, v, stream, (uint32_t)total);
        }
    }
}
extern "C" __global__ __launch_bounds__(256) void transpose_tiled_v4(uint32_t* __restrict__ out, const uint32_t* __restrict__ in,
                                                                     TransposeParams P) {
    transpose_v4_body(out, in, P, blockIdx.x, blockIdx.y, blockIdx.z, gridDim.y);
}

// 128 x 128 tiles for large arrays: runs of 512 contiguous bytes on both sides, sixteen 16-byte loads
// in flight per thread. Same conditions as transpose_tiled_v4.
__device__ __forceinline__ void transpose_v4_t128_body(uint32_t* __restrict__ out, const uint32_t* __restrict__ in, const TransposeParams& P,
                                                       const uint32_t bx, const uint32_t by, const uint32_t bz, const uint32_t gy) {
    __shared__ uint32_t tile[128][129];
    const uint32_t t32 = threadIdx.x & 31u, tr = threadIdx.x >> 5;        // 32 vectors per tile row, 8 rows per pass
    const uint32_t j0 = bx * 128u, i0 = ((by + bx) % gy) * 128u, b = bz;
    const uint32_t* src = in + (int64_t)b * P.sb;
    const uint64_t total = (uint64_t)without_stream_bit(P.B) * P.I * P.J * 4u;      // (below 4 GiB when the host asks for streaming)
    const bool stream = streams_result(P.B);
    u32x4 v[16];
#pragma unroll
    for (uint32_t p = 0; p < 16; ++p) {
        const uint32_t j = j0 + tr + 8u * p, i = i0 + 4u * t32;
        v[p] = u32x4{0u, 0u, 0u, 0u};
        if (i < P.I && j < P.J) v[p] = *reinterpret_cast<const u32x4*>(src + (uint64_t)j * P.sj + i);
    }
#pragma unroll
    for (uint32_t p = 0; p < 16; ++p) {
        uint32_t* row = tile[tr + 8u * p] + 4u * t32;
        row[0] = v[p].x; row[1] = v[p].y; row[2] = v[p].z; row[3] = v[p].w;
    }
    __syncthreads();
#pragma unroll
    for (uint32_t p = 0; p < 16; ++p) {
        const uint32_t i = i0 + tr + 8u * p, j = j0 + 4u * t32;
        if (i < P.I && j < P.J) {
            u32x4 w;
            w.x = tile[4u * t32][tr + 8u * p]; w.y = tile[4u * t32 + 1u][tr + 8u * p];
            w.z = tile[4u * t32 + 2u][tr + 8u * p]; w.w = tile[4u * t32 + 3u][tr + 8u * p];
            store_x4(out, (uint64_t)b * P.I * P.J + (uint64_t)i * P.J + j, w, stream, (uint32_t)total);
        }
    }
}
extern "C" __global__ __launch_bounds__(256) void transpose_tiled_v4_t128(uint32_t* __restrict__ out, const uint32_t* __restrict__ in,
                                                                          TransposeParams P) {
    transpose_v4_t128_body(out, in, P, blockIdx.x, blockIdx.y, blockIdx.z, gridDim.y);
}

// Several independent copies of this kind in ONE launch (the kernels of a network's convolutions, transposed for
// the backward pass: dozens of launches of a few microseconds each). As for the batched chains above, the host
// writes one entry per copy into a table in device memory and workgroup b belongs to the last entry whose
// first_block is <= b; its place in that copy's own (grid_x, grid_y, B) grid follows from b - first_block.
struct TransposeBatchEntry {
    uint32_t        first_block, grid_x;
    uint32_t*       out;
    const uint32_t* in;
    TransposeParams P;
    uint32_t        grid_y;
};
static_assert(sizeof(TransposeBatchEntry) == 48, "the host lays the table out with 48-byte entries");

template <bool BIG>
__device__ __forceinline__ void transpose_batch_body(const TransposeBatchEntry* __restrict__ table, uint32_t entries) {
    uint32_t lo = 0, hi = entries;
    while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) >> 1;
        if (table[mid].first_block <= blockIdx.x) lo = mid; else hi = mid;
    }
    lo = __builtin_amdgcn_readfirstlane(lo);
    const TransposeBatchEntry& e = table[lo];
    const uint32_t local = blockIdx.x - e.first_block, bx = local % e.grid_x, rest = local / e.grid_x;
    const uint32_t by = rest % e.grid_y, bz = rest / e.grid_y;
    if constexpr (BIG) transpose_v4_t128_body(e.out, e.in, e.P, bx, by, bz, e.grid_y);
    else transpose_v4_body(e.out, e.in, e.P, bx, by, bz, e.grid_y);
}
extern "C" __global__ __launch_bounds__(256) void transpose_tiled_batch_v4(const TransposeBatchEntry* __restrict__ table, uint32_t entries) {
    transpose_batch_body<false>(table, entries);
}
extern "C" __global__ __launch_bounds__(256) void transpose_tiled_batch_v4_t128(const TransposeBatchEntry* __restrict__ table, uint32_t entries) {
    transpose_batch_body<true>(table, entries);
}
