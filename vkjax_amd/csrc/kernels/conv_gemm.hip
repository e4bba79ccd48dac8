// fp32 implicit-GEMM convolution / matrix product on the MFMA units (v_mfma_f32_32x32x2_f32).
//
//   C[m, n] = sum_k A(m, k) * B(k, n)       m = (batch, out_y, out_x), n = out feature,
//                                           k = (kernel_y, kernel_x, in feature), in feature fastest
//   A(m, k) = lhs[b, y*SH + ky*DH - PH, x*SW + kx*DW - PW, c]   (zero outside; lhs dilation = only
//                                                               multiples of LH/LW exist)
//   B(k, n) = rhs[ky, kx, c, n]
//
// Both operands and the result are addressed through element strides, so any
// ConvDimensionNumbers permutation, and dot_general with either contracting dimension, run
// through the same kernel; the *_FAST template flags enable 16-byte loads when the feature
// axis is contiguous. It supersedes the reference's scalar kernels conv2d.comp and
// dot_general.comp (reference: vkjax/ops.py:277-297, 463-487; vkjax/shaders/conv2d.comp:44-95;
// vkjax/shaders/dot_general.comp:10-34).
//
// Block = WGM x WGN waves, each wave owns TM x TN tiles of 32x32; block tile BM x BN with
// BM = 32*WGM*TM, BN = 32*WGN*TN, K step BK (32 or 64). A and B tiles are staged through LDS
// (A: [BM][BK+4] so a lane reads 4 consecutive k with one 16-byte LDS load without bank
// conflicts; B: [BK][BN+4]); the next tiles are prefetched into registers while the MFMAs of
// the current one run. The sum over k is order-free, so lanes 0-31 take the first half of a k
// tile and lanes 32-63 the second half, which is what makes the 16-byte A reads possible.
// After the k loop an optional chain of element-wise steps (per-feature vectors, full-size
// tensors or scalars as operands) is applied to the accumulators before the single store.
//
// The fp32 MFMA executes on the same lanes as ordinary vector instructions: measured, a wave's
// vector instruction issues only once per 64-cycle MFMA of another wave on the same SIMD. Every
// vector instruction therefore costs MFMA throughput, and the 16-byte paths are written to need
// almost none: addresses are split into a per-thread part that is computed once per block and a
// per-k-tile part that is wave-uniform and travels in the scalar offset operand of the buffer
// instruction; taps that fall into the padding are looked up in a per-row bit mask built once;
// rows and columns outside the matrices are caught by the range check of the buffer descriptor
// (an out-of-range load returns zeros, an out-of-range store is dropped); row decoding uses
// multiply-high division by constants prepared on the host.
#include "common.h"

#define CONV_MAX_EPI 6
#define CONV_OOB 0x80000000u     // byte offset beyond any descriptor: loads give 0, stores are dropped

enum EwOpConv : uint32_t {
#define EW_OP(name, num) CEW_##name = num,
#include "ew_opcodes.h"
#undef EW_OP
};

// Argument block. The fields up to wo_shift are used by every variant and are fetched into
// scalar registers in one batch when a block starts; the rest is only read by the generic
// (strided) paths, where it is needed.
struct ConvParams {
    int32_t M, N, K;
    int32_t Ho, Wo;                 // M = batch * Ho * Wo
    int32_t H, W, Cin;              // lhs spatial size (undilated) and features
    int32_t KH, KW;
    int32_t SH, SW, PH, PW, DH, DW;
    int32_t xs_b, xs_h, xs_w;       // lhs strides in elements
    int32_t tiles_m, tiles_n;
    uint32_t flags;                 // bit0: out is row-major [M, N]; bit1: m is the input row index itself
                                    // (batch = Wo = 1, stride 1, no padding: no row decode, no masks); bit2: some kernel taps of some
                                    // rows fall outside the input; bits 8-11: number of epilogue
                                    // steps; bits 12-15: 0, or 1 + t: the value after t template steps
                                    // (t = 0, or t = 1 after `acc - vector`) is ALSO stored, laid out like
                                    // out, to the array the last epilogue pointer slot names;
                                    // bits 16-19: 1 + index of the first kind-3 step, or 0;
                                    // bits 20-24: the steps are, in this order, a subset of
                                    // (acc - vector, * vector, + vector, + full tensor, max(acc, scalar)):
                                    // bit 20+k set = template step k is present;
                                    // bits 25-28: M tiles per block (at least 1);
                                    // bits 29-31: four-waves-per-tile kernels: 0, or 1 + log2 of the number of XCD columns
    uint32_t epi_desc[2];           // 10 bits per step, steps 0-2 in [0], 3-5 in [1]: bits 0-7 opcode * 2 +
                                    // (operand is the left argument), bits 8-9 kind: 1 scalar,
                                    // 2 per-feature vector [N], 3 full tensor laid out like out
    uint32_t x_bytes, w_bytes, out_bytes;   // sizes for the buffer descriptors (each below 2^31)
    uint32_t howo_magic, howo_shift;        // n / (Ho*Wo) = mulhi(n, magic) >> shift for 0 <= n < 2^31
    uint32_t wo_magic, wo_shift;            // same for Wo; magic 0 stands for a divisor of 1
    int32_t LH, LW, xs_c;           // lhs dilation and feature stride
    int32_t ws_r, ws_s, ws_c, ws_n; // rhs strides
    int32_t os_b, os_h, os_w, os_n; // out strides
    int32_t split_tiles_m;          // mixed kernels only: the first split_tiles_m M tiles (of 64 rows) are computed as 64 x 64
                                    // tiles, the rows behind them as 32 x 32 tiles by the blocks that follow in the grid
    int32_t k_split_steps;          // four-waves-per-tile kernels only: 0, or the k steps (of 128) one block sums. The grid then holds
                                    // ceil(k steps / k_split_steps) blocks per tile; those of slice s store their sums, without an
                                    // epilogue, to the s-th [M, N] matrix behind out, and a later launch adds the slices
    int32_t m_blocks;               // lean kernels: 0, or the number of blocks that share the M tiles of one N tile as evenly as whole
                                    // tiles allow: every block takes m_each = tiles_m / m_blocks consecutive tiles, the first
                                    // m_extra = tiles_m % m_blocks blocks one more; the M tiles per block in the flags are then
                                    // ignored. For grids sized to what the GPU holds at once.
    int32_t m_each, m_extra;
};

// The part of the output a block's tile number refers to: a grid of tiles_m x tiles_n tiles whose first row is
// m_base, handed to the blocks from first_block on.
struct ConvRegion { int first_block, tiles_m, tiles_n, m_base; };

// LDS of one block: A tile, B tile, per-column epilogue operands, row offsets (floats)
template <int WGM, int WGN, int TM, int TN, int BK>
constexpr int conv_pool_floats() { return 32 * WGM * TM * (BK + 4) + BK * (32 * WGN * TN + 4) + CONV_MAX_EPI * 32 * WGN * TN + 32 * WGM * TM; }

struct ConvEpiPtrs { const float* p[CONV_MAX_EPI]; };

// One per-feature epilogue operand may be computed instead of read: the value for column n is
//     v = first[n]; v = op_k(v, operand_k[n]) for k < nsteps      (each array a vector [N] or a single value)
// which lets the small chain that prepares a batch-norm scale (gamma * rsqrt(var + eps)) run inside
// the convolution that consumes it instead of as a launch of its own.
#define CONV_MAX_DERIVED 3
struct ConvDerivedPtrs { const float* p[CONV_MAX_DERIVED + 1]; };   // first, then the operand of each step (null where a step has none)
struct ConvDerived {
    uint32_t step;                          // the epilogue step whose operand this is
    uint32_t nsteps;                        // 0: nothing is derived
    uint32_t vector_mask;                   // bit k: array k is a vector [N] (else one value)
    uint32_t op[CONV_MAX_DERIVED];          // add / sub / mul / div / max / min / neg / rsqrt / sqrt, float
    uint32_t left[CONV_MAX_DERIVED];        // the operand is the left argument
};

// LEAN: the variant for the common case, with the rarely needed paths compiled out (they cost
// registers, and with them resident waves, even when not taken): both operands on the 16-byte
// path, k tiles that never straddle kernel taps, a row-major result, an epilogue that fits the
// straight-line template.
template <int WGM, int WGN, int TM, int TN, int BK, bool A_FAST, bool B_FAST, bool LEAN, int KSW = 1>
__device__ __forceinline__ void conv_gemm_body(float* __restrict__ pool, const ConvRegion region, float* __restrict__ out, const float* __restrict__ x,
                                               const float* __restrict__ w, const ConvEpiPtrs& epi,
                                               const ConvDerivedPtrs& Dp, const ConvParams& Pk, const ConvDerived& Dk) {
    // KSW > 1: KSW groups of WGM x WGN waves share one block tile, each taking a 1/KSW slice of every k
    // step; their accumulators are added through LDS before the epilogue. For products whose handful of
    // tiles would otherwise leave most of a CU's four MFMA units idle (a wave can drive only one).
    static_assert(KSW == 1 || (LEAN && TM == 1 && TN == 1), "k-split blocks exist for the lean single-tile form only");
    constexpr int BM = 32 * WGM * TM, BN = 32 * WGN * TN, NT = 64 * WGM * WGN * KSW;
    constexpr int LDA = BK + 4, LDB = BN + 4;
    static_assert((BM * LDA) % 4 == 0 && (BK * LDB) % 4 == 0, "16-byte alignment of the LDS tiles");
    float* const As = pool;                         // [BM][LDA]
    float* const Bs = As + BM * LDA;                // [BK][LDB]
    float* const Es = Bs + BK * LDB;                // [CONV_MAX_EPI][BN]: per-column operands of the epilogue steps
    int*   const Rs = reinterpret_cast<int*>(Es + CONV_MAX_EPI * BN);   // [BM]: row offsets of outputs that are not row-major

    // Copy the hot part of the argument block into scalar registers once, at the very start. Left
    // to itself the compiler fetches each field right before its first use; under load every such
    // fetch costs about a microsecond, and the prologue and the epilogue would each chain several.
    struct {
        int32_t M, N, K, Ho, Wo, H, W, Cin, KH, KW, SH, SW, PH, PW, DH, DW, xs_b, xs_h, xs_w, tiles_m, tiles_n, m_blocks, m_each, m_extra;
        uint32_t flags, epi_desc[2], x_bytes, w_bytes, out_bytes, howo_magic, howo_shift, wo_magic, wo_shift;
    } P;
#define CONV_PIN(f) P.f = Pk.f; asm volatile("" : "+s"(P.f));
    asm volatile("" : "+s"(out), "+s"(x), "+s"(w));
#pragma unroll
    for (int q = 0; q < CONV_MAX_EPI; ++q) asm volatile("" :: "s"(epi.p[q]));
    CONV_PIN(M) CONV_PIN(N) CONV_PIN(K) CONV_PIN(Ho) CONV_PIN(Wo) CONV_PIN(H) CONV_PIN(W) CONV_PIN(Cin)
    CONV_PIN(KH) CONV_PIN(KW) CONV_PIN(SH) CONV_PIN(SW) CONV_PIN(PH) CONV_PIN(PW) CONV_PIN(DH) CONV_PIN(DW)
    CONV_PIN(xs_b) CONV_PIN(xs_h) CONV_PIN(xs_w) CONV_PIN(tiles_m) CONV_PIN(tiles_n) CONV_PIN(flags)
    CONV_PIN(epi_desc[0]) CONV_PIN(epi_desc[1]) CONV_PIN(x_bytes) CONV_PIN(w_bytes) CONV_PIN(out_bytes)
    CONV_PIN(howo_magic) CONV_PIN(howo_shift) CONV_PIN(wo_magic) CONV_PIN(wo_shift) CONV_PIN(m_blocks) CONV_PIN(m_each) CONV_PIN(m_extra)
#undef CONV_PIN
    static_assert(CONV_MAX_EPI == 6, "descriptor packing");
    auto step_desc = [&](int e) -> uint32_t { return ((e < 3 ? P.epi_desc[0] : P.epi_desc[1]) >> (10 * (e < 3 ? e : e - 3))) & 1023u; };
    const bool c_contig = LEAN || (P.flags & 1u), flat_rows = P.flags & 2u, masked = P.flags & 4u;
    const int nepi = (P.flags >> 8) & 15u, epi_first_full = (int)((P.flags >> 16) & 15u) - 1;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kw = wave / (WGM * WGN), wm = (wave % (WGM * WGN)) / WGN, wn = wave % WGN;
    const int l32 = lane & 31, half = lane >> 5;
    // A single 32 x 32 tile whose k steps are shared by KSW waves: every wave loads, parks in LDS and consumes its
    // own slice of a k step, so the k loop needs no barrier between the waves; they drift apart and one wave's
    // MFMAs cover the others' load latencies (a block of these kernels is usually alone on its CU).
    constexpr bool WAVE_PRIVATE = KSW > 1 && WGM == 1 && WGN == 1 && A_FAST;
    constexpr int  BKW_ = BK / KSW;
    // thread -> (row within a pass, 16-byte vector within the row) of the A tile, (k row, vector) of the B tile
    const int a_r0 = WAVE_PRIVATE ? lane / (BKW_ / 4) : tid / (BK / 4);
    const int a_kv = WAVE_PRIVATE ? kw * (BKW_ / 4) + lane % (BKW_ / 4) : tid % (BK / 4);
    const int b_r0 = WAVE_PRIVATE ? kw * BKW_ + lane / (BN / 4) : tid / (BN / 4);
    const int b_nv = WAVE_PRIVATE ? lane % (BN / 4) : tid % (BN / 4);
    auto tile_barrier = [&]() {
        if constexpr (WAVE_PRIVATE) __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");   // LDS accesses of a wave execute in order
        else __syncthreads();
    };

    // A block works through up to `chunk` consecutive M tiles of one N tile, one after the other,
    // as one flat sequence of k steps: while a step is computed the loads of the next one are in
    // flight, also across the boundary between two M tiles. Only the first tile of a block pays
    // the latency of the argument fetch, the address set-up and the first loads in full.
    // Consecutive block ids go to different XCDs (8 of them, each with its own L2). Hand every
    // XCD a contiguous range of work so that the N-tiles of one M-tile share an L2.
    const int chunk = LEAN ? (P.flags >> 25) & 15u : 1;         // the general variants take one tile per block
    const int m_blocks = LEAN && KSW == 1 ? P.m_blocks : 0;
    // (every wave runs this once per block on the CU's one scalar unit: divisors that are powers of two, the usual
    // case for the M tiles per block and the number of N tiles, cost a shift instead of the long division sequence)
    auto div_small = [](int n, int d) { return (d & (d - 1)) == 0 ? n >> __builtin_ctz((unsigned)d) : n / d; };
    const int chunks_m = m_blocks > 0 ? m_blocks : div_small(region.tiles_m + chunk - 1, chunk);
    int work = (int)blockIdx.x - region.first_block;
    // K_SPLIT kernels can share a tile's contraction among several blocks (for products with so few tiles that most
    // CUs would stay idle while a few fetch all the weights): slice s sums k steps [kbase, kbase + ktiles)
    constexpr bool K_SPLIT = KSW > 1 && BK == 128;
    int kbase = 0, ktiles = max(1, (P.K + BK - 1) / BK);       // K = 0 runs as one k step whose loads are all out of range
    if constexpr (K_SPLIT) {
        const int per = Pk.k_split_steps;
        if (per > 0) {
            const int tiles = chunks_m * region.tiles_n, slice = work / tiles;
            work -= slice * tiles;
            kbase = slice * per;
            ktiles = min(per, ktiles - kbase);
            out += (size_t)slice * (size_t)P.M * (size_t)P.N;
        }
    }
    // Four-waves-per-tile kernels (products with few tiles, often with the kernel operand as the large one): the host may
    // ask for the XCDs to be laid over the tile grid as 8 / xn rows of xn columns (flags bits 29-31 hold 1 + log2 xn),
    // each XCD owning a rectangle of tiles_m / (8 / xn) x tiles_n / xn tiles (both divisible; the host checks). An XCD's
    // L2 then fetches 1 / (8 / xn) of the rows of A and 1 / xn of the columns of B, instead of a few rows of A and
    // all of B.
    const int xcd_code = KSW > 1 ? (int)(P.flags >> 29) : 0;
    int chunk_m, tile_n;
    if (xcd_code > 0) {
        const int xn = 1 << (xcd_code - 1), sub_n = div_small(region.tiles_n, xn);
        const int x = work & 7, l = work >> 3, xi = x >> (xcd_code - 1), xj = x & (xn - 1);
        const int sub_m = region.tiles_m >> (4 - xcd_code);                     // tiles_m / (8 / xn)
        const int lm = div_small(l, sub_n);
        chunk_m = xi * sub_m + lm;
        tile_n  = xj * sub_n + (l - lm * sub_n);
    } else {
        const int total = chunks_m * region.tiles_n, per = total / 8;
        if (per > 0 && work < per * 8) work = (work & 7) * per + (work >> 3);
        chunk_m = div_small(work, region.tiles_n);
        tile_n  = work - chunk_m * region.tiles_n;
    }
    int tile_m0 = chunk_m * chunk, nsub = LEAN ? min(chunk, region.tiles_m - tile_m0) : 1;
    if (m_blocks > 0) {
        tile_m0 = chunk_m * P.m_each + min(chunk_m, P.m_extra);
        nsub    = P.m_each + (chunk_m < P.m_extra ? 1 : 0);
    }
    const int n0 = tile_n * BN;
    const int HoWo = P.Ho * P.Wo;

    // The 16-byte A path addresses the input from (PH, PW) positions before its start, so that
    // the offset of a row's top-left tap is never negative (a negative offset is out of range
    // for the descriptor even when a later addition brings it back).
    const uint32_t x_bias = A_FAST ? (uint32_t)(P.PH * P.xs_h + P.PW * P.xs_w) * 4u : 0u;
    const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(reinterpret_cast<const char*>(x) - x_bias, P.x_bytes + x_bias),
                                 w_rsrc = make_rsrc(w, P.w_bytes), o_rsrc = make_rsrc(out, P.out_bytes);

    // Scalar and per-feature epilogue operands are fetched once per block and parked in LDS, so that the epilogue
    // never waits on global memory for them. Thread t fetches column t of every step. Every step issues one load,
    // whatever its kind, so that none waits for the one before: an absent operand, one that is derived below, or a
    // full tensor (read in the epilogue) has a descriptor of size 0, which reads nothing and returns 0.
    // Where a block is alone on its CU (the four-waves-per-tile kernels) they are requested right behind the first
    // k tile's loads: one round trip to memory for both. Elsewhere they go first, and the other blocks' work covers them.
    constexpr bool EPI_BEHIND_TILES = KSW > 1;
    float e_reg[CONV_MAX_EPI], d_in[CONV_MAX_DERIVED + 1];
    uint32_t e_bytes[CONV_MAX_EPI], e_scale[CONV_MAX_EPI];       // (the same in every lane: worked out before the lanes part)
#pragma unroll
    for (int e = 0; e < CONV_MAX_EPI; ++e) {
        const uint32_t kind = step_desc(e) >> 8;                 // 0 beyond the last step
        const uint32_t present = epi.p[e] != nullptr ? 1u : 0u;
        e_bytes[e] = (uint32_t)__builtin_amdgcn_readfirstlane((int)(kind == 1 ? 4u * present : kind == 2 ? (uint32_t)P.N * 4u * present : 0u));
        e_scale[e] = kind == 2 ? 4u : 0u;
    }
    auto request_epilogue_operands = [&]() {
        if (tid < BN) {
#pragma unroll
            for (int e = 0; e < CONV_MAX_EPI; ++e)
                e_reg[e] = buffer_load_x1(make_rsrc(epi.p[e], e_bytes[e]), (uint32_t)(n0 + tid) * e_scale[e]);
            if (Dk.nsteps) {
                // the arrays of the derived operand: combined once the first k tile's loads are on their way (combining
                // them at once would hold the wave, and with it the block's first barrier, for a round trip to memory)
#pragma unroll
                for (int k = 0; k <= CONV_MAX_DERIVED; ++k) {
                    const bool vec = (Dk.vector_mask >> k) & 1u;
                    d_in[k] = buffer_load_x1(make_rsrc(Dp.p[k], Dp.p[k] == nullptr ? 0u : vec ? (uint32_t)P.N * 4u : 4u),
                                             vec ? (uint32_t)(n0 + tid) * 4u : 0u);
                }
            }
        }
    };
    if constexpr (!EPI_BEHIND_TILES) request_epilogue_operands();
    // the first full-size operand (a residual input) is fetched for a whole tile at once, while
    // the tile's last k step is computed (for the largest tile that would not fit the register
    // file: it loads sub-tile by sub-tile in the epilogue)
    constexpr bool PREFETCH_FULL = !LEAN && TM * TN <= 2;
    const int first_full = (PREFETCH_FULL && c_contig) ? epi_first_full : -1;
    const float* full_ptr = epi.p[0];
#pragma unroll
    for (int t = 1; t < CONV_MAX_EPI; ++t) full_ptr = epi_first_full == t ? epi.p[t] : full_ptr;
    const __amdgpu_buffer_rsrc_t f_rsrc = make_rsrc(full_ptr, P.out_bytes);

    // ---------------- per-thread load assignment ----------------
    // A fast: 16-byte vectors along k. A generic: one row, a run of consecutive k.
    constexpr int A_VPR   = BK / 4;                 // vectors per row
    constexpr int A_RSTEP = WAVE_PRIVATE ? 64 / (BKW_ / 4) : NT / A_VPR;   // rows between a thread's vectors
    constexpr int A_NV    = BM / A_RSTEP;           // vectors per thread
    constexpr int A_KG    = NT / BM;                // generic: k groups
    constexpr int A_KPT   = BK / A_KG;              // generic: k per thread
    constexpr int A_ROWS  = A_FAST ? A_NV : 1;
    // fast: byte offset of (row, tap 0, this thread's k vector) from the biased base, out of range for rows beyond M;
    //       bit t of a_inv set = tap t = ky*KW + kx of that row lies outside the input
    // generic: element offset of the row's batch and the input coordinates of its tap 0
    uint32_t a_voff[A_ROWS], a_inv[A_ROWS];
    int a_off0 = 0, a_hi0 = 0, a_wi0 = 0;
    // When a k tile never straddles two kernel taps (Cin % BK == 0, or there is only one tap) the
    // tap (ky, kx) and first feature of a tile are the same for the whole block and live in
    // scalar registers.
    const bool uniform_taps = LEAN || (A_FAST && (P.Cin % BK == 0 || P.KH * P.KW == 1));
    int t_r = 0, t_s = 0, t_c = 0;                  // uniform tile position
    // otherwise every thread tracks the position of its own first k
    int ak = 0, ac = 0, as_ = 0, ar = 0;
    // per-thread state for the M tile that starts at row m0, positioned at its first k tile
    auto setup_rows = [&](int m0) {
#pragma unroll
        for (int p = 0; p < A_ROWS; ++p) {
            const int row = A_FAST ? (a_r0 + p * A_RSTEP) : (tid % BM);
            const int m = m0 + row;
            if (A_FAST && flat_rows) {
                a_voff[p] = m < P.M ? (uint32_t)(m * P.xs_h + a_kv * 4) * 4u : CONV_OOB;
                a_inv[p]  = 0u;
                continue;
            }
            int b = 0, ho = m, wo = 0;
            if (!flat_rows) {
                b = magic_div(m, P.howo_magic, P.howo_shift);
                const int r2 = m - b * HoWo;
                ho = magic_div(r2, P.wo_magic, P.wo_shift);
                wo = r2 - ho * P.Wo;
            }
            const int hi0 = ho * P.SH - P.PH, wi0 = wo * P.SW - P.PW;
            if constexpr (A_FAST) {
                a_voff[p] = m < P.M ? (uint32_t)(b * P.xs_b + ho * P.SH * P.xs_h + wo * P.SW * P.xs_w + a_kv * 4) * 4u : CONV_OOB;
                a_inv[p]  = 0u;
                if (masked) {
                    uint32_t wbad = 0u;
                    for (int s = 0; s < P.KW; ++s) wbad |= ((uint32_t)(wi0 + s * P.DW) >= (uint32_t)P.W ? 1u : 0u) << s;
                    const uint32_t wall = (2u << (P.KW - 1)) - 1u;
                    for (int r = 0; r < P.KH; ++r)
                        a_inv[p] |= ((uint32_t)(hi0 + r * P.DH) >= (uint32_t)P.H ? wall : wbad) << (r * P.KW);
                }
            } else {
                a_voff[p] = 0u; a_inv[p] = 0u;
                a_off0 = b * P.xs_b;
                a_hi0 = m < P.M ? hi0 : -(1 << 28);
                a_wi0 = m < P.M ? wi0 : -(1 << 28);
            }
        }
        t_r = 0; t_s = 0; t_c = 0;
        if constexpr (K_SPLIT) {
            if (kbase > 0) {                          // a later slice of the contraction starts at its own tap and feature
                const int k0 = kbase * BK, rs = k0 / P.Cin;
                t_c = k0 - rs * P.Cin; t_r = rs / P.KW; t_s = rs - t_r * P.KW;
            }
        }
        ak = A_FAST ? a_kv * 4 : (tid / BM) * A_KPT;
        const int rs = ak / P.Cin;
        ac = ak - rs * P.Cin; ar = rs / P.KW; as_ = rs - ar * P.KW;
    };

    constexpr int B_VPR   = BN / 4;
    constexpr int B_RSTEP = WAVE_PRIVATE ? 64 / B_VPR : NT / B_VPR;
    constexpr int B_NV    = (WAVE_PRIVATE ? BKW_ : BK) / B_RSTEP;
    constexpr int B_KG    = NT / BN;                // generic: k groups
    constexpr int B_KPT   = BK / B_KG;
    // B fast: byte offset of this thread's first vector in tile 0, or out of range for columns >= N
    const int      b_n    = n0 + b_nv * 4;
    const uint32_t b_voff = b_n < P.N ? (uint32_t)(b_r0 * P.N + b_n) * 4u : CONV_OOB;

    // what a thread has requested of the coming k step(s): one step ahead, two for the wave-private tiles, whose
    // single block per CU has nothing else to cover a load's latency with
    // (not for the small tiles of the mixed kernels, k step 64: their registers decide how many blocks share a CU;
    // nor with element-wise loads of B, whose 16 values per step and stage would spill)
    constexpr int STAGES = WAVE_PRIVATE && BK >= 128 && B_FAST ? 2 : 1;
    f32x4 a_reg[STAGES][A_FAST ? A_NV : 1];
    float a_sreg[A_FAST ? 1 : A_KPT];
    f32x4 b_reg[STAGES][B_FAST ? B_NV : 1];
    float b_sreg[STAGES][B_FAST ? 1 : B_KPT];

    auto load_tiles = [&](int k0, int st = 0) {
        // ---- A ----
        if constexpr (A_FAST) {
            if (uniform_taps) {
                // everything that changes from tile to tile is wave-uniform
                const uint32_t soff = (uint32_t)(t_r * P.DH * P.xs_h + t_s * P.DW * P.xs_w + t_c) * 4u;
                const bool     tail = k0 + BK > P.K;                 // only with a single tap
                if (!masked && !tail) {
                    // the common case issues the loads with no vector arithmetic at all
#pragma unroll
                    for (int p = 0; p < A_NV; ++p) a_reg[st][p] = buffer_load_x4(x_rsrc, a_voff[p], soff);
                } else {
                    const uint32_t sh   = 31u - (uint32_t)(t_r * P.KW + t_s);
                    const bool     kbad = tail && k0 + a_kv * 4 >= P.K;
#pragma unroll
                    for (int p = 0; p < A_NV; ++p) {
                        const uint32_t v = a_voff[p] | ((a_inv[p] << sh) & CONV_OOB);
                        a_reg[st][p] = buffer_load_x4(x_rsrc, kbad ? CONV_OOB : v, soff);
                    }
                }
            } else {
                const uint32_t koff = (uint32_t)(ar * P.DH * P.xs_h + as_ * P.DW * P.xs_w + ac - a_kv * 4) * 4u;
                const uint32_t sh   = 31u - (uint32_t)(ar * P.KW + as_);
                const bool     kok  = ak < P.K;
#pragma unroll
                for (int p = 0; p < A_NV; ++p) {
                    uint32_t v = (a_voff[p] + koff) | (a_voff[p] & CONV_OOB);
                    if (masked) v |= (a_inv[p] << sh) & CONV_OOB;
                    a_reg[st][p] = buffer_load_x4(x_rsrc, kok ? v : CONV_OOB);
                }
            }
        } else {
            int c = ac, s = as_, r = ar, k = ak;
#pragma unroll
            for (int j = 0; j < A_KPT; ++j) {
                int hi = a_hi0 + r * P.DH, wi = a_wi0 + s * P.DW;
                bool ok = hi >= 0 && wi >= 0 && k < P.K;
                if (Pk.LH > 1) { ok = ok && (hi % Pk.LH == 0); hi /= Pk.LH; }
                if (Pk.LW > 1) { ok = ok && (wi % Pk.LW == 0); wi /= Pk.LW; }
                ok = ok && hi < P.H && wi < P.W;
                a_sreg[j] = ok ? x[a_off0 + hi * P.xs_h + wi * P.xs_w + c * Pk.xs_c] : 0.f;
                ++k; ++c;
                if (c == P.Cin) { c = 0; ++s; if (s == P.KW) { s = 0; ++r; } }
            }
        }
        // ---- B ----
        if constexpr (B_FAST) {
            // rows k >= K fall beyond the descriptor and read as zeros
#pragma unroll
            for (int p = 0; p < B_NV; ++p)
                b_reg[st][p] = buffer_load_x4(w_rsrc, b_voff, (uint32_t)(k0 + p * B_RSTEP) * (uint32_t)P.N * 4u);
        } else {
            const int n = n0 + tid % BN;
            int k = k0 + (tid / BN) * B_KPT;
            const int rs = k / P.Cin;
            int c = k - rs * P.Cin, r = rs / P.KW, s = rs - r * P.KW;
#pragma unroll
            for (int j = 0; j < B_KPT; ++j) {
                b_sreg[st][j] = (k < P.K && n < P.N) ? w[r * Pk.ws_r + s * Pk.ws_s + c * Pk.ws_c + n * Pk.ws_n] : 0.f;
                ++k; ++c;
                if (c == P.Cin) { c = 0; ++s; if (s == P.KW) { s = 0; ++r; } }
            }
        }
        // advance to the next k tile
        if (uniform_taps) {
            t_c += BK;
            if (t_c >= P.Cin) { t_c = 0; ++t_s; if (t_s == P.KW) { t_s = 0; ++t_r; } }
        } else {
            ak += BK; ac += BK;
            while (ac >= P.Cin) { ac -= P.Cin; ++as_; if (as_ == P.KW) { as_ = 0; ++ar; } }
        }
    };

    auto store_tiles = [&](int st = 0) {
        if constexpr (A_FAST) {
#pragma unroll
            for (int p = 0; p < A_NV; ++p) {
                const int row = a_r0 + p * A_RSTEP, kv = a_kv;
                *reinterpret_cast<f32x4*>(&As[row * LDA + kv * 4]) = a_reg[st][p];
            }
        } else {
            const int row = tid % BM, kb = (tid / BM) * A_KPT;
#pragma unroll
            for (int j = 0; j < A_KPT; ++j) As[row * LDA + kb + j] = a_sreg[j];
        }
        if constexpr (B_FAST) {
#pragma unroll
            for (int p = 0; p < B_NV; ++p) {
                const int kr = b_r0 + p * B_RSTEP, nv = b_nv;
                *reinterpret_cast<f32x4*>(&Bs[kr * LDB + nv * 4]) = b_reg[st][p];
            }
        } else {
            const int n = tid % BN, kb = (tid / BN) * B_KPT;
#pragma unroll
            for (int j = 0; j < B_KPT; ++j) Bs[(kb + j) * LDB + n] = b_sreg[st][j];
        }
    };

    // Calls fn(v, per-lane byte offset, uniform byte offset) for the 16 accumulator elements a
    // lane holds of sub-tile (i, j) of the M tile at row m0: element v is row 8*(v/4) + 4*half +
    // v%4, column l32. The offsets are out of range outside the matrix. For a row-major result
    // one per-lane offset serves all 16 (the row goes into the uniform part, and rows beyond M lie
    // beyond the descriptor's size). The lane id and the row pitch go through opaque copies so
    // that this arithmetic is redone at each use instead of occupying registers for the whole
    // loop. Byte offsets fit 31 bits: the host refuses larger tensors.
    auto sub_tile = [&](int m0, int i, int j, auto&& fn) {
        int l = l32;
        asm volatile("" : "+v"(l));
        const int n  = n0 + (wn * TN + j) * 32 + l;
        const int r0 = (wm * TM + i) * 32 + 4 * half;
        if (c_contig) {
            const uint32_t base = n < P.N ? (uint32_t)((m0 + r0) * P.N + n) * 4u : CONV_OOB;
            uint32_t rowb = (uint32_t)P.N * 4u;
            asm volatile("" : "+s"(rowb));
#pragma unroll
            for (int v = 0; v < 16; ++v) fn(v, base, (uint32_t)(8 * (v / 4) + (v % 4)) * rowb);
        } else {
            const int* ro = Rs + r0 + (l - l32);
            const int  cn = n < P.N ? n * Pk.os_n : -(1 << 30);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = ro[8 * (v / 4) + (v % 4)];
                fn(v, (r >= 0 && cn >= 0) ? (uint32_t)(r + cn) * 4u : CONV_OOB, 0u);
            }
        }
    };

    float full[PREFETCH_FULL ? TM : 1][PREFETCH_FULL ? TN : 1][16];
    setup_rows(region.m_base + tile_m0 * BM);
    load_tiles(kbase * BK);
    if constexpr (EPI_BEHIND_TILES) request_epilogue_operands();
    if (tid < BN) {
        if (Dk.nsteps) {
            // the derived operand: same arithmetic, operation by operation, as the element-wise kernel
            float v = d_in[0];
#pragma unroll
            for (int k = 0; k < CONV_MAX_DERIVED; ++k) {
                if (k < (int)Dk.nsteps) {
                    const float a = Dk.left[k] ? d_in[k + 1] : v, b = Dk.left[k] ? v : d_in[k + 1];
                    switch (Dk.op[k]) {
                        case CEW_ADD_F:   v = a + b; break;
                        case CEW_SUB_F:   v = a - b; break;
                        case CEW_MUL_F:   v = a * b; break;
                        case CEW_DIV_F:   v = a / b; break;
                        case CEW_MAX_F:   v = (a > b || a != a) ? a : b; break;
                        case CEW_MIN_F:   v = (a < b || a != a) ? a : b; break;
                        case CEW_NEG_F:   v = -v; break;
                        case CEW_RSQRT_F: v = 1.0f / sqrtf(v); break;
                        case CEW_SQRT_F:  v = sqrtf(v); break;
                        default: break;
                    }
                }
            }
#pragma unroll
            for (int e = 0; e < CONV_MAX_EPI; ++e)
                if (e == (int)Dk.step) e_reg[e] = v;
        }
#pragma unroll
        for (int e = 0; e < CONV_MAX_EPI; ++e)
            if (e < nepi) Es[e * BN + tid] = e_reg[e];           // published by the barriers of the first k step
    }

    f32x16 acc[TM][TN];
    // one k step on the tiles in LDS. Lanes 0-31 consume the first half of the tile's k range,
    // lanes 32-63 the second half. Fragments are double-buffered in registers: the LDS reads of
    // group g+1 are in flight while the MFMAs of group g execute.
    auto compute = [&]() {
        constexpr int BKW = BK / KSW, G = BKW / 8;               // this wave's slice of the k step
        f32x4 af[2][TM];
        float bf[2][TN][4];
        auto load_frags = [&](int g, int buf) {
            const int kk = kw * BKW + half * (BKW / 2) + g * 4;
#pragma unroll
            for (int i = 0; i < TM; ++i)
                af[buf][i] = *reinterpret_cast<const f32x4*>(&As[((wm * TM + i) * 32 + l32) * LDA + kk]);
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) bf[buf][j][q] = Bs[(kk + q) * LDB + (wn * TN + j) * 32 + l32];
        };
        load_frags(0, 0);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (g + 1 < G) load_frags(g + 1, (g + 1) & 1);
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[g & 1][i][q], bf[g & 1][j][q], acc[i][j], 0, 0, 0);
        }
    };

    for (int sub = 0; sub < nsub; ++sub) {
        const int m0 = region.m_base + (tile_m0 + sub) * BM;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = f32x16{};
        if constexpr (STAGES == 2) {
            // Two k steps of loads in flight per wave, the stages alternating (written out twice: the stage is a
            // compile-time index into the registers). The waves meet once, behind the first store, which also
            // publishes the epilogue operands parked in LDS, and again before the reduction reuses the tiles.
            if (ktiles > 1) load_tiles((kbase + 1) * BK, 1);
            for (int kt = 0; kt < ktiles; kt += 2) {
                store_tiles(0);
                if (kt == 0) __syncthreads(); else tile_barrier();
                if (kt + 2 < ktiles) load_tiles((kbase + kt + 2) * BK, 0);
                compute();
                tile_barrier();
                if (kt + 1 < ktiles) {
                    store_tiles(1);
                    tile_barrier();
                    if (kt + 3 < ktiles) load_tiles((kbase + kt + 3) * BK, 1);
                    compute();
                    tile_barrier();
                }
            }
            __syncthreads();
        } else {
            // all k steps but the last: the next step's loads are in flight during the MFMAs
            for (int kt = 1; kt < ktiles; ++kt) {
                store_tiles();
                tile_barrier();
                load_tiles((kbase + kt) * BK);
                compute();
                tile_barrier();
            }
            // last k step: the loads in flight are those of the next M tile's first step and of
            // the residual operand
            store_tiles();
            __syncthreads();                 // (also where wave-private tiles publish the epilogue operands parked in LDS)
            if (sub + 1 < nsub) {
                setup_rows(m0 + BM);
                load_tiles(kbase * BK);
            }
            if (first_full >= 0) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        sub_tile(m0, i, j, [&](int v, uint32_t vo, uint32_t so) {
                            full[PREFETCH_FULL ? i : 0][PREFETCH_FULL ? j : 0][v] = buffer_load_x1(f_rsrc, vo, so);
                        });
            }
            compute();
            __syncthreads();
        }

        // ---------------- epilogue + store of the finished M tile ----------------
        // Outputs that are not a row-major [M, N] matrix need (batch, y, x) of every row: decoded
        // once per row into LDS, -1 for rows beyond M.
        if (!c_contig) {
            for (int r = tid; r < BM; r += NT) {
                const int m = m0 + r;
                const int b = m / HoWo, r2 = m - b * HoWo, ho = r2 / P.Wo, wo = r2 - ho * P.Wo;
                Rs[r] = m < P.M ? b * Pk.os_b + ho * Pk.os_h + wo * Pk.os_w : -1;
            }
            __syncthreads();
        }
        // From here on the accumulators are handled as separate scalars: element-wise updates of a
        // 16-register MFMA tuple make the compiler copy the whole tuple at every step.
        float c[TM][TN][16];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) c[i][j][v] = acc[i][j][v];
        if constexpr (KSW > 1) {
            // the k slices meet in the first group of waves (the LDS space of the A and B tiles is free after the last step)
            static_assert((KSW - 1) * WGM * WGN * 16 * 64 <= BM * LDA + BK * LDB, "reduction buffer does not fit the A and B tiles (B follows A)");
            float* red = As + ((kw - 1) * WGM * WGN + wm * WGN + wn) * 16 * 64 + lane;
            if (kw > 0) {
#pragma unroll
                for (int v = 0; v < 16; ++v) red[v * 64] = c[0][0][v];
            }
            __syncthreads();
            if (kw > 0) continue;                                 // nsub == 1 for these kernels: the wave is done
#pragma unroll
            for (int s = 1; s < KSW; ++s)
#pragma unroll
                for (int v = 0; v < 16; ++v) c[0][0][v] += As[((s - 1) * WGM * WGN + wm * WGN + wn) * 16 * 64 + v * 64 + lane];
        }
        const uint32_t slots = (P.flags >> 20) & 31u;
        if (LEAN || slots) {
            // The usual chains (bias, batch norm, residual add, ReLU in that order, each optional) run
            // as straight-line code: every step is one pass over a sub-tile's 16 values, in place.
            const int e_mul = __builtin_popcount(slots & 1u), e_add = __builtin_popcount(slots & 3u),
                      e_max = __builtin_popcount(slots & 15u);
            const int tap = (int)((P.flags >> 12) & 15u) - 1;          // -1: no second result
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    float (&y)[16] = c[i][j];
                    const int col = (wn * TN + j) * 32 + l32;
                    // without a prefetched copy the residual operand is requested first and used
                    // after the per-feature steps
                    float ov[16];
                    if ((slots & 8u) && !(PREFETCH_FULL && first_full >= 0))
                        sub_tile(m0, i, j, [&](int v, uint32_t vo, uint32_t so) { ov[v] = buffer_load_x1_nt(f_rsrc, vo, so); });   // read once: kept out of the caches (-0.8 % on ResNet-50's step)
                    // a second result: the value as it stands before or after the first step
#define CONV_TAP_STORE() sub_tile(m0, i, j, [&](int v, uint32_t vo, uint32_t so) {                                   \
                            buffer_store_x1(y[v], make_rsrc(epi.p[CONV_MAX_EPI - 1], P.out_bytes), vo, so); })
                    if (tap == 0) CONV_TAP_STORE();
                    if (slots & 1u) {
                        const float o = Es[col];
#pragma unroll
                        for (int v = 0; v < 16; ++v) y[v] = y[v] - o;
                        if (tap == 1) CONV_TAP_STORE();
                    }
#undef CONV_TAP_STORE
                    if (slots & 2u) {
                        const float o = Es[e_mul * BN + col];
#pragma unroll
                        for (int v = 0; v < 16; ++v) y[v] = y[v] * o;
                    }
                    if (slots & 4u) {
                        const float o = Es[e_add * BN + col];
#pragma unroll
                        for (int v = 0; v < 16; ++v) y[v] = y[v] + o;
                    }
                    if (slots & 8u) {
                        if (PREFETCH_FULL && first_full >= 0) {
#pragma unroll
                            for (int v = 0; v < 16; ++v) y[v] = y[v] + full[PREFETCH_FULL ? i : 0][PREFETCH_FULL ? j : 0][v];
                        } else {
#pragma unroll
                            for (int v = 0; v < 16; ++v) y[v] = y[v] + ov[v];
                        }
                    }
                    if (slots & 16u) {
                        const float o = Es[e_max * BN + col];          // the same value in every lane
                        if (__builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, o != o ? 1.f : 0.f)) == 0) {
                            // max(y, o) that returns a NaN y, for o known not to be NaN: one compare
#pragma unroll
                            for (int v = 0; v < 16; ++v) y[v] = !(y[v] <= o) ? y[v] : o;
                        } else {
#pragma unroll
                            for (int v = 0; v < 16; ++v) y[v] = (y[v] > o || y[v] != y[v]) ? y[v] : o;
                        }
                    }
                }
        } else if constexpr (!LEAN) {
            // any other chain: one uniform branch per step and sub-tile, not per element
            auto apply = [&](uint32_t code, float (&y)[16], auto&& operand) {
#define EPI_LOOP(expr) _Pragma("unroll") for (int v = 0; v < 16; ++v) { const float a = y[v], o = operand(v); y[v] = (expr); }
                switch (code) {                                          // bit0: operand on the left
                    case CEW_ADD_F * 2: case CEW_ADD_F * 2 + 1: EPI_LOOP(a + o) break;
                    case CEW_MUL_F * 2: case CEW_MUL_F * 2 + 1: EPI_LOOP(a * o) break;
                    case CEW_SUB_F * 2:     EPI_LOOP(a - o) break;
                    case CEW_SUB_F * 2 + 1: EPI_LOOP(o - a) break;
                    case CEW_DIV_F * 2:     EPI_LOOP(a / o) break;
                    case CEW_DIV_F * 2 + 1: EPI_LOOP(o / a) break;
                    case CEW_MAX_F * 2:     EPI_LOOP((a > o || a != a) ? a : o) break;
                    case CEW_MAX_F * 2 + 1: EPI_LOOP((o > a || o != o) ? o : a) break;
                    case CEW_MIN_F * 2:     EPI_LOOP((a < o || a != a) ? a : o) break;
                    case CEW_MIN_F * 2 + 1: EPI_LOOP((o < a || o != o) ? o : a) break;
                    default: __builtin_unreachable();                    // the host fuses no other operation
                }
#undef EPI_LOOP
            };
            // The step loop stays rolled: one copy of the step code keeps the kernel small.
#pragma nounroll
            for (int e = 0; e < nepi; ++e) {
                const uint32_t kind = step_desc(e) >> 8;
                const uint32_t code = step_desc(e) & 255u;
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        if (kind == 3) {
                            if (PREFETCH_FULL && e == first_full) {
                                apply(code, c[i][j], [&](int v) { return full[PREFETCH_FULL ? i : 0][PREFETCH_FULL ? j : 0][v]; });
                            } else {
                                float ov[16];
                                // (the pointer table is re-read from the argument block: indexing the by-value
                                // argument with a run-time value would make the compiler copy it to scratch memory)
                                const float* const* table = reinterpret_cast<const float* const*>(
                                    reinterpret_cast<const char*>(__builtin_amdgcn_kernarg_segment_ptr()) + 24);
                                const __amdgpu_buffer_rsrc_t g_rsrc = make_rsrc(table[e], P.out_bytes);
                                sub_tile(m0, i, j, [&](int v, uint32_t vo, uint32_t so) { ov[v] = buffer_load_x1(g_rsrc, vo, so); });
                                apply(code, c[i][j], [&](int v) { return ov[v]; });
                            }
                        } else {
                            // one value per column: used straight from its register
                            const float o1 = Es[e * BN + (wn * TN + j) * 32 + l32];
                            apply(code, c[i][j], [&](int) { return o1; });
                        }
                    }
            }
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                sub_tile(m0, i, j, [&](int v, uint32_t vo, uint32_t so) { buffer_store_x1(c[i][j][v], o_rsrc, vo, so); });
        if (!c_contig) __syncthreads();          // Rs is rewritten for the next M tile
    }
}

#define CONV_KERNEL(name, WGM, WGN, TM, TN, BK, AF, BF, LEAN, ...)                                          \
    extern "C" __global__ __launch_bounds__(64 * WGM * WGN * (1, ##__VA_ARGS__)) __attribute__((amdgpu_waves_per_eu(2))) void name( \
        float* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,                   \
        ConvEpiPtrs epi, ConvDerivedPtrs dp, ConvParams P, ConvDerived D) {                                  \
        __shared__ __attribute__((aligned(16))) float pool[conv_pool_floats<WGM, WGN, TM, TN, BK>()];        \
        const ConvRegion all{0, P.tiles_m, P.tiles_n, 0};                                                    \
        conv_gemm_body<WGM, WGN, TM, TN, BK, AF, BF, LEAN, ##__VA_ARGS__>(pool, all, out, x, w, epi, dp, P, D); \
    }

// name = conv_gemm_<BM>x<BN>x<BK>_<a><b>  with a/b = f (16-byte loads) or g (generic strided loads),
//        conv_gemm_<BM>x<BN>x<BK>_lean for the common-case variant
#define CONV_TILE(tag, WGM, WGN, TM, TN, BK)                                      \
    CONV_KERNEL(conv_gemm_##tag##_lean, WGM, WGN, TM, TN, BK, true, true, true)   \
    CONV_KERNEL(conv_gemm_##tag##_ff, WGM, WGN, TM, TN, BK, true, true, false)    \
    CONV_KERNEL(conv_gemm_##tag##_fg, WGM, WGN, TM, TN, BK, true, false, false)   \
    CONV_KERNEL(conv_gemm_##tag##_gf, WGM, WGN, TM, TN, BK, false, true, false)   \
    CONV_KERNEL(conv_gemm_##tag##_gg, WGM, WGN, TM, TN, BK, false, false, false)

CONV_TILE(64x64x32, 2, 2, 1, 1, 32)
CONV_TILE(64x64x64, 2, 2, 1, 1, 64)
CONV_TILE(32x32x32, 1, 1, 1, 1, 32)
CONV_TILE(32x32x64, 1, 1, 1, 1, 64)
// one 32 x 32 tile per block, the k step of 128 split over four waves (chunk 1; see KSW above)
CONV_KERNEL(conv_gemm_32x32x128_ks4, 1, 1, 1, 1, 128, true, true, true, 4)
// the same with element-wise loads of the kernel operand (an output width that is no multiple of 4)
CONV_KERNEL(conv_gemm_32x32x128_ks4g, 1, 1, 1, 1, 128, true, false, true, 4)
// the same with a 64-long k step, for windows over 64 (or 192, ...) input features, whose taps a 128-long step would straddle
CONV_KERNEL(conv_gemm_32x32x64_ks4, 1, 1, 1, 1, 64, true, true, true, 4)
// Mixed tiling for layers whose 64 x 64 tiles do not divide evenly among the CUs (784 tiles on 256 CUs: a CU
// with four tiles sets the time, the average is 3.06). The first P.split_tiles_m M tiles are computed as 64 x 64
// tiles, as many as fill every CU equally; the rows behind them as 32 x 32 tiles of a quarter of the work each
// (four waves sharing every 64-long k step), which spread over the CUs in finer units. Both kinds of block have 256
// threads and share one LDS pool; with the 64-long step the kernel needs 127 registers, so four blocks fit a CU
// (the 128-long step of conv_gemm_32x32x128_ks4 takes 149: three blocks, and the small tiles would wait for
// the large ones). One M tile per block (chunk 1).
#define CONV_MIX_KERNEL(name, BK)                                                                              \
    extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void name(            \
        float* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,                   \
        ConvEpiPtrs epi, ConvDerivedPtrs dp, ConvParams P, ConvDerived D) {                                  \
        constexpr int big = conv_pool_floats<2, 2, 1, 1, BK>(), small = conv_pool_floats<1, 1, 1, 1, 64>(); \
        __shared__ __attribute__((aligned(16))) float pool[big > small ? big : small];                       \
        const int n_big = P.split_tiles_m * P.tiles_n;                                                       \
        if ((int)blockIdx.x < n_big) {                                                                       \
            const ConvRegion r{0, P.split_tiles_m, P.tiles_n, 0};                                            \
            conv_gemm_body<2, 2, 1, 1, BK, true, true, true>(pool, r, out, x, w, epi, dp, P, D);             \
        } else {                                                                                             \
            const int m_base = P.split_tiles_m * 64;                                                         \
            const ConvRegion r{n_big, (P.M - m_base + 31) / 32, (P.N + 31) / 32, m_base};                    \
            conv_gemm_body<1, 1, 1, 1, 64, true, true, true, 4>(pool, r, out, x, w, epi, dp, P, D);         \
        }                                                                                                    \
    }
CONV_MIX_KERNEL(conv_gemm_64x64x32_mix, 32)
CONV_MIX_KERNEL(conv_gemm_64x64x64_mix, 64)

// ---------------------------------------------------------------------------------------------
// Convolutions of dense images with very few features (an RGB stem: 7 x 7 x 3, stride 2). The general kernel
// above assembles the A tile element by element for them: 1650 vector instructions per 64 x 64 tile against
// 80 MFMAs, and the two share the SIMDs' issue slots (counters: the vector ALUs busy 56 % of the kernel's time).
// Here a block copies the image rows its 64 output positions touch into LDS once (16-byte loads of whole
// rows, zero borders written beside them) and the MFMA operands are read straight from that patch: the
// KW * Cin values one kernel row reads for an output position are contiguous there, so the address of A(m, k)
// is a per-lane base plus a compile-time offset. The whole kernel (KH * RLP rows, RLP = KW * Cin rounded up to
// even, the extra row zero) sits in LDS for the block's lifetime; a block walks the tiles in steps of the grid.
//   KH: kernel rows; RLP: padded run length; PR: image rows of a patch (>= KH + SH, a tile spans two output rows
//   at most); NVEC: 16-byte vectors a thread fetches per patch.
// Requirements (the host checks them): pixels dense ([B, H, W, Cin], W * Cin % 4 == 0), no dilation, M % 64 == 0,
// Ho * Wo % 64 == 0 (a tile lies in one image), Wo >= 64, N <= 64, row-major result, template epilogue without a
// full-size operand, KW * Cin in (RLP - 2, RLP], KH + SH <= PR, PR * W * Cin / 4 <= 256 * NVEC.
struct ConvStemParams {
    int32_t M, N, K;
    int32_t Ho, Wo, H, W, Cin, KH, KW, SH, SW, PH, PW;
    int32_t pitch;                  // floats per patch row: left border, W * Cin values, right border (a multiple of 4)
    int32_t left;                   // floats of left border (>= PW * Cin, a multiple of 4)
    uint32_t flags;                 // bits 20-24: template epilogue steps as in ConvParams.flags (bit 23 never)
    uint32_t x_bytes, w_bytes, out_bytes;
    uint32_t howo_magic, howo_shift, wo_magic, wo_shift;
};

// NWM: 32-row sub-tiles of a block's tile (2: 64 output positions, 256 threads; 4: 128 positions, 512 threads - the
// kernel and the patch take the same room in LDS either way, so the larger block brings twice the waves per CU).
template <int KH, int RLP, int PR, int NVEC, int NWM = 2>
__device__ __forceinline__ void conv_stem_body(float* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
                                               const ConvEpiPtrs& epi, const ConvDerivedPtrs& Dp, const ConvStemParams& P,
                                               const ConvDerived& Dk, float* __restrict__ Ws, float* __restrict__ Ps, float* __restrict__ Es) {
    constexpr int BN = 64, LDB = BN + 4, G = RLP / 2, BM = 32 * NWM, NT = 128 * NWM;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, half = lane >> 5;
    const int RL = P.KW * P.Cin, WC = P.W * P.Cin, vecs_per_row = WC >> 2, HoWo = P.Ho * P.Wo;
    const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, P.x_bytes), w_rsrc = make_rsrc(w, P.w_bytes), o_rsrc = make_rsrc(out, P.out_bytes);

    // the kernel: Ws[ky * RLP + j][n] = w[ky, j, n] for j < KW * Cin, zero behind
    for (int e = tid; e < KH * RLP * (BN / 4); e += NT) {
        const int row = e / (BN / 4), n4 = (e - row * (BN / 4)) * 4, ky = row / RLP, j = row - ky * RLP;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (j < RL) {
            const uint32_t off = (uint32_t)((ky * RL + j) * P.N + n4) * 4u;
            if (n4 + 3 < P.N) v = buffer_load_x4(w_rsrc, off);
            else {
#pragma unroll
                for (int q = 0; q < 4; ++q) v[q] = n4 + q < P.N ? buffer_load_x1(w_rsrc, off + 4u * q) : 0.f;
            }
        }
        *reinterpret_cast<f32x4*>(&Ws[row * LDB + n4]) = v;
    }
    // the borders of the patch rows stay zero
    for (int e = tid; e < PR * P.pitch; e += NT) {
        const int c = e % P.pitch;
        if (c < P.left || c >= P.left + WC) Ps[e] = 0.f;
    }
    // per-column epilogue operands (see conv_gemm_body)
    const int nepi = __builtin_popcount((P.flags >> 20) & 31u);
    if (tid < BN) {
        float e_reg[CONV_MAX_EPI];
#pragma unroll
        for (int e = 0; e < CONV_MAX_EPI; ++e) {
            e_reg[e] = 0.f;
            if (e < nepi) {
                const uint32_t present = epi.p[e] != nullptr ? 1u : 0u;
                // template steps in order: vector, vector, vector, (full tensor: never here), scalar
                const bool scalar = e == nepi - 1 && ((P.flags >> 24) & 1u);
                e_reg[e] = scalar ? buffer_load_x1(make_rsrc(epi.p[e], 4u * present), 0u)
                                  : buffer_load_x1(make_rsrc(epi.p[e], (uint32_t)P.N * 4u * present), (uint32_t)tid * 4u);
            }
        }
        if (Dk.nsteps) {
            float in[CONV_MAX_DERIVED + 1];
#pragma unroll
            for (int k = 0; k <= CONV_MAX_DERIVED; ++k) {
                const bool vec = (Dk.vector_mask >> k) & 1u;
                in[k] = buffer_load_x1(make_rsrc(Dp.p[k], Dp.p[k] == nullptr ? 0u : vec ? (uint32_t)P.N * 4u : 4u), vec ? (uint32_t)tid * 4u : 0u);
            }
            float v = in[0];
#pragma unroll
            for (int k = 0; k < CONV_MAX_DERIVED; ++k) {
                if (k < (int)Dk.nsteps) {
                    const float a = Dk.left[k] ? in[k + 1] : v, b = Dk.left[k] ? v : in[k + 1];
                    switch (Dk.op[k]) {
                        case CEW_ADD_F:   v = a + b; break;
                        case CEW_SUB_F:   v = a - b; break;
                        case CEW_MUL_F:   v = a * b; break;
                        case CEW_DIV_F:   v = a / b; break;
                        case CEW_MAX_F:   v = (a > b || a != a) ? a : b; break;
                        case CEW_MIN_F:   v = (a < b || a != a) ? a : b; break;
                        case CEW_NEG_F:   v = -v; break;
                        case CEW_RSQRT_F: v = 1.0f / sqrtf(v); break;
                        case CEW_SQRT_F:  v = sqrtf(v); break;
                        default: break;
                    }
                }
            }
#pragma unroll
            for (int e = 0; e < CONV_MAX_EPI; ++e)
                if (e == (int)Dk.step) e_reg[e] = v;
        }
#pragma unroll
        for (int e = 0; e < CONV_MAX_EPI; ++e)
            if (e < nepi) Es[e * BN + tid] = e_reg[e];
    }

    const int tiles = P.M / BM;
    // the image rows of the patch of tile t: requested into registers, written to LDS later
    f32x4 pv[NVEC];
    auto patch_geometry = [&](int t, int& b, int& ho0, int& hi0) {
        const int m0 = t * BM;
        b = magic_div(m0, P.howo_magic, P.howo_shift);
        ho0 = magic_div(m0 - b * HoWo, P.wo_magic, P.wo_shift);
        hi0 = ho0 * P.SH - P.PH;
    };
    // Which image row and which 16 bytes of it a thread fetches, and where they go in the patch, is the same for every
    // tile: worked out once, outside the tile loop.
    int      p_row[NVEC];            // patch row of the thread's q-th vector; PR and above: nothing to fetch
    uint32_t p_from[NVEC];           // byte offset of the vector behind the patch's first image row
    int      p_to[NVEC];             // where it goes in the patch (floats)
#pragma unroll
    for (int q = 0; q < NVEC; ++q) {
        const int v = tid + q * NT, r = v / vecs_per_row, c4 = v - r * vecs_per_row;
        p_row[q]  = r;
        p_from[q] = (uint32_t)(r * WC + c4 * 4) * 4u;
        p_to[q]   = r * P.pitch + P.left + c4 * 4;
    }
    auto request_patch = [&](int t) {
        int b, ho0, hi0;
        patch_geometry(t, b, ho0, hi0);
        const uint32_t first_row = (uint32_t)((b * P.H + hi0) * WC) * 4u;       // (wraps for rows above the image, which are not fetched)
#pragma unroll
        for (int q = 0; q < NVEC; ++q) {
            const bool ok = p_row[q] < PR && (uint32_t)(hi0 + p_row[q]) < (uint32_t)P.H;
            pv[q] = buffer_load_x4(x_rsrc, ok ? first_row + p_from[q] : CONV_OOB);   // zeros outside the image
        }
    };
    auto park_patch = [&]() {
#pragma unroll
        for (int q = 0; q < NVEC; ++q)
            if (p_row[q] < PR) *reinterpret_cast<f32x4*>(&Ps[p_to[q]]) = pv[q];
    };

    int t = blockIdx.x;
    if (t < tiles) request_patch(t);
    for (; t < tiles; t += gridDim.x) {
        __syncthreads();                              // the previous tile's reads of the patch are over (first pass: the fills above)
        park_patch();
        __syncthreads();
        if (t + (int)gridDim.x < tiles) request_patch(t + gridDim.x);   // in flight during this tile's MFMAs
        int b, ho0, hi0;
        patch_geometry(t, b, ho0, hi0);
        // this lane's output position and where its kernel row 0 starts in the patch
        const int m  = t * BM + wm * 32 + l32;
        const int r2 = m - b * HoWo, ho = magic_div(r2, P.wo_magic, P.wo_shift), wo = r2 - ho * P.Wo;
        const float* a_base = Ps + (ho - ho0) * P.SH * P.pitch + P.left + (wo * P.SW - P.PW) * P.Cin + half;
        const float* b_base = Ws + half * LDB + wn * 32 + l32;
        f32x16 acc = {};
#pragma unroll
        for (int ky = 0; ky < KH; ++ky) {
            const float* a_row = a_base + ky * P.pitch;
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float a = a_row[2 * g];
                // the padding position behind an odd run is a neighbouring pixel, not a zero: 0 * Inf would be NaN
                if (g == G - 1 && 2 * g + half >= RL) a = 0.f;
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b_base[(ky * RLP + 2 * g) * LDB], acc, 0, 0, 0);
            }
        }
        // epilogue: (acc - vector) * vector + vector, max(., scalar), each optional, then the store
        float y[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) y[v] = acc[v];
        const uint32_t slots = (P.flags >> 20) & 31u;
        const int col = wn * 32 + l32;
        const int e_mul = __builtin_popcount(slots & 1u), e_add = __builtin_popcount(slots & 3u), e_max = __builtin_popcount(slots & 15u);
        const uint32_t base = col < P.N ? (uint32_t)((t * BM + wm * 32 + 4 * half) * P.N + col) * 4u : CONV_OOB;
        const uint32_t rowb = (uint32_t)P.N * 4u;
        // a second result (bits 12-15 of the flags, as in conv_gemm_body): the value as it stands before (1) or after (2) the first step
        const int tap = (int)((P.flags >> 12) & 15u) - 1;
        const auto tap_store = [&]() {
            const auto t_rsrc = make_rsrc(epi.p[CONV_MAX_EPI - 1], P.out_bytes);
#pragma unroll
            for (int v = 0; v < 16; ++v) buffer_store_x1(y[v], t_rsrc, base, (uint32_t)(8 * (v / 4) + (v % 4)) * rowb);
        };
        if (tap == 0) tap_store();
        if (slots & 1u) {
            const float o = Es[col];
#pragma unroll
            for (int v = 0; v < 16; ++v) y[v] = y[v] - o;
            if (tap == 1) tap_store();
        }
        if (slots & 2u) {
            const float o = Es[e_mul * BN + col];
#pragma unroll
            for (int v = 0; v < 16; ++v) y[v] = y[v] * o;
        }
        if (slots & 4u) {
            const float o = Es[e_add * BN + col];
#pragma unroll
            for (int v = 0; v < 16; ++v) y[v] = y[v] + o;
        }
        if (slots & 16u) {
            const float o = Es[e_max * BN + col];
#pragma unroll
            for (int v = 0; v < 16; ++v) y[v] = (y[v] > o || y[v] != y[v]) ? y[v] : o;
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) buffer_store_x1(y[v], o_rsrc, base, (uint32_t)(8 * (v / 4) + (v % 4)) * rowb);
    }
}

#define CONV_STEM_PATCH_FLOATS 6272          // PR rows of at most 696 floats (W * Cin = 672 with borders), + slack
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void conv_gemm_stem_7x22(
        float* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
        ConvEpiPtrs epi, ConvDerivedPtrs dp, ConvStemParams P, ConvDerived D) {
    __shared__ __attribute__((aligned(16))) float Ws[7 * 22 * 68];
    __shared__ __attribute__((aligned(16))) float Ps[CONV_STEM_PATCH_FLOATS];
    __shared__ float Es[CONV_MAX_EPI * 64];
    conv_stem_body<7, 22, 9, 6>(out, x, w, epi, dp, P, D, Ws, Ps, Es);
}
// 128 output positions per tile (they reach into three output rows at most: 11 image rows), 8 waves per block
#define CONV_STEM_PATCH_FLOATS_M128 7680
extern "C" __global__ __launch_bounds__(512) void conv_gemm_stem_7x22_m128(
        float* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
        ConvEpiPtrs epi, ConvDerivedPtrs dp, ConvStemParams P, ConvDerived D) {
    __shared__ __attribute__((aligned(16))) float Ws[7 * 22 * 68];
    __shared__ __attribute__((aligned(16))) float Ps[CONV_STEM_PATCH_FLOATS_M128];
    __shared__ float Es[CONV_MAX_EPI * 64];
    conv_stem_body<7, 22, 11, 4, 4>(out, x, w, epi, dp, P, D, Ws, Ps, Es);
}

// ---------------------------------------------------------------------------------------------
// Products with at most 16 output features (a classifier's last layer): out = x [M, K] . w [K, N], one wave per
// row of x, on the vector ALUs. A 32-column MFMA tile would be mostly padding, and for the few rows of a small
// batch the launch is all latency: this kernel runs a few hundred instructions per wave, all its loads are in
// flight together, and the softmax (and arg-max) that usually follows can run on the row before it is stored.
//
// Lane l multiplies x[row][k] for k = 4l .. 4l+3 (+ 256, + 512, ...) with the rows k of w, which are 4N consecutive
// floats, into N running sums with fused multiply-adds, in ascending k; the lanes' sums are then added by a
// butterfly (xor 32, 16, ..., 1), so that every lane holds all N results. Epilogue: the steps of the straight-line
// epilogue of conv_gemm_body that take a per-feature vector or a single value; then, with bit 29 of the flags, the
// softmax of the row exactly as softmax_rows_v1 / _v4 computes it for a row of N values (the maximum, exp(x - max)
// added in the order of the row-sum kernel, one division per value), and, if the last pointer slot is not null,
// the arg-max of the probabilities (first occurrence; a NaN wins).
// Needs K % 4 == 0, rows of x that start at multiples of 4 floats, dense w and out; the host checks.
struct DenseRowsParams {
    int32_t M, N, K;
    int32_t x_pitch;                // floats between two rows of x
    uint32_t flags;                 // bits 20-22 and 24: template epilogue steps as in ConvParams.flags; bit 29: softmax
    uint32_t x_bytes, w_bytes, out_bytes;
};

template <int N>
__device__ __forceinline__ void dense_rows_body(float* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
                                                const ConvEpiPtrs& epi, const DenseRowsParams& P) {
    const int lane = threadIdx.x & 63, row = (int)blockIdx.x * 4 + (int)(threadIdx.x >> 6);
    if (row >= P.M) return;                                            // whole wave leaves together
    const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, P.x_bytes), w_rsrc = make_rsrc(w, P.w_bytes), o_rsrc = make_rsrc(out, P.out_bytes);
    const uint32_t slots = (P.flags >> 20) & 31u;
    const int e_mul = __builtin_popcount(slots & 1u), e_add = __builtin_popcount(slots & 3u), e_max = __builtin_popcount(slots & 15u);
    // epilogue operands: requested before the products, used after them
    float o_sub[N], o_mul[N], o_add[N], o_max = 0.f;
#pragma unroll
    for (int n = 0; n < N; ++n) {
        o_sub[n] = buffer_load_x1(make_rsrc(epi.p[0], (slots & 1u) ? (uint32_t)N * 4u : 0u), (uint32_t)n * 4u);
        o_mul[n] = buffer_load_x1(make_rsrc(epi.p[e_mul], (slots & 2u) ? (uint32_t)N * 4u : 0u), (uint32_t)n * 4u);
        o_add[n] = buffer_load_x1(make_rsrc(epi.p[e_add], (slots & 4u) ? (uint32_t)N * 4u : 0u), (uint32_t)n * 4u);
    }
    if (slots & 16u) o_max = buffer_load_x1(make_rsrc(epi.p[e_max], 4u), 0u);

    float acc[N];
#pragma unroll
    for (int n = 0; n < N; ++n) acc[n] = 0.f;
    const uint32_t xrow = (uint32_t)row * (uint32_t)P.x_pitch * 4u;
    for (int k0 = 0; k0 < P.K; k0 += 512) {
        f32x4 xv[2], wv[2][N];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int  k4 = k0 + u * 256 + lane * 4;
            const bool in = k4 < P.K;                                  // beyond K: zeros, which leave the sums as they are
            xv[u] = buffer_load_x4(x_rsrc, in ? xrow + (uint32_t)k4 * 4u : CONV_OOB);
#pragma unroll
            for (int j = 0; j < N; ++j) wv[u][j] = buffer_load_x4(w_rsrc, in ? (uint32_t)(k4 * N + 4 * j) * 4u : CONV_OOB);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int n = 0; n < N; ++n) acc[n] = __builtin_fmaf(xv[u][q], wv[u][(q * N + n) / 4][(q * N + n) % 4], acc[n]);
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) {
        float o[N];
#pragma unroll
        for (int n = 0; n < N; ++n) o[n] = __shfl_xor(acc[n], s, 64);
#pragma unroll
        for (int n = 0; n < N; ++n) acc[n] = acc[n] + o[n];
    }
    float y[N];
#pragma unroll
    for (int n = 0; n < N; ++n) {
        float v = acc[n];
        if (slots & 1u) v = v - o_sub[n];
        if (slots & 2u) v = v * o_mul[n];
        if (slots & 4u) v = v + o_add[n];
        if (slots & 16u) v = (v > o_max || v != v) ? v : o_max;
        y[n] = v;
    }
    if (P.flags & (1u << 29)) {
        float m = -INFINITY;                                           // a NaN wins
#pragma unroll
        for (int n = 0; n < N; ++n) m = (y[n] > m || y[n] != y[n]) ? y[n] : m;
        float e[16];
#pragma unroll
        for (int n = 0; n < 16; ++n) e[n] = n < N ? expf(y[n < N ? n : 0] - m) : 0.f;
        float total;
        if constexpr (N % 4 == 0) {
            // the 16-byte row-sum kernel: lane l holds (e[4l] + e[4l+1]) + (e[4l+2] + e[4l+3]), then lanes xor 2, xor 1
            float a[4];
#pragma unroll
            for (int l = 0; l < 4; ++l) a[l] = (e[4 * l] + e[4 * l + 1]) + (e[4 * l + 2] + e[4 * l + 3]);
            total = (a[0] + a[2]) + (a[1] + a[3]);
        } else {
            // the 4-byte row-sum kernel: lane l holds e[l], then lanes xor 8, 4, 2, 1 (xor 32 and 16 add zeros)
            float a[16];
#pragma unroll
            for (int l = 0; l < 16; ++l) a[l] = e[l];
#pragma unroll
            for (int s = 8; s >= 1; s >>= 1)
#pragma unroll
                for (int l = 0; l < s; ++l) a[l] = a[l] + a[l + s];
            total = a[0];
        }
#pragma unroll
        for (int n = 0; n < N; ++n) y[n] = e[n] / total;
        // arg-max: the first occurrence of the maximum; a NaN replaces any number and is never replaced
        uint32_t best = 0;
        float bv = y[0];
#pragma unroll
        for (int n = 1; n < N; ++n) {
            const bool better = y[n] > bv || (y[n] != y[n] && bv == bv);
            bv = better ? y[n] : bv;
            best = better ? (uint32_t)n : best;
        }
        uint32_t* const arg_out = reinterpret_cast<uint32_t*>(const_cast<float*>(epi.p[CONV_MAX_EPI - 1]));
        if (arg_out != nullptr && lane == 0) arg_out[row] = best;
    }
    float mine = 0.f;
#pragma unroll
    for (int n = 0; n < N; ++n) mine = lane == n ? y[n] : mine;
    buffer_store_x1(mine, o_rsrc, lane < N ? (uint32_t)(row * N + lane) * 4u : CONV_OOB);
}

extern "C" __global__ __launch_bounds__(256) void dense_rows_n16(float* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
                                                                ConvEpiPtrs epi, DenseRowsParams P) {
    switch (P.N) {
#define DENSE_ROWS_CASE(n) case n: dense_rows_body<n>(out, x, w, epi, P); break;
        DENSE_ROWS_CASE(1) DENSE_ROWS_CASE(2) DENSE_ROWS_CASE(3) DENSE_ROWS_CASE(4) DENSE_ROWS_CASE(5) DENSE_ROWS_CASE(6)
        DENSE_ROWS_CASE(7) DENSE_ROWS_CASE(8) DENSE_ROWS_CASE(9) DENSE_ROWS_CASE(10) DENSE_ROWS_CASE(11) DENSE_ROWS_CASE(12)
        DENSE_ROWS_CASE(13) DENSE_ROWS_CASE(14) DENSE_ROWS_CASE(15) DENSE_ROWS_CASE(16)
#undef DENSE_ROWS_CASE
        default: break;
    }
}
