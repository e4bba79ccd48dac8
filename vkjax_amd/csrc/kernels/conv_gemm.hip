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
// The 16-byte paths read through buffer descriptors: a masked-out load is an out-of-range
// offset that returns zeros, so padding, tile tails and partial tiles need no branches.
// After the k loop an optional chain of element-wise steps (per-feature vectors, full-size
// tensors or scalars as operands) is applied to the accumulators before the single store.
#include "common.h"

#define CONV_MAX_EPI 6
#define CONV_OOB 0x80000000u     // byte offset beyond any descriptor: loads give 0, stores are dropped

enum EwOpConv : uint32_t {
#define EW_OP(name, num) CEW_##name = num,
#include "ew_opcodes.h"
#undef EW_OP
};

struct ConvParams {
    int32_t M, N, K;
    int32_t Ho, Wo;                 // M = batch * Ho * Wo
    int32_t H, W, Cin;              // lhs spatial size (undilated) and features
    int32_t KH, KW;
    int32_t SH, SW, PH, PW, DH, DW, LH, LW;
    int32_t xs_b, xs_h, xs_w, xs_c; // lhs strides in elements
    int32_t ws_r, ws_s, ws_c, ws_n; // rhs strides
    int32_t os_b, os_h, os_w, os_n; // out strides
    int32_t c_contig;               // out is row-major [M, N]
    int32_t tiles_m, tiles_n;
    uint32_t nepi;                  // number of epilogue steps
    uint32_t epi_op[CONV_MAX_EPI];
    uint32_t epi_flags[CONV_MAX_EPI];   // bit1: operand is the left argument
    uint32_t epi_kind[CONV_MAX_EPI];    // 0 none, 1 scalar, 2 per-feature vector [N], 3 full tensor laid out like out
    int32_t  epi_first_full;            // index of the first kind-3 step, or -1
    int32_t  flat_rows;                 // m is the row index itself (batch = Wo = 1): no row decode
    uint32_t x_bytes, w_bytes, out_bytes;   // sizes for the buffer descriptors (each below 2^31)
};

struct ConvEpiPtrs { const float* p[CONV_MAX_EPI]; };

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ f32x4 buffer_load_x4(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 0));
}
__device__ __forceinline__ float buffer_load_x1(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, byte_off, 0, 0));
}
__device__ __forceinline__ void buffer_store_x1(float v, __amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), r, byte_off, 0, 0);
}

template <int WGM, int WGN, int TM, int TN, int BK, bool A_FAST, bool B_FAST>
__device__ __forceinline__ void conv_gemm_body(float* __restrict__ out, const float* __restrict__ x,
                                               const float* __restrict__ w, const ConvEpiPtrs& epi,
                                               const ConvParams& Pk) {
    constexpr int BM = 32 * WGM * TM, BN = 32 * WGN * TN, NT = 64 * WGM * WGN;
    constexpr int LDA = BK + 4, LDB = BN + 4;
    __shared__ __attribute__((aligned(16))) float As[BM * LDA];
    __shared__ __attribute__((aligned(16))) float Bs[BK * LDB];
    __shared__ float Es[CONV_MAX_EPI * BN];         // per-column operands of the epilogue steps

    // Copy the argument block into scalar registers once, at the very start. Left to itself the
    // compiler fetches each field right before its first use; under load every such fetch costs
    // about a microsecond, and the prologue and the epilogue would each chain several of them.
    ConvParams P;
#define CONV_PIN(f) P.f = Pk.f; asm volatile("" : "+s"(P.f));
    CONV_PIN(M) CONV_PIN(N) CONV_PIN(K) CONV_PIN(Ho) CONV_PIN(Wo) CONV_PIN(H) CONV_PIN(W) CONV_PIN(Cin)
    CONV_PIN(KH) CONV_PIN(KW) CONV_PIN(SH) CONV_PIN(SW) CONV_PIN(PH) CONV_PIN(PW) CONV_PIN(DH) CONV_PIN(DW)
    CONV_PIN(LH) CONV_PIN(LW) CONV_PIN(xs_b) CONV_PIN(xs_h) CONV_PIN(xs_w) CONV_PIN(xs_c) CONV_PIN(ws_r) CONV_PIN(ws_s)
    CONV_PIN(ws_c) CONV_PIN(ws_n) CONV_PIN(os_b) CONV_PIN(os_h) CONV_PIN(os_w) CONV_PIN(os_n) CONV_PIN(c_contig) CONV_PIN(tiles_m)
    CONV_PIN(tiles_n) CONV_PIN(nepi) CONV_PIN(epi_first_full) CONV_PIN(flat_rows) CONV_PIN(x_bytes) CONV_PIN(w_bytes) CONV_PIN(out_bytes)
#pragma unroll
    for (int q = 0; q < CONV_MAX_EPI; ++q) {
        CONV_PIN(epi_op[q]) CONV_PIN(epi_flags[q]) CONV_PIN(epi_kind[q])
        asm volatile("" :: "s"(epi.p[q]));
    }
#undef CONV_PIN
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int l32 = lane & 31, half = lane >> 5;

    // Consecutive block ids go to different XCDs (8 of them, each with its own L2). Hand every
    // XCD a contiguous range of tiles so that the N-tiles of one M-tile share an L2.
    int tile = blockIdx.x;
    {
        const int total = P.tiles_m * P.tiles_n, per = total / 8;
        if (per > 0 && tile < per * 8) tile = (tile & 7) * per + (tile >> 3);
    }
    const int tile_m = tile / P.tiles_n, tile_n = tile - tile_m * P.tiles_n;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int HoWo = P.Ho * P.Wo;

    const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, P.x_bytes), w_rsrc = make_rsrc(w, P.w_bytes),
                                 o_rsrc = make_rsrc(out, P.out_bytes);

    // Scalar and per-feature epilogue operands are fetched once per block, at its very start, and
    // parked in LDS behind the first k tile's loads, so that the epilogue never waits on global
    // memory for them.
    constexpr int E_PER_THREAD = (CONV_MAX_EPI * BN + NT - 1) / NT;
    float e_reg[E_PER_THREAD];
#pragma unroll
    for (int q = 0; q < E_PER_THREAD; ++q) {
        const int idx = tid + q * NT;
        e_reg[q] = 0.f;
        if (idx < (int)P.nepi * BN) {
            const int e = idx / BN, n = n0 + idx - e * BN;
            // pick step e's descriptor with selects: indexing the argument block with a run-time
            // value would move the whole block from scalar registers to scratch memory
            uint32_t kind = P.epi_kind[0];
            const float* src = epi.p[0];
#pragma unroll
            for (int t = 1; t < CONV_MAX_EPI; ++t) {
                kind = e == t ? P.epi_kind[t] : kind;
                src  = e == t ? epi.p[t] : src;
            }
            if (kind == 1) e_reg[q] = src[0];
            else if (kind == 2 && n < P.N) e_reg[q] = src[n];
        }
    }

    // ---------------- per-thread load assignment ----------------
    // A fast: 16-byte vectors along k. A generic: one row, a run of consecutive k.
    constexpr int A_VPR   = BK / 4;                 // vectors per row
    constexpr int A_RSTEP = NT / A_VPR;             // rows between a thread's vectors
    constexpr int A_NV    = BM / A_RSTEP;           // vectors per thread
    constexpr int A_KG    = NT / BM;                // generic: k groups
    constexpr int A_KPT   = BK / A_KG;              // generic: k per thread
    constexpr int A_ROWS  = A_FAST ? A_NV : 1;
    // row state: element offset of (row, ky = kx = c = 0) and the input coordinates of that corner
    int a_off[A_ROWS], a_hi0[A_ROWS], a_wi0[A_ROWS];
#pragma unroll
    for (int p = 0; p < A_ROWS; ++p) {
        const int row = A_FAST ? (tid / A_VPR + p * A_RSTEP) : (tid % BM);
        const int m = m0 + row;
        if (m < P.M) {
            int b = 0, ho = m, wo = 0;
            if (!P.flat_rows) { b = m / HoWo; const int r2 = m - b * HoWo; ho = r2 / P.Wo; wo = r2 - ho * P.Wo; }
            a_hi0[p] = ho * P.SH - P.PH;
            a_wi0[p] = wo * P.SW - P.PW;
            a_off[p] = b * P.xs_b + (A_FAST ? a_hi0[p] * P.xs_h + a_wi0[p] * P.xs_w + (tid % A_VPR) * 4 : 0);
        } else {
            a_off[p] = 0; a_hi0[p] = -(1 << 28); a_wi0[p] = -(1 << 28);
        }
    }
    // When a k tile never straddles two kernel taps (Cin % BK == 0) the tap (ky, kx) and first
    // feature of a tile are the same for the whole block and live in scalar registers.
    const bool uniform_taps = A_FAST && (P.Cin % BK == 0);
    int t_r = 0, t_s = 0, t_c = 0;                  // uniform tile position
    // otherwise every thread tracks the position of its own first k
    int ak = A_FAST ? (tid % A_VPR) * 4 : (tid / BM) * A_KPT;
    int ac, as_, ar;
    {
        const int rs = ak / P.Cin;
        ac = ak - rs * P.Cin; ar = rs / P.KW; as_ = rs - ar * P.KW;
    }

    constexpr int B_VPR   = BN / 4;
    constexpr int B_RSTEP = NT / B_VPR;
    constexpr int B_NV    = BK / B_RSTEP;
    constexpr int B_KG    = NT / BN;                // generic: k groups
    constexpr int B_KPT   = BK / B_KG;
    // B fast: byte offset of this thread's first vector in tile 0, or out of range for columns >= N
    const int      b_n    = n0 + (tid % B_VPR) * 4;
    const uint32_t b_off0 = b_n < P.N ? (uint32_t)(((tid / B_VPR) * P.N + b_n) * 4) : CONV_OOB;

    f32x4 a_reg[A_FAST ? A_NV : 1];
    float a_sreg[A_FAST ? 1 : A_KPT];
    f32x4 b_reg[B_FAST ? B_NV : 1];
    float b_sreg[B_FAST ? 1 : B_KPT];

    auto load_tiles = [&](int k0) {
        // ---- A ----
        if constexpr (A_FAST) {
            int r, s, koff;                          // tap of this thread's vector and its element offset
            bool kok = true;
            if (uniform_taps) {
                r = t_r; s = t_s;
                koff = t_r * P.DH * P.xs_h + t_s * P.DW * P.xs_w + t_c;
            } else {
                r = ar; s = as_;
                koff = ar * P.DH * P.xs_h + as_ * P.DW * P.xs_w + ac - (tid % A_VPR) * 4;
                kok = ak < P.K;
            }
            const int dh = r * P.DH, dw = s * P.DW;
#pragma unroll
            for (int p = 0; p < A_NV; ++p) {
                const bool ok = kok && (uint32_t)(a_hi0[p] + dh) < (uint32_t)P.H && (uint32_t)(a_wi0[p] + dw) < (uint32_t)P.W;
                a_reg[p] = buffer_load_x4(x_rsrc, ok ? (uint32_t)(a_off[p] + koff) * 4u : CONV_OOB);
            }
        } else {
            int c = ac, s = as_, r = ar, k = ak;
#pragma unroll
            for (int j = 0; j < A_KPT; ++j) {
                int hi = a_hi0[0] + r * P.DH, wi = a_wi0[0] + s * P.DW;
                bool ok = hi >= 0 && wi >= 0 && k < P.K;
                if (P.LH > 1) { ok = ok && (hi % P.LH == 0); hi /= P.LH; }
                if (P.LW > 1) { ok = ok && (wi % P.LW == 0); wi /= P.LW; }
                ok = ok && hi < P.H && wi < P.W;
                a_sreg[j] = ok ? x[a_off[0] + hi * P.xs_h + wi * P.xs_w + c * P.xs_c] : 0.f;
                ++k; ++c;
                if (c == P.Cin) { c = 0; ++s; if (s == P.KW) { s = 0; ++r; } }
            }
        }
        // ---- B ----
        if constexpr (B_FAST) {
            // rows k >= K fall beyond the descriptor and read as zeros
            const uint32_t base = b_off0 == CONV_OOB ? CONV_OOB : b_off0 + (uint32_t)k0 * (uint32_t)P.N * 4u;
#pragma unroll
            for (int p = 0; p < B_NV; ++p)
                b_reg[p] = buffer_load_x4(w_rsrc, base == CONV_OOB ? CONV_OOB : base + (uint32_t)(p * B_RSTEP) * (uint32_t)P.N * 4u);
        } else {
            const int n = n0 + tid % BN;
            int k = k0 + (tid / BN) * B_KPT;
            const int rs = k / P.Cin;
            int c = k - rs * P.Cin, r = rs / P.KW, s = rs - r * P.KW;
#pragma unroll
            for (int j = 0; j < B_KPT; ++j) {
                b_sreg[j] = (k < P.K && n < P.N) ? w[r * P.ws_r + s * P.ws_s + c * P.ws_c + n * P.ws_n] : 0.f;
                ++k; ++c;
                if (c == P.Cin) { c = 0; ++s; if (s == P.KW) { s = 0; ++r; } }
            }
        }
        // advance to the next k tile
        if (uniform_taps) {
            t_c += BK;
            if (t_c == P.Cin) { t_c = 0; ++t_s; if (t_s == P.KW) { t_s = 0; ++t_r; } }
        } else {
            ak += BK; ac += BK;
            while (ac >= P.Cin) { ac -= P.Cin; ++as_; if (as_ == P.KW) { as_ = 0; ++ar; } }
        }
    };

    auto store_tiles = [&]() {
        if constexpr (A_FAST) {
#pragma unroll
            for (int p = 0; p < A_NV; ++p) {
                const int row = tid / A_VPR + p * A_RSTEP, kv = tid % A_VPR;
                *reinterpret_cast<f32x4*>(&As[row * LDA + kv * 4]) = a_reg[p];
            }
        } else {
            const int row = tid % BM, kb = (tid / BM) * A_KPT;
#pragma unroll
            for (int j = 0; j < A_KPT; ++j) As[row * LDA + kb + j] = a_sreg[j];
        }
        if constexpr (B_FAST) {
#pragma unroll
            for (int p = 0; p < B_NV; ++p) {
                const int kr = tid / B_VPR + p * B_RSTEP, nv = tid % B_VPR;
                *reinterpret_cast<f32x4*>(&Bs[kr * LDB + nv * 4]) = b_reg[p];
            }
        } else {
            const int n = tid % BN, kb = (tid / BN) * B_KPT;
#pragma unroll
            for (int j = 0; j < B_KPT; ++j) Bs[(kb + j) * LDB + n] = b_sreg[j];
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    const int ktiles = (P.K + BK - 1) / BK;
    load_tiles(0);
#pragma unroll
    for (int q = 0; q < E_PER_THREAD; ++q)
        if (tid + q * NT < (int)P.nepi * BN) Es[tid + q * NT] = e_reg[q];
    if (ktiles == 0) __syncthreads();            // otherwise the barriers of the k loop publish Es
    for (int kt = 0; kt < ktiles; ++kt) {
        store_tiles();
        __syncthreads();
        if (kt + 1 < ktiles) load_tiles((kt + 1) * BK);
        // lanes 0-31 consume the first half of the tile's k range, lanes 32-63 the second half.
        // Fragments are double-buffered in registers: the LDS reads of group g+1 are in flight
        // while the MFMAs of group g execute.
        constexpr int G = BK / 8;
        f32x4 af[2][TM];
        float bf[2][TN][4];
        auto load_frags = [&](int g, int buf) {
            const int kk = half * (BK / 2) + g * 4;
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
        __syncthreads();
    }

    // ---------------- epilogue + store ----------------
    // accumulator element v of a lane: row = 8*(v/4) + 4*half + v%4, column = l32.
    // Byte offsets fit 31 bits: the host refuses larger tensors.
    const bool whole_tile = m0 + BM <= P.M && n0 + BN <= P.N;
    // Outputs that are not a row-major [M, N] matrix need (batch, y, x) of every row: decoded once
    // per row into the LDS space of the A tile (free after the k loop), -1 for rows beyond M.
    int* const row_off = reinterpret_cast<int*>(As);
    if (!P.c_contig) {
        for (int r = tid; r < BM; r += NT) {
            const int m = m0 + r;
            const int b = m / HoWo, r2 = m - b * HoWo, ho = r2 / P.Wo, wo = r2 - ho * P.Wo;
            row_off[r] = m < P.M ? b * P.os_b + ho * P.os_h + wo * P.os_w : -1;
        }
        __syncthreads();
    }
    auto elem_offset = [&](int i, int j, int v) -> uint32_t {
        const int n = n0 + (wn * TN + j) * 32 + l32;
        const int r = (wm * TM + i) * 32 + 4 * half + 8 * (v / 4) + (v % 4);
        if (P.c_contig) {
            const int m = m0 + r;
            return (whole_tile || (m < P.M && n < P.N)) ? (uint32_t)(m * P.N + n) * 4u : CONV_OOB;
        }
        const int ro = row_off[r];
        return (ro >= 0 && n < P.N) ? (uint32_t)(ro + n * P.os_n) * 4u : CONV_OOB;
    };
    // the first full-size operand (a residual input) is fetched for the whole tile at once
    // (for the largest tile that would not fit the register file: it loads sub-tile by sub-tile)
    constexpr bool PREFETCH_FULL = TM * TN <= 2;
    float full[PREFETCH_FULL ? TM : 1][PREFETCH_FULL ? TN : 1][16];
    const int first_full = PREFETCH_FULL ? P.epi_first_full : -1;
    if (PREFETCH_FULL && first_full >= 0) {
        const float* fp = epi.p[0];
#pragma unroll
        for (int t = 1; t < CONV_MAX_EPI; ++t) fp = first_full == t ? epi.p[t] : fp;
        const __amdgpu_buffer_rsrc_t f_rsrc = make_rsrc(fp, P.out_bytes);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    full[PREFETCH_FULL ? i : 0][PREFETCH_FULL ? j : 0][v] = buffer_load_x1(f_rsrc, elem_offset(i, j, v));
    }
#pragma unroll
    for (int e = 0; e < CONV_MAX_EPI; ++e) {             // unrolled: the step descriptors stay in scalar registers
        if (e >= (int)P.nepi) break;
        const uint32_t kind = P.epi_kind[e];
        const uint32_t code = P.epi_op[e] * 2u + ((P.epi_flags[e] >> 1) & 1u);   // bit0: operand on the left
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                float ov[16];
                if (kind == 3) {
                    if (PREFETCH_FULL && e == first_full) {
#pragma unroll
                        for (int v = 0; v < 16; ++v) ov[v] = full[PREFETCH_FULL ? i : 0][PREFETCH_FULL ? j : 0][v];
                    } else {
                        const __amdgpu_buffer_rsrc_t f_rsrc = make_rsrc(epi.p[e], P.out_bytes);
#pragma unroll
                        for (int v = 0; v < 16; ++v) ov[v] = buffer_load_x1(f_rsrc, elem_offset(i, j, v));
                    }
                } else {
                    const float o1 = Es[e * BN + (wn * TN + j) * 32 + l32];
#pragma unroll
                    for (int v = 0; v < 16; ++v) ov[v] = o1;
                }
#define EPI_LOOP(expr)                                              \
                _Pragma("unroll") for (int v = 0; v < 16; ++v) {    \
                    const float y = acc[i][j][v], o = ov[v];        \
                    acc[i][j][v] = (expr);                          \
                }
                switch (code) {                              // one uniform branch per step, not per element
                    case CEW_ADD_F * 2: case CEW_ADD_F * 2 + 1: EPI_LOOP(y + o) break;
                    case CEW_MUL_F * 2: case CEW_MUL_F * 2 + 1: EPI_LOOP(y * o) break;
                    case CEW_SUB_F * 2:     EPI_LOOP(y - o) break;
                    case CEW_SUB_F * 2 + 1: EPI_LOOP(o - y) break;
                    case CEW_DIV_F * 2:     EPI_LOOP(y / o) break;
                    case CEW_DIV_F * 2 + 1: EPI_LOOP(o / y) break;
                    case CEW_MAX_F * 2:     EPI_LOOP((y > o || y != y) ? y : o) break;
                    case CEW_MAX_F * 2 + 1: EPI_LOOP((o > y || o != o) ? o : y) break;
                    case CEW_MIN_F * 2:     EPI_LOOP((y < o || y != y) ? y : o) break;
                    case CEW_MIN_F * 2 + 1: EPI_LOOP((o < y || o != o) ? o : y) break;
                    default: break;
                }
#undef EPI_LOOP
            }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) buffer_store_x1(acc[i][j][v], o_rsrc, elem_offset(i, j, v));
}

#define CONV_KERNEL(name, WGM, WGN, TM, TN, BK, AF, BF)                                                     \
    extern "C" __global__ __launch_bounds__(64 * WGM * WGN) __attribute__((amdgpu_waves_per_eu(2))) void name( \
        float* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,                   \
        ConvEpiPtrs epi, ConvParams P) {                                                                     \
        conv_gemm_body<WGM, WGN, TM, TN, BK, AF, BF>(out, x, w, epi, P);                                     \
    }

// name = conv_gemm_<BM>x<BN>x<BK>_<a><b>  with a/b = f (16-byte loads) or g (generic strided loads)
#define CONV_TILE(tag, WGM, WGN, TM, TN, BK)                               \
    CONV_KERNEL(conv_gemm_##tag##_ff, WGM, WGN, TM, TN, BK, true, true)    \
    CONV_KERNEL(conv_gemm_##tag##_fg, WGM, WGN, TM, TN, BK, true, false)   \
    CONV_KERNEL(conv_gemm_##tag##_gf, WGM, WGN, TM, TN, BK, false, true)   \
    CONV_KERNEL(conv_gemm_##tag##_gg, WGM, WGN, TM, TN, BK, false, false)

CONV_TILE(128x128x32, 2, 2, 2, 2, 32)
CONV_TILE(128x64x32, 2, 2, 2, 1, 32)
CONV_TILE(64x64x32, 2, 2, 1, 1, 32)
CONV_TILE(64x64x64, 2, 2, 1, 1, 64)
CONV_TILE(32x32x32, 1, 1, 1, 1, 32)
CONV_TILE(32x32x64, 1, 1, 1, 1, 64)
