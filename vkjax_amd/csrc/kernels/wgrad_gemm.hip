// fp32 "TN" implicit GEMM on the MFMA units: C[m, n] = sum over p of A[p, m] * B[p, n], where p runs
// over the pixels (image, y, x) of a convolution's output and
//     A[p, m] = X[image, y*SH + ky*DH - PH, x*SW + kx*DW - PW, ci]    m = (ky*KW + kx)*C + ci   (0 outside X)
//     B[p, n] = G[p, n]
// i.e. the kernel gradient dW[ky, kx, ci, co] of an NHWC / HWIO convolution from its input X and the
// cotangent G of its output, and, with a 1x1 window, the product X^T G of two row-major matrices
// contracted over their rows (the weight gradient of a dense layer). Autodiff emits both as a
// convolution / dot_general whose contraction index is the slowest-varying one of both operands;
// the general implicit-GEMM kernel would read them one element per cache line.
//
// Both operands are read along their contiguous dimension (16 bytes per lane when C resp. N allow)
// and parked k-major in LDS, which is the order the MFMA operands want: lane l of a wave supplies
// A[k = l / 32][m = l % 32] and B[k = l / 32][n = l % 32] from consecutive addresses.
// The contraction is long (pixels) and the result small, so it is split over gridDim.z: slice z
// contracts pixels [z * pix_per_split, (z + 1) * pix_per_split) and writes its own [M, N] partial
// result; the host adds the slices with a column reduction. Tile 64 x 64 x 32, four waves (2 x 2).
#include "common.h"

#define WG_OOB 0x80000000u

struct WgradParams {
    int32_t  pixels, M, N;             // contraction length (images * Ho * Wo); M = KH * KW * C
    int32_t  Ho, Wo, H, W, C, KW;
    int32_t  SH, SW, PH, PW, DH, DW;
    int32_t  pix_per_split;            // multiple of 32
    uint32_t howo_magic, howo_shift, wo_magic, wo_shift, c_magic, c_shift, kw_magic, kw_shift;
    uint32_t x_bytes, g_bytes;
};

template <bool VEC_A, bool VEC_B>
__device__ __forceinline__ void wgrad_body(float* __restrict__ out, const float* __restrict__ x, const float* __restrict__ g,
                                           const WgradParams& P) {
    constexpr int BM = 64, BN = 64, BK = 32, LD = 68;
    __shared__ float As[BK * LD], Bs[BK * LD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, half = lane >> 5;
    const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;
    const int kbeg = blockIdx.z * P.pix_per_split, kend = min(P.pixels, kbeg + P.pix_per_split);
    const int nk = kbeg < kend ? (kend - kbeg + BK - 1) / BK : 0;
    const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, P.x_bytes), g_rsrc = make_rsrc(g, P.g_bytes);

    // this thread's column group (four consecutive m resp. n) and its two pixel rows of every tile
    const int cg = tid & 15, prow = tid >> 4;
    constexpr int NA = VEC_A ? 1 : 4;
    int a_dy[NA], a_dx[NA], a_ci[NA];
    bool a_ok[NA];
#pragma unroll
    for (int q = 0; q < NA; ++q) {
        const int m   = m0 + 4 * cg + q;
        const int tap = magic_div(m, P.c_magic, P.c_shift);
        const int ky  = magic_div(tap, P.kw_magic, P.kw_shift);
        a_ci[q] = m - tap * P.C;
        a_dy[q] = ky * P.DH - P.PH;
        a_dx[q] = (tap - ky * P.KW) * P.DW - P.PW;
        a_ok[q] = m < P.M;
    }
    const int n = n0 + 4 * cg;
    const int HoWo = P.Ho * P.Wo;

    float ra[2][4], rb[2][4];
    auto load_tiles = [&](int kt) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int p = kbeg + kt * BK + prow + 16 * j;
            const bool p_ok = p < kend;
            const int img = magic_div(p, P.howo_magic, P.howo_shift);
            const int r   = p - img * HoWo;
            const int ho  = magic_div(r, P.wo_magic, P.wo_shift);
            const int wo  = r - ho * P.Wo;
            const int y0 = ho * P.SH, x0 = wo * P.SW;
#pragma unroll
            for (int q = 0; q < NA; ++q) {
                const int y = y0 + a_dy[q], xx = x0 + a_dx[q];
                const bool ok = p_ok && a_ok[q] && (uint32_t)y < (uint32_t)P.H && (uint32_t)xx < (uint32_t)P.W;
                const uint32_t off = ok ? (uint32_t)(((img * P.H + y) * P.W + xx) * P.C + a_ci[q]) * 4u : WG_OOB;
                if constexpr (VEC_A) {
                    const f32x4 v = buffer_load_x4(x_rsrc, off);
                    ra[j][0] = v.x; ra[j][1] = v.y; ra[j][2] = v.z; ra[j][3] = v.w;
                } else {
                    ra[j][q] = buffer_load_x1(x_rsrc, off);
                }
            }
            if constexpr (VEC_B) {
                const f32x4 v = buffer_load_x4(g_rsrc, (p_ok && n < P.N) ? (uint32_t)(p * P.N + n) * 4u : WG_OOB);
                rb[j][0] = v.x; rb[j][1] = v.y; rb[j][2] = v.z; rb[j][3] = v.w;
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    rb[j][q] = buffer_load_x1(g_rsrc, (p_ok && n + q < P.N) ? (uint32_t)(p * P.N + n + q) * 4u : WG_OOB);
            }
        }
    };
    auto store_tiles = [&]() {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            *reinterpret_cast<f32x4*>(&As[(prow + 16 * j) * LD + 4 * cg]) = f32x4{ra[j][0], ra[j][1], ra[j][2], ra[j][3]};
            *reinterpret_cast<f32x4*>(&Bs[(prow + 16 * j) * LD + 4 * cg]) = f32x4{rb[j][0], rb[j][1], rb[j][2], rb[j][3]};
        }
    };

    f32x16 acc = f32x16{};
    if (nk > 0) load_tiles(0);
    for (int kt = 0; kt < nk; ++kt) {
        store_tiles();
        __syncthreads();
        if (kt + 1 < nk) load_tiles(kt + 1);
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            const float a = As[(kk + half) * LD + wm * 32 + l32];
            const float b = Bs[(kk + half) * LD + wn * 32 + l32];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
        }
        __syncthreads();
    }
    // element v of the accumulator: row 8 * (v / 4) + 4 * half + v % 4, column l32 of the wave's 32 x 32 block
    float c[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) c[v] = acc[v];
    const int col = n0 + wn * 32 + l32;
    float* const slice = out + (size_t)blockIdx.z * P.M * P.N;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 32 + 8 * (v / 4) + 4 * half + (v % 4);
        if (row < P.M && col < P.N) slice[(size_t)row * P.N + col] = c[v];
    }
}

#define WGRAD_KERNEL(name, VA, VB)                                                                          \
    extern "C" __global__ __launch_bounds__(256) void name(float* __restrict__ out, const float* __restrict__ x, \
                                                           const float* __restrict__ g, WgradParams P) {    \
        wgrad_body<VA, VB>(out, x, g, P);                                                                   \
    }
// suffix: a = 16-byte loads of X (C % 4 == 0), b = 16-byte loads of G (N % 4 == 0), s = single words
WGRAD_KERNEL(wgrad_gemm_64x64_aa, true, true)
WGRAD_KERNEL(wgrad_gemm_64x64_as, true, false)
WGRAD_KERNEL(wgrad_gemm_64x64_sa, false, true)
WGRAD_KERNEL(wgrad_gemm_64x64_ss, false, false)
