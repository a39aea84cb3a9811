// 16-way batched GEMM of the Winograd domain on MFMA (gfx950, wave64).
//
//   Mo[xi][k][p] = sum_c U[xi][c][k] * V[xi][c][p]          xi = 0..15
//
// fp32 path: v_mfma_f32_32x32x2_f32.  Operand registers of that instruction for
// lane l:  a = A[i = l%32][kk = l/32],  b = B[kk = l/32][j = l%32];  the 16
// accumulator registers r hold D[i = 8*(r/4) + 4*(l/32) + r%4][j = l%32].
// With A = U^T (i = filter) and B = V (j = tile) a wave store of one register
// is a contiguous run of tiles.
#pragma once
#include "common.hpp"
#include "transforms.hpp"

namespace wino {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Block tile 128 filters x 128 tiles, 4 waves in a 2x2 arrangement, each wave
// 64x64 = 2x2 MFMA tiles.  Reduction is consumed 16 channels at a time from LDS,
// double-buffered: the next slab travels HBM -> registers while the current one
// feeds the MFMAs, then registers -> the other LDS buffer, one barrier per slab.
constexpr int GEMM_BM = 128, GEMM_BN = 128, GEMM_KC = 16;

__global__ __launch_bounds__(256) void gemm_f32_128x128_kernel(const float* __restrict__ U,
                                                                const float* __restrict__ V,
                                                                float* __restrict__ Mo, int Cp, int Kp, long Pp) {
    __shared__ float As[2][GEMM_KC][GEMM_BM];
    __shared__ float Bs[2][GEMM_KC][GEMM_BN];

    const int xi = blockIdx.z;
    const long p0 = (long)blockIdx.x * GEMM_BN;
    const int k0 = blockIdx.y * GEMM_BM;
    const float* Ub = U + (size_t)xi * Cp * Kp + k0;
    const float* Vb = V + (size_t)xi * Cp * Pp + p0;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;

    // global -> LDS mapping: thread moves rows (tid/32) and (tid/32 + 8), 4 floats at column 4*(tid%32)
    const int lrow = tid >> 5, lcol = (tid & 31) * 4;

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    floatx4 ra[2], rb[2];
    auto gload = [&](int ch) {
        const int c0 = ch * GEMM_KC;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            ra[h] = *reinterpret_cast<const floatx4*>(Ub + (size_t)(c0 + lrow + 8 * h) * Kp + lcol);
            rb[h] = *reinterpret_cast<const floatx4*>(Vb + (size_t)(c0 + lrow + 8 * h) * Pp + lcol);
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            *reinterpret_cast<floatx4*>(&As[buf][lrow + 8 * h][lcol]) = ra[h];
            *reinterpret_cast<floatx4*>(&Bs[buf][lrow + 8 * h][lcol]) = rb[h];
        }
    };

    const int nch = Cp / GEMM_KC;
    gload(0);
    lstore(0);
    __syncthreads();

    for (int ch = 0; ch < nch; ++ch) {
        const int buf = ch & 1;
        if (ch + 1 < nch) gload(ch + 1);
#pragma unroll
        for (int kk = 0; kk < GEMM_KC / 2; ++kk) {
            float a[2], b[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                a[t] = As[buf][kk * 2 + lh][wm * 64 + t * 32 + l32];
                b[t] = Bs[buf][kk * 2 + lh][wn * 64 + t * 32 + l32];
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (ch + 1 < nch) lstore(buf ^ 1);
        __syncthreads();
    }

    float* Mb = Mo + (size_t)xi * Kp * Pp;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = k0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
                const long col = p0 + wn * 64 + j * 32 + l32;
                Mb[(size_t)row * Pp + col] = acc[i][j][r];
            }
}

// =============================================================================
// GEMM with the output transform in its epilogue.
//
// A workgroup owns a 64-filter x 64-tile patch for ALL 16 Winograd coordinates:
// each of its 4 waves keeps sixteen 32x32 MFMA accumulators (256 accumulation
// registers, the whole AGPR file of a wave), so when the reduction over
// channels ends every lane holds the 16 coordinates of its (filter, tile) pairs
// and applies A^T(.)A in registers; the product tensor never reaches HBM.
//
// Reduction runs KC channels at a time through LDS ([xi][KC][64] for U and for
// V), double-buffered through registers as in the plain GEMM.
//
// SWAP = false: MFMA rows = filters, lanes = tiles  (stores contiguous along the
//               tile axis: NCHW, or CHWN with batch-minor tiles)
// SWAP = true : MFMA rows = tiles, lanes = filters  (stores contiguous along K: NHWC)
//
// Workgroup -> patch mapping is XCD-aware: consecutive workgroup ids go to the
// 8 XCDs round-robin, so the ids that land on one XCD walk the filter tiles of
// one tile patch first; the V slab they share then stays in that XCD's L2.
// =============================================================================
constexpr int GO_KC = 8;
constexpr int GO_T = 64;   // patch edge (filters and tiles)
constexpr size_t GO_LDS_BYTES = 2ull * 2 * 16 * GO_KC * GO_T * sizeof(float);

template <typename OutT>
__device__ __forceinline__ void store_tile_outputs(OutT* __restrict__ y, const ActStrides& ys, int n, int k, int ty,
                                                   int tx, int Ho, int Wo, float y00, float y01, float y10, float y11,
                                                   int relu) {
    if (relu) {
        y00 = fmaxf(y00, 0.f); y01 = fmaxf(y01, 0.f); y10 = fmaxf(y10, 0.f); y11 = fmaxf(y11, 0.f);
    }
    const int oh = 2 * ty, ow = 2 * tx;
    OutT* yp = y + n * ys.n + k * ys.c + oh * ys.h + ow * ys.w;
    const bool w1 = ow + 1 < Wo, h1 = oh + 1 < Ho;
    yp[0] = from_f32<OutT>(y00);
    if (w1) yp[ys.w] = from_f32<OutT>(y01);
    if (h1) {
        yp[ys.h] = from_f32<OutT>(y10);
        if (w1) yp[ys.h + ys.w] = from_f32<OutT>(y11);
    }
}

template <typename OutT, bool SWAP>
__global__ __launch_bounds__(256) void gemm_out_f32_kernel(const float* __restrict__ U, const float* __restrict__ V,
                                                           OutT* __restrict__ y, ActStrides ys, int N, int K, int Ho,
                                                           int Wo, int th, int tw, long P, int Cp, int Kp, long Pp,
                                                           int order, int relu, int kTiles, int pTiles) {
    // 2 stages x (U slab + V slab) x 16 x KC x 64 floats = 128 KB: dynamic LDS
    extern __shared__ float go_smem[];
    typedef float (*slab_t)[16][GO_KC][GO_T];
    slab_t Us = reinterpret_cast<slab_t>(go_smem);
    slab_t Vs = reinterpret_cast<slab_t>(go_smem + 2 * 16 * GO_KC * GO_T);

    const int b = blockIdx.x;
    const int xcd = b & 7, j = b >> 3;
    const int ktile = j % kTiles;
    const int ptile = (j / kTiles) * 8 + xcd;
    if (ptile >= pTiles) return;
    const int k0 = ktile * GO_T;
    const long p0 = (long)ptile * GO_T;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;

    floatx16 acc[16];
#pragma unroll
    for (int xi = 0; xi < 16; ++xi)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[xi][r] = 0.f;

    // global -> LDS: 128 rows (xi, c) of 64 floats per operand = 2048 float4, 8 per thread per operand
    floatx4 ru[8], rv[8];
    const int q4 = (tid & 15) * 4;      // column inside the 64-wide row
    const int rbase = tid >> 4;         // 0..15, rows rbase + 16*i
    auto gload = [&](int ch) {
        const int c0 = ch * GO_KC;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = rbase + 16 * i;            // 0..127
            const int xi = row / GO_KC, c = row % GO_KC;
            ru[i] = *reinterpret_cast<const floatx4*>(U + ((size_t)xi * Cp + c0 + c) * Kp + k0 + q4);
            rv[i] = *reinterpret_cast<const floatx4*>(V + ((size_t)xi * Cp + c0 + c) * Pp + p0 + q4);
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = rbase + 16 * i;
            const int xi = row / GO_KC, c = row % GO_KC;
            *reinterpret_cast<floatx4*>(&Us[buf][xi][c][q4]) = ru[i];
            *reinterpret_cast<floatx4*>(&Vs[buf][xi][c][q4]) = rv[i];
        }
    };

    const int nch = Cp / GO_KC;
    gload(0);
    lstore(0);
    __syncthreads();

    for (int ch = 0; ch < nch; ++ch) {
        const int buf = ch & 1;
        if (ch + 1 < nch) gload(ch + 1);
#pragma unroll
        for (int xi = 0; xi < 16; ++xi) {
#pragma unroll
            for (int kk = 0; kk < GO_KC / 2; ++kk) {
                const float fu = Us[buf][xi][kk * 2 + lh][(SWAP ? wn : wm) * 32 + l32];
                const float fv = Vs[buf][xi][kk * 2 + lh][(SWAP ? wm : wn) * 32 + l32];
                acc[xi] = __builtin_amdgcn_mfma_f32_32x32x2f32(SWAP ? fv : fu, SWAP ? fu : fv, acc[xi], 0, 0, 0);
            }
        }
        if (ch + 1 < nch) lstore(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: A^T (.) A on the 16 accumulators, then store ----------------------
    if (!SWAP) {
        const long p = p0 + wn * 32 + l32;
        if (p >= P) return;
        int n, ty, tx;
        decode_tile(p, order, N, th, tw, n, ty, tx);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int k = k0 + wm * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
            if (k >= K) continue;
            float m[16];
#pragma unroll
            for (int xi = 0; xi < 16; ++xi) m[xi] = acc[xi][r];
            float y00, y01, y10, y11;
            output_tile_transform(m, y00, y01, y10, y11);
            store_tile_outputs<OutT>(y, ys, n, k, ty, tx, Ho, Wo, y00, y01, y10, y11, relu);
        }
    } else {
        const int k = k0 + wn * 32 + l32;
        if (k >= K) return;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const long p = p0 + wm * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
            if (p >= P) continue;
            int n, ty, tx;
            decode_tile(p, order, N, th, tw, n, ty, tx);
            float m[16];
#pragma unroll
            for (int xi = 0; xi < 16; ++xi) m[xi] = acc[xi][r];
            float y00, y01, y10, y11;
            output_tile_transform(m, y00, y01, y10, y11);
            store_tile_outputs<OutT>(y, ys, n, k, ty, tx, Ho, Wo, y00, y01, y10, y11, relu);
        }
    }
}

}  // namespace wino
