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

}  // namespace wino
