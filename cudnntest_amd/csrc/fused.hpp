// Single-kernel Winograd F(2x2,3x3) convolution: input transform, 16-coordinate
// multiply-accumulate over channels and output transform in one launch, with no
// transformed-input or product tensor in HBM.  The structure of the reference's
// fusedTest/winotrans.cuh:1452 (Winofuse4433): per channel slab, half of the
// work is "load a raw input patch, B^T d B in registers, scatter to LDS", the
// other half "copy the pre-transformed filter slab to LDS", then every
// accumulator advances, and A^T(.)A runs on the accumulators at the end -- here
// for 4x4 tiles, all three layouts, zero padding, any C and K, on MFMA.
//
// A workgroup owns 64 filters x 64 tiles for all 16 coordinates: each of its 4
// waves keeps sixteen 32x32 MFMA accumulators (256 AGPRs), so the output
// transform runs in registers (winograd_epilogue in gemm.hpp).  Per k-group
// (GC = 2*CV channels):
//   U slab  <- HBM by direct-to-LDS loads (pre-transformed filters, as in the reference)
//   V slab  <- built in the kernel: each thread owns UNITS (tile, channel) pairs, keeps
//              their 16 raw input values in registers one k-group ahead, transforms
//              them and writes the 16 coordinates into the idle LDS stage.
#pragma once
#include "gemm.hpp"

namespace wino {

// LANES_ON_CHANNELS = false: lanes walk tiles (coalesced when W or N is the contiguous axis)
// LANES_ON_CHANNELS = true : lanes walk the GC channels of a k-group first (NHWC)
template <typename T, bool SWAP, bool LANES_ON_CHANNELS>
__global__ __launch_bounds__(256) void fused_conv_kernel(const T* __restrict__ x, const T* __restrict__ U,
                                                         T* __restrict__ y, ActStrides xs, ActStrides ys, int N,
                                                         int C, int K, int H, int W, int pad, int Ho, int Wo, int th,
                                                         int tw, long P, int Cp, int Kp, int order, int relu,
                                                         int kTiles, int pTiles) {
    typedef typename Mma<T>::vec vec;
    constexpr int CV = ChanVec<T>::n;
    constexpr int GC = 2 * CV;                 // channels per k-group
    constexpr int UNITS = 64 * GC / 256;       // (tile, channel) pairs per thread: 2 (fp32) or 4 (16-bit)
    // s_waitcnt vmcnt(VM) lgkmcnt(0): at most VM (the x loads of one k-group, capped by the 6-bit field) still in flight
    constexpr int VM = 16 * UNITS < 63 ? 16 * UNITS : 63;
    constexpr int WAIT_IMM = (VM & 0xF) | (0x7 << 4) | (0 << 8) | ((VM >> 4) << 14);
    __shared__ vec Us0[16][2][GO_T], Us1[16][2][GO_T];
    __shared__ vec Vs0[16][2][GO_T], Vs1[16][2][GO_T];

    const int b = blockIdx.x;
    const int xcd = b & 7, j = b >> 3;
    const int ktile = j % kTiles;
    const int ptile = (j / kTiles) * 8 + xcd;
    if (ptile >= pTiles) return;
    const int k0 = ktile * GO_T;
    const long p0 = (long)ptile * GO_T;
    const int CQ = Cp / CV;
    const int ngrp = CQ / 2;
    const vec* Ug = reinterpret_cast<const vec*>(U);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;

    // ---- this thread's (tile, channel) units: fixed for the whole kernel ----------------
    int u_tile[UNITS], u_ch[UNITS];            // tile index inside the patch, channel inside the k-group
    unsigned u_row[UNITS][4], u_col[UNITS][4]; // element offsets of the patch rows (incl. image) and columns, clamped inside
    unsigned u_mask[UNITS];                    // bit i*4+j set when position (i, j) lies inside the image
#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
        if (LANES_ON_CHANNELS) {
            u_ch[u] = tid % GC;
            u_tile[u] = tid / GC + u * (256 / GC);
        } else {
            u_tile[u] = tid & 63;
            u_ch[u] = (tid >> 6) * UNITS + u;
        }
        const long p = p0 + u_tile[u];
        int n = 0, ty = 0, tx = 0;
        const bool pvalid = p < P;
        if (pvalid) decode_tile(p, order, N, th, tw, n, ty, tx);
        u_mask[u] = 0;
        unsigned rmask = 0, cmask = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int ih = 2 * ty - pad + i, iw = 2 * tx - pad + i;
            if (ih >= 0 && ih < H) rmask |= 1u << i;
            if (iw >= 0 && iw < W) cmask |= 1u << i;
            const int ihc = ih < 0 ? 0 : (ih >= H ? H - 1 : ih);     // clamped: the load stays inside x, the
            const int iwc = iw < 0 ? 0 : (iw >= W ? W - 1 : iw);     // value is discarded through u_mask
            u_row[u][i] = (unsigned)(n * xs.n + ihc * xs.h);
            u_col[u][i] = (unsigned)(iwc * xs.w);
        }
        if (pvalid) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if ((rmask >> i) & 1u) u_mask[u] |= cmask << (4 * i);
        }
    }

    floatx16 acc[16];
#pragma unroll
    for (int xi = 0; xi < 16; ++xi)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[xi][r] = 0.f;

    typedef std::integral_constant<int, 0> par0_t;
    typedef std::integral_constant<int, 1> par1_t;

    // Raw input patches of the k-group after the one being multiplied.
    T xr[UNITS][16];
    auto x_load_unit = [&](int g, int u) {
        const int c = g * GC + u_ch[u];
        const unsigned coff = c < C ? (unsigned)(c * xs.c) : 0u;   // channel padding: masked out in v_piece
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const unsigned ro = u_row[u][i] + coff;
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) xr[u][i * 4 + jj] = x[ro + u_col[u][jj]];
        }
    };
    // Building stage S of V from the staged patches, cut into 16 pieces so that one
    // piece can ride in the shadow of each coordinate's MFMAs:
    //   pieces 0 .. 2*UNITS-1 : per unit, mask the patch (zero padding) then B^T d B
    //   the remaining pieces  : the LDS writes, a few coordinates each; the first UNITS
    //                           of them also refill the patches with k-group `gload`
    float vt[UNITS][16];
    float dpatch[4][4];
    auto v_piece = [&](auto par, int g, int gload, int piece) {
        constexpr int S = decltype(par)::value;
        constexpr int NW = 16 - 2 * UNITS;                 // pieces that write
        constexpr int PER = (16 + NW - 1) / NW;            // coordinates per writing piece
        if (piece < 2 * UNITS) {
            const int u = piece >> 1;
            if ((piece & 1) == 0) {
                const bool cok = g * GC + u_ch[u] < C;
                const unsigned m = cok ? u_mask[u] : 0u;
#pragma unroll
                for (int q = 0; q < 16; ++q) dpatch[q >> 2][q & 3] = ((m >> q) & 1u) ? to_f32(xr[u][q]) : 0.f;
            } else {
                input_tile_transform(dpatch, vt[u]);
            }
            return;
        }
        const int w = piece - 2 * UNITS;
        if (w < UNITS && gload >= 0) x_load_unit(gload, w);
#pragma unroll
        for (int t = 0; t < PER; ++t) {
            const int xi = w * PER + t;
            if (xi >= 16) continue;
            if (LANES_ON_CHANNELS) {
#pragma unroll
                for (int u = 0; u < UNITS; ++u) {
                    const int h = u_ch[u] / CV, e = u_ch[u] % CV;
                    T* dst = reinterpret_cast<T*>(S ? &Vs1[xi][h][u_tile[u]] : &Vs0[xi][h][u_tile[u]]);
                    dst[e] = from_f32<T>(vt[u][xi]);
                }
            } else {
                // the thread's UNITS channels are consecutive elements of one channel vector: one 8-byte write
                struct alignas(8) Chunk { T e[UNITS]; };
                static_assert(sizeof(Chunk) == 8, "chunk must be 8 bytes");
                const int h = u_ch[0] / CV, e0 = u_ch[0] % CV;
                Chunk ck;
#pragma unroll
                for (int u = 0; u < UNITS; ++u) ck.e[u] = from_f32<T>(vt[u][xi]);
                T* dst = reinterpret_cast<T*>(S ? &Vs1[xi][h][u_tile[0]] : &Vs0[xi][h][u_tile[0]]);
                *reinterpret_cast<Chunk*>(dst + e0) = ck;
            }
        }
    };
    auto u_load = [&](auto par, int g) {
        constexpr int S = decltype(par)::value;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = wave + 4 * i;            // 0..31, wave-uniform
            const int xi = row >> 1, h = row & 1;
            const vec* usrc = Ug + ((size_t)xi * CQ + 2 * g + h) * Kp + k0 + lane;
            vec* udst = S ? &Us1[xi][h][0] : &Us0[xi][h][0];
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)usrc,
                                             (__attribute__((address_space(3))) void*)udst, 16, 0, 0);
        }
    };

    vec fu[3], fv[3];
    auto iteration = [&](auto par, int g) {
        constexpr int S = decltype(par)::value;
        typedef std::integral_constant<int, 1 - S> other_t;
        auto frag_load = [&](int xi) {
            fu[xi % 3] = S ? Us1[xi][lh][(SWAP ? wn : wm) * 32 + l32] : Us0[xi][lh][(SWAP ? wn : wm) * 32 + l32];
            fv[xi % 3] = S ? Vs1[xi][lh][(SWAP ? wm : wn) * 32 + l32] : Vs0[xi][lh][(SWAP ? wm : wn) * 32 + l32];
        };
        const int g1 = g + 1 < ngrp ? g + 1 : g;      // surplus work on the last group is never read
        const int g2 = g + 2 < ngrp ? g + 2 : g1;
        // filter rows of group g+1 first (the whole iteration to land); the raw patches of
        // group g+2 are requested as soon as those of g+1 have been consumed
        u_load(other_t{}, g1);
        frag_load(0);
        frag_load(1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int xi = 0; xi < 16; ++xi) {
            if (xi + 2 < 16) frag_load(xi + 2);
            v_piece(other_t{}, g1, g2, xi);
            if (SWAP) Mma<T>::run(fv[xi % 3], fu[xi % 3], acc[xi]);
            else Mma<T>::run(fu[xi % 3], fv[xi % 3], acc[xi]);
            __builtin_amdgcn_sched_barrier(0);
        }
        // the filter rows of the next stage must be in LDS (they were issued before the x
        // loads, and loads retire in order); the younger x loads may stay in flight
        __builtin_amdgcn_s_waitcnt(WAIT_IMM);
        __syncthreads();
    };

    // prologue: stage 0 of both slabs, and the raw patches of group 1 in flight
    u_load(par0_t{}, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < UNITS; ++u) x_load_unit(0, u);
#pragma unroll
    for (int piece = 0; piece < 16; ++piece) v_piece(par0_t{}, 0, ngrp > 1 ? 1 : 0, piece);
    __builtin_amdgcn_s_waitcnt(WAIT_IMM);
    __syncthreads();

    for (int g = 0; g < ngrp; g += 2) {   // ngrp is even: Cp is a multiple of 4 channel vectors
        iteration(par0_t{}, g);
        iteration(par1_t{}, g + 1);
    }

    winograd_epilogue<T, SWAP>(acc, y, ys, N, K, Ho, Wo, th, tw, P, order, relu, k0, p0, wm, wn, l32, lh);
}

}  // namespace wino
