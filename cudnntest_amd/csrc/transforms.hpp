// Winograd F(2x2,3x3) transform kernels: U = G g G^T, V = B^T d B, y = A^T Mo A.
// All three are HBM-bandwidth bound; arithmetic is fp32 whatever the storage type.
//
//   B^T = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 1 0 -1]
//   G   = [1 0 0; 1/2 1/2 1/2; 1/2 -1/2 1/2; 0 0 1]
//   A^T = [1 1 1 0; 0 1 -1 -1]
//
// Operand layouts written here (CV = 16 / sizeof(T) channels per 16-byte vector):
//   U[xi][Cp/CV][Kp][CV]     V[xi][Cp/CV][Pp][CV]
#pragma once
#include "common.hpp"

namespace wino {

// ---- register-level 1-D transforms ------------------------------------------
__device__ __forceinline__ void bt4(float d0, float d1, float d2, float d3, float& o0, float& o1, float& o2,
                                    float& o3) {
    o0 = d0 - d2;
    o1 = d1 + d2;
    o2 = d2 - d1;
    o3 = d1 - d3;
}

// v (16, row-major 4x4) = B^T d B, rows first then columns
__device__ __forceinline__ void input_tile_transform(const float d[4][4], float* v) {
    float t[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) bt4(d[0][j], d[1][j], d[2][j], d[3][j], t[0][j], t[1][j], t[2][j], t[3][j]);
#pragma unroll
    for (int i = 0; i < 4; ++i) bt4(t[i][0], t[i][1], t[i][2], t[i][3], v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
}

// u (16, row-major 4x4) = G g G^T
__device__ __forceinline__ void filter_tile_transform(const float g[3][3], float* u) {
    float t[4][3];
#pragma unroll
    for (int s = 0; s < 3; ++s) {
        t[0][s] = g[0][s];
        t[1][s] = 0.5f * (g[0][s] + g[1][s] + g[2][s]);
        t[2][s] = 0.5f * (g[0][s] - g[1][s] + g[2][s]);
        t[3][s] = g[2][s];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        u[4 * i + 0] = t[i][0];
        u[4 * i + 1] = 0.5f * (t[i][0] + t[i][1] + t[i][2]);
        u[4 * i + 2] = 0.5f * (t[i][0] - t[i][1] + t[i][2]);
        u[4 * i + 3] = t[i][2];
    }
}

// y (2x2) = A^T m A
__device__ __forceinline__ void output_tile_transform(const float m[16], float& y00, float& y01, float& y10,
                                                      float& y11) {
    float r0[4], r1[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        r0[j] = m[j] + m[4 + j] + m[8 + j];
        r1[j] = m[4 + j] - m[8 + j] - m[12 + j];
    }
    y00 = r0[0] + r0[1] + r0[2];
    y01 = r0[1] - r0[2] - r0[3];
    y10 = r1[0] + r1[1] + r1[2];
    y11 = r1[1] - r1[2] - r1[3];
}

// ---- filter transform ---------------------------------------------------------
// One thread per (filter k, channel vector cq), k fastest: each of its 16 stores
// is a 16-byte vector and a wave's stores are contiguous.  The grid covers the
// padded (Cp/CV) x Kp rectangle and the padding is written as zeros, which is
// what lets the GEMM run without masks on the reduction dimension.
// The 3x3 taps of filter k for the CV channels of vector cq, as fp32; zeros where the filter or a channel does not exist.
template <typename T>
__device__ __forceinline__ void filter_taps_load(const T* __restrict__ w, const FltStrides& s, int K, int C, int k, int cq,
                                                 float (&g)[ChanVec<T>::n][3][3]) {
    constexpr int CV = ChanVec<T>::n;
    // all CV channels of this vector exist, and the filter bank allows 16-byte loads
    const bool full = k < K && (cq + 1) * CV <= C && (reinterpret_cast<uintptr_t>(w) & 15) == 0;
    if (full && s.c == 9 && s.s == 1 && (C * 9) % CV == 0) {
        // [K][C][3][3]: the CV channels of this thread are 9*CV contiguous elements -> nine 16-byte loads
        const Pack16<T>* wp = reinterpret_cast<const Pack16<T>*>(w + k * s.k + (long)cq * CV * 9);
#pragma unroll
        for (int i = 0; i < 9; ++i) {
            const Pack16<T> pk = wp[i];
#pragma unroll
            for (int j = 0; j < CV; ++j) {
                const int f = i * CV + j;                 // flat index: channel f/9, tap f%9
                g[f / 9][(f % 9) / 3][f % 3] = to_f32(pk.e[j]);
            }
        }
    } else if (full && s.c == 1 && C % CV == 0) {
        // [K][3][3][C]: each tap holds the CV channels contiguously -> one 16-byte load per tap
#pragma unroll
        for (int r = 0; r < 3; ++r)
#pragma unroll
            for (int q = 0; q < 3; ++q) {
                const Pack16<T> pk = *reinterpret_cast<const Pack16<T>*>(w + k * s.k + r * s.r + q * s.s + cq * CV);
#pragma unroll
                for (int e = 0; e < CV; ++e) g[e][r][q] = to_f32(pk.e[e]);
            }
    } else {
        // any strides ([C][3][3][K]: lanes along k read contiguously).  All 9*CV loads are issued
        // from clamped addresses before the first use and masked afterwards: a load under a branch
        // is waited for on its own, and this kernel is all latency.
        T raw[CV][9];
#pragma unroll
        for (int e = 0; e < CV; ++e) {
            const int c = cq * CV + e;
            const T* wp = w + (k < K ? k : K - 1) * s.k + (c < C ? c : C - 1) * s.c;
#pragma unroll
            for (int t = 0; t < 9; ++t) raw[e][t] = wp[(t / 3) * s.r + (t % 3) * s.s];
        }
#pragma unroll
        for (int e = 0; e < CV; ++e) {
            const unsigned m = (k < K && cq * CV + e < C) ? 0xFFFFFFFFu : 0u;
#pragma unroll
            for (int t = 0; t < 9; ++t) g[e][t / 3][t % 3] = mask_keep(to_f32(raw[e][t]), m);
        }
    }
}

template <typename T>
__device__ __forceinline__ void filter_transform_thread(const T* __restrict__ w, T* __restrict__ U, FltStrides s,
                                                        int K, int C, int Kp, int Cp, int k, int cq) {
    constexpr int CV = ChanVec<T>::n;
    float u[CV][16];
    float g[CV][3][3];
    filter_taps_load<T>(w, s, K, C, k, cq, g);
#pragma unroll
    for (int e = 0; e < CV; ++e) filter_tile_transform(g[e], u[e]);
    const size_t plane = (size_t)Cp * Kp;   // elements per coordinate
    T* up = U + ((size_t)cq * Kp + k) * CV;
#pragma unroll
    for (int xi = 0; xi < 16; ++xi) {
        float v[CV];
#pragma unroll
        for (int e = 0; e < CV; ++e) v[e] = u[e][xi];
        store_chan_vec<T>(up + xi * plane, v);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void filter_transform_kernel(const T* __restrict__ w, T* __restrict__ U,
                                                                FltStrides s, int K, int C, int Kp, int Cp) {
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k < Kp) filter_transform_thread<T>(w, U, s, K, C, Kp, Cp, k, blockIdx.y);
}

// A filter bank to transform in the same launch as an input transform (w == nullptr: none).  A layer call
// needs both before its GEMM, the filter transform is a few microseconds of latency-bound work, and a launch
// of its own costs about as much again: the input transform's grid gets one more z-slice for it.
struct FilterJob {
    const void* w;
    void* U;
    FltStrides s;
    int K, C, Kp, Cp;
};

// The filter job of a launch whose grid.x was extended past in_blocks: those workgroups (all y) share the
// Kp x Cp/CV threads of the job, filters fastest.
template <typename T, int NT>
__device__ __forceinline__ void filter_job_blocks(const FilterJob& fj, int in_blocks) {
    constexpr int CV = ChanVec<T>::n;
    const long work = (long)fj.Kp * (fj.Cp / CV);
    const long nthreads = (long)(gridDim.x - in_blocks) * gridDim.y * NT;
    for (long i = ((long)(blockIdx.x - in_blocks) * gridDim.y + blockIdx.y) * NT + threadIdx.x; i < work; i += nthreads)
        filter_transform_thread<T>((const T*)fj.w, (T*)fj.U, fj.s, fj.K, fj.C, fj.Kp, fj.Cp, (int)(i % fj.Kp),
                                   (int)(i / fj.Kp));
}

// ---- input transform, layout-generic ---------------------------------------------
// One thread per (tile p, channel vector cq), p fastest: every store is a
// 16-byte vector and a wave's stores form a contiguous 1 KB run of V.  Reads go
// through the activation strides, so the kernel is correct for every layout and
// tile order; it is the fast path when the source's contiguous axis runs along
// p (NCHW rows, CHWN with batch-minor tiles).
template <typename T>
__global__ __launch_bounds__(256) void input_transform_generic_kernel(const T* __restrict__ x, T* __restrict__ V,
                                                                       ActStrides s, int N, int C, int H, int W,
                                                                       int pad, int th, int tw, long P, long Pp,
                                                                       int Cp, int order, FilterJob fj,
                                                                       int in_blocks, int cq_fast) {
    constexpr int CV = ChanVec<T>::n;
    if (fj.w && (int)blockIdx.x >= in_blocks) {
        filter_job_blocks<T, 256>(fj, in_blocks);
        return;
    }
    // Workgroups are dispatched along x first.  cq_fast re-deals the ids so that the channel vectors of one run of
    // tiles follow each other instead of the tile runs of one channel vector (faster while x and V together fit the
    // last-level cache, slower beyond: measured on CHWN sources).
    long pb = blockIdx.x;
    int cq = blockIdx.y;
    if (cq_fast) {
        const long lin = (long)blockIdx.y * in_blocks + blockIdx.x;
        pb = lin / gridDim.y;
        cq = (int)(lin - pb * gridDim.y);
    }
    const long p = pb * blockDim.x + threadIdx.x;
    if (p >= P) return;
    int n, ty, tx;
    decode_tile(p, order, N, th, tw, n, ty, tx);
    const int h0 = 2 * ty - pad, w0 = 2 * tx - pad;
    // Branch-free halo handling: every load goes to a clamped (always valid) address and
    // the value is kept or zeroed by a mask, so all CV*16 loads are in flight together.
    long roff[4], coff[4];
    unsigned rkeep[4], ckeep[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int ih = h0 + i, iw = w0 + i;
        rkeep[i] = (ih >= 0 && ih < H) ? 0xffffffffu : 0u;
        ckeep[i] = (iw >= 0 && iw < W) ? 0xffffffffu : 0u;
        roff[i] = (long)(ih < 0 ? 0 : (ih >= H ? H - 1 : ih)) * s.h;
        coff[i] = (long)(iw < 0 ? 0 : (iw >= W ? W - 1 : iw)) * s.w;
    }
    float v[CV][16];
#pragma unroll
    for (int e = 0; e < CV; ++e) {
        const int c = cq * CV + e;
        const unsigned chkeep = c < C ? 0xffffffffu : 0u;
        const T* xp = x + n * s.n + (c < C ? c : C - 1) * s.c;
        float d[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                d[i][j] = mask_keep(to_f32(xp[roff[i] + coff[j]]), rkeep[i] & ckeep[j] & chkeep);
        input_tile_transform(d, v[e]);
    }
    const size_t plane = (size_t)Cp * Pp;
    T* vp = V + ((size_t)cq * Pp + p) * CV;
#pragma unroll
    for (int xi = 0; xi < 16; ++xi) {
        float o[CV];
#pragma unroll
        for (int e = 0; e < CV; ++e) o[e] = v[e][xi];
        store_chan_vec<T>(vp + xi * plane, o);
    }
}

// ---- input transform, NCHW source, LDS-staged ----------------------------------------
// A workgroup takes one image n, one channel vector cq and a TR x TC block of
// tiles.  The (2*TR+2) x (2*TC+2) input halo of each of its CV channels is read
// once, along W (contiguous), into LDS with the zero padding materialised; each
// thread then builds its tile from LDS (lanes walk tx, two columns apart:
// conflict-free) and issues 16 coalesced 16-byte stores.
//
// VEC = elements per lane and load in the halo copy: 1, or 2 for 2-byte types
// when W is even (4-byte loads of image-aligned column pairs).
template <typename T> __device__ __forceinline__ void lds_row4(const T* p, float* d);
template <> __device__ __forceinline__ void lds_row4<float>(const float* p, float* d) {
    const float2 a = *reinterpret_cast<const float2*>(p);
    const float2 b = *reinterpret_cast<const float2*>(p + 2);
    d[0] = a.x; d[1] = a.y; d[2] = b.x; d[3] = b.y;
}
template <> __device__ __forceinline__ void lds_row4<f16_t>(const f16_t* p, float* d) {
    struct alignas(4) P2 { f16_t a, b; };
    const P2 u = *reinterpret_cast<const P2*>(p), v = *reinterpret_cast<const P2*>(p + 2);
    d[0] = (float)u.a; d[1] = (float)u.b; d[2] = (float)v.a; d[3] = (float)v.b;
}
template <> __device__ __forceinline__ void lds_row4<bf16_t>(const bf16_t* p, float* d) {
    const uint32_t u = *reinterpret_cast<const uint32_t*>(p), v = *reinterpret_cast<const uint32_t*>(p + 2);
    d[0] = __uint_as_float(u << 16); d[1] = __uint_as_float(u & 0xffff0000u);
    d[2] = __uint_as_float(v << 16); d[3] = __uint_as_float(v & 0xffff0000u);
}

// The 16 coordinates of one tile for the CV channels of a vector, built from LDS planes [ch][rows][ldsW] that hold
// the zero padding (`base`: the tile's first element in the first plane, at an even column), and stored as 16
// vectors of V, `plane` elements apart.
template <typename T>
__device__ __forceinline__ void tile_from_lds_store(const T* base, int per_ch, int ldsW, T* vp, size_t plane) {
    constexpr int CV = ChanVec<T>::n;
    auto tile_of = [&](int ch, float (&out)[16]) {
        float d[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) lds_row4<T>(base + ch * per_ch + i * ldsW, d[i]);
        input_tile_transform(d, out);
    };
    if constexpr (sizeof(T) == 2) {
        // 8 channels x 16 coordinates: rounded and packed two channels to a register as they are produced (64
        // registers instead of 128 fp32 values held until the stores)
        uint32_t wd[16][CV / 2];
#pragma unroll
        for (int ch = 0; ch < CV; ++ch) {
            float vc[16];
            tile_of(ch, vc);
#pragma unroll
            for (int xi = 0; xi < 16; ++xi) {
                const uint32_t bits = __builtin_bit_cast(uint16_t, from_f32<T>(vc[xi]));
                wd[xi][ch / 2] = (ch & 1) ? (wd[xi][ch / 2] | bits << 16) : bits;
            }
        }
#pragma unroll
        for (int xi = 0; xi < 16; ++xi)
            *reinterpret_cast<uint4*>(vp + xi * plane) = make_uint4(wd[xi][0], wd[xi][1], wd[xi][2], wd[xi][3]);
    } else {
        float v[CV][16];
#pragma unroll
        for (int ch = 0; ch < CV; ++ch) tile_of(ch, v[ch]);
#pragma unroll
        for (int xi = 0; xi < 16; ++xi) {
            float o[CV];
#pragma unroll
            for (int e = 0; e < CV; ++e) o[e] = v[e][xi];
            store_chan_vec<T>(vp + xi * plane, o);
        }
    }
}

// the F(4x4,3x3) pieces the tiled NCHW kernel uses with M = 4 (transforms_f4.hpp)
template <typename T>
__device__ __forceinline__ void filter_transform_f4_thread(const T* __restrict__ w, T* __restrict__ U, const FltStrides& s, int K,
                                                           int C, int Kp, int Cp, int k, int cq);
__device__ __forceinline__ void tile_from_lds_store_f4(const float* base, int per_ch, int ldsW, float* vp, size_t plane);

// M = 2: F(2x2,3x3) tiles, 4x4 pixels every 2.  M = 4: F(4x4,3x3) tiles, 6x6 pixels every 4 (fp32 only); the halo
// copy is the same code, the filter job and the tile arithmetic are the F(4x4) ones.
template <typename T, int VEC, int M = 2>
__global__ __launch_bounds__(256) void input_transform_nchw_kernel(const T* __restrict__ x, T* __restrict__ V, int N,
                                                                   int C, int H, int W, int pad, int th, int tw,
                                                                   long Pp, int Cp, int TR, int TC, int colBlocks,
                                                                   int chunkLog2, FilterJob fj) {
    constexpr int CV = ChanVec<T>::n;
    extern __shared__ __attribute__((aligned(16))) unsigned char in_smem_raw[];
    T* in_smem = reinterpret_cast<T*>(in_smem_raw);   // [CV][rows][ldsW], the storage type
    if (fj.w && blockIdx.z == 0) {
        // the first z-slice transforms the filter bank: channel vector blockIdx.y (the layer's C), filters strided
        for (int k = blockIdx.x * 256 + threadIdx.x; k < fj.Kp; k += gridDim.x * 256) {
            if constexpr (M == 4) filter_transform_f4_thread<T>((const T*)fj.w, (T*)fj.U, fj.s, fj.K, fj.C, fj.Kp, fj.Cp, k, blockIdx.y);
            else filter_transform_thread<T>((const T*)fj.w, (T*)fj.U, fj.s, fj.K, fj.C, fj.Kp, fj.Cp, k, blockIdx.y);
        }
        return;
    }
    const int cq = blockIdx.y, n = fj.w ? blockIdx.z - 1 : blockIdx.z;
    const int rb = blockIdx.x / colBlocks, cb = blockIdx.x % colBlocks;
    const int ty0 = rb * TR, tx0 = cb * TC;
    const int rows = M * TR + 2;
    const int ldsW = M * TC + 2;          // even
    const int h0 = M * ty0 - pad, w0 = M * tx0 - pad;
    const int tid = threadIdx.x;

    const int per_ch = rows * ldsW;
    // Halo copy.  A unit is 64*VEC consecutive columns of one halo row; wave w takes
    // units w, w+4, ...  Loads are issued in batches of CV x MAXU before any of
    // them is written to LDS, so a wave keeps that many HBM requests in flight.
    // With VEC = 2 a lane loads the image-aligned pair (iw, iw+1), iw even.
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);     // wave-uniform: keeps the unit arithmetic on the scalar unit
    constexpr int MAXU = M == 4 ? 8 : 6;               // (6x6 tiles of 56 x 56 fp32 planes: 8 measured 66.7 against 70.1 us, 15 67.4)
    const int nunits = rows << chunkLog2;
    const int cmask = (1 << chunkLog2) - 1;
    const int wbase = VEC == 2 ? (w0 & ~1) : w0;       // first loaded image column (even for VEC = 2)
    // Every load is unconditional, from an address clamped into the image, and its bits are
    // ANDed with an all-ones / zero mask afterwards (zero padding, channel padding, units past
    // the halo): loads under a branch are waited for one by one.
    typedef typename std::conditional<sizeof(T) * VEC == 4, uint32_t, uint16_t>::type raw_t;
    typedef typename std::conditional<sizeof(T) == 4, uint32_t, uint16_t>::type elem_t;
    elem_t* smem_bits = reinterpret_cast<elem_t*>(in_smem_raw);
    auto copy_batch = [&](auto nb_c, int u0) {
        constexpr int NB = decltype(nb_c)::value;
        raw_t buf[CV][NB];
        unsigned keep[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int u = min(u0 + wv + 4 * i, nunits - 1);   // a unit past the halo repeats the last one (not stored)
            const int r = u >> chunkLog2;
            const int iw = wbase + (((u & cmask) << 6) + lane) * VEC;
            const int ih = h0 + r;
            // a pair is inside the image or outside it as a whole (W even, iw even)
            const bool ok = ih >= 0 && ih < H && iw >= 0 && iw < W;
            keep[i] = ok ? 0xFFFFFFFFu : 0u;
            const int ihc = min(max(ih, 0), H - 1), iwc = min(max(iw, 0), W - VEC);
#pragma unroll
            for (int ch = 0; ch < CV; ++ch) {
                const int c = min(cq * CV + ch, C - 1);
                buf[ch][i] = *reinterpret_cast<const raw_t*>(x + (((size_t)n * C + c) * H + ihc) * W + iwc);
            }
        }
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int u = u0 + wv + 4 * i;
            const int r = u >> chunkLog2;
            const int q0 = wbase - w0 + (((u & cmask) << 6) + lane) * VEC;   // LDS column of the first element
            if (u < nunits) {
#pragma unroll
                for (int ch = 0; ch < CV; ++ch) {
                    const unsigned m = cq * CV + ch < C ? keep[i] : 0u;
                    const unsigned bits = __float_as_uint(mask_keep(__uint_as_float((unsigned)buf[ch][i]), m));
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const int q = q0 + e;
                        if (q >= 0 && q < ldsW)
                            smem_bits[ch * per_ch + r * ldsW + q] = (elem_t)(bits >> (8 * sizeof(T) * e));
                    }
                }
            }
        }
    };
    int u0 = 0;
    for (; u0 + 4 * MAXU <= nunits; u0 += 4 * MAXU) copy_batch(std::integral_constant<int, MAXU>{}, u0);
    // the remainder in the smallest batch that holds it: a unit past the halo still costs its loads
    const int rem = nunits - u0;
    if (rem > 16) copy_batch(std::integral_constant<int, MAXU>{}, u0);
    else if (rem > 8) copy_batch(std::integral_constant<int, 4>{}, u0);
    else if (rem > 0) copy_batch(std::integral_constant<int, 2>{}, u0);
    __syncthreads();

    const int tr = tid / TC, tc = tid % TC;
    const int ty = ty0 + tr, tx = tx0 + tc;
    if (tr >= TR || ty >= th || tx >= tw) return;
    const long p = ((long)n * th + ty) * tw + tx;
    const size_t plane = (size_t)Cp * Pp;
    T* vp = V + ((size_t)cq * Pp + p) * CV;
    if constexpr (M == 4) {
        static_assert(M != 4 || sizeof(T) == 4, "the F(4x4) tiles of this kernel are fp32");
        tile_from_lds_store_f4(reinterpret_cast<const float*>(in_smem) + (4 * tr) * ldsW + 4 * tc, per_ch, ldsW,
                               reinterpret_cast<float*>(vp), plane);
    } else {
        tile_from_lds_store<T>(in_smem + (2 * tr) * ldsW + 2 * tc, per_ch, ldsW, vp, plane);
    }
}

// ---- input transform, NCHW source, small images -------------------------------------
// Images whose tiles do not fill a workgroup (th*tw <= 128): a workgroup takes one image and NQ = 256 / (th*tw)
// consecutive channel vectors.  Their channel planes are one contiguous run of the source, read word by word
// (VEC elements per 4-byte or 2-byte word, a row being W / VEC words) with consecutive lanes on consecutive words,
// and scattered into LDS planes [ch][2*th+2][2*tw+2] whose zero padding was written beforehand; thread
// (channel vector, tile) then builds its tile as in the tiled kernel.  A thread walks the run 256 words at a
// time; (stepC, stepH, stepW) is that stride split into planes, rows and words by the host, so the position of a
// word costs two compares instead of two divisions.  M as in the tiled kernel.
// QUAD (fp32): a row is W / 4 pieces of 16 bytes (W a multiple of 4, x 16-byte aligned, at most 16 pieces per thread:
// the host checks) and all of a thread's pieces are requested before the first is written to LDS -- a quarter of the
// load instructions and one round trip to memory instead of one per batch (N = 64, C = 512, 28 x 28 in F(4x4) tiles:
// 79 -> 72 us).
template <typename T, int VEC, int M = 2, bool QUAD = false>
__global__ __launch_bounds__(256) void input_transform_nchw_small_kernel(const T* __restrict__ x, T* __restrict__ V,
                                                                         int C, int H, int W, int pad, int th, int tw,
                                                                         long Pp, int Cp, int NQ, int groups,
                                                                         int in_blocks, int stepC, int stepH,
                                                                         int stepW, FilterJob fj) {
    constexpr int CV = ChanVec<T>::n;
    constexpr int NB = M == 4 ? 16 : 8;                // loads in flight per thread (fp32 28 x 28 planes: 16 measured 72 against 75 us)
    extern __shared__ __attribute__((aligned(16))) unsigned char in_smem_raw[];
    int bid = blockIdx.x;
    if constexpr (M == 4) {
        // the filter job's workgroups come first: they run beside the input's, not after them
        const int job_blocks = gridDim.x - in_blocks;
        if (bid < job_blocks) {
            const long id = (long)bid * 256 + threadIdx.x;
            if (id < (long)fj.Kp * (fj.Cp / CV))
                filter_transform_f4_thread<T>((const T*)fj.w, (T*)fj.U, fj.s, fj.K, fj.C, fj.Kp, fj.Cp, (int)(id % fj.Kp), (int)(id / fj.Kp));
            return;
        }
        bid -= job_blocks;
    } else if (fj.w && bid >= in_blocks) {
        filter_job_blocks<T, 256>(fj, in_blocks);
        return;
    }
    typedef typename std::conditional<sizeof(T) * VEC == 4, uint32_t, uint16_t>::type raw_t;
    typedef typename std::conditional<sizeof(T) == 4, uint32_t, uint16_t>::type elem_t;
    T* in_smem = reinterpret_cast<T*>(in_smem_raw);
    elem_t* smem_bits = reinterpret_cast<elem_t*>(in_smem_raw);
    const int tid = threadIdx.x;
    const int n = bid / groups, cq0 = (bid - n * groups) * NQ;
    const int nq = min(NQ, Cp / CV - cq0);             // channel vectors of this workgroup
    const int c0 = cq0 * CV;
    const int nch = max(min(nq * CV, C - c0), 0);      // channels that exist; the others stay zero
    const int rows = M * th + 2, ldsW = M * tw + 2, per_ch = rows * ldsW;
    const int Ww = W / VEC;
    const int words = nch * H * Ww;
    const raw_t* xw = reinterpret_cast<const raw_t*>(x + ((size_t)n * C + c0) * H * W);

    if constexpr (QUAD) {
        static_assert(!QUAD || (sizeof(T) == 4 && VEC == 1), "16-byte pieces of fp32 rows");
        constexpr int MAXP = 16;
        const int Wq = W / 4, pieces = nch * H * Wq;
        const uint4* xq = reinterpret_cast<const uint4*>(xw);
        uint4 buf4[MAXP];
#pragma unroll
        for (int i = 0; i < MAXP; ++i) buf4[i] = xq[min(tid + 256 * i, max(pieces - 1, 0))];
        {
            const int nvec = nq * CV * per_ch * (int)sizeof(T) / 16;   // per_ch is a multiple of 4 elements
            uint4* z = reinterpret_cast<uint4*>(in_smem_raw);
            for (int i = tid; i < nvec; i += 256) z[i] = make_uint4(0, 0, 0, 0);
        }
        __syncthreads();
        // piece -> (channel, row, piece of the row): divisions by multiplication, exact for the 4096 pieces at most
        const unsigned inv_row = (65536u + (unsigned)Wq - 1u) / (unsigned)Wq;
        const unsigned inv_pl = (0x1000000u + (unsigned)(H * Wq) - 1u) / (unsigned)(H * Wq);
#pragma unroll
        for (int i = 0; i < MAXP; ++i) {
            const int pi = tid + 256 * i;
            if (pi < pieces) {
                const int ch = (int)(((unsigned long long)pi * inv_pl) >> 24), rem = pi - ch * H * Wq;
                const int h = (int)(((unsigned)rem * inv_row) >> 16), wq = rem - h * Wq;
                elem_t* d = smem_bits + ch * per_ch + (h + pad) * ldsW + 4 * wq + pad;
                d[0] = buf4[i].x; d[1] = buf4[i].y; d[2] = buf4[i].z; d[3] = buf4[i].w;
            }
        }
        __syncthreads();
    } else {
        int idx = tid;
        int ch = tid / (H * Ww);
        int h = (tid - ch * H * Ww) / Ww;
        int w = tid - ch * H * Ww - h * Ww;
        raw_t buf[NB];
        int dst[NB];                                       // LDS element index of the word's first element, -1: past the run
        auto load_batch = [&]() {
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                buf[i] = xw[min(idx, words - 1)];          // always a valid address; a word past the run is not stored
                dst[i] = idx < words ? ch * per_ch + (h + pad) * ldsW + w * VEC + pad : -1;
                idx += 256;
                w += stepW;
                if (w >= Ww) { w -= Ww; ++h; }
                h += stepH;
                if (h >= H) { h -= H; ++ch; }
                ch += stepC;
            }
        };
        if (words > 0) load_batch();
        {
            const int nvec = nq * CV * per_ch * (int)sizeof(T) / 16;   // per_ch is a multiple of 4 elements
            uint4* z = reinterpret_cast<uint4*>(in_smem_raw);
            for (int i = tid; i < nvec; i += 256) z[i] = make_uint4(0, 0, 0, 0);
        }
        __syncthreads();
        for (int done = 0; done < words;) {
#pragma unroll
            for (int i = 0; i < NB; ++i)
                if (dst[i] >= 0) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) smem_bits[dst[i] + e] = (elem_t)(buf[i] >> (8 * sizeof(T) * e));
                }
            done += NB * 256;
            if (done < words) load_batch();
        }
        __syncthreads();
    }

    const int tiles = th * tw;
    const int q = tid / tiles, t = tid - q * tiles;
    if (q >= nq) return;
    const int ty = t / tw, tx = t - ty * tw;
    const long p = (long)n * tiles + t;
    T* vp = V + ((size_t)(cq0 + q) * Pp + p) * CV;
    if constexpr (M == 4) {
        static_assert(M != 4 || sizeof(T) == 4, "the F(4x4) tiles of this kernel are fp32");
        tile_from_lds_store_f4(reinterpret_cast<const float*>(in_smem) + q * CV * per_ch + (4 * ty) * ldsW + 4 * tx, per_ch, ldsW,
                               reinterpret_cast<float*>(vp), (size_t)Cp * Pp);
    } else {
        tile_from_lds_store<T>(in_smem + q * CV * per_ch + (2 * ty) * ldsW + 2 * tx, per_ch, ldsW, vp, (size_t)Cp * Pp);
    }
}

// ---- input transform, NHWC source, LDS-transposed ---------------------------------------
// Reads run along C (contiguous in NHWC), stores along p, so the block
// transposes through LDS.  A workgroup takes one image, TR tile rows, TC
// consecutive tx and NQ channel vectors (C % CV == 0, checked by the host):
// phase 1 copies the (2*TR+2) x (2*TC+2) pixel halo, 16 bytes per (pixel, cq)
// with cq fastest across lanes, all loads of a thread issued from clamped
// addresses before the first LDS write and masked afterwards (zero padding,
// channel padding); phase 2 gives thread (tile column, cq) its TR tiles one
// after the other, 16 pixels each as 16-byte LDS reads (even/odd columns kept
// apart so lanes walking tx read consecutive vectors), and stores 16 coalesced
// vectors of V per tile.
template <typename T, int TC, int NQ, int TR>
__global__ __launch_bounds__(TC * NQ) void input_transform_nhwc_kernel(const T* __restrict__ x, T* __restrict__ V,
                                                                       int N, int C, int H, int W, int pad, int th,
                                                                       int tw, long Pp, int Cp, int colBlocks,
                                                                       int rowBlocks, FilterJob fj, int in_blocks) {
    constexpr int CV = ChanVec<T>::n;
    if (fj.w && (int)blockIdx.x >= in_blocks) {
        filter_job_blocks<T, TC * NQ>(fj, in_blocks);
        return;
    }
    constexpr int HALF = TC + 1;                       // columns of one parity
    constexpr int ROWS = 2 * TR + 2, COLS = 2 * TC + 2;
    constexpr int NT = TC * NQ;
    constexpr int UNITS = ROWS * COLS * NQ;            // 16-byte vectors in the halo
    constexpr int NLOAD = (UNITS + NT - 1) / NT;
    __shared__ uint4 sm[NQ][ROWS][2][HALF];            // [cq][row][col parity][col/2]
    static_assert(sizeof(Pack16<T>) == sizeof(uint4), "vector size");
    const int cq0 = blockIdx.y * NQ;
    const int cb = blockIdx.x % colBlocks, rowid = blockIdx.x / colBlocks;
    const int rb = rowid % rowBlocks, n = rowid / rowBlocks;
    const int ty0 = rb * TR, tx0 = cb * TC;
    const int h0 = 2 * ty0 - pad, w0 = 2 * tx0 - pad;
    const int tid = threadIdx.x;
    const int CQ = Cp / CV, CQreal = C / CV;

    {
        uint4 buf[NLOAD];
        unsigned keep[NLOAD];
#pragma unroll
        for (int i = 0; i < NLOAD; ++i) {
            const int e = min(tid + i * NT, UNITS - 1);      // a unit past the halo repeats the last one (not stored)
            const int q = e % NQ, col = (e / NQ) % COLS, r = e / (NQ * COLS);
            const int ih = h0 + r, iw = w0 + col, cq = cq0 + q;
            keep[i] = (ih >= 0 && ih < H && iw >= 0 && iw < W && cq < CQreal) ? 0xFFFFFFFFu : 0u;
            const int ihc = min(max(ih, 0), H - 1), iwc = min(max(iw, 0), W - 1), cqc = min(cq, CQreal - 1);
            buf[i] = *reinterpret_cast<const uint4*>(x + (((size_t)n * H + ihc) * W + iwc) * C + cqc * CV);
        }
#pragma unroll
        for (int i = 0; i < NLOAD; ++i) {
            const int e = tid + i * NT;
            if (e < UNITS) {
                const int q = e % NQ, col = (e / NQ) % COLS, r = e / (NQ * COLS);
                uint4 v;
                v.x = __float_as_uint(mask_keep(__uint_as_float(buf[i].x), keep[i]));
                v.y = __float_as_uint(mask_keep(__uint_as_float(buf[i].y), keep[i]));
                v.z = __float_as_uint(mask_keep(__uint_as_float(buf[i].z), keep[i]));
                v.w = __float_as_uint(mask_keep(__uint_as_float(buf[i].w), keep[i]));
                sm[q][r][col & 1][col >> 1] = v;
            }
        }
    }
    __syncthreads();

    const int tc = tid % TC, q = tid / TC;
    const int tx = tx0 + tc, cq = cq0 + q;
    if (tx >= tw || cq >= CQ) return;
    const size_t plane = (size_t)Cp * Pp;
    for (int tr = 0; tr < TR; ++tr) {
        const int ty = ty0 + tr;
        if (ty >= th) break;
        float v[CV][16];
        {
            float d[CV][4][4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint4 raw = sm[q][2 * tr + i][j & 1][tc + (j >> 1)];
                    Pack16<T> pk;
                    __builtin_memcpy(&pk, &raw, sizeof(pk));
#pragma unroll
                    for (int e = 0; e < CV; ++e) d[e][i][j] = to_f32(pk.e[e]);
                }
#pragma unroll
            for (int e = 0; e < CV; ++e) input_tile_transform(d[e], v[e]);
        }
        const long p = ((long)n * th + ty) * tw + tx;
        T* vp = V + ((size_t)cq * Pp + p) * CV;
#pragma unroll
        for (int xi = 0; xi < 16; ++xi) {
            float o[CV];
#pragma unroll
            for (int e = 0; e < CV; ++e) o[e] = v[e][xi];
            store_chan_vec<T>(vp + xi * plane, o);
        }
    }
}

// ---- output transform, layout-generic ---------------------------------------------
// One thread per (tile p, filter k), p fastest: the 16 loads of a wave are
// contiguous runs of Mo[xi][k][.].  Stores go through the destination strides.
template <typename T>
__device__ __forceinline__ void output_tile_store(T* __restrict__ y, const ActStrides& s, int n, int k, int ty, int tx,
                                                  int Ho, int Wo, float (&o)[2][2], const Epilogue& ep) {
    const float bk = bias_of<T>(ep, k);
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            o[a][b] += bk;
            if (ep.relu) o[a][b] = fmaxf(o[a][b], 0.f);
        }
    if (ep.pool) {                               // s describes the pooled tensor; a window cut by the edge is dropped
        if (2 * ty + 1 < Ho && 2 * tx + 1 < Wo)
            y[n * s.n + k * s.c + ty * s.h + tx * s.w] = from_f32<T>(fmaxf(fmaxf(o[0][0], o[0][1]), fmaxf(o[1][0], o[1][1])));
        return;
    }
    T* yp = y + n * s.n + k * s.c;
    if (s.w == 1 && (Wo & 1) == 0 && (s.h & 1) == 0 && (s.c & 1) == 0 && (s.n & 1) == 0 &&
        (reinterpret_cast<uintptr_t>(y) & (2 * sizeof(T) - 1)) == 0) {
        // W-contiguous destination with even rows: the two outputs of a tile row go out as one store
        struct alignas(2 * sizeof(T)) Pair { T a, b; };
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            const int oh = 2 * ty + a;
            if (oh < Ho) {
                Pair pr{from_f32<T>(o[a][0]), from_f32<T>(o[a][1])};
                *reinterpret_cast<Pair*>(yp + oh * s.h + 2 * tx) = pr;
            }
        }
        return;
    }
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const int oh = 2 * ty + a, ow = 2 * tx + b;
            if (oh < Ho && ow < Wo) yp[oh * s.h + ow * s.w] = from_f32<T>(o[a][b]);
        }
}

template <typename T>
__global__ __launch_bounds__(256) void output_transform_generic_kernel(const float* __restrict__ Mo,
                                                                        T* __restrict__ y, ActStrides s, int N,
                                                                        int K, int Ho, int Wo, int th, int tw,
                                                                        long P, long Pp, int Kp, int order,
                                                                        Epilogue ep, int splits) {
    const long p = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const int k = blockIdx.y;
    if (p >= P || k >= K) return;
    const size_t plane = (size_t)Kp * Pp;
    const float* mp = Mo + (size_t)k * Pp + p;
    float m[16];
#pragma unroll
    for (int xi = 0; xi < 16; ++xi) m[xi] = mp[xi * plane];
    for (int sp = 1; sp < splits; ++sp)          // partial products of a reduction cut into runs, in a fixed order
#pragma unroll
        for (int xi = 0; xi < 16; ++xi) m[xi] += mp[((size_t)sp * 16 + xi) * plane];
    float o[2][2];
    output_tile_transform(m, o[0][0], o[0][1], o[1][0], o[1][1]);
    int n, ty, tx;
    decode_tile(p, order, N, th, tw, n, ty, tx);
    output_tile_store<T>(y, s, n, k, ty, tx, Ho, Wo, o, ep);
}

// ---- output transform from the K-contiguous product Mo[xi][Pp][Kp] ------------------------
// One thread per (filter k, tile p), k fastest: loads are contiguous along K and
// so are the stores of a K-contiguous destination (NHWC).
template <typename T>
__global__ __launch_bounds__(256) void output_transform_pk_kernel(const float* __restrict__ Mo, T* __restrict__ y,
                                                                   ActStrides s, int N, int K, int Ho, int Wo, int th,
                                                                   int tw, long P, long Pp, int Kp, int order,
                                                                   Epilogue ep, int splits) {
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    const long p = (long)blockIdx.y * blockDim.y + threadIdx.y;
    if (k >= K || p >= P) return;
    const size_t plane = (size_t)Kp * Pp;
    const float* mp = Mo + (size_t)p * Kp + k;
    float m[16];
#pragma unroll
    for (int xi = 0; xi < 16; ++xi) m[xi] = mp[xi * plane];
    for (int sp = 1; sp < splits; ++sp)
#pragma unroll
        for (int xi = 0; xi < 16; ++xi) m[xi] += mp[((size_t)sp * 16 + xi) * plane];
    float o[2][2];
    output_tile_transform(m, o[0][0], o[0][1], o[1][0], o[1][1]);
    int n, ty, tx;
    decode_tile(p, order, N, th, tw, n, ty, tx);
    output_tile_store<T>(y, s, n, k, ty, tx, Ho, Wo, o, ep);
}

// ---- plain layout permutation -------------------------------------------------------
// Walks the destination linearly (coalesced stores) and gathers from the source.
template <typename T>
__global__ __launch_bounds__(256) void permute_gather_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                              ActStrides a, int dst_layout, int N, int C, int H,
                                                              int W) {
    const long total = (long)N * C * H * W;
    long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    long n, c, h, w, r;
    switch (dst_layout) {
    case WINO_NHWC: c = e % C; r = e / C; w = r % W; r /= W; h = r % H; n = r / H; break;
    case WINO_CHWN: n = e % N; r = e / N; w = r % W; r /= W; h = r % H; c = r / H; break;
    default: w = e % W; r = e / W; h = r % H; r /= H; c = r % C; n = r / C; break;
    }
    out[e] = in[n * a.n + c * a.c + h * a.h + w * a.w];
}

// Layout permutation through an LDS tile: a tensor seen as [R][A][B] with the source contiguous along A and the
// destination contiguous along B (the six layout pairs all have this shape: e.g. NCHW -> NHWC is R = n,
// A = h*w, B = c).  A workgroup moves a TA x TB (A x B) tile of 4096 elements -- 64 x 64, or 32 x 128 / 128 x 32
// when one of the axes is the batch of 32 or fewer: lanes read along A, write along B, in runs of up to 512 bytes;
// the tile is padded by one column so that neither side has bank conflicts.
struct PermuteDims {
    long nA, nB, nR;          // extents
    long sB, sR;              // source strides of B and R (A has stride 1)
    long dA, dR;              // destination strides of A and R (B has stride 1)
};

template <typename T, int TA, int TB>
__global__ __launch_bounds__(256) void permute_tiled_kernel(const T* __restrict__ in, T* __restrict__ out, PermuteDims d,
                                                             int tilesA, int tilesB) {
    static_assert(TA * TB == 4096 && TA >= 32 && TB >= 32, "tile shape");
    __shared__ T tile[TB][TA + 1];
    long t = blockIdx.x;
    const int ta = (int)(t % tilesA);
    t /= tilesA;
    const int tb = (int)(t % tilesB);
    const long r = t / tilesB;
    const long a0 = (long)ta * TA, b0 = (long)tb * TB;
    const T* src = in + r * d.sR;
    T* dst = out + r * d.dR;
    {
        const int lx = threadIdx.x % TA, ly = threadIdx.x / TA;      // lanes along A
#pragma unroll 4
        for (int i = ly; i < TB; i += 256 / TA) {
            const long a = a0 + lx, b = b0 + i;
            if (a < d.nA && b < d.nB) tile[i][lx] = src[b * d.sB + a];
        }
    }
    __syncthreads();
    {
        const int lx = threadIdx.x % TB, ly = threadIdx.x / TB;      // lanes along B
#pragma unroll 4
        for (int i = ly; i < TA; i += 256 / TB) {
            const long a = a0 + i, b = b0 + lx;
            if (a < d.nA && b < d.nB) dst[a * d.dA + b] = tile[lx][i];
        }
    }
}

// The same for 2-byte elements, two at a time: lanes read 4-byte pairs along A and write 4-byte pairs along B
// (one element per lane moves 128 bytes per wave and instruction, half of what the fp32 kernel moves, and
// measured 3.1 TB/s against 5.4).  Needs even extents and strides, so that every pair is 4-byte aligned
// relative to the tensor; the tile holds 8192 elements (TA x TB = 128 x 64, 64 x 128, or 32 x 256 / 256 x 32).
template <int TA, int TB>
__global__ __launch_bounds__(256) void permute_tiled_pairs_kernel(const uint16_t* __restrict__ in,
                                                                   uint16_t* __restrict__ out, PermuteDims d,
                                                                   int tilesA, int tilesB) {
    static_assert(TA * TB == 8192 && TA >= 32 && TB >= 32, "tile shape");
    constexpr int PITCH = TA + 2;                                   // elements; rows stay 4-byte aligned
    __shared__ __attribute__((aligned(4))) uint16_t tile[TB * PITCH];
    long t = blockIdx.x;
    const int ta = (int)(t % tilesA);
    t /= tilesA;
    const int tb = (int)(t % tilesB);
    const long r = t / tilesB;
    const long a0 = (long)ta * TA, b0 = (long)tb * TB;
    const uint16_t* src = in + r * d.sR;
    uint16_t* dst = out + r * d.dR;
    {
        constexpr int LX = TA / 2;
        const int lx = threadIdx.x % LX, ly = threadIdx.x / LX;     // lanes along A, a pair each
#pragma unroll 4
        for (int i = ly; i < TB; i += 256 / LX) {
            const long a = a0 + 2 * lx, b = b0 + i;
            if (a < d.nA && b < d.nB)
                *reinterpret_cast<uint32_t*>(&tile[i * PITCH + 2 * lx]) =
                    *reinterpret_cast<const uint32_t*>(src + b * d.sB + a);
        }
    }
    __syncthreads();
    {
        constexpr int LX = TB / 2;
        const int lx = threadIdx.x % LX, ly = threadIdx.x / LX;     // lanes along B, a pair each
#pragma unroll 4
        for (int i = ly; i < TA; i += 256 / LX) {
            const long a = a0 + i, b = b0 + 2 * lx;
            if (a < d.nA && b < d.nB) {
                const uint32_t lo = tile[(2 * lx) * PITCH + i], hi = tile[(2 * lx + 1) * PITCH + i];
                *reinterpret_cast<uint32_t*>(dst + a * d.dA + b) = lo | hi << 16;
            }
        }
    }
}

}  // namespace wino
