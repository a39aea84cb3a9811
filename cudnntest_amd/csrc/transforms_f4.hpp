// Winograd F(4x4,3x3) transform kernels -- the reference's own tile size
// (6x6 input tiles, 36 coordinates, 4x4 outputs per tile):
//   comparison/wrapedConv_NCHW.cuh:836-855 (B^T d B), :879-899 (G g G^T), :1084-1101 (A^T m A)
//
//   B^T = [ 4  0 -5  0 1 0 ]   G = [ 1/4    0     0  ]   A^T = [ 1 1  1 1  1 0 ]
//         [ 0 -4 -4  1 1 0 ]       [-1/6  -1/6  -1/6 ]         [ 0 1 -1 2 -2 0 ]
//         [ 0  4 -4 -1 1 0 ]       [-1/6   1/6  -1/6 ]         [ 0 1  1 4  4 0 ]
//         [ 0 -2 -1  2 1 0 ]       [ 1/24  1/12  1/6 ]         [ 0 1 -1 8 -8 1 ]
//         [ 0  2 -1 -2 1 0 ]       [ 1/24 -1/12  1/6 ]
//         [ 0  4  0 -5 0 1 ]       [ 0     0     1   ]
//
// Operand layouts are those of the F(2x2) path with 36 coordinates instead of 16:
//   U[36][Cp/CV][Kp][CV]   V[36][Cp/CV][Pp][CV]   Mo[36][Kp][Pp] (or [36][Pp][Kp])
// with th = ceil(Ho/4), tw = ceil(Wo/4), P = N*th*tw.
#pragma once
#include "common.hpp"

namespace wino {

__device__ __forceinline__ void bt6(const float d[6], float o[6]) {
    o[0] = 4.f * d[0] - 5.f * d[2] + d[4];
    o[1] = -4.f * (d[1] + d[2]) + d[3] + d[4];
    o[2] = 4.f * (d[1] - d[2]) - d[3] + d[4];
    o[3] = -2.f * d[1] - d[2] + 2.f * d[3] + d[4];
    o[4] = 2.f * d[1] - d[2] - 2.f * d[3] + d[4];
    o[5] = 4.f * d[1] - 5.f * d[3] + d[5];
}

// v (36, row-major 6x6) = B^T d B
__device__ __forceinline__ void input_tile_transform_f4(const float d[6][6], float* v) {
    float t[6][6];
#pragma unroll
    for (int j = 0; j < 6; ++j) {
        float col[6], o[6];
#pragma unroll
        for (int i = 0; i < 6; ++i) col[i] = d[i][j];
        bt6(col, o);
#pragma unroll
        for (int i = 0; i < 6; ++i) t[i][j] = o[i];
    }
#pragma unroll
    for (int i = 0; i < 6; ++i) bt6(t[i], v + 6 * i);
}

__device__ __forceinline__ void g6(float g0, float g1, float g2, float o[6]) {
    o[0] = 0.25f * g0;
    o[1] = (-g0 - g1 - g2) * (1.f / 6.f);
    o[2] = (-g0 + g1 - g2) * (1.f / 6.f);
    o[3] = g0 * (1.f / 24.f) + g1 * (1.f / 12.f) + g2 * (1.f / 6.f);
    o[4] = g0 * (1.f / 24.f) - g1 * (1.f / 12.f) + g2 * (1.f / 6.f);
    o[5] = g2;
}

// u (36) = G g G^T
__device__ __forceinline__ void filter_tile_transform_f4(const float g[3][3], float* u) {
    float t[6][3];
#pragma unroll
    for (int s = 0; s < 3; ++s) {
        float o[6];
        g6(g[0][s], g[1][s], g[2][s], o);
#pragma unroll
        for (int i = 0; i < 6; ++i) t[i][s] = o[i];
    }
#pragma unroll
    for (int i = 0; i < 6; ++i) g6(t[i][0], t[i][1], t[i][2], u + 6 * i);
}

__device__ __forceinline__ void at6(const float m[6], float o[4]) {
    o[0] = m[0] + m[1] + m[2] + m[3] + m[4];
    o[1] = m[1] - m[2] + 2.f * (m[3] - m[4]);
    o[2] = m[1] + m[2] + 4.f * (m[3] + m[4]);
    o[3] = m[1] - m[2] + 8.f * (m[3] - m[4]) + m[5];
}

// y (4x4) = A^T m A
__device__ __forceinline__ void output_tile_transform_f4(const float m[36], float y[4][4]) {
    float t[4][6];
#pragma unroll
    for (int j = 0; j < 6; ++j) {
        float col[6], o[4];
#pragma unroll
        for (int i = 0; i < 6; ++i) col[i] = m[6 * i + j];
        at6(col, o);
#pragma unroll
        for (int a = 0; a < 4; ++a) t[a][j] = o[a];
    }
#pragma unroll
    for (int a = 0; a < 4; ++a) at6(t[a], y[a]);
}

// ---- filter transform: thread per (filter k, channel vector), k fastest -----------------------------------
// The CV channels of a vector one after the other (36 live values each), their results gathered into one
// 16-byte store per coordinate: a wave writes 1 KB runs of U.
template <typename T>
__device__ __forceinline__ void filter_transform_f4_thread(const T* __restrict__ w, T* __restrict__ U, const FltStrides& s, int K,
                                                           int C, int Kp, int Cp, int k, int cq) {
    constexpr int CV = ChanVec<T>::n;
    T out[36][CV];
    float g[CV][3][3];
    filter_taps_load<T>(w, s, K, C, k, cq, g);                // 16-byte loads where the bank's layout has them
#pragma unroll
    for (int e = 0; e < CV; ++e) {
        float u[36];
        filter_tile_transform_f4(g[e], u);
#pragma unroll
        for (int xi = 0; xi < 36; ++xi) out[xi][e] = from_f32<T>(u[xi]);
    }
    const size_t plane = (size_t)Cp * Kp;
    T* up = U + ((size_t)cq * Kp + k) * CV;
#pragma unroll
    for (int xi = 0; xi < 36; ++xi) {
        uint4 v;
        __builtin_memcpy(&v, out[xi], 16);
        *reinterpret_cast<uint4*>(up + xi * plane) = v;
    }
}

template <typename T>
__global__ __launch_bounds__(64) void filter_transform_f4_kernel(const T* __restrict__ w, T* __restrict__ U,
                                                                  FltStrides s, int K, int C, int Kp, int Cp) {
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k < Kp) filter_transform_f4_thread<T>(w, U, s, K, C, Kp, Cp, k, blockIdx.y);
}

// A whole-layer call gives the filter bank's transform to the input transform's launch (the FilterJob of the
// F(2x2) kernels): one more z-slice of its grid -- slice 0, which is dispatched first, so the job runs beside the
// input's workgroups and not after them -- whose workgroups share the Kp x Cp/CV threads of the job, filters
// fastest, and leave at once when there is none left for them.
template <typename T>
__device__ __forceinline__ void filter_job_f4(const FilterJob& fj) {
    constexpr int CV = ChanVec<T>::n;
    const long id = ((long)blockIdx.y * gridDim.x + blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= (long)fj.Kp * (fj.Cp / CV)) return;
    filter_transform_f4_thread<T>((const T*)fj.w, (T*)fj.U, fj.s, fj.K, fj.C, fj.Kp, fj.Cp, (int)(id % fj.Kp), (int)(id / fj.Kp));
}

// ---- input transform, fp32 NCHW source: the tiled kernel of transforms.hpp with M = 4 ------------------------------
// Its second phase: the 6x6 pixels of one tile for the 4 channels of a vector, from LDS planes [ch][rows][ldsW]
// (`base`: the tile's first pixel in the first plane, at an even column: 8-byte reads), to 36 vectors of V.
__device__ __forceinline__ void tile_from_lds_store_f4(const float* base, int per_ch, int ldsW, float* vp, size_t plane) {
    float v[4][36];
#pragma unroll
    for (int ch = 0; ch < 4; ++ch) {
        float d[6][6];
#pragma unroll
        for (int i = 0; i < 6; ++i)
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const float2 a = *reinterpret_cast<const float2*>(base + ch * per_ch + i * ldsW + 2 * j);
                d[i][2 * j] = a.x;
                d[i][2 * j + 1] = a.y;
            }
        input_tile_transform_f4(d, v[ch]);
    }
#pragma unroll
    for (int xi = 0; xi < 36; ++xi)
        *reinterpret_cast<float4*>(vp + xi * plane) = make_float4(v[0][xi], v[1][xi], v[2][xi], v[3][xi]);
}

// ---- input transform, layout-generic -------------------------------------------------------
// Thread per (channel-in-vector e, tile p, channel vector cq) with e fastest: the CV lanes of
// one tile write the CV elements of one 16-byte vector, so a wave's store is one contiguous
// run of V.  One channel per thread keeps the 36 + 36 live values in registers.  Loads go to
// clamped addresses and are masked afterwards (all 36 in flight together).
template <typename T>
__global__ __launch_bounds__(256) void input_transform_f4_generic_kernel(const T* __restrict__ x, T* __restrict__ V,
                                                                          ActStrides s, int N, int C, int H, int W,
                                                                          int pad, int th, int tw, long P, long Pp,
                                                                          int Cp, int order, FilterJob fj) {
    constexpr int CV = ChanVec<T>::n;
    if (gridDim.z == 2 && blockIdx.z == 0) {                 // dispatched first: the job runs under the input's workgroups
        filter_job_f4<T>(fj);
        return;
    }
    const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const int e = (int)(gid % CV);
    const long p = gid / CV;
    const int cq = blockIdx.y;
    if (p >= P) return;
    const int c = cq * CV + e;
    int n, ty, tx;
    decode_tile(p, order, N, th, tw, n, ty, tx);
    const int h0 = 4 * ty - pad, w0 = 4 * tx - pad;
    long roff[6], coff[6];
    unsigned rkeep[6], ckeep[6];
#pragma unroll
    for (int i = 0; i < 6; ++i) {
        const int ih = h0 + i, iw = w0 + i;
        rkeep[i] = (ih >= 0 && ih < H) ? 0xffffffffu : 0u;
        ckeep[i] = (iw >= 0 && iw < W) ? 0xffffffffu : 0u;
        roff[i] = (long)(ih < 0 ? 0 : (ih >= H ? H - 1 : ih)) * s.h;
        coff[i] = (long)(iw < 0 ? 0 : (iw >= W ? W - 1 : iw)) * s.w;
    }
    const unsigned chkeep = c < C ? 0xffffffffu : 0u;
    const T* xp = x + n * s.n + (c < C ? c : C - 1) * s.c;
    float d[6][6], v[36];
#pragma unroll
    for (int i = 0; i < 6; ++i)
#pragma unroll
        for (int j = 0; j < 6; ++j) d[i][j] = mask_keep(to_f32(xp[roff[i] + coff[j]]), rkeep[i] & ckeep[j] & chkeep);
    input_tile_transform_f4(d, v);
    const size_t plane = (size_t)Cp * Pp;
    T* vp = V + ((size_t)cq * Pp + p) * CV + e;
#pragma unroll
    for (int xi = 0; xi < 36; ++xi) vp[xi * plane] = from_f32<T>(v[xi]);
}

// ---- input transform, fp32, tiles in batch-minor order (CHWN sources) ------------------------------------------
// Thread per (tile, channel vector): the four channels of the vector one after the other (36 loads in flight each
// time), then 36 stores of 16 bytes.  With the batch fastest along the lanes a load instruction reads 256 contiguous
// bytes of a pixel row of x and a store writes 1 KB of a coordinate plane -- a quarter of the memory instructions of
// the thread-per-channel kernel above, which is what a CU runs out of first there (N = 32, C = 256, 56 x 56 from
// CHWN: 72 against 85 us).  Byte offsets inside a channel plane of x and inside a coordinate plane of V are 32-bit
// (the host checks).
__global__ __launch_bounds__(256) void input_transform_f4_vec_kernel(const float* __restrict__ x, float* __restrict__ V,
                                                                      ActStrides s, int N, int C, int H, int W, int pad,
                                                                      int th, int tw, long P, long Pp, int Cp, int order,
                                                                      FilterJob fj) {
    if (gridDim.z == 2 && blockIdx.z == 0) {                 // dispatched first: the job runs under the input's workgroups
        filter_job_f4<float>(fj);
        return;
    }
    const long p = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const int cq = blockIdx.y;
    if (p >= P) return;
    int n, ty, tx;
    decode_tile(p, order, N, th, tw, n, ty, tx);
    const int h0 = 4 * ty - pad, w0 = 4 * tx - pad;
    unsigned roff[6], coff[6], rkeep[6], ckeep[6];
#pragma unroll
    for (int i = 0; i < 6; ++i) {
        const int ih = h0 + i, iw = w0 + i;
        rkeep[i] = (ih >= 0 && ih < H) ? 0xffffffffu : 0u;
        ckeep[i] = (iw >= 0 && iw < W) ? 0xffffffffu : 0u;
        roff[i] = (unsigned)((ih < 0 ? 0 : (ih >= H ? H - 1 : ih)) * s.h) * 4u;
        coff[i] = (unsigned)((iw < 0 ? 0 : (iw >= W ? W - 1 : iw)) * s.w + n * s.n) * 4u;
    }
    float v[4][36];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int c = cq * 4 + e;
        const unsigned chkeep = c < C ? 0xffffffffu : 0u;
        const char* xp = reinterpret_cast<const char*>(x) + (size_t)(c < C ? c : C - 1) * s.c * sizeof(float);   // uniform
        float raw[6][6], d[6][6];
#pragma unroll
        for (int i = 0; i < 6; ++i)
#pragma unroll
            for (int j = 0; j < 6; ++j) raw[i][j] = *reinterpret_cast<const float*>(xp + (roff[i] + coff[j]));
#pragma unroll
        for (int i = 0; i < 6; ++i)
#pragma unroll
            for (int j = 0; j < 6; ++j) d[i][j] = mask_keep(raw[i][j], rkeep[i] & ckeep[j] & chkeep);
        input_tile_transform_f4(d, v[e]);
    }
    const size_t plane_bytes = (size_t)Cp * Pp * sizeof(float);
    char* vb = reinterpret_cast<char*>(V) + (size_t)cq * Pp * 16;
    const unsigned voff = (unsigned)p * 16u;
#pragma unroll
    for (int xi = 0; xi < 36; ++xi) {
        *reinterpret_cast<float4*>(vb + voff) = make_float4(v[0][xi], v[1][xi], v[2][xi], v[3][xi]);
        vb += plane_bytes;
    }
}

// ---- input transform, fp32 NHWC source, batch-major tiles: a row of tiles staged in LDS ------------------------
// In NHWC the channels of a pixel are contiguous and the pixels of a tile are not: a thread per (tile, channel)
// gathers 4-byte pieces 4 pixels apart.  Here a workgroup takes one image, one tile row, a block of at most 14 tile
// columns and CC channels: the 6 x (4*tiles + 2) pixels it needs are loaded 16 bytes per lane, CC/4 lanes per pixel
// (every load unconditional from a clamped address and masked afterwards -- all of a lane's loads issued
// before the first mask, under a branch that is uniform for the workgroup: with the loads inside a per-lane branch
// the compiler waits for each one before it issues the next, 91 against 73 us on N = 32, C = 256, 56 x 56), and
// stored to LDS with a pixel pitch of CC + 1 words.  Then one thread per (channel of a vector,
// tile, channel vector), channel fastest as in the layout-generic kernel: its 36 LDS reads hit distinct banks across
// the wave (bank = 4*tile + channel + const), and the 4 lanes of a vector and the 16 tiles of a wave write 256
// contiguous bytes of each coordinate plane of V.
// Blocks of 16 channels (64-byte pieces of a pixel, 24 KB of LDS, six workgroups to a CU) against 32 and 8, one run,
// N = 32, C = 256, 56 x 56: 71 us against 75.5 and 79.
constexpr int F4N_CC = 16, F4N_TCB = 14;
template <int CC>
__global__ __launch_bounds__(256) void input_transform_f4_nhwc_kernel(const float* __restrict__ x, float* __restrict__ V,
                                                                       int N, int C, int H, int W, int pad, int th,
                                                                       int tw, long Pp, int Cp, int colBlocks, FilterJob fj) {
    constexpr int PITCH = CC + 1, L = CC / 4, PP = 256 / L, NQ = (6 * (4 * F4N_TCB + 2) + PP - 1) / PP;   // lanes of a pixel, pixels of a pass, passes
    __shared__ float sm[6 * (4 * F4N_TCB + 2) * PITCH];
    const int zjob = gridDim.z - N;                          // 1 with a filter job: slice 0, dispatched first
    if (zjob && blockIdx.z == 0) {
        filter_job_f4<float>(fj);
        return;
    }
    const int tid = threadIdx.x;
    // Workgroup ids go round-robin to the 8 XCDs, each with an L2 of its own.  Re-dealt so that an XCD takes a
    // contiguous eighth of the (image, channel block, tile row) sequence: neighbouring tile rows share two of their
    // six pixel rows, and their 224-byte runs of a coordinate plane of V lie next to each other.
    int bx = blockIdx.x, by = blockIdx.y, n = blockIdx.z - zjob;
    {
        const unsigned total = gridDim.x * gridDim.y * (unsigned)N;
        if ((total & 7u) == 0) {
            const unsigned lin = bx + gridDim.x * (by + gridDim.y * (unsigned)n);
            const unsigned re = (lin & 7u) * (total >> 3) + (lin >> 3);
            bx = re % gridDim.x;
            by = (re / gridDim.x) % gridDim.y;
            n = re / (gridDim.x * gridDim.y);
        }
    }
    const int ty = bx / colBlocks, cb = bx - ty * colBlocks;
    const int c0 = by * CC;
    const int tx0 = cb * F4N_TCB, ntx = min(F4N_TCB, tw - tx0);
    const int wlb = 4 * ntx + 2;                             // pixel columns of the block
    const int h0 = 4 * ty - pad, w0 = 4 * tx0 - pad;
    // ---- pixels -> LDS
    const int npix = 6 * wlb;                                // <= 348: NQ passes of PP pixels at most
    const int ch4 = tid & (L - 1), pl = tid / L;             // 16-byte piece of the CC channels; pixel of a pass
    const unsigned inv_wlb = (65536u + (unsigned)wlb - 1u) / (unsigned)wlb;      // pix / wlb = pix * inv_wlb >> 16 for pix < 348
    const char* const xn = reinterpret_cast<const char*>(x) + (size_t)n * H * W * C * sizeof(float);   // the image (uniform)
    const int c = c0 + 4 * ch4;
    const bool vec = (C & 3) == 0 && c0 + CC <= C;         // uniform: every lane of the workgroup loads 16 bytes
    float4 raw[NQ];
    unsigned keep[NQ];
    if (vec) {
        // (all loads first, unconditionally, from clamped addresses; the masks afterwards: the loads are in flight together)
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int pix = min(pl + PP * q, npix - 1);
            const int r = (int)(((unsigned)pix * inv_wlb) >> 16), col = pix - r * wlb;
            const int ih = h0 + r, iw = w0 + col;
            const bool ok = ih >= 0 && ih < H && iw >= 0 && iw < W;
            const int ihc = min(max(ih, 0), H - 1), iwc = min(max(iw, 0), W - 1);
            keep[q] = ok ? 0xFFFFFFFFu : 0u;
            const unsigned off = (unsigned)((ihc * W + iwc) * C + c) * 4u;       // byte offset in the image (< 2^32: the host checks)
            raw[q] = *reinterpret_cast<const float4*>(xn + off);
        }
#pragma unroll
        for (int q = 0; q < NQ; ++q)
            raw[q] = make_float4(mask_keep(raw[q].x, keep[q]), mask_keep(raw[q].y, keep[q]), mask_keep(raw[q].z, keep[q]), mask_keep(raw[q].w, keep[q]));
    } else {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int pix = min(pl + PP * q, npix - 1);
            const int r = (int)(((unsigned)pix * inv_wlb) >> 16), col = pix - r * wlb;
            const int ih = h0 + r, iw = w0 + col;
            const bool ok = ih >= 0 && ih < H && iw >= 0 && iw < W;
            const int ihc = min(max(ih, 0), H - 1), iwc = min(max(iw, 0), W - 1);
            const unsigned kp = ok ? 0xFFFFFFFFu : 0u;
            const unsigned off = (unsigned)((ihc * W + iwc) * C) * 4u;
            float e[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) e[k] = mask_keep(*reinterpret_cast<const float*>(xn + (off + (unsigned)min(c + k, C - 1) * 4u)), c + k < C ? kp : 0u);
            raw[q] = make_float4(e[0], e[1], e[2], e[3]);
        }
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        const int pix = pl + PP * q;
        if (pix < npix) {
            float* d = sm + pix * PITCH + 4 * ch4;
            d[0] = raw[q].x; d[1] = raw[q].y; d[2] = raw[q].z; d[3] = raw[q].w;
        }
    }
    __syncthreads();
    // ---- tiles
    const size_t vplane_bytes = (size_t)Cp * Pp * sizeof(float);
    const int nvec = min(CC, Cp - c0) / 4;               // channel vectors of this workgroup (Cp is a multiple of 16)
    const long p0 = ((long)n * th + ty) * tw + tx0;
    const unsigned inv_ntx = (65536u + (unsigned)ntx - 1u) / (unsigned)ntx;
    // a thread's 36 stores: a uniform plane base that moves on by a plane, and one 32-bit offset (a plane is < 2^32 bytes)
    char* const vbase = reinterpret_cast<char*>(V) + ((size_t)(c0 / 4) * Pp + p0) * 16;
    for (int idx = tid; idx < nvec * ntx * 4; idx += 256) {
        const int e = idx & 3, it = idx >> 2;
        const int ql = (int)(((unsigned)it * inv_ntx) >> 16), t = it - ql * ntx;
        const float* src = sm + (4 * t) * PITCH + 4 * ql + e;
        float d[6][6], v[36];
#pragma unroll
        for (int i = 0; i < 6; ++i) {
            const float* row = src + i * wlb * PITCH;
#pragma unroll
            for (int j = 0; j < 6; ++j) d[i][j] = row[j * PITCH];
        }
        input_tile_transform_f4(d, v);
        const unsigned voff = (unsigned)(((size_t)ql * Pp + t) * 16 + e * 4);
        char* vb = vbase;
#pragma unroll
        for (int xi = 0; xi < 36; ++xi) {
            *reinterpret_cast<float*>(vb + voff) = v[xi];
            vb += vplane_bytes;
        }
    }
}

// The 4x4 outputs o of tile (n, ty, tx) and filter k on their way out: bias, ReLU, 2x2 max pooling (s then describes
// the pooled tensor, Ho/2 x Wo/2, a tile gives 2x2 pooled values and a window cut by the border is dropped), stores --
// one 4-element store per output row where the destination is W-contiguous with rows a multiple of 4 wide.
template <typename T>
__device__ __forceinline__ void store_tile_f4(T* __restrict__ y, const ActStrides& s, int n, int k, int ty, int tx, int Ho,
                                              int Wo, float (&o)[4][4], const Epilogue& ep, float bv) {
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            o[a][b] += bv;
            if (ep.relu) o[a][b] = fmaxf(o[a][b], 0.f);
        }
    T* yp = y + n * s.n + k * s.c;
    if (ep.pool) {
        const int Hq = Ho / 2, Wq = Wo / 2;
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const int ph = 2 * ty + a, pw = 2 * tx + b;
                const float v = fmaxf(fmaxf(o[2 * a][2 * b], o[2 * a][2 * b + 1]), fmaxf(o[2 * a + 1][2 * b], o[2 * a + 1][2 * b + 1]));
                if (ph < Hq && pw < Wq) yp[ph * s.h + pw * s.w] = from_f32<T>(v);
            }
        return;
    }
    if (s.w == 1 && (Wo & 3) == 0 && (s.h & 3) == 0 && (s.c & 3) == 0 && (s.n & 3) == 0 &&
        (reinterpret_cast<uintptr_t>(y) & (4 * sizeof(T) - 1)) == 0) {
        // W-contiguous destination, rows a multiple of 4 wide: one 4-element store per output row
        struct alignas(4 * sizeof(T)) Quad { T e[4]; };
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int oh = 4 * ty + a;
            if (oh < Ho) {
                Quad q;
#pragma unroll
                for (int b = 0; b < 4; ++b) q.e[b] = from_f32<T>(o[a][b]);
                *reinterpret_cast<Quad*>(yp + oh * s.h + 4 * tx) = q;
            }
        }
        return;
    }
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int oh = 4 * ty + a, ow = 4 * tx + b;
            if (oh < Ho && ow < Wo) yp[oh * s.h + ow * s.w] = from_f32<T>(o[a][b]);
        }
}

// ---- output transform ------------------------------------------------------------------------------
// PK = false: Mo[36][Kp][Pp], thread per (tile p, filter k), p fastest
// PK = true : Mo[36][Pp][Kp], thread per (filter k, tile p), k fastest
// Bias, ReLU and 2x2 max pooling as in the F(2x2) output stage: with pooling, s describes the pooled tensor
// (Ho/2 x Wo/2) and a tile gives 2x2 pooled values; a window cut by the border is dropped.
template <typename T, bool PK>
__global__ __launch_bounds__(256) void output_transform_f4_kernel(const float* __restrict__ Mo, T* __restrict__ y,
                                                                   ActStrides s, int N, int K, int Ho, int Wo, int th,
                                                                   int tw, long P, long Pp, int Kp, int order,
                                                                   Epilogue ep) {
    long p;
    int k;
    if (PK) {
        k = blockIdx.x * blockDim.x + threadIdx.x;
        p = (long)blockIdx.y * blockDim.y + threadIdx.y;
    } else {
        p = (long)blockIdx.x * blockDim.x + threadIdx.x;
        k = blockIdx.y;
    }
    if (p >= P || k >= K) return;
    const size_t plane = (size_t)Kp * Pp;
    const float* mp = PK ? Mo + (size_t)p * Kp + k : Mo + (size_t)k * Pp + p;
    float m[36];
#pragma unroll
    for (int xi = 0; xi < 36; ++xi) m[xi] = mp[xi * plane];
    float o[4][4];
    output_tile_transform_f4(m, o);
    int n, ty, tx;
    decode_tile(p, order, N, th, tw, n, ty, tx);
    store_tile_f4<T>(y, s, n, k, ty, tx, Ho, Wo, o, ep, bias_of<T>(ep, k));
}

}  // namespace wino
