// Direct 3x3 convolution of 2-byte tensors (f16 / bf16) as an implicit GEMM on the 16-bit matrix instruction,
// fp32 accumulation.  With 2-byte operands the Winograd pipelines are bound by memory on both sides of the
// transformed input (16*P*C elements written and read again for 2.25x fewer multiplies), while the direct product
//     y[k][q] = sum over (tap, c) of W[k][tap][c] * x[c][q + tap]
// reads x once and needs no transform at all: the 9 taps of a pixel are the same LDS tile read at 9 offsets.
// The stage replaced is the reference's batched GEMM (comparison/GEMM.cuh:124-253); the reference's own
// direct-convolution-in-a-tile kernel is Conv_fuse (fusedTest/winotrans.cuh:1868).
//
// A tile is 64 filters x a block of BR x BC output pixels (BR*BC <= 128*NPG, chosen by the host); a workgroup
// (4 waves) computes one tile after the other, a wave 64 filters x NPG groups of 32 pixels: 2 x NPG accumulators
// of v_mfma_f32_32x32x16, filters on the rows, pixels on the lanes, so a store instruction writes runs of y along w.  The channel reduction runs in
// stages of 16 channels (one k-step of the instruction per tap); per stage LDS holds
//     Fs[9 taps][2 channel vectors][64 filters]          16-byte vectors of 8 channels, from the packed bank
//     Xs[2 channel vectors][LR rows][PW pixel slots]     the block's input rows with halo, zero padding included
// in two buffers.  The packed filter bank W9[tap][Cp/8][Kp][8] travels HBM -> LDS directly
// (global_load_lds_dwordx4, as in gemm_rows_kernel); the input is NCHW, so 8 channels of a pixel are 8 different
// planes: a thread loads, for a pair of neighbouring columns, one 4-byte word from each of the 8 planes
// (coalesced along w), regroups them into the two pixels' channel vectors with 8 byte-permutes and writes two
// 16-byte vectors.  The loads of stage s+1 are issued before the multiplies of stage s and written to LDS after.
//
// The grid is persistent: two workgroups per CU, each walking its share of the tiles, and the stages of all its
// tiles form ONE pipeline -- the first stage of the next tile is requested during the last stage of the current
// one, so only the very first stage of a workgroup waits for memory, and a tile's stores are issued while the
// other workgroup of the CU multiplies.  Workgroup ids go round-robin to the 8 XCDs; the ids of an XCD take the
// filter tiles of one pixel block one after the other, so the block's input is fetched into that XCD's L2 once.
//
// Rows are "global" output rows g = n*Ho + oh, so a block may hold the last rows of one image and the first of
// the next (small images: 14x14 puts several images into one block); in LDS every image brings its own zero
// rows above and below (row slot = (n - n0)*(Ho + 2) + oh + r - oh0), so taps never read a neighbour's rows.
#pragma once
#include "common.hpp"
#include "gemm.hpp"

namespace wino {

constexpr int D16_FBYTES = 9 * 2 * 64 * 16;                   // filter stage: 18 KB
constexpr int D16_PLANE = 704;                                // pixel slots per channel-vector plane of a stage
constexpr int D16_BUF = D16_FBYTES + 2 * D16_PLANE * 16;      // 40 KB per buffer, two buffers, two workgroups per CU
constexpr int D16_KT = 64;                                    // filters per workgroup

struct D16Geom {
    int N, C, K, H, W, pad, Ho, Wo;
    int BR, BC;            // output rows x columns of a block
    int WC;                // (8-wave kernel) waves side by side in a block
    int ds;                // (8-wave kernel) pixel slots between the tap columns: 1, or N for CHWN tensors taken as one image of width W * N
    int PW, LR;            // LDS: pixel slots per row (BC + 2), rows (BR + 2 + 2 per image boundary a block can span)
    int PP;                // column pairs loaded per row
    int colBlocks, rowBlocks, kTiles;
    int maxcross;          // image boundaries a block can span
    int a4, b3;            // (8-wave kernel) b3 > 0: every image is a4 blocks whose waves own 4 rows and b3 blocks whose waves own 3
    int CQ, Kp;            // channel vectors (a multiple of 4) and padded filters of the packed bank
    long G;                // N * Ho output rows
};

// ---- 2x2 / stride-2 maximum of a tensor the direct kernels wrote unpooled ------------------------------------
// The 8-wave kernel pools in its stores where a window's columns sit in neighbouring lanes; in a CHWN tensor they are N
// elements apart, in different waves, and the kernels for layers of at most four channels do not pool.  Such a layer is
// convolved unpooled (bias and ReLU applied) into scratch and one of these kernels follows.
// max(round(v)) = round(max(v)): the same bits as a kernel that pooled before it rounded.
// [outer][Ho][Wo][inner] (CHWN: K, N; NHWC: N, K): a thread takes VEC inner elements of one window.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void pool2_inner_kernel(const T* __restrict__ t, T* __restrict__ y, int Ho, int Wo, int N,
                                                          long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int nv = N / VEC, Hp = Ho >> 1, Wp = Wo >> 1;
    const int n0 = (int)(i % nv) * VEC;
    long r = i / nv;
    const int pw = (int)(r % Wp);
    r /= Wp;
    const int ph = (int)(r % Hp);
    const long k = r / Hp;
    const T* src = t + ((k * Ho + 2 * ph) * Wo + 2 * pw) * (long)N + n0;
    struct alignas(VEC * sizeof(T)) Vec { T v[VEC]; };
    const Vec a = *reinterpret_cast<const Vec*>(src), b = *reinterpret_cast<const Vec*>(src + N);
    const Vec c = *reinterpret_cast<const Vec*>(src + (long)Wo * N), d = *reinterpret_cast<const Vec*>(src + (long)Wo * N + N);
    Vec o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) o.v[e] = from_f32<T>(fmaxf(fmaxf(to_f32(a.v[e]), to_f32(b.v[e])), fmaxf(to_f32(c.v[e]), to_f32(d.v[e]))));
    *reinterpret_cast<Vec*>(y + ((k * Hp + ph) * Wp + pw) * (long)N + n0) = o;
}
// [planes][Ho][Wo] (NCHW: N x K planes): a thread takes VEC neighbouring windows of a row pair, 2 VEC contiguous
// elements of each row (VEC > 1: Wo a multiple of 2 VEC and both tensors aligned to the pieces).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void pool2_rows_kernel(const T* __restrict__ t, T* __restrict__ y, int Ho, int Wo, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int Hp = Ho >> 1, Wp = Wo >> 1, wv = Wp / VEC;
    const int pw0 = (int)(i % wv) * VEC;
    long r = i / wv;
    const int ph = (int)(r % Hp);
    const long plane = r / Hp;
    const T* src = t + (plane * Ho + 2 * ph) * (long)Wo + 2 * pw0;
    struct alignas(2 * VEC * sizeof(T)) In { T v[2 * VEC]; };
    struct alignas(VEC * sizeof(T)) Out { T v[VEC]; };
    const In a = *reinterpret_cast<const In*>(src), b = *reinterpret_cast<const In*>(src + Wo);
    Out o;
#pragma unroll
    for (int e = 0; e < VEC; ++e)
        o.v[e] = from_f32<T>(fmaxf(fmaxf(to_f32(a.v[2 * e]), to_f32(a.v[2 * e + 1])), fmaxf(to_f32(b.v[2 * e]), to_f32(b.v[2 * e + 1]))));
    *reinterpret_cast<Out*>(y + (plane * Hp + ph) * (long)Wp + pw0) = o;
}

// ---- filter bank -> W9[tap][Cp/8][Kp][8] (zero padded) --------------------------------------------------
// One thread per (filter, channel vector).  VEC = 1: the bank is [K][C][3][3] with C a multiple of 8 and a 16-byte
// aligned base, so the 72 values of a thread are 144 contiguous, aligned bytes: nine 16-byte loads instead of 72
// two-byte ones a filter apart.  VEC = 2: [K][3][3][C], same conditions: a tap's 8 channels are one 16-byte load and
// go out as they are.
template <typename T, int VEC>
__global__ __launch_bounds__(64) void direct16_pack_kernel(const T* __restrict__ w, T* __restrict__ W9, FltStrides s,
                                                           int K, int C, int Kp, int CQ) {
    const int k = blockIdx.x * 64 + threadIdx.x, cq = blockIdx.y;
    if (k >= Kp) return;
    unsigned short raw[72];                                  // [channel of the vector][tap]
    const bool kin = k < K;
    if (VEC == 2) {
        const bool in = kin && cq * 8 < C;
        const uint4* src = reinterpret_cast<const uint4*>(w + (size_t)(kin ? k : K - 1) * 9 * C + (cq * 8 < C ? cq * 8 : 0));
        uint4 v[9];
#pragma unroll
        for (int t = 0; t < 9; ++t) v[t] = src[(size_t)t * (C / 8)];
#pragma unroll
        for (int t = 0; t < 9; ++t)
            *reinterpret_cast<uint4*>(W9 + (((size_t)t * CQ + cq) * Kp + k) * 8) = in ? v[t] : make_uint4(0, 0, 0, 0);
        return;
    }
    if (VEC == 1) {
        uint4 v[9];
        const uint4* src = reinterpret_cast<const uint4*>(w + ((size_t)(kin ? k : K - 1) * C + (cq * 8 < C ? cq * 8 : 0)) * 9);
#pragma unroll
        for (int i = 0; i < 9; ++i) v[i] = src[i];
        __builtin_memcpy(raw, v, sizeof(raw));
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int c = cq * 8 + e;
            const T* wp = w + (kin ? k : K - 1) * s.k + (c < C ? c : C - 1) * s.c;
#pragma unroll
            for (int t = 0; t < 9; ++t) {
                const T val = wp[(t / 3) * s.r + (t % 3) * s.s];
                __builtin_memcpy(&raw[e * 9 + t], &val, 2);
            }
        }
    }
#pragma unroll
    for (int t = 0; t < 9; ++t) {
        unsigned short pk[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) pk[e] = (kin && cq * 8 + e < C) ? raw[e * 9 + t] : (unsigned short)0;    // +0.0 in both formats
        uint4 out;
        __builtin_memcpy(&out, pk, 16);
        *reinterpret_cast<uint4*>(W9 + (((size_t)t * CQ + cq) * Kp + k) * 8) = out;
    }
}


// ROWS: the block is 16 rows x 32 columns (PW = 34), every wave owns 4 consecutive output rows of one image
// (the host offers it when Ho is a multiple of 4), so pixel group j, filter row r reads input row j + r of the
// wave's six: the pixel fragment of an input row is fetched once and multiplied into up to three groups --
// 18 pixel fragments per stage instead of 36.
template <typename T, int NPG, bool ROWS>
__global__ __launch_bounds__(256, 2) void direct16_kernel(const T* __restrict__ x, const T* __restrict__ W9,
                                                          T* __restrict__ y, D16Geom g, Epilogue ep) {
    typedef typename Mma<T>::vec vec;
    constexpr int NTASK = 3;
    extern __shared__ __attribute__((aligned(16))) unsigned char d16_smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int HW = g.H * g.W, Hp = g.Ho + 2;
    const int nst = g.CQ / 2;                               // stages of 16 channels per tile (even: Cp is a multiple of 32)

    // ---- this workgroup's tiles: sequence items s = s0, s0 + sstep, ... < send of its XCD ------------------
    const int xcd = blockIdx.x & 7;
    const int sstep = gridDim.x >> 3;
    const int npb = g.colBlocks * g.rowBlocks;              // pixel blocks; block pbx*8 + xcd belongs to this XCD
    const int send = ((npb - xcd + 7) >> 3) * g.kTiles;
    struct Tile {
        int k0, c0, n0, oh0;
    };
    auto decode = [&](int s) {
        const int pbx = s / g.kTiles, kt = s - pbx * g.kTiles;
        const int pb = pbx * 8 + xcd;
        const int rb = pb / g.colBlocks, cb = pb - rb * g.colBlocks;
        const long g0 = (long)rb * g.BR;
        const int n0 = (int)(g0 / g.Ho);
        return Tile{kt * D16_KT, cb * g.BC, n0, (int)(g0 - (long)n0 * g.Ho)};
    };

    // ---- input tasks of this thread: (channel vector v, LDS row, column pair); what does not depend on the tile ----
    const int ntask = 2 * g.LR * g.PP;
    int tpk[NTASK];                                         // LDS row | (first column of the pair relative to c0, + 8) << 12 | v << 20
    int ldsw[NTASK];                                        // LDS byte offset of the pair's first slot inside a buffer (a multiple of 16)
                                                            // | bit 0 / 1: slot 0 / 1 exists; < 0: no task
#pragma unroll
    for (int q = 0; q < NTASK; ++q) {
        const int t = tid + 256 * q;
        const int m = t % g.PP, rr = t / g.PP;
        const int lr = rr % g.LR, v = min(rr / g.LR, 1);
        const int slot0 = 2 * m - g.pad;                    // the pair (c0 + 2m - 2 pad, + 1) sits in slots (2m - pad, + 1)
        tpk[q] = lr | (2 * m - 2 * g.pad + 8) << 12 | v << 20;
        const int wr = (slot0 >= 0 && slot0 < g.PW ? 1 : 0) | (slot0 + 1 >= 0 && slot0 + 1 < g.PW ? 2 : 0);
        ldsw[q] = t < ntask ? (((v * D16_PLANE + lr * g.PW + slot0) * 16 + D16_FBYTES) | wr) : -1;
    }
    // ---- this lane's pixels inside a block ----------------------------------------------------------------
    int ppk[NPG];                                           // row << 8 | column
#pragma unroll
    for (int j = 0; j < NPG; ++j) {
        const int p = (wave * NPG + j) * 32 + l32;
        ppk[j] = (p / g.BC) << 8 | (p % g.BC);
    }
    const int rowb = g.PW * 16;                             // bytes between LDS rows

    // ---- the tile being loaded: offsets and masks of this thread's tasks, filter rows, channel base --------------
    unsigned xoff[NTASK];                                   // byte offset from (image n0, the stage's first channel), a multiple
                                                            // of 4 | bit 0: the pair lies inside the image
    constexpr int FROWS = 5;                                // 18 filter rows of 64 vectors per stage: wave w takes rows w, w + 4, ...
    uint64_t fptr = 0;                                      // row `wave` of the stage to request; row + 4 is two taps further
    const unsigned lane_off = lane * 16;
    const uint64_t fstep = (uint64_t)2 * g.Kp * 16, frow4 = (uint64_t)2 * g.CQ * g.Kp * 16;
    const char* xs = nullptr;                               // image n0, first channel of the stage to request
    const uint64_t xstep = (uint64_t)16 * HW * 2;
    const unsigned hw2 = (unsigned)(HW * 2);
    auto prep_load = [&](const Tile& t) {
#pragma unroll
        for (int q = 0; q < NTASK; ++q) {
            const int lr = tpk[q] & 0xFFF, v = tpk[q] >> 20;
            const int qq = t.oh0 + lr;                      // padded row index counted from image n0
            int dn = 0;
            for (int k = 1; k <= g.maxcross; ++k) dn += qq >= k * Hp ? 1 : 0;
            const int ih = qq - dn * Hp - g.pad;
            const int iw = t.c0 + ((tpk[q] >> 12) & 0xFF) - 8;
            const bool in = ldsw[q] >= 0 && t.n0 + dn < g.N && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
            const int ihc = min(max(ih, 0), g.H - 1), iwc = min(max(iw, 0), g.W - 2);
            const int dnc = min(dn, g.N - 1 - t.n0);
            xoff[q] = ((unsigned)((dnc * g.C * g.H + ihc) * g.W + iwc) * 2u + (unsigned)(v * 8 * HW * 2)) | (in ? 1u : 0u);
        }
        xs = reinterpret_cast<const char*>(x) + (size_t)t.n0 * g.C * HW * 2;
        fptr = reinterpret_cast<uint64_t>(W9 + (((size_t)(wave >> 1) * g.CQ + (wave & 1)) * g.Kp + t.k0) * 8);
    };
    auto f_load = [&](auto bufc) {
        constexpr int B = decltype(bufc)::value;
        uint64_t fp = fptr;
#pragma unroll
        for (int q = 0; q < FROWS; ++q) {
            const int row = wave + 4 * q;
            if (row < 18) dma_row(fp, lane_off, d16_smem + B * D16_BUF + row * 1024);
            fp += frow4;
        }
        fptr += fstep;
    };
    uint32_t raw[NTASK][8];
    // A stage's second channel vector may lie past C: the first one is loaded instead, and masked.  So may the whole
    // stage (the bank is padded to 32 channels, C is a multiple of 8: C = 8, 40, 72, ...): the first stage's channels
    // are loaded then -- xs has moved on by cs stages -- so that no address leaves the tensor.
    auto stage_base = [&](int cs) { return cs * 16 < g.C ? xs : xs - (size_t)cs * xstep; };
    auto x_load = [&](int cs) {
        const char* const xb = stage_base(cs);
#pragma unroll
        for (int q = 0; q < NTASK; ++q) {
            const int v = tpk[q] >> 20;
            const bool vok = cs * 16 + v * 8 < g.C;
            unsigned off = (xoff[q] & ~3u) - (vok ? 0u : (unsigned)v * 8u * hw2);
#pragma unroll
            for (int e = 0; e < 8; ++e) {     // a scalar base and a 32-bit offset per load
                raw[q][e] = *reinterpret_cast<const uint32_t*>(xb + off);
                off += hw2;
            }
        }
        xs += xstep;
    };
    // The same requests one at a time, for issuing between the multiplies of a stage: piece 0..4 a filter row,
    // piece 5 + 8q + e channel e of task q.  (A wave that issues its ~30 requests in one go sits in the issue
    // queue for as long as the multiplies of half a stage take.)
    unsigned poff[NTASK];
    auto load_piece = [&](auto bufc, int idx, int cs) {
        constexpr int B = decltype(bufc)::value;
        if (idx < FROWS) {
            const int row = wave + 4 * idx;
            if (row < 18) dma_row(fptr + (uint64_t)idx * frow4, lane_off, d16_smem + B * D16_BUF + row * 1024);
        } else if (idx < FROWS + 8 * NTASK) {
            const int q = (idx - FROWS) >> 3, e = (idx - FROWS) & 7;
            if (e == 0) {
                const int v = tpk[q] >> 20;
                const bool vok = cs * 16 + v * 8 < g.C;
                poff[q] = (xoff[q] & ~3u) - (vok ? 0u : (unsigned)v * 8u * hw2);
            }
            raw[q][e] = *reinterpret_cast<const uint32_t*>(stage_base(cs) + poff[q]);
            poff[q] += hw2;
        }
    };
    auto loads_done = [&]() {
        fptr += fstep;
        xs += xstep;
    };
    auto x_commit = [&](auto bufc, int cs) {                // cs: the stage x_load was called with
        constexpr int B = decltype(bufc)::value;
#pragma unroll
        for (int q = 0; q < NTASK; ++q) {
            if (ldsw[q] < 0) continue;
            const bool keep = (xoff[q] & 1u) && cs * 16 + (tpk[q] >> 20) * 8 < g.C;
            const uint32_t km = keep ? 0xFFFFFFFFu : 0u;
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t a = raw[q][2 * e] & km, b = raw[q][2 * e + 1] & km;
                lo[e] = __builtin_amdgcn_perm(b, a, 0x05040100u);     // (a.lo16, b.lo16): the pair's first pixel
                hi[e] = __builtin_amdgcn_perm(b, a, 0x07060302u);     // (a.hi16, b.hi16): its second pixel
            }
            unsigned char* dst = d16_smem + B * D16_BUF + (ldsw[q] & ~15);
            if (ldsw[q] & 1) *reinterpret_cast<uint4*>(dst) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            if (ldsw[q] & 2) *reinterpret_cast<uint4*>(dst + 16) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        }
    };

    // ---- the tile being multiplied: LDS address of tap (0, 0) per 32-pixel group, where its outputs go ----------
    int xaddr[NPG];
    int yoff[NPG];                                          // element offset of (n, k0, oh, ow) in y, < 0: no pixel
    int k0c = 0;
    auto prep_pix = [&](const Tile& t) {
        k0c = t.k0;
        const long g0 = (long)t.n0 * g.Ho + t.oh0;
#pragma unroll
        for (int j = 0; j < NPG; ++j) {
            const int prow = ppk[j] >> 8, pcol = ppk[j] & 0xFF;
            const bool ok = prow < g.BR && g0 + prow < g.G && t.c0 + pcol < g.Wo;
            const int prc = ok ? prow : 0, pcc = ok ? pcol : 0;
            const int ohp = t.oh0 + prc;
            int dn = 0;
            for (int k = 1; k <= g.maxcross; ++k) dn += ohp >= k * g.Ho ? 1 : 0;
            const int oh = ohp - dn * g.Ho;
            const int L = dn * Hp + oh - t.oh0;
            xaddr[j] = ((lh * D16_PLANE) + L * g.PW + pcc) * 16 + D16_FBYTES;
            yoff[j] = ok ? (int)((((long)(t.n0 + dn) * g.K + t.k0) * g.Ho + oh) * g.Wo + t.c0 + pcc) : -1;
        }
    };

    floatx16 acc[2][NPG];
    // ---- one stage of multiplies: 9 taps x (2 filter fragments x NPG pixel fragments) ----------------------
    // more: the next stage's requests go out between this stage's multiplies (wave-uniform)
    auto compute = [&](auto bufc, auto firstc, bool more, int cs_next) {
        constexpr int B = decltype(bufc)::value;
        typedef std::integral_constant<int, 1 - B> otherbuf_t;
        constexpr bool FIRST = decltype(firstc)::value;     // the tile's first stage starts from zero accumulators
        const unsigned char* fs = d16_smem + B * D16_BUF + (lh * 64 + l32) * 16;
        const unsigned char* xsb = d16_smem + B * D16_BUF;
        if constexpr (ROWS) {
            static_assert(!ROWS || NPG == 4, "four rows per wave");
            constexpr int RB = 34 * 16;                     // bytes between LDS rows
            const unsigned char* xw = xsb + xaddr[0];       // the wave's first input row, this lane's column
            // 18 steps (filter column s, input row rho), each one pixel fragment and 2 to 6 multiplies.  The order
            // is pinned: the pixel fragment of step t+2 and the filter fragments that the following steps need are
            // requested before the multiplies of step t (a wave's LDS latency is covered by its own multiplies only
            // if the requests are already out), filter row r of the next column as soon as its last use has issued.
            vec a[3][2], b[3];
            auto lda = [&](int r, int s) {
#pragma unroll
                for (int i = 0; i < 2; ++i) a[r][i] = *reinterpret_cast<const vec*>(fs + (3 * r + s) * 2048 + i * 512);
            };
            auto ldb = [&](int t) { b[t % 3] = *reinterpret_cast<const vec*>(xw + (t % 6) * RB + (t / 6) * 16); };
            lda(0, 0);
            ldb(0);
            lda(1, 0);
            ldb(1);
            lda(2, 0);
#pragma unroll
            for (int t = 0; t < 18; ++t) {
                const int s = t / 6, rho = t % 6;
                if (more) {
                    constexpr int NPIECE = FROWS + 8 * NTASK;        // 29 over 18 steps: two per step, then one
                    const int first = t < 11 ? 2 * t : 22 + (t - 11);
                    load_piece(otherbuf_t{}, first, cs_next);
                    if (t < 11) load_piece(otherbuf_t{}, first + 1, cs_next);
                    static_assert(NPIECE == 29, "pieces per stage");
                }
                if (t + 2 < 18) ldb(t + 2);
                if (rho == 4 && s < 2) lda(0, s + 1);
                if (rho == 5 && s < 2) lda(1, s + 1);
                if (rho == 0 && s > 0) lda(2, s);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int r = rho - j;
                    if (r < 0 || r > 2) continue;
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        if (FIRST && s == 0 && r == 0) {
#pragma unroll
                            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
                        }
                        Mma<T>::run(a[r][i], b[t % 3], acc[i][j]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (more) loads_done();
            return;
        }
        if (more) {
            f_load(otherbuf_t{});
            x_load(cs_next);
        }
#pragma unroll
        for (int tap = 0; tap < 9; ++tap) {
            const int r = tap / 3, s = tap % 3;
            vec a[2], b[NPG];
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = *reinterpret_cast<const vec*>(fs + tap * 2048 + i * 512);
#pragma unroll
            for (int j = 0; j < NPG; ++j) b[j] = *reinterpret_cast<const vec*>(xsb + xaddr[j] + r * rowb + s * 16);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < NPG; ++j) {
                    if (FIRST && tap == 0) {
#pragma unroll
                        for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
                    }
                    Mma<T>::run(a[i], b[j], acc[i][j]);
                }
        }
    };

    // ---- stores: register r of acc[i][j] is filter k0 + 32*i + 8*(r/4) + 4*lh + r%4, the lane's pixel of group j ----
    // Offsets into y are 32-bit element offsets (the host checks the tensor size) that run along with the filter
    // index: from one register pair to the next the filter advances by 2 or by 6.
    const unsigned kstride = (unsigned)(g.Ho * g.Wo);
    // W-contiguous rows of even length from an aligned base: two neighbouring lanes hold neighbouring columns, and
    // exchange values so that each stores one 4-byte pair -- the even lane for filter r, the odd lane for filter r+1
    const bool pairs = (g.Wo & 1) == 0 && (reinterpret_cast<uintptr_t>(y) & 3) == 0;
    const bool odd = lane & 1;
    // KFULL: no filter of the tile lies past K (no per-store test); a lane without a pixel (yoff < 0) sits the
    // whole group out, and so does its pair partner: both columns of a pair exist or neither
    auto stores_t = [&](auto kfullc) {
        constexpr bool KFULL = decltype(kfullc)::value;
        const int kfirst = 4 * lh + ((pairs && odd) ? 1 : 0);
#pragma unroll
        for (int j = 0; j < NPG; ++j) {
            if (yoff[j] < 0) continue;
            unsigned o = (unsigned)yoff[j] + (unsigned)kfirst * kstride - ((pairs && odd) ? 1u : 0u);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int r2 = 0; r2 < 16; r2 += 2) {
                    const int kk = 32 * i + 8 * (r2 >> 2) + 4 * lh + (r2 & 3);     // filter of register r2; r2 + 1: the next one
                    float v0 = acc[i][j][r2], v1 = acc[i][j][r2 + 1];
                    if (ep.bias) {
                        v0 += bias_of<T>(ep, KFULL ? k0c + kk : min(k0c + kk, g.K - 1));
                        v1 += bias_of<T>(ep, KFULL ? k0c + kk + 1 : min(k0c + kk + 1, g.K - 1));
                    }
                    if (ep.relu) { v0 = fmaxf(v0, 0.f); v1 = fmaxf(v1, 0.f); }
                    if (pairs) {
                        const float got = swap_lane_pairs(odd ? v0 : v1);
                        const float lo = odd ? got : v0, hi = odd ? v1 : got;
                        struct alignas(4) Pair { T a, b; };
                        if (KFULL || k0c + kk + (odd ? 1 : 0) < g.K)
                            *reinterpret_cast<Pair*>(y + o) = Pair{from_f32<T>(lo), from_f32<T>(hi)};
                    } else {
                        if (KFULL || k0c + kk < g.K) y[o] = from_f32<T>(v0);
                        if (KFULL || k0c + kk + 1 < g.K) y[o + kstride] = from_f32<T>(v1);
                    }
                    o += ((r2 & 2) ? 6u : 2u) * kstride;
                    __builtin_amdgcn_sched_barrier(0);   // one register pair at a time: nothing of the next pair is hoisted up here
                }
        }
    };
    auto stores = [&]() {
        if (k0c + D16_KT <= g.K) stores_t(std::true_type{});      // wave-uniform
        else stores_t(std::false_type{});
    };

    typedef std::integral_constant<int, 0> b0_t;
    typedef std::integral_constant<int, 1> b1_t;
    int s_ld = (int)(blockIdx.x >> 3), ld_cs = 0;           // the stage to request next: (sequence item, stage)
    if (s_ld >= send) return;
    bool ld_valid = true;
    prep_load(decode(s_ld));
    f_load(b0_t{});
    x_load(0);
    x_commit(b0_t{}, 0);
    ld_cs = 1;
    auto stage = [&](auto bufc, auto firstc) {
        constexpr int B = decltype(bufc)::value;
        typedef std::integral_constant<int, 1 - B> other_t;
        __builtin_amdgcn_s_waitcnt(0x0070);              // vmcnt(0) lgkmcnt(0): this wave's share of the stage is in LDS
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        compute(bufc, firstc, ld_valid, ld_cs);
        if (ld_valid) {
            x_commit(other_t{}, ld_cs);
            if (++ld_cs == nst) {                        // on to the next tile of this workgroup, if there is one
                ld_cs = 0;
                s_ld += sstep;
                ld_valid = s_ld < send;
                if (ld_valid) prep_load(decode(s_ld));
            }
        }
    };
    for (int s = (int)(blockIdx.x >> 3); s < send; s += sstep) {
        prep_pix(decode(s));
        stage(b0_t{}, std::true_type{});
        stage(b1_t{}, std::false_type{});
        for (int cs = 2; cs < nst; cs += 2) {
            stage(b0_t{}, std::false_type{});
            stage(b1_t{}, std::false_type{});
        }
        stores();
    }
}

}  // namespace wino
