// Single-kernel Winograd F(2x2,3x3) convolution: input transform, 16-coordinate
// multiply-accumulate over channels and output transform in one launch, with no
// transformed-input or product tensor in HBM.  The structure of the reference's
// fusedTest/winotrans.cuh:1452 (Winofuse4433): per channel slab, half of the
// work is "load a raw input patch, transform it in registers, scatter to LDS",
// the other half "copy the pre-transformed filter slab to LDS", then the
// accumulators advance, and A^T(.)A runs on the accumulators -- here for 4x4
// tiles, all three layouts, zero padding, any C and K, on MFMA.
#pragma once
#include "gemm.hpp"

namespace wino {

// =============================================================================
// The kernel has the row-at-a-time structure of gemm_rows_kernel: a workgroup
// owns 64 filters x 64 tiles, keeps the 4 coordinates of ONE row i of the 4x4
// coordinate grid resident, folds the row into the output tile when its channel
// reduction ends, and is small enough (one wave ~ 240 registers, 32-64 KB of
// LDS) for two workgroups to share a CU.  The filter rows of a stage travel
// HBM -> LDS directly, as in gemm_rows_kernel; the tile rows are built here.
//
// Row i of V = B^T d B needs only two rows of the raw patch:
//     (B^T d)_i = d_ra + sg * d_rb,   (ra, rb, sg) = (0,2,-), (1,2,+), (2,1,-), (1,3,-)
// followed by the column transform.  Per stage (NC = NV*CV channels of one row) a
// thread owns one tile and UN = NC/4 consecutive channels, requests their 2 x 4 raw
// values at the start of the stage before, transforms them during that stage's last
// MFMA runs, and writes the four coordinates as one UN-element chunk each.  (Register
// loads that stay in flight across a wait on direct-to-LDS loads gain nothing: while
// such a load is pending the compiler turns every vmcnt wait into vmcnt(0).)  The raw input is read four times in total (once per row), from
// L2 after the first.
//
// How a thread reads its 2 x 4 x UN raw values (the load path, not HBM, bounds this kernel):
//   XM_SCALAR  one element per load, any strides; lanes walk tiles (coalesced for CHWN)
//   XM_CHANVEC channels contiguous (NHWC) and C % UN == 0: the UN channels of a position are
//              one load, and 4 neighbouring lanes cover the NC channels of a position
//   XM_ROW     columns contiguous (NCHW) and W >= 4: the 4 columns of a patch row are one
//              load that starts at a column clamped into [0, W-4]; lanes of edge tiles pick
//              their columns out of the shifted quadruple
// =============================================================================
enum { XM_SCALAR = 0, XM_CHANVEC = 1, XM_ROW = 2 };

// b in the lanes whose bit is set in the lane mask m, a in the others.  Opaque to the optimiser on
// purpose: written with ?: on a per-lane index, the compiler turns the column shuffle of XM_ROW into
// an indexed array in scratch memory.
__device__ __forceinline__ float lane_select(float a, float b, unsigned long m) {
    float r;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "s"(m));
    return r;
}

template <typename T> struct alignas(sizeof(T)) Quad { T v[4]; };

template <typename T, bool SWAP, int XM, int NVG>
__global__ __launch_bounds__(256, 2) void fused_rows_kernel(const T* __restrict__ x, const T* __restrict__ U,
                                                            T* __restrict__ y, ActStrides xs, ActStrides ys, int N,
                                                            int C, int K, int H, int W, int pad, int Ho, int Wo,
                                                            int th, int tw, long P, int Cp, int Kp, int order,
                                                            Epilogue ep, int kTiles, int pTiles, int xcd_map) {
    typedef typename Mma<T>::vec vec;
    constexpr int CV = ChanVec<T>::n;
    constexpr int NV = 2 * NVG;                // channel vectors per stage and coordinate
    constexpr int NC = NV * CV;                // channels per stage
    constexpr int UN = NC / 4;                 // channels per thread (64 tiles x NC channels over 256 threads)
    static_assert(CV % UN == 0, "a thread's channels must lie inside one channel vector");
    typedef typename std::conditional<UN * sizeof(T) == 16, uint4, uint2>::type chunk_t;   // UN channels
    static_assert(sizeof(chunk_t) == UN * sizeof(T), "chunk size");
    constexpr int VPAD = XM == XM_CHANVEC ? 2 : 0;   // V rows padded where lanes walk channel vectors first
    __shared__ vec Us0[4][NV][GO_T], Us1[4][NV][GO_T];
    __shared__ vec Vs0[4][NV][GO_T + VPAD], Vs1[4][NV][GO_T + VPAD];

    const int b = blockIdx.x;
    // Workgroup ids go round-robin to the 8 XCDs.  The ids of one XCD walk the filter tiles of a
    // tile patch first (they share its raw input), then CONSECUTIVE tile patches: neighbouring
    // patches are neighbouring tile rows, whose raw input rows overlap, and an XCD has its own L2.
    // (With few tile patches that order would leave XCDs idle: the host then asks for the plain one.)
    const int xcd = xcd_map ? b & 7 : 0, jb = xcd_map ? b >> 3 : b;
    const int ktile = jb % kTiles;
    const int ptile = xcd * ((pTiles + 7) / 8) + jb / kTiles;
    if (ptile >= pTiles) return;
    const int k0 = ktile * GO_T;
    const long p0 = (long)ptile * GO_T;
    const int CQ = Cp / CV;
    const int nst = CQ / NV;                   // stages per row (even)
    const vec* Ug = reinterpret_cast<const vec*>(U);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform, so addresses built from it stay on the scalar unit
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;

    // ---- this thread's tile and channels: fixed for the whole kernel --------------------
    const int tile = XM == XM_CHANVEC ? tid >> 2 : tid & 63;
    const int ch0 = (XM == XM_CHANVEC ? tid & 3 : wave) * UN;       // first of its UN channels inside a stage (wave-uniform unless XM_CHANVEC)
    unsigned u_col[4];                         // XM_ROW: [0] = offset of the clamped first column; else the 4 clamped columns
    unsigned cw[4];                            // all ones when column j of the patch lies inside the image (and the tile exists)
    unsigned img_off;                          // element offset of the tile's image
    int ih0;                                   // image row of patch row 0
    int dcol = 0;                              // XM_ROW: patch column j is element j + dcol of the loaded quadruple
    {
        const long p = p0 + tile;
        int n = 0, ty = 0, tx = 0;
        const bool pvalid = p < P;
        if (pvalid) decode_tile(p, order, N, th, tw, n, ty, tx);
        img_off = (unsigned)(n * xs.n);
        ih0 = 2 * ty - pad;
        const int iw0 = 2 * tx - pad;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int iw = iw0 + i;
            cw[i] = (pvalid && iw >= 0 && iw < W) ? 0xFFFFFFFFu : 0u;
            const int iwc = iw < 0 ? 0 : (iw >= W ? W - 1 : iw);     // clamped: the load stays inside x, the
            u_col[i] = (unsigned)(iwc * xs.w);                       // value is discarded through the masks
        }
        if (XM == XM_ROW) {
            // The quadruple starts at column iw0 even where that lies outside the row: the elements it
            // then takes from the neighbouring row are zeroed through cw.  Only where it could leave
            // the TENSOR (first image at its left edge, last image at its right edge) is it moved
            // inside the row, and the columns are put back in place with lane selects.
            const bool fix = (n == 0 && iw0 < 0) || (n == N - 1 && iw0 + 3 > W - 1);
            const int s0 = fix ? min(max(iw0, 0), W - 4) : iw0;
            dcol = iw0 - s0;                   // fix lanes: -1 at the left edge, 1 or 2 at the right edge; else 0
            u_col[0] = (unsigned)s0;
        }
    }
    // lane masks of the edge tiles (wave-uniform 64-bit values, fixed for the whole kernel)
    const unsigned long laneL = __ballot(dcol == -1), laneR1 = __ballot(dcol == 1), laneR2 = __ballot(dcol == 2);
    const bool any_fix = (laneL | laneR1 | laneR2) != 0;     // wave-uniform; false for all but a few waves of the grid

    floatx16 acc[4];
    floatx16 yo[4];                            // y00, y01, y10, y11
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc[j][r] = 0.f; yo[j][r] = 0.f; }

    typedef std::integral_constant<int, 0> par0_t;
    typedef std::integral_constant<int, 1> par1_t;

    // ---- raw rows ra, rb of the patch for the next stage -----------------------------------
    // x_prep fixes the stage to request (offsets, masks, sign); x_load_unit / x_load_all issue the
    // loads; v_unit turns the staged values of one channel into row i of B^T d B; v_write stores
    // the four coordinates into stage S of V.
    // DEEP (2-byte operands): a stage's MFMAs are too short to cover the latency of the raw rows requested at its
    // head, and a stage took as long as a trip to memory.  There the raw rows are requested TWO stages ahead, into
    // two register sets that alternate with the stage parity, and the filter rows travel through registers (with a
    // direct-to-LDS load pending the compiler would wait for every load in flight, the newest raw rows included).
    constexpr bool DEEP = sizeof(T) == 2 && XM != XM_CHANVEC;   // (channel-vector loads: two k-groups per stage measured faster, and both do not fit the registers)
    constexpr int NSET = DEEP ? 2 : 1;
    typedef std::integral_constant<int, 0> set0_t;
    typedef std::integral_constant<int, 1> set1_t;
    // The raw values stay as loaded (packed quadruples / channel chunks) until v_unit takes them apart: split at
    // the load, the unpacking of 2-byte elements would sit right behind the load and wait for it.
    T xa[XM == XM_SCALAR ? NSET : 1][4][UN], xb[XM == XM_SCALAR ? NSET : 1][4][UN];   // XM_SCALAR: [set][column][channel]
    Quad<T> qa_[XM == XM_ROW ? NSET : 1][UN], qb_[XM == XM_ROW ? NSET : 1][UN];        // XM_ROW: [set][channel], 4 columns each
    chunk_t ca_[XM == XM_CHANVEC ? NSET : 1][4], cb_[XM == XM_CHANVEC ? NSET : 1][4];  // XM_CHANVEC: [set][column], UN channels each
    unsigned ma_c[NSET], mb_c[NSET], cok_c[NSET];   // all ones when patch row ra / rb lies inside the image; bit u: channel u is real
    float sg_c[NSET];
    unsigned ma_n = 0, mb_n = 0, cok_n, ra_off = 0, rb_off = 0;
    float sg_n = 0.f;
    int c_n;
    auto x_prep = [&](int row_i, int st) {
        if (st == 0) {                             // the raw rows, their masks and the sign change with the Winograd row only
            const int ra = row_i == 0 ? 0 : (row_i == 2 ? 2 : 1);
            const int rb = row_i < 2 ? 2 : (row_i == 2 ? 1 : 3);
            const int iha = ih0 + ra, ihb = ih0 + rb;
            ma_n = (iha >= 0 && iha < H) ? 0xFFFFFFFFu : 0u;
            mb_n = (ihb >= 0 && ihb < H) ? 0xFFFFFFFFu : 0u;
            ra_off = img_off + (unsigned)(min(max(iha, 0), H - 1) * xs.h);
            rb_off = img_off + (unsigned)(min(max(ihb, 0), H - 1) * xs.h);
            if (XM == XM_ROW) {                    // byte offsets of the two quadruples inside a channel plane
                ra_off = (ra_off + u_col[0]) * (unsigned)sizeof(T);
                rb_off = (rb_off + u_col[0]) * (unsigned)sizeof(T);
            }
            sg_n = row_i == 1 ? 1.f : -1.f;
        }
        c_n = st * NC + ch0;
        cok_n = 0;
#pragma unroll
        for (int u = 0; u < UN; ++u) cok_n |= (c_n + u < C) ? 1u << u : 0u;
    };
    auto x_load_unit = [&](auto set, int u) {  // XM_SCALAR, XM_ROW
        constexpr int Q = decltype(set)::value;
        const unsigned coff = ((cok_n >> u) & 1u) ? (unsigned)((c_n + u) * xs.c) : 0u;
        if (XM == XM_ROW) {
            // channel plane: a wave-uniform (scalar) base; the lane adds its 32-bit byte offset
            const char* plane = reinterpret_cast<const char*>(x) + (size_t)coff * sizeof(T);
            qa_[XM == XM_ROW ? Q : 0][u] = *reinterpret_cast<const Quad<T>*>(plane + ra_off);
            qb_[XM == XM_ROW ? Q : 0][u] = *reinterpret_cast<const Quad<T>*>(plane + rb_off);
        } else {
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                xa[XM == XM_SCALAR ? Q : 0][jj][u] = x[ra_off + coff + u_col[jj]];
                xb[XM == XM_SCALAR ? Q : 0][jj][u] = x[rb_off + coff + u_col[jj]];
            }
        }
    };
    auto x_load_all = [&](auto set) {          // XM_CHANVEC: C % UN == 0, all UN channels real or none
        constexpr int Q = decltype(set)::value;
        const unsigned coff = cok_n ? (unsigned)c_n : 0u;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            ca_[XM == XM_CHANVEC ? Q : 0][jj] = *reinterpret_cast<const chunk_t*>(x + (ra_off + coff + u_col[jj]));
            cb_[XM == XM_CHANVEC ? Q : 0][jj] = *reinterpret_cast<const chunk_t*>(x + (rb_off + coff + u_col[jj]));
        }
    };
    auto take_next = [&](auto set) {
        constexpr int Q = decltype(set)::value;
        ma_c[Q] = ma_n; mb_c[Q] = mb_n; cok_c[Q] = cok_n; sg_c[Q] = sg_n;
    };
    T out[4][UN];
    auto v_unit = [&](auto set, int u) {
        constexpr int Q = decltype(set)::value;
        const bool ok = (cok_c[Q] >> u) & 1u;
        const unsigned mau = ok ? ma_c[Q] : 0u, mbu = ok ? mb_c[Q] : 0u;
        float da[4], db[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if constexpr (XM == XM_ROW) {
                da[q] = to_f32(qa_[Q][u].v[q]);
                db[q] = to_f32(qb_[Q][u].v[q]);
            } else if constexpr (XM == XM_CHANVEC) {
                T ea[UN], eb[UN];
                __builtin_memcpy(ea, &ca_[Q][q], sizeof(chunk_t));
                __builtin_memcpy(eb, &cb_[Q][q], sizeof(chunk_t));
                da[q] = to_f32(ea[u]);
                db[q] = to_f32(eb[u]);
            } else {
                da[q] = to_f32(xa[Q][q][u]);
                db[q] = to_f32(xb[Q][q][u]);
            }
        }
        if (XM == XM_ROW) {
            // patch column j = element j + dcol of the quadruple; elements that fall outside it are
            // columns outside the image, zeroed by cw below
            auto pick = [&](float (&d)[4]) {
                const float e0 = lane_select(lane_select(d[0], d[2], laneR2), d[1], laneR1);
                const float e1 = lane_select(lane_select(lane_select(d[1], d[3], laneR2), d[2], laneR1), d[0], laneL);
                const float e2 = lane_select(lane_select(d[2], d[3], laneR1), d[1], laneL);
                const float e3 = lane_select(d[3], d[2], laneL);
                d[0] = e0; d[1] = e1; d[2] = e2; d[3] = e3;
            };
            if (any_fix) {
                pick(da);
                pick(db);
            }
        }
        float r[4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
            r[jj] = mask_keep(fmaf(sg_c[Q], mask_keep(db[jj], mbu), mask_keep(da[jj], mau)), cw[jj]);
        out[0][u] = from_f32<T>(r[0] - r[2]);
        out[1][u] = from_f32<T>(r[1] + r[2]);
        out[2][u] = from_f32<T>(r[2] - r[1]);
        out[3][u] = from_f32<T>(r[1] - r[3]);
    };
    auto v_write = [&](auto par) {
        constexpr int S = decltype(par)::value;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            T* dst = reinterpret_cast<T*>(S ? &Vs1[j][ch0 / CV][tile] : &Vs0[j][ch0 / CV][tile]);
            chunk_t ck;
            __builtin_memcpy(&ck, out[j], sizeof(chunk_t));
            *reinterpret_cast<chunk_t*>(dst + ch0 % CV) = ck;
        }
    };
    // Building the next stage of V is cut into pieces that ride between the MFMA runs of the
    // current stage (two workgroups of a CU run in lockstep, so VALU work that is not interleaved
    // with a wave's own MFMAs does not overlap anybody's): pieces 0 .. WP-1 each transform UPP
    // channels and request their values for the stage after; piece WP writes the stage.
    constexpr int NR = 4 * NVG;                // MFMA runs per stage
    constexpr int UPP = (UN + NR - 2) / (NR - 1);
    constexpr int WP = (UN + UPP - 1) / UPP;
    static_assert(WP < NR, "pieces must fit the runs");
    auto v_piece = [&](auto par, auto set, int piece) {     // set: the raw rows to transform; par: the stage of V they become
        if (piece < WP) {
#pragma unroll
            for (int u = piece * UPP; u < (piece + 1) * UPP && u < UN; ++u) v_unit(set, u);
        } else if (piece == WP) {
            v_write(par);
        }
    };
    auto x_load_stage = [&](auto set, int row_i, int st) {
        x_prep(row_i, st);
        take_next(set);
        if (XM == XM_CHANVEC) x_load_all(set);
        else {
#pragma unroll
            for (int u = 0; u < UN; ++u) x_load_unit(set, u);
        }
    };
    // ---- the filter rows of a stage: 4*NV rows of 64 vectors, wave w issues rows w, w+4, ... --
    // one running scalar address per row slot, as in gemm_rows_kernel; u_load requests the stage
    // (ni, nstg) and moves the addresses to the one after it
    const unsigned lane_off = lane * 16;
    uint64_t uptr[NV];
    const uint64_t stepU = (uint64_t)NV * Kp * 16, wrapU = (uint64_t)(NV + 3 * CQ) * Kp * 16;
#pragma unroll
    for (int q = 0; q < NV; ++q) {
        const int r = wave + 4 * q;
        const int j = r / NV, v = r % NV;
        uptr[q] = reinterpret_cast<uint64_t>(Ug + ((size_t)j * CQ + v) * Kp + k0);
    }
    auto u_load = [&](auto par, int row_i, int st) {
        constexpr int S = decltype(par)::value;
        const bool last = row_i == 3 && st == nst - 1;               // the clamped stage past the end repeats it
        const uint64_t inc = last ? 0 : (st == nst - 1 ? wrapU : stepU);
#pragma unroll
        for (int q = 0; q < NV; ++q) {
            const int r = wave + 4 * q;
            const int j = r / NV, v = r % NV;
            dma_row(uptr[q], lane_off, S ? &Us1[j][v][0] : &Us0[j][v][0]);
            uptr[q] += inc;
        }
    };
    // DEEP: the filter rows as register loads (requested at the head of a stage, written to LDS at its tail)
    vec ureg[DEEP ? NV : 1];
    auto u_req = [&](int row_i, int st) {
        typedef __attribute__((address_space(1))) const vec* gvec_p;
        const bool last = row_i == 3 && st == nst - 1;
        const uint64_t inc = last ? 0 : (st == nst - 1 ? wrapU : stepU);
#pragma unroll
        for (int q = 0; q < NV; ++q) {
            ureg[DEEP ? q : 0] = *reinterpret_cast<gvec_p>(uptr[q] + lane_off);
            uptr[q] += inc;
        }
    };
    auto u_commit = [&](auto par) {
        constexpr int S = decltype(par)::value;
#pragma unroll
        for (int q = 0; q < NV; ++q) {
            const int r = wave + 4 * q;
            const int j = r / NV, v = r % NV;
            (S ? Us1 : Us0)[j][v][lane] = ureg[DEEP ? q : 0];
        }
    };
    int ni = 0, nstg = 0;                      // (row, stage) of the filter rows to request: the one after the stage being multiplied
    int xi_ = 0, xst_ = 0;                     // (row, stage) of the raw rows to request: the same, or one further (DEEP)
    auto advance = [&]() {
        if (++nstg == nst) { nstg = 0; ++ni; }
        if (ni > 3) { ni = 3; nstg = nst - 1; }      // past the end: repeat the last stage (never read)
    };
    auto advance_x = [&]() {
        if (++xst_ == nst) { xst_ = 0; ++xi_; }
        if (xi_ > 3) { xi_ = 3; xst_ = nst - 1; }
    };
    vec fu[2], fv[2];
    // first: the stage opens a Winograd row, its MFMAs start from a zero accumulator
    auto iteration = [&](auto par, auto first) {
        constexpr int S = decltype(par)::value;
        constexpr bool FIRST = decltype(first)::value;
        typedef std::integral_constant<int, 1 - S> other_t;
        auto frag_load = [&](int r) {
            const int j = r & 3, v = 2 * (r >> 2) + lh;
            fu[r & 1] = S ? Us1[j][v][(SWAP ? wn : wm) * 32 + l32] : Us0[j][v][(SWAP ? wn : wm) * 32 + l32];
            fv[r & 1] = S ? Vs1[j][v][(SWAP ? wm : wn) * 32 + l32] : Vs0[j][v][(SWAP ? wm : wn) * 32 + l32];
        };
        // the next stage: filter rows and raw patch rows requested first, multiplied stage in between,
        // the raw rows transformed and written during the last MFMA runs.  DEEP: the raw rows requested here
        // are those of the stage after the next (set S); the ones transformed below arrived a stage ago (set 1-S)
        typedef std::integral_constant<int, DEEP ? S : 0> lset_t;
        typedef std::integral_constant<int, DEEP ? 1 - S : 0> vset_t;
        if constexpr (DEEP) u_req(ni, nstg);
        else u_load(other_t{}, ni, nstg);
        x_load_stage(lset_t{}, xi_, xst_);
        advance();
        advance_x();
        frag_load(0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            if (r + 1 < NR) frag_load(r + 1);
            if (r >= NR - 1 - WP) v_piece(other_t{}, vset_t{}, r - (NR - 1 - WP));
            if (FIRST && r < 4) {
#pragma unroll
                for (int q = 0; q < 16; ++q) acc[r][q] = 0.f;
            }
            if (SWAP) Mma<T>::run(fv[r & 1], fu[r & 1], acc[r & 3]);
            else Mma<T>::run(fu[r & 1], fv[r & 1], acc[r & 3]);
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (DEEP) {
            u_commit(other_t{});                     // (the compiler waits for exactly these loads)
            __builtin_amdgcn_s_waitcnt(0xC07F);      // lgkmcnt(0) only: the newest raw rows stay in flight
        } else {
            __builtin_amdgcn_s_waitcnt(0x0070);      // vmcnt(0) lgkmcnt(0)
        }
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");               // no LDS access moves across the barrier
    };

    // prologue: stage (0, 0) of both operands in LDS (DEEP: and the raw rows of the stage after it requested)
    x_load_stage(set0_t{}, 0, 0);
    advance_x();
    if constexpr (DEEP) {
        u_req(0, 0);
        x_load_stage(set1_t{}, xi_, xst_);
        advance_x();
    } else {
        u_load(par0_t{}, 0, 0);
    }
    advance();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int piece = 0; piece <= WP; ++piece) v_piece(par0_t{}, set0_t{}, piece);
    if constexpr (DEEP) u_commit(par0_t{});
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(DEEP ? 0xC07F : 0x0070);
    __syncthreads();

    for (int i = 0; i < 4; ++i) {
        iteration(par0_t{}, std::true_type{});
        iteration(par1_t{}, std::false_type{});
        for (int st = 2; st < nst; st += 2) {
            iteration(par0_t{}, std::false_type{});
            iteration(par1_t{}, std::false_type{});
        }
        rows_fold<false>(acc, yo, i);
    }
    rows_store<T, SWAP>(yo, y, ys, N, K, Ho, Wo, th, tw, P, order, ep, k0, p0, wm, wn, l32, lh);
}

}  // namespace wino
