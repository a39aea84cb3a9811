// 16-way batched GEMM of the Winograd domain on MFMA (gfx950, wave64).
//
//   Mo[xi][k][p] = sum_c U[xi][c][k] * V[xi][c][p]          xi = 0..15
//
// Operands arrive as 16-byte channel vectors, U[xi][Cp/CV][Kp][CV] and
// V[xi][Cp/CV][Pp][CV]; HBM -> LDS copies and LDS -> register fetches are all
// 16-byte accesses in the same arrangement.
//
// MFMA register conventions (32x32 family), lane l, l32 = l%32, lh = l/32:
//   fp32  v_mfma_f32_32x32x2_f32 :  a = A[i=l32][kk=lh]        b = B[kk=lh][j=l32]
//   16bit v_mfma_f32_32x32x16_*  :  a = A[i=l32][8*lh .. +7]   b = B[8*lh .. +7][j=l32]
//   accumulator register r holds D[i = 8*(r/4) + 4*lh + r%4][j = l32].
// A "k-group" is the pair of channel vectors (2g, 2g+1) taken by the lane halves
// lh = 0 and 1: 8 channels for fp32 (4 MFMAs, one per vector element), 16
// channels for f16/bf16 (one MFMA).  The sum over channels does not care which
// channel a lane half takes as long as both operands agree.
#pragma once
#include <type_traits>

#include "common.hpp"
#include "transforms.hpp"

namespace wino {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

template <typename T> struct Mma;
template <> struct Mma<float> {
    typedef floatx4 vec;
    static __device__ __forceinline__ void run(const vec& a, const vec& b, floatx16& acc) {
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], acc, 0, 0, 0);
    }
};
template <> struct Mma<f16_t> {
    typedef halfx8 vec;
    static __device__ __forceinline__ void run(const vec& a, const vec& b, floatx16& acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
    }
};
template <> struct Mma<bf16_t> {
    typedef bf16x8 vec;
    static __device__ __forceinline__ void run(const vec& a, const vec& b, floatx16& acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
    }
};

// One direct-to-LDS load of 64 channel vectors (1 KB): lane l moves the 16 bytes at sbase + 16*l to
// lds_dst + 16*l.  sbase is wave-uniform (a scalar register pair, advanced with scalar adds): at
// 16-bit MFMA rates the address arithmetic of these loads, vector or scalar, costs as much as the
// multiplies of a stage, so the kernels keep one running address per load slot instead of
// recomputing row * pitch products.
// The instruction is written out rather than taken from the compiler's builtin: the compiler counts the builtin
// as an access of unknown kind, and while one is in flight (in these kernels: always) it can no longer tell in
// which order LDS reads return, so that every wait for an LDS read becomes a wait for ALL of them -- the read
// issued one instruction earlier included, which leaves a wave's matrix pipe idle for an LDS round trip at
// every step.  Written out, the load is invisible to that bookkeeping: every kernel that uses it waits for its
// rows itself (s_waitcnt vmcnt before the workgroup's barrier), which they did already.
// M0 is written here and not named as a clobber: it is a reserved register for this compiler (which refuses it on a
// clobber list as undefined behaviour), never holds a value across instructions, and is set by the compiler itself
// right before each of its own uses.
__device__ __forceinline__ void dma_row(uint64_t sbase, unsigned lane_off, void* lds_dst) {
    const unsigned dst = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)lds_dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(lane_off), "s"(sbase) : "memory");
}

// a wave-uniform 64-bit value, for the compiler too (scalar registers): values that are uniform by construction
// (derived from the workgroup id and kernel arguments through a cursor the compiler keeps in memory) still have to
// reach the scalar operands of dma_row
__device__ __forceinline__ uint64_t uniform64(uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
}

constexpr int GEMM_BM = 128, GEMM_BN = 128;

constexpr int GO_T = 64;   // patch edge (filters and tiles)

// The 2x2 outputs of tile (n, ty, tx), filter k.  pair: the destination is W-contiguous with even
// rows and an aligned base (checked once per kernel by pair_stores_ok), so the two outputs of a tile row
// go out as one store.
template <typename OutT> __device__ __forceinline__ bool pair_stores_ok(const OutT* y, const ActStrides& ys, int Wo) {
    return ys.w == 1 && (Wo & 1) == 0 && (ys.h & 1) == 0 && (ys.c & 1) == 0 && (ys.n & 1) == 0 &&
           (reinterpret_cast<uintptr_t>(y) & (2 * sizeof(OutT) - 1)) == 0;
}

template <typename OutT>
__device__ __forceinline__ void store_tile_outputs(OutT* __restrict__ y, const ActStrides& ys, int n, int k, int ty,
                                                   int tx, int Ho, int Wo, float y00, float y01, float y10, float y11,
                                                   const Epilogue& ep, float bias, bool pair) {
    y00 += bias; y01 += bias; y10 += bias; y11 += bias;
    if (ep.relu) {
        y00 = fmaxf(y00, 0.f); y01 = fmaxf(y01, 0.f); y10 = fmaxf(y10, 0.f); y11 = fmaxf(y11, 0.f);
    }
    const int oh = 2 * ty, ow = 2 * tx;
    const bool w1 = ow + 1 < Wo, h1 = oh + 1 < Ho;
    if (ep.pool) {                               // ys describes the pooled tensor; a window cut by the edge is dropped
        if (w1 && h1) y[n * ys.n + k * ys.c + ty * ys.h + tx * ys.w] = from_f32<OutT>(fmaxf(fmaxf(y00, y01), fmaxf(y10, y11)));
        return;
    }
    OutT* yp = y + n * ys.n + k * ys.c + oh * ys.h + ow * ys.w;
    if (pair) {
        struct alignas(2 * sizeof(OutT)) Pair { OutT a, b; };
        *reinterpret_cast<Pair*>(yp) = Pair{from_f32<OutT>(y00), from_f32<OutT>(y01)};
        if (h1) *reinterpret_cast<Pair*>(yp + ys.h) = Pair{from_f32<OutT>(y10), from_f32<OutT>(y11)};
        return;
    }
    yp[0] = from_f32<OutT>(y00);
    if (w1) yp[ys.w] = from_f32<OutT>(y01);
    if (h1) {
        yp[ys.h] = from_f32<OutT>(y10);
        if (w1) yp[ys.h + ys.w] = from_f32<OutT>(y11);
    }
}

// Row i of the 4x4 product tile (its four coordinates in acc) folded into the four outputs
// y00, y01, y10, y11 of the tile, then acc cleared if CLEAR:  A^T = [1 1 1 0; 0 1 -1 -1], column i =
// (c0, c1); the products with 0 and +-1 are exact.
template <bool CLEAR> __device__ __forceinline__ void rows_fold(floatx16 (&acc)[4], floatx16 (&yo)[4], int i) {
    const float c0 = i < 3 ? 1.f : 0.f;
    const float c1 = i == 0 ? 0.f : (i == 1 ? 1.f : -1.f);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const float t0 = acc[0][r] + acc[1][r] + acc[2][r];
        const float t1 = acc[1][r] - acc[2][r] - acc[3][r];
        yo[0][r] = fmaf(c0, t0, yo[0][r]);
        yo[1][r] = fmaf(c0, t1, yo[1][r]);
        yo[2][r] = fmaf(c1, t0, yo[2][r]);
        yo[3][r] = fmaf(c1, t1, yo[3][r]);
        if (CLEAR) {
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j][r] = 0.f;
        }
    }
}

// Stores of a wave's 32x32 patch of output tiles: register r is MFMA row 8*(r/4) + 4*lh + r%4,
// the lane's l32 the MFMA column.
template <typename T, bool SWAP>
__device__ __forceinline__ void rows_store(const floatx16 (&yo)[4], T* __restrict__ y, const ActStrides& ys, int N,
                                           int K, int Ho, int Wo, int th, int tw, long P, int order, const Epilogue& ep, int k0,
                                           long p0, int wm, int wn, int l32, int lh) {
    const bool pair = !ep.pool && pair_stores_ok(y, ys, Wo);
    if (!SWAP) {
        const long p = p0 + wn * 32 + l32;
        if (p >= P) return;
        int n, ty, tx;
        decode_tile(p, order, N, th, tw, n, ty, tx);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int k = k0 + wm * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
            if (k >= K) continue;
            store_tile_outputs<T>(y, ys, n, k, ty, tx, Ho, Wo, yo[0][r], yo[1][r], yo[2][r], yo[3][r], ep, bias_of<T>(ep, k), pair);
        }
    } else {
        const int k = k0 + wn * 32 + l32;
        if (k >= K) return;
        const float bk = bias_of<T>(ep, k);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const long p = p0 + wm * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
            if (p >= P) continue;
            int n, ty, tx;
            decode_tile(p, order, N, th, tw, n, ty, tx);
            store_tile_outputs<T>(y, ys, n, k, ty, tx, Ho, Wo, yo[0][r], yo[1][r], yo[2][r], yo[3][r], ep, bk, pair);
        }
    }
}

// f(integral_constant<int, S>) for every S of the sequence, in order
template <int... S, class F> __device__ __forceinline__ void for_each_const(std::integer_sequence<int, S...>, F&& f) {
    (f(std::integral_constant<int, S>{}), ...);
}

// =============================================================================
// GEMM with the output transform in its epilogue, one Winograd ROW at a time.
//
// A workgroup owns a 64-filter x 64-tile patch; only the 4 coordinates of one
// row i of the 4x4 coordinate grid are resident at a time: a wave
// keeps four 32x32 MFMA accumulators (64 AGPRs) and, in VGPRs, the four output
// planes y00, y01, y10, y11 of its (filter, tile) pairs.  When the channel
// reduction of row i ends, the row is folded into the outputs,
//     T_b = (A^T-column transform of m_i0..m_i3)_b,   y_ab += (A^T)_{a i} * T_b,
// and the accumulators restart for row i+1.  A wave needs ~160 registers instead
// of 512, so three workgroups share a CU: their barriers and load latencies
// overlap, and three times as many waves pull operands from L2 (one 4-wave
// workgroup per CU cannot draw more than ~38 B/clk, which is what a kernel that
// keeps all 16 coordinates resident -- one wave per SIMD -- needs at fp32 MFMA
// peak; that variant measured 8-14 % slower on every shape).
//
// A stage is NVG k-groups of one row: [4][2*NVG][64] channel vectors of U and of V,
// moved HBM -> LDS by global_load_lds_dwordx4.  The 4 * nst stages of a patch form
// one pipeline that runs across the row boundaries, through a ring of RING LDS
// stages with RING-1 of them in flight: the operands of a stage come from HBM or a
// remote L2 slice and need longer than one stage of MFMAs to arrive (a 3-deep ring
// measured 7-17 % faster than double buffering with 2-byte operands, a 4-deep one
// 2-4 % with fp32).  The ring slot is a compile-time index (loop unrolled RING
// times, remainder peeled) and every slot is an array of its own, so the compiler
// can tell the slot being filled from the one being read.  The stage barrier is a
// bare s_barrier: __syncthreads() carries a release fence for which the compiler
// drains every pending direct-to-LDS load.
//
// A workgroup alone on its CU needs the MFMA time of a whole patch (55 us for C = 256 in fp32),
// and that is what a last round of a few workgroups costs while the other CUs idle.  The host
// therefore appends the patches of a last round that fills at most 60 % of the resident workgroups
// as TAIL workgroups: four per patch, one Winograd row each, combined by the last one to arrive.
// =============================================================================
template <typename T, bool SWAP, int NVG, int RING>
__global__ __launch_bounds__(256, 2) void gemm_rows_kernel(const T* __restrict__ U, const T* __restrict__ V,
                                                           T* __restrict__ y, ActStrides ys, int N, int K,
                                                           int Ho, int Wo, int th, int tw, long P, int Cp,
                                                           int Kp, long Pp, int order, Epilogue ep, int kTiles,
                                                           int pTiles, int main_ids, float* __restrict__ tail_part,
                                                           int* __restrict__ tail_cnt, int xcd_map) {
    typedef typename Mma<T>::vec vec;
    constexpr int CV = ChanVec<T>::n;
    constexpr int NV = 2 * NVG;
    static_assert(RING == 3 || RING == 4, "ring depth");
    __shared__ vec Us0[4][NV][GO_T], Us1[4][NV][GO_T], Us2[4][NV][GO_T], Us3[RING > 3 ? 4 : 1][NV][GO_T];
    __shared__ vec Vs0[4][NV][GO_T], Vs1[4][NV][GO_T], Vs2[4][NV][GO_T], Vs3[RING > 3 ? 4 : 1][NV][GO_T];
    auto uslot = [&](auto sl) -> vec(*)[NV][GO_T] {
        constexpr int S = decltype(sl)::value;
        if constexpr (S == 0) return Us0; else if constexpr (S == 1) return Us1; else if constexpr (S == 2) return Us2; else return Us3;
    };
    auto vslot = [&](auto sl) -> vec(*)[NV][GO_T] {
        constexpr int S = decltype(sl)::value;
        if constexpr (S == 0) return Vs0; else if constexpr (S == 1) return Vs1; else if constexpr (S == 2) return Vs2; else return Vs3;
    };

    // Workgroup ids >= main_ids are TAIL workgroups: the patches of the last, partly filled round are
    // cut four ways -- one Winograd row per workgroup (a quarter of the reduction) -- so the whole chip
    // works on them instead of a few CUs; tq = patch of the tail, trow = its row.  The four workgroups
    // of a patch have ids 8 apart (the same XCD); they follow the whole patches in the same launch, so
    // they start as soon as CUs run out of whole patches.
    const bool TAIL = (int)blockIdx.x >= main_ids;
    const int tb = (int)blockIdx.x - main_ids;
    const int tq = TAIL ? (tb >> 5) * 8 + (tb & 7) : 0;
    const int trow = TAIL ? (tb >> 3) & 3 : 0;
    const int b = TAIL ? main_ids + tq : (int)blockIdx.x;
    // xcd_map: ids go round-robin to the 8 XCDs, and the ids of one XCD walk the filter tiles of a tile patch
    // before the next patch (one XCD's L2 serves the patch's V to all of them).  With few tile patches that
    // would leave XCDs idle (one patch: seven of eight), so the host then asks for the plain order.
    const int xcd = xcd_map ? b & 7 : 0, jb = xcd_map ? b >> 3 : b;
    const int ktile = jb % kTiles;
    const int ptile = (jb / kTiles) * (xcd_map ? 8 : 1) + xcd;
    if (ptile >= pTiles) return;
    const int k0 = ktile * GO_T;
    const long p0 = (long)ptile * GO_T;
    const int CQ = Cp / CV;
    const int nst = CQ / NV;
    const int total = TAIL ? nst : 4 * nst;
    const vec* Ug = reinterpret_cast<const vec*>(U);
    const vec* Vg = reinterpret_cast<const vec*>(V);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;

    floatx16 acc[4], yo[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc[j][r] = 0.f; yo[j][r] = 0.f; }

    const unsigned lane_off = lane * 16;
    uint64_t sptr[2 * NV];
    const uint64_t stepU = (uint64_t)NV * Kp * 16, wrapU = (uint64_t)(NV + 3 * CQ) * Kp * 16;
    const uint64_t stepV = (uint64_t)NV * Pp * 16, wrapV = (uint64_t)(NV + 3 * CQ) * Pp * 16;
#pragma unroll
    for (int q = 0; q < 2 * NV; ++q) {
        const int r = wave + 4 * q;
        const int opnd = q / NV;
        const int j = (r / NV) & 3, v = r % NV;
        const size_t cvec = (size_t)(4 * trow + j) * CQ + v;
        sptr[q] = opnd ? reinterpret_cast<uint64_t>(Vg + cvec * Pp + p0) : reinterpret_cast<uint64_t>(Ug + cvec * Kp + k0);
    }
    int issued = 0, in_row = 0;
    auto stage_load = [&](auto sl) {
        ++issued;
        const bool wrap = ++in_row == nst, last = issued >= total;
        if (wrap) in_row = 0;
        const uint64_t incU = last ? 0 : (wrap ? wrapU : stepU), incV = last ? 0 : (wrap ? wrapV : stepV);
#pragma unroll
        for (int q = 0; q < 2 * NV; ++q) {
            const int r = wave + 4 * q;
            const int opnd = q / NV;
            const int j = (r / NV) & 3, v = r % NV;
            dma_row(sptr[q], lane_off, opnd ? &vslot(sl)[j][v][0] : &uslot(sl)[j][v][0]);
            sptr[q] += opnd ? incV : incU;
        }
    };
    constexpr int LPW = 2 * NV;                       // loads per wave and stage
    constexpr int WV = (RING - 2) * LPW;              // the newest RING-2 stages may still be in flight
    constexpr int WAIT_IMM = (WV & 0xF) | (0x7 << 4) | (0xF << 8) | ((WV >> 4) << 14);
    int row = trow, cst = 0;                          // Winograd row and stage of it being multiplied
    auto iteration = [&](auto sl) {
        constexpr int S = decltype(sl)::value;
        __builtin_amdgcn_s_waitcnt(WAIT_IMM);
        __builtin_amdgcn_s_barrier();                 // stage S landed for every wave; slot S-1 is free
        asm volatile("" ::: "memory");
        // the stage's fragments are requested first, all of them, and the loads of the stage RING-1 ahead
        // are issued while they travel: a wave's own LDS latency is not covered by its own MFMAs otherwise
        vec fu[NVG][4], fv[NVG][4];
#pragma unroll
        for (int g = 0; g < NVG; ++g)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                fu[g][j] = uslot(sl)[j][2 * g + lh][(SWAP ? wn : wm) * 32 + l32];
                fv[g][j] = vslot(sl)[j][2 * g + lh][(SWAP ? wm : wn) * 32 + l32];
            }
        __builtin_amdgcn_sched_barrier(0);
        stage_load(std::integral_constant<int, (S + RING - 1) % RING>{});
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < NVG; ++g)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (SWAP) Mma<T>::run(fv[g][j], fu[g][j], acc[j]);
                else Mma<T>::run(fu[g][j], fv[g][j], acc[j]);
            }
        __builtin_amdgcn_sched_barrier(0);
        if (++cst == nst) {
            cst = 0;
            rows_fold<true>(acc, yo, row);
            ++row;
        }
    };

    for_each_const(std::make_integer_sequence<int, RING - 1>{}, stage_load);
    int s = 0;
    for (; s + RING <= total; s += RING) for_each_const(std::make_integer_sequence<int, RING>{}, iteration);
    // total = 4*nst is even; with RING = 3 up to two stages remain, in slots 0 and 1; with RING = 4 none or two
    if (s < total) iteration(std::integral_constant<int, 0>{});
    if (s + 1 < total) iteration(std::integral_constant<int, 1>{});
    if (RING == 4 && s + 2 < total) iteration(std::integral_constant<int, 2>{});
    __builtin_amdgcn_s_waitcnt(0x0F70);               // the surplus requests of the last stages
    if (TAIL) {
        // Every workgroup leaves its row's contribution in tail_part[patch][row][register][thread]; the
        // one that arrives last (a counter per patch, returned to zero for the next launch) adds the four
        // rows in the order 0..3 -- so the result does not depend on who was last -- and stores the patch.
        // The partial sums travel as device-scope relaxed atomic stores and loads (coherent across the
        // chip's L2 slices without flushing them: a device-scope fence writes the whole L2 back); the
        // stores have completed (vmcnt) before the workgroup's arrival is counted.
        float* mine = tail_part + ((size_t)(tq * 4 + trow) * 64) * 256 + tid;
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                __hip_atomic_store(mine + (a * 16 + r) * 256, yo[a][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __shared__ int s_last;
        __builtin_amdgcn_s_waitcnt(0x0F70);           // vmcnt(0): this wave's partial sums are in memory
        __syncthreads();
        if (tid == 0) {
            const int old = __hip_atomic_fetch_add(&tail_cnt[tq], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = old == 3;
            if (old == 3) __hip_atomic_store(&tail_cnt[tq], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (!s_last) return;
        const float* all = tail_part + ((size_t)(tq * 4) * 64) * 256 + tid;
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float* e = all + (a * 16 + r) * 256;
                const float e0 = __hip_atomic_load(e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const float e1 = __hip_atomic_load(e + 64 * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const float e2 = __hip_atomic_load(e + 2 * 64 * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const float e3 = __hip_atomic_load(e + 3 * 64 * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                yo[a][r] = ((e0 + e1) + e2) + e3;
            }
    }
    rows_store<T, SWAP>(yo, y, ys, N, K, Ho, Wo, th, tw, P, order, ep, k0, p0, wm, wn, l32, lh);
}

// =============================================================================
// Plain batched GEMM, product written to HBM as Mo[xi][Kp][Pp] (fp32).
//
// Block tile 128 filters x 128 tiles, 4 waves in a 2x2 arrangement, each wave
// 64x64 = 2x2 MFMA tiles.  The reduction is consumed NV channel vectors at a
// time from a ring of RING LDS stages; the stages travel HBM -> LDS directly
// (global_load_lds_dwordx4: one instruction moves 64 channel vectors = 1 KB,
// lane l to LDS row base + 16*l), RING-1 of them in flight, from running scalar
// addresses; no staging registers, no LDS store instructions; one wait and one
// bare s_barrier per stage (the pipeline of gemm_rows_kernel).  Measured: 4 deep
// for fp32 (1-5 % faster than register-staged double buffering), 3 deep for 2-byte
// operands (the layers that take this kernel are small: N=32, C=K=512, H=14 in bf16 runs
// 30.8 us 2 deep, 28.2 us 3 deep, 30.7 us 4 deep; large layers are bound by the fp32
// product store and measure the same at 2 and 3).
//
// XCD-aware tile order: consecutive workgroup ids go round-robin to the 8 XCDs, so
// the ids that share an XCD walk the filter tiles of one tile column first and the
// V slab they share is fetched from HBM once, into that XCD's L2.
//
// PK = false: product stored as Mo[xi][Kp][Pp] (MFMA rows = filters, lanes = tiles)
// PK = true : product stored as Mo[xi][Pp][Kp] (MFMA rows = tiles, lanes = filters), for
//             destinations whose contiguous axis is K (NHWC)
// =============================================================================
template <typename T, int NV, bool PK, int RING>
__global__ __launch_bounds__(256) void gemm_128x128_kernel(const T* __restrict__ U, const T* __restrict__ V,
                                                                float* __restrict__ Mo, int Cp, int Kp, long Pp,
                                                                int kTiles, int pTiles, int split_chunks, int xcd_map) {
    typedef typename Mma<T>::vec vec;
    constexpr int CV = ChanVec<T>::n;
    static_assert(RING >= 2 && RING <= 4, "ring depth");
    __shared__ vec As0[NV][GEMM_BM], As1[NV][GEMM_BM], As2[RING > 2 ? NV : 1][GEMM_BM], As3[RING > 3 ? NV : 1][GEMM_BM];
    __shared__ vec Bs0[NV][GEMM_BN], Bs1[NV][GEMM_BN], Bs2[RING > 2 ? NV : 1][GEMM_BN], Bs3[RING > 3 ? NV : 1][GEMM_BN];
    auto aslot = [&](auto sl) -> vec(*)[GEMM_BM] {
        constexpr int S = decltype(sl)::value;
        if constexpr (S == 0) return As0; else if constexpr (S == 1) return As1; else if constexpr (S == 2) return As2; else return As3;
    };
    auto bslot = [&](auto sl) -> vec(*)[GEMM_BN] {
        constexpr int S = decltype(sl)::value;
        if constexpr (S == 0) return Bs0; else if constexpr (S == 1) return Bs1; else if constexpr (S == 2) return Bs2; else return Bs3;
    };
    const int xi = blockIdx.y;
    const int b = blockIdx.x;
    // as in gemm_rows_kernel, but the XCD that takes slot s of a group of 8 tile columns moves on by one with every
    // coordinate: with pTiles not a multiple of 8 the last group is partly empty, and the XCDs whose slots are filled
    // there would otherwise carry a whole tile column more than the others in every one of the 16 or 36 planes
    // (49 tile columns: 7 against 6, the kernel's duration is the 7)
    const int xcd = xcd_map ? (b + xi) & 7 : 0, jj = xcd_map ? b >> 3 : b;
    const int ktile = jj % kTiles;
    const int ptile = (jj / kTiles) * (xcd_map ? 8 : 1) + xcd;
    if (ptile >= pTiles) return;
    const long p0 = (long)ptile * GEMM_BN;
    const int k0 = ktile * GEMM_BM;
    const int CQ = Cp / CV;
    // blockIdx.z: which run of split_chunks stages (NV channel vectors each) of the reduction this workgroup
    // sums; its product goes to copy blockIdx.z of Mo (the host makes every run non-empty)
    const int c_first = blockIdx.z * split_chunks;
    const int nch = min(split_chunks, CQ / NV - c_first);
    const vec* Ub = reinterpret_cast<const vec*>(U) + ((size_t)xi * CQ + (size_t)c_first * NV) * Kp + k0;
    const vec* Vb = reinterpret_cast<const vec*>(V) + ((size_t)xi * CQ + (size_t)c_first * NV) * Pp + p0;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // a stage is 2*NV rows of 128 vectors = 4*NV pieces of 64 vectors; wave w issues pieces w, w+4, ...
    const unsigned lane_off = lane * 16;
    uint64_t sptr[NV];
    const uint64_t stepU = (uint64_t)NV * Kp * 16, stepV = (uint64_t)NV * Pp * 16;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int piece = wave + 4 * i;
        const int opnd = i / (NV / 2);               // = piece / (2*NV), known at compile time
        const int row = (piece >> 1) % NV, half = piece & 1;
        sptr[i] = opnd ? reinterpret_cast<uint64_t>(Vb + (size_t)row * Pp + half * 64)
                       : reinterpret_cast<uint64_t>(Ub + (size_t)row * Kp + half * 64);
    }
    int issued = 0;
    auto stage_load = [&](auto sl) {
        const bool last = ++issued >= nch;           // past the end: the last stage again (never read)
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int piece = wave + 4 * i;
            const int opnd = i / (NV / 2);
            const int row = (piece >> 1) % NV, half = piece & 1;
            dma_row(sptr[i], lane_off, opnd ? &bslot(sl)[row][half * 64] : &aslot(sl)[row][half * 64]);
            sptr[i] += last ? 0 : (opnd ? stepV : stepU);
        }
    };
    constexpr int WV = (RING - 2) * NV;
    constexpr int WAIT_IMM = (WV & 0xF) | (0x7 << 4) | (0xF << 8) | ((WV >> 4) << 14);
    auto iteration = [&](auto sl) {
        __builtin_amdgcn_s_waitcnt(WAIT_IMM);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        stage_load(std::integral_constant<int, (decltype(sl)::value + RING - 1) % RING>{});
        __builtin_amdgcn_sched_barrier(0);
        vec a[2][2], bq[2][2];
        auto frag_load = [&](int g) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const vec fa = aslot(sl)[2 * g + lh][(PK ? wn : wm) * 64 + q * 32 + l32];
                const vec fb = bslot(sl)[2 * g + lh][(PK ? wm : wn) * 64 + q * 32 + l32];
                a[g & 1][q] = PK ? fb : fa;
                bq[g & 1][q] = PK ? fa : fb;
            }
        };
        frag_load(0);
#pragma unroll
        for (int g = 0; g < NV / 2; ++g) {
            if (g + 1 < NV / 2) frag_load(g + 1);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) Mma<T>::run(a[g & 1][i], bq[g & 1][j], acc[i][j]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    for_each_const(std::make_integer_sequence<int, RING - 1>{}, stage_load);
    int s = 0;
    for (; s + RING <= nch; s += RING) for_each_const(std::make_integer_sequence<int, RING>{}, iteration);
    if (s < nch) iteration(std::integral_constant<int, 0>{});
    if (s + 1 < nch) iteration(std::integral_constant<int, 1>{});
    if (RING > 3 && s + 2 < nch) iteration(std::integral_constant<int, 2>{});
    __builtin_amdgcn_s_waitcnt(0x0F70);

    float* Mb = Mo + ((size_t)blockIdx.z * gridDim.y + xi) * Kp * Pp;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ri = wm * 64 + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);   // MFMA row
                const int ci = wn * 64 + j * 32 + l32;                               // MFMA column (lane)
                if (PK) Mb[(size_t)(p0 + ri) * Kp + k0 + ci] = acc[i][j][r];
                else Mb[(size_t)(k0 + ri) * Pp + p0 + ci] = acc[i][j][r];
            }
}

// =============================================================================
// The same GEMM as one resident set of workgroups that WALK the (coordinate, tile column) pairs.
//
// gemm_128x128_kernel starts and ends a workgroup per (tile, coordinate): three stages of loads in flight before
// its first multiply, 64 KB of product stores after its last -- about 6 us of a 33 us workgroup when the reduction
// is 256 channels long.  Here the grid is the resident set (two workgroups per CU).  The pairs, tile column fastest,
// are dealt round-robin to GROUPS of kTiles workgroups -- the filter tiles of a pair, on one XCD, so that its L2
// serves the shared V slab; at any time the whole chip works on a few neighbouring coordinates, whose U planes stay
// in the L2s -- and a workgroup runs its pairs as ONE pipeline: the load ring moves on to the next pair's rows when
// the current pair's last stage has been requested, and at the end of a pair's reduction the workgroup stores the
// product and clears its accumulators while those loads are in flight.
// =============================================================================
template <typename T, int NV, bool PK, int RING>
__global__ __launch_bounds__(256, 2) void gemm_128x128_walk_kernel(const T* __restrict__ U, const T* __restrict__ V,
                                                                   float* __restrict__ Mo, int Cp, int Kp, long Pp,
                                                                   int kTiles, int pTiles, int nxi, int groups) {
    typedef typename Mma<T>::vec vec;
    constexpr int CV = ChanVec<T>::n;
    static_assert(RING >= 3 && RING <= 4, "ring depth");
    __shared__ vec As0[NV][GEMM_BM], As1[NV][GEMM_BM], As2[NV][GEMM_BM], As3[RING > 3 ? NV : 1][GEMM_BM];
    __shared__ vec Bs0[NV][GEMM_BN], Bs1[NV][GEMM_BN], Bs2[NV][GEMM_BN], Bs3[RING > 3 ? NV : 1][GEMM_BN];
    auto aslot = [&](auto sl) -> vec(*)[GEMM_BM] {
        constexpr int S = decltype(sl)::value;
        if constexpr (S == 0) return As0; else if constexpr (S == 1) return As1; else if constexpr (S == 2) return As2; else return As3;
    };
    auto bslot = [&](auto sl) -> vec(*)[GEMM_BN] {
        constexpr int S = decltype(sl)::value;
        if constexpr (S == 0) return Bs0; else if constexpr (S == 1) return Bs1; else if constexpr (S == 2) return Bs2; else return Bs3;
    };
    const int b = blockIdx.x;
    const int xcd = b & 7, v = b >> 3;                   // ids go round-robin to the XCDs
    const int gl = v / kTiles, ktile = v - gl * kTiles;
    const int grp = gl * 8 + xcd;
    const int units = pTiles * nxi;                      // pairs, q = xi * pTiles + tile column
    if (grp >= groups || grp >= units) return;
    const int mine = (units - grp + groups - 1) / groups;    // pairs grp, grp + groups, ...
    const int k0 = ktile * GEMM_BM;
    const int CQ = Cp / CV, nch = CQ / NV;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;
    const unsigned lane_off = lane * 16;
    const uint64_t stepU = (uint64_t)NV * Kp * 16, stepV = (uint64_t)NV * Pp * 16;
    constexpr int WV = (RING - 2) * NV;
    constexpr int WAIT_IMM = (WV & 0xF) | (0x7 << 4) | (0xF << 8) | ((WV >> 4) << 14);

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // ---- load side: the pair whose rows are being requested
    uint64_t sptr[NV];
    int lq = grp, lst = 0;                               // pair and stage of it to request next
    auto point_at = [&](int q) {
        const int xi = q / pTiles, ptile = q - xi * pTiles;
        const vec* Ub = reinterpret_cast<const vec*>(U) + (size_t)xi * CQ * Kp + k0;
        const vec* Vb = reinterpret_cast<const vec*>(V) + (size_t)xi * CQ * Pp + (size_t)ptile * GEMM_BN;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int piece = wave + 4 * i;
            const int opnd = i / (NV / 2);
            const int row = (piece >> 1) % NV, half = piece & 1;
            sptr[i] = opnd ? reinterpret_cast<uint64_t>(Vb + (size_t)row * Pp + half * 64)
                           : reinterpret_cast<uint64_t>(Ub + (size_t)row * Kp + half * 64);
        }
    };
    point_at(lq);
    auto stage_load = [&](auto sl) {
        // past the last pair: the last stage again (never read)
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int piece = wave + 4 * i;
            const int opnd = i / (NV / 2);
            const int row = (piece >> 1) % NV, half = piece & 1;
            dma_row(sptr[i], lane_off, opnd ? &bslot(sl)[row][half * 64] : &aslot(sl)[row][half * 64]);
        }
        if (++lst == nch) {
            lst = 0;
            if (lq + groups < units) {
                lq += groups;
                point_at(lq);
            } else {
                lst = nch - 1;                           // stay on the last stage
            }
        } else {
#pragma unroll
            for (int i = 0; i < NV; ++i) sptr[i] += (i / (NV / 2)) ? stepV : stepU;
        }
    };
    // ---- compute side
    int cq = grp, cst = 0;
    auto iteration = [&](auto sl) {
        __builtin_amdgcn_s_waitcnt(WAIT_IMM);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        stage_load(std::integral_constant<int, (decltype(sl)::value + RING - 1) % RING>{});
        __builtin_amdgcn_sched_barrier(0);
        vec a[2][2], bq[2][2];
        auto frag_load = [&](int g) {
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                const vec fa = aslot(sl)[2 * g + lh][(PK ? wn : wm) * 64 + qq * 32 + l32];
                const vec fb = bslot(sl)[2 * g + lh][(PK ? wm : wn) * 64 + qq * 32 + l32];
                a[g & 1][qq] = PK ? fb : fa;
                bq[g & 1][qq] = PK ? fa : fb;
            }
        };
        frag_load(0);
#pragma unroll
        for (int g = 0; g < NV / 2; ++g) {
            if (g + 1 < NV / 2) frag_load(g + 1);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) Mma<T>::run(a[g & 1][i], bq[g & 1][j], acc[i][j]);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (++cst == nch) {                              // the pair's reduction is complete: store it, start the next
            cst = 0;
            const int xi = cq / pTiles, ptile = cq - xi * pTiles;
            cq += groups;
            const long p0 = (long)ptile * GEMM_BN;
            // (the row pitch is made opaque here: the 64 store addresses of a thread would otherwise be computed
            // ahead of the loop and kept in registers across it -- 300 registers, one workgroup per CU)
            long pitch = PK ? (long)Kp : Pp;
            asm volatile("" : "+s"(pitch));
            float* Mb = Mo + (size_t)xi * Kp * Pp +
                        (PK ? (size_t)(p0 + wm * 64 + 4 * lh) * pitch + k0 + wn * 64 + l32
                            : (size_t)(k0 + wm * 64 + 4 * lh) * pitch + p0 + wn * 64 + l32);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float* row = Mb + (size_t)(i * 32 + 8 * (r >> 2) + (r & 3)) * pitch;      // MFMA row; lanes: columns
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        row[j * 32] = acc[i][j][r];
                        acc[i][j][r] = 0.f;
                    }
                }
        }
    };
    const int total = mine * nch;
    for_each_const(std::make_integer_sequence<int, RING - 1>{}, stage_load);
    int s = 0;
    for (; s + RING <= total; s += RING) for_each_const(std::make_integer_sequence<int, RING>{}, iteration);
    if (s < total) iteration(std::integral_constant<int, 0>{});
    if (s + 1 < total) iteration(std::integral_constant<int, 1>{});
    if (RING > 3 && s + 2 < total) iteration(std::integral_constant<int, 2>{});
    __builtin_amdgcn_s_waitcnt(0x0F70);                  // the surplus requests of the last stages
}

// =============================================================================
// The walking GEMM with the product stores of a pair spread over the first stages of the NEXT pair.
//
// In gemm_128x128_walk_kernel a wave stores its 64 x 64 block of a finished pair in one burst of 64 instructions,
// 19 % of its time, during which it multiplies nothing; the matrix pipe of a SIMD idles whenever both of its waves are
// out of their multiplies.  Here the finished accumulators move to a second register set and are stored two
// instructions at a time behind the multiplies of the next pair's first RING stages (a quarter of the block per
// stage: the ring slot names the quarter, so the reduction must be a multiple of RING stages long); only a
// workgroup's last pair is stored in a burst.  224 registers instead of 160: still two workgroups per CU.
// =============================================================================
template <typename T, int NV, bool PK, int RING>
__global__ __launch_bounds__(256, 2) void gemm_128x128_walk_spread_kernel(const T* __restrict__ U, const T* __restrict__ V,
                                                                          float* __restrict__ Mo, int Cp, int Kp, long Pp,
                                                                          int kTiles, int pTiles, int nxi, int groups) {
    typedef typename Mma<T>::vec vec;
    constexpr int CV = ChanVec<T>::n;
    static_assert(RING == 4 && NV == 4, "a quarter of the block per ring slot, eight (group, i, j) steps per stage");
    __shared__ vec As0[NV][GEMM_BM], As1[NV][GEMM_BM], As2[NV][GEMM_BM], As3[NV][GEMM_BM];
    __shared__ vec Bs0[NV][GEMM_BN], Bs1[NV][GEMM_BN], Bs2[NV][GEMM_BN], Bs3[NV][GEMM_BN];
    auto aslot = [&](auto sl) -> vec(*)[GEMM_BM] {
        constexpr int S = decltype(sl)::value;
        if constexpr (S == 0) return As0; else if constexpr (S == 1) return As1; else if constexpr (S == 2) return As2; else return As3;
    };
    auto bslot = [&](auto sl) -> vec(*)[GEMM_BN] {
        constexpr int S = decltype(sl)::value;
        if constexpr (S == 0) return Bs0; else if constexpr (S == 1) return Bs1; else if constexpr (S == 2) return Bs2; else return Bs3;
    };
    const int b = blockIdx.x;
    const int xcd = b & 7, v = b >> 3;                   // ids go round-robin to the XCDs
    const int gl = v / kTiles, ktile = v - gl * kTiles;
    const int grp = gl * 8 + xcd;
    const int units = pTiles * nxi;                      // pairs, q = xi * pTiles + tile column
    if (grp >= groups || grp >= units) return;
    const int mine = (units - grp + groups - 1) / groups;    // pairs grp, grp + groups, ...
    const int k0 = ktile * GEMM_BM;
    const int CQ = Cp / CV, nch = CQ / NV;               // a multiple of RING (the host checks)

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;
    const unsigned lane_off = lane * 16;
    const uint64_t stepU = (uint64_t)NV * Kp * 16, stepV = (uint64_t)NV * Pp * 16;
    constexpr int WV = (RING - 2) * NV;

    floatx16 acc[2][2], prv[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = prv[i][j][r] = 0.f;

    // ---- load side: the pair whose rows are being requested (as in gemm_128x128_walk_kernel)
    uint64_t sptr[NV];
    int lq = grp, lst = 0;
    auto point_at = [&](int q) {
        const int xi = q / pTiles, ptile = q - xi * pTiles;
        const vec* Ub = reinterpret_cast<const vec*>(U) + (size_t)xi * CQ * Kp + k0;
        const vec* Vb = reinterpret_cast<const vec*>(V) + (size_t)xi * CQ * Pp + (size_t)ptile * GEMM_BN;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int piece = wave + 4 * i;
            const int opnd = i / (NV / 2);
            const int row = (piece >> 1) % NV, half = piece & 1;
            sptr[i] = opnd ? reinterpret_cast<uint64_t>(Vb + (size_t)row * Pp + half * 64)
                           : reinterpret_cast<uint64_t>(Ub + (size_t)row * Kp + half * 64);
        }
    };
    point_at(lq);
    auto stage_load = [&](auto sl) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int piece = wave + 4 * i;
            const int opnd = i / (NV / 2);
            const int row = (piece >> 1) % NV, half = piece & 1;
            dma_row(sptr[i], lane_off, opnd ? &bslot(sl)[row][half * 64] : &aslot(sl)[row][half * 64]);
        }
        if (++lst == nch) {
            lst = 0;
            if (lq + groups < units) {
                lq += groups;
                point_at(lq);
            } else {
                lst = nch - 1;                           // past the last pair: the last stage again (never read)
            }
        } else {
#pragma unroll
            for (int i = 0; i < NV; ++i) sptr[i] += (i / (NV / 2)) ? stepV : stepU;
        }
    };
    // ---- compute side
    long pitch = PK ? (long)Kp : Pp;                     // (opaque: the store addresses are not to be computed ahead
    asm volatile("" : "+s"(pitch));                      //  of the loop and kept in registers across it)
    auto block_of = [&](int q) {                         // this lane's corner of pair q's 64 x 64 block
        const int xi = q / pTiles, ptile = q - xi * pTiles;
        const long p0 = (long)ptile * GEMM_BN;
        return Mo + (size_t)xi * Kp * Pp + (PK ? (size_t)(p0 + wm * 64 + 4 * lh) * pitch + k0 + wn * 64 + l32
                                               : (size_t)(k0 + wm * 64 + 4 * lh) * pitch + p0 + wn * 64 + l32);
    };
    float* Mprev = nullptr;
    // store n = 0..63 of the previous pair's block: rows i = n / 32, register (n / 2) % 16, half n % 2
    // (n is a constant once the loops around the call are unrolled)
    auto store_one = [&](int n) {
        const int i = n >> 5, r = (n >> 1) & 15, j = n & 1;
        Mprev[(size_t)(i * 32 + 8 * (r >> 2) + (r & 3)) * pitch + j * 32] = prv[i][j][r];
        prv[i][j][r] = 0.f;
    };
    // The wait before the barrier is for the rows this wave requested three stages ago: "all but my newest WV
    // operations" -- interleaved stores only make it wait for more than it must.
    auto stage = [&](auto sl, auto with_stores) {
        constexpr int S = decltype(sl)::value;
        constexpr bool ST = decltype(with_stores)::value;
        __builtin_amdgcn_s_waitcnt((WV & 0xF) | (0x7 << 4) | (0xF << 8) | ((WV >> 4) << 14));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        stage_load(std::integral_constant<int, (decltype(sl)::value + RING - 1) % RING>{});
        __builtin_amdgcn_sched_barrier(0);
        vec a[2][2], bq[2][2];
        auto frag_load = [&](int g) {
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                const vec fa = aslot(sl)[2 * g + lh][(PK ? wn : wm) * 64 + qq * 32 + l32];
                const vec fb = bslot(sl)[2 * g + lh][(PK ? wm : wn) * 64 + qq * 32 + l32];
                a[g & 1][qq] = PK ? fb : fa;
                bq[g & 1][qq] = PK ? fa : fb;
            }
        };
        frag_load(0);
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            if (g == 0) frag_load(1);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    Mma<T>::run(a[g & 1][i], bq[g & 1][j], acc[i][j]);
                    if constexpr (ST) {              // two of the quarter's sixteen stores behind every step
                        const int n = 16 * S + 2 * (4 * g + 2 * i + j);
                        __builtin_amdgcn_sched_barrier(0);
                        store_one(n);
                        store_one(n + 1);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    for_each_const(std::make_integer_sequence<int, RING - 1>{}, stage_load);
    int cq = grp;
#pragma unroll 1
    for (int pair = 0; pair < mine; ++pair) {
        // the first RING stages carry the previous pair's stores (spread over two or four times as many stages,
        // 8 or 4 stores to a stage, measured 1-3 % slower)
        if (pair > 0) for_each_const(std::make_integer_sequence<int, RING>{}, [&](auto sl) { stage(sl, std::true_type{}); });
        else for_each_const(std::make_integer_sequence<int, RING>{}, [&](auto sl) { stage(sl, std::false_type{}); });
#pragma unroll 1
        for (int st = RING; st < nch; st += RING)
            for_each_const(std::make_integer_sequence<int, RING>{}, [&](auto sl) { stage(sl, std::false_type{}); });
        // the pair's reduction is complete: its sums move to the second register set
        Mprev = block_of(cq);
        cq += groups;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    prv[i][j][r] = acc[i][j][r];
                    acc[i][j][r] = 0.f;
                }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                  // the surplus requests of the last stages
    // the last pair's block, in one go
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float* row = Mprev + (size_t)(i * 32 + 8 * (r >> 2) + (r & 3)) * pitch;
#pragma unroll
            for (int j = 0; j < 2; ++j) row[j * 32] = prv[i][j][r];
        }
}

}  // namespace wino
