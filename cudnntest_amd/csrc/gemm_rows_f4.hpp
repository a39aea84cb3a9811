// F(4x4,3x3): the 36-way GEMM with the output transform A^T (.) A in its epilogue -- no product tensor in HBM.
//
//   y[k][tile][a][b] = sum_{i,j} A^T[a][i] A^T[b][j]  sum_c U[6i+j][c][k] V[6i+j][c][tile]
//
// What the reference's fused kernels do per thread (fusedTest/winotrans.cuh:1530-1574: 36 running products, A^T acc A
// in registers, 16 stores), arranged for the matrix cores: a (filter, tile) pair needs its 36 products at once, and the
// 32x32 MFMA tile with its 16 sums per lane and coordinate leaves no room for that.  So, as in gemm_rows_kernel:
//
//   * one Winograd ROW of the 6x6 coordinate grid is resident at a time: six accumulators per pair, and at the end of
//     the row's channel reduction the row is folded into the pair's sixteen outputs,
//         T_b = sum_j A^T[b][j] m_ij,        y_ab += A^T[a][i] T_b,
//     22 registers per pair instead of 36 + 16;
//   * 16x16x4 MFMA tiles (4 sums per lane): a wave owns 32 x 16 pairs -- 8 per lane, 176 accumulator registers -- so
//     two waves share a SIMD; a workgroup is 8 waves = a 64 x 64 patch, one workgroup per CU;
//   * a stage is one row x 16 channels: [6][4][64] channel vectors of U and of V (48 KB), HBM -> LDS by
//     global_load_lds_dwordx4 into a ring of three, two stages in flight.
//
// Scheduling.  A patch is 6 * C/16 stages -- 123 us of a CU at C = 256 -- and a VGG layer has one to two patches per
// CU, so whole patches per workgroup would leave the chip half idle in the last round.  The grid is instead one
// persistent workgroup per CU, and every workgroup gets the same number of STAGES: the sequence of all stages of an
// XCD's patches (filter tile major, so that the U rows of a filter tile stay in that XCD's L2 while its workgroups
// stream their tiles' V) is cut into equal runs.  A run begins and ends in the middle of patches; the fold is linear,
// so a part of a patch gives a partial sum of its outputs.  The workgroup that holds a patch's END owns it: the
// others leave their partial outputs in scratch (device-scope relaxed atomic stores, then an arrival counter), the
// owner adds them in workgroup order and stores the patch, so the result does not depend on timing.  Order inside a
// run: first the part of the patch that continues in the next workgroup (a contributor's part: written at once, its
// owner never waits long), then the whole patches, last the part whose beginning lies in the previous workgroups
// (by then their parts were written long ago).  A workgroup only ever waits for lower workgroup ids of its own XCD,
// for something they do first and without waiting themselves; the wait is bounded all the same.
#pragma once
#include "gemm.hpp"
#include "transforms_f4.hpp"

namespace wino {

constexpr int GF4_T = 64;                              // patch edge (filters and tiles)
constexpr int GF4_RING = 3;
constexpr int GF4_PLANE = 4 * GF4_T * 16;              // bytes of one coordinate of a stage: [4 vectors][64] x 16 B
constexpr int GF4_OPND = 6 * GF4_PLANE;                // one operand's stage: 24 KB
constexpr int GF4_LDS = GF4_RING * 2 * GF4_OPND;       // 144 KB
constexpr int GF4_PART = 128 * 512;                    // floats of a patch's partial outputs: [128 registers][512 threads]

// dma_row with the LDS destination as a byte address in a scalar register (no pointer conversion per request)
__device__ __forceinline__ void dma_row_to(uint64_t sbase, unsigned lane_off, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(lane_off), "s"(sbase) : "memory");
}

// SWAP = false: MFMA rows (registers) = filters, columns (lanes) = tiles -- for destinations contiguous along tiles
// SWAP = true : MFMA rows = tiles, columns = filters -- for NHWC destinations (lanes write along K)
template <bool SWAP>
__global__ __launch_bounds__(512, 1) void gemm_rows_f4_kernel(const float* __restrict__ U, const float* __restrict__ V,
                                                              float* __restrict__ y, ActStrides ys, int N, int K, int Ho,
                                                              int Wo, int th, int tw, long P, int Cp, int Kp, long Pp,
                                                              int order, Epilogue ep, int kTiles, int pTiles,
                                                              int nparts, float* __restrict__ part,
                                                              int* __restrict__ cnt, int spin_limit) {
    extern __shared__ __attribute__((aligned(16))) unsigned char gf4_smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave >> 2, wc = wave & 3;             // the wave's 32 rows and 16 columns of the patch
    const int l16 = lane & 15, lq = lane >> 4;
    const int CQ = Cp / 4, nst = CQ / 4;                 // channel vectors; stages of a row
    const int PL = 6 * nst;                              // stages of a patch

    // ---- this workgroup's run of its XCD's stage sequence ---------------------------------------------------
    const int xcd = blockIdx.x & 7, jw = blockIdx.x >> 3, Sx = gridDim.x >> 3;
    const long Np = (long)kTiles * pTiles;
    if (xcd >= nparts) return;                            // (fewer patches than XCDs)
    const long q0 = xcd * Np / nparts, q1 = (xcd + 1) * Np / nparts;   // patches of this XCD, q = ktile * pTiles + ptile
    const long Tx = (q1 - q0) * PL;
    const long ra = jw * Tx / Sx, rb = (jw + 1) * Tx / Sx;
    if (ra >= rb) return;
    // three segments, in the order they are run: the part of the last patch (continued by the next workgroup),
    // the whole patches, the rest of the first patch (begun by the previous workgroups)
    const long hstart = rb / PL * PL;
    // (the run ends with a patch: no first segment; the whole run lies inside a patch that goes on: nothing else)
    const long at0 = rb == hstart ? rb : (hstart <= ra ? ra : hstart), len0 = rb - at0;
    const long low_end = rb - len0;
    const long at1 = min((ra + PL - 1) / PL * PL, low_end), len1 = low_end - at1;
    const long at2 = ra, len2 = at1 - ra;
    const int total = (int)(rb - ra);
    const int slot_me = xcd * Sx + jw;

    // a position of the sequence: segment and what is left of it, Winograd row and stage of the row, filter and tile
    // patch; a step tells what changed (the load side keeps running addresses and only re-derives them per patch)
    struct Cur {
        int seg, left, row, cst, kt, pt;
    };
    auto seek = [&](Cur& c, int seg) __attribute__((always_inline)) {     // the first stage of segment `seg` or, if that is empty, of the next
        if (seg == 0 && len0 == 0) seg = 1;
        if (seg == 1 && len1 == 0) seg = 2;
        if (seg == 2 && len2 == 0) seg = 3;
        c.seg = seg;
        if (seg >= 3) return false;
        c.left = (int)(seg == 0 ? len0 : (seg == 1 ? len1 : len2));
        const long g = seg == 0 ? at0 : (seg == 1 ? at1 : at2);
        const int patch = (int)(g / PL);
        const int t = (int)(g - (long)patch * PL);
        c.row = t / nst;
        c.cst = t - c.row * nst;
        const long q = q0 + patch;
        c.kt = (int)(q / pTiles);
        c.pt = (int)(q - (long)c.kt * pTiles);
        return true;
    };
    enum { STEP_STAGE = 0, STEP_ROW = 1, STEP_PATCH = 2, STEP_END = 3 };
    auto step = [&](Cur& c) __attribute__((always_inline)) {
        if (--c.left == 0) {
            Cur n = c;
            if (!seek(n, c.seg + 1)) {
                c.left = 1;                               // the last stage of the run: stay on it
                return (int)STEP_END;
            }
            c = n;
            return (int)STEP_PATCH;
        }
        if (++c.cst < nst) return (int)STEP_STAGE;
        c.cst = 0;
        if (++c.row < 6) return (int)STEP_ROW;
        c.row = 0;
        if (++c.pt == pTiles) {
            c.pt = 0;
            ++c.kt;
        }
        return (int)STEP_PATCH;
    };

    // ---- load side: 48 rows of 1 KB per stage, six per wave ----------------------------------------------------
    // row r = wave + 8 q of a stage: operand r / 24 (U, V), coordinate (r % 24) / 4 of the row, channel vector r % 4
    const unsigned lane_off = lane * 16;
    const unsigned lds_base = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)gf4_smem);
    const uint64_t kp16 = (uint64_t)Kp * 16, pp16 = (uint64_t)Pp * 16;
    uint64_t row_off[6];
    unsigned row_dst[6];
#pragma unroll
    for (int q = 0; q < 6; ++q) {
        const int r = wave + 8 * q, opnd = q / 3, rr = r - 24 * opnd;
        const int j = rr >> 2, v = rr & 3;
        row_off[q] = (uint64_t)(j * CQ + v) * (opnd ? pp16 : kp16);
        row_dst[q] = lds_base + opnd * GF4_OPND + rr * 1024;
    }
    Cur lc;
    seek(lc, 0);
    uint64_t ub, vb;                                      // (row, coordinate 0, stage) of the load cursor's patch in U and in V
    auto point = [&]() __attribute__((always_inline)) {
        const uint64_t first = (uint64_t)(6 * lc.row) * CQ + (uint64_t)lc.cst * 4;
        ub = uniform64(reinterpret_cast<uint64_t>(U) + first * kp16 + (uint64_t)lc.kt * (GF4_T * 16));
        vb = uniform64(reinterpret_cast<uint64_t>(V) + first * pp16 + (uint64_t)lc.pt * (GF4_T * 16));
    };
    point();
    const uint64_t stepU = 4 * kp16, stepV = 4 * pp16, rowU = (uint64_t)(5 * CQ + 4) * kp16, rowV = (uint64_t)(5 * CQ + 4) * pp16;
    auto issue = [&](int slot) __attribute__((always_inline)) {
        const unsigned sl = (unsigned)slot * (2 * GF4_OPND);
#pragma unroll
        for (int q = 0; q < 6; ++q)
            dma_row_to((q < 3 ? ub : vb) + row_off[q], lane_off, sl + row_dst[q]);
        const int what = step(lc);                        // past the end: the last stage again (never read)
        if (what == STEP_STAGE) {
            ub += stepU;
            vb += stepV;
        } else if (what == STEP_ROW) {
            ub += rowU;
            vb += rowV;
        } else if (what == STEP_PATCH) {
            point();
        }
    };

    // ---- compute side ----------------------------------------------------------------------------------------
    floatx4 acc[6][2], out[16][2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int j = 0; j < 6; ++j) acc[j][h] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ab = 0; ab < 16; ++ab) out[ab][h] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    const int r_lds = (SWAP ? GF4_OPND : 0) + ((lq * GF4_T) + wr * 32 + l16) * 16;      // row operand: U (V when SWAP)
    const int c_lds = (SWAP ? 0 : GF4_OPND) + ((lq * GF4_T) + wc * 16 + l16) * 16;
    auto multiply = [&](int slot, int wslot) __attribute__((always_inline)) {
        const unsigned char* rbase = gf4_smem + slot * (2 * GF4_OPND) + r_lds;
        const unsigned char* cbase = gf4_smem + slot * (2 * GF4_OPND) + c_lds;
        floatx4 fr[2][2], fc[2];
        auto frag = [&](int j) __attribute__((always_inline)) {
            fr[j & 1][0] = *reinterpret_cast<const floatx4*>(rbase + j * GF4_PLANE);
            fr[j & 1][1] = *reinterpret_cast<const floatx4*>(rbase + j * GF4_PLANE + 256);
            fc[j & 1] = *reinterpret_cast<const floatx4*>(cbase + j * GF4_PLANE);
        };
        frag(0);
#pragma unroll
        for (int j = 0; j < 6; ++j) {
            if (j + 1 < 6) frag(j + 1);
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    acc[j][h] = __builtin_amdgcn_mfma_f32_16x16x4f32(fr[j & 1][h][e], fc[j & 1][e], acc[j][h], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (j == 0) {                                 // the next requests behind the first coordinate's multiplies
                issue(wslot);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    // the six coordinates of row i (complete or not: the fold is linear) into the outputs, accumulators cleared
    auto fold = [&](int i) __attribute__((always_inline)) {
        // column i of A^T = [1 1 1 1 1 0; 0 1 -1 2 -2 0; 0 1 1 4 4 0; 0 1 -1 8 -8 1]
        const float sgn = (i == 2 || i == 4) ? -1.f : 1.f, mag = i >= 3 ? 2.f : 1.f;
        const float c0 = i < 5 ? 1.f : 0.f;
        const float c1 = (i == 0 || i == 5) ? 0.f : sgn * mag;
        const float c2 = (i == 0 || i == 5) ? 0.f : mag * mag;
        const float c3 = i == 0 ? 0.f : (i == 5 ? 1.f : sgn * mag * mag * mag);
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float m0 = acc[0][h][r], m1 = acc[1][h][r], m2 = acc[2][h][r], m3 = acc[3][h][r], m4 = acc[4][h][r],
                            m5 = acc[5][h][r];
                const float s12 = m1 + m2, d12 = m1 - m2, s34 = m3 + m4, d34 = m3 - m4;
                float t[4];
                t[0] = m0 + s12 + s34;
                t[1] = fmaf(2.f, d34, d12);
                t[2] = fmaf(4.f, s34, s12);
                t[3] = fmaf(8.f, d34, d12) + m5;
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    out[b][h][r] = fmaf(c0, t[b], out[b][h][r]);
                    out[4 + b][h][r] = fmaf(c1, t[b], out[4 + b][h][r]);
                    out[8 + b][h][r] = fmaf(c2, t[b], out[8 + b][h][r]);
                    out[12 + b][h][r] = fmaf(c3, t[b], out[12 + b][h][r]);
                }
#pragma unroll
                for (int j = 0; j < 6; ++j) acc[j][h][r] = 0.f;
            }
    };
    // register (ab, h, r) of this thread in a partial-output block
    auto part_at = [&](float* base, int ab, int h, int r) __attribute__((always_inline)) { return base + ((ab * 2 + h) * 4 + r) * 512 + tid; };
    // a contributor's part is complete: its partial outputs to scratch, then the owner's arrival counter
    auto hand_over = [&]() __attribute__((always_inline)) {
        float* mine = part + (size_t)slot_me * GF4_PART;
#pragma unroll
        for (int ab = 0; ab < 16; ++ab)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    __hip_atomic_store(part_at(mine, ab, h, r), out[ab][h][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    out[ab][h][r] = 0.f;
                }
        __builtin_amdgcn_s_waitcnt(0x0F70);               // vmcnt(0): this wave's values have been performed
        __syncthreads();
        if (tid == 0) {
            const long pend = (rb / PL + 1) * PL;         // the patch ends here; its owner holds stage pend - 1
            const int owner = (int)((pend * Sx - 1) / Tx);
            __hip_atomic_fetch_add(&cnt[xcd * Sx + owner], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };
    // the owner of a patch whose beginning lies in the previous workgroups: their partial outputs, in workgroup order
    auto gather = [&]() __attribute__((always_inline)) {
        const long pbeg = ra / PL * PL;                   // the patch begins here, in workgroup `first`
        const int first = (int)(((pbeg + 1) * Sx - 1) / Tx);
        const int want = jw - first;
        if (tid == 0) {
            int spins = 0;
            while (__hip_atomic_load(&cnt[slot_me], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want && spins < spin_limit) {
                __builtin_amdgcn_s_sleep(32);
                ++spins;
            }
            __hip_atomic_store(&cnt[slot_me], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);     // zero for the next launch
        }
        __syncthreads();
        for (int c = first; c < jw; ++c) {
            float* theirs = part + (size_t)(xcd * Sx + c) * GF4_PART;
#pragma unroll
            for (int ab = 0; ab < 16; ++ab)
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        out[ab][h][r] += __hip_atomic_load(part_at(theirs, ab, h, r), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };
    // the outputs of the patch at (k0, p0): bias, ReLU, pooling and stores, outputs cleared
    auto store_patch = [&](int k0, long p0) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int ri = wr * 32 + h * 16 + 4 * lq + r, ci = wc * 16 + l16;        // row and column of the patch
                const int k = k0 + (SWAP ? ci : ri);
                const long p = p0 + (SWAP ? ri : ci);
                float o[4][4];
#pragma unroll
                for (int ab = 0; ab < 16; ++ab) {
                    o[ab >> 2][ab & 3] = out[ab][h][r];
                    out[ab][h][r] = 0.f;
                }
                if (k < K && p < P) {
                    int n, ty, tx;
                    decode_tile(p, order, N, th, tw, n, ty, tx);
                    store_tile_f4<float>(y, ys, n, k, ty, tx, Ho, Wo, o, ep, bias_of<float>(ep, k));
                }
            }
    };

    Cur cc;
    seek(cc, 0);
    constexpr int WAIT_IMM = (6 & 0xF) | (0x7 << 4) | (0xF << 8);          // vmcnt(6): all but this wave's newest stage
    issue(0);
    issue(1);
    int slot = 0;                                         // ring slot of the stage being multiplied (one loop body for all three)
#pragma unroll 1
    for (int s = 0; s < total; ++s) {
        __builtin_amdgcn_s_waitcnt(WAIT_IMM);
        __builtin_amdgcn_s_barrier();                     // the stage landed for every wave; the slot before it is free
        asm volatile("" ::: "memory");
        multiply(slot, slot == 0 ? GF4_RING - 1 : slot - 1);
        const bool seg_end = cc.left == 1, row_end = cc.cst == nst - 1;
        if (seg_end || row_end) {
            fold(cc.row);
            if (seg_end && cc.seg == 0) {
                hand_over();
            } else if (row_end && cc.row == 5) {
                if (cc.seg == 2) gather();
                store_patch(cc.kt * GF4_T, (long)cc.pt * GF4_T);
            }
        }
        step(cc);
        slot = slot == GF4_RING - 1 ? 0 : slot + 1;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                   // the surplus requests of the last stages
}

}  // namespace wino
