// Direct 3x3 convolution of 2-byte NCHW (and, with the template flag further down, NHWC) tensors, the kernel for large
// images (see direct16.hpp for the method):
// one workgroup of 8 waves per CU, tiles of 64*WF filters x 8/WF waves of 4 rows x 32 columns of output pixels, the
// waves side by side until they span the image's width (then stacked).
//
// What binds the 4-wave kernel of direct16.hpp on large layers is the rate at which a CU draws operands from L2
// (a wave that issues a stage's requests waits in the CU's request path for as long as the multiplies of half a
// stage take, and the waves of a workgroup all issue at once), so this one moves fewer bytes per multiply, asks for
// them earlier, and lets its waves take turns:
//   * WF = 2: 128 filters share a block's input (the two filter halves are two groups of 4 waves), 59 KB per stage
//     and CU instead of 82 KB;
//   * the 160 KB of LDS hold a ring of THREE filter stages and two input stages: the filter rows of stage s+2 are
//     requested during stage s and have a whole stage to arrive, and so has the input of stage s+2, which waits in
//     registers until it is written to LDS during stage s+1;
//   * every wave owns 4 consecutive output rows of one image (the host offers the kernel when Ho is a multiple of
//     4), so pixel group j, filter row r reads input row j + r of the wave's six: a pixel fragment is fetched once
//     and multiplied into up to three groups (18 pixel fragments per stage instead of 36);
//   * a wave does everything that is not a multiply (LDS writes of the input it holds, its requests) in one go,
//     once per stage, at one of four points of the stage that differs between the two waves of a SIMD: the other
//     wave multiplies meanwhile, and only two waves of the CU issue requests at a time;
//   * a block spans the image's width where 8/WF waves of 32 columns can (W <= 256 / WF): the rows a block needs are
//     then one contiguous run of each channel plane, and a wave's request covers whole cache lines (a request that
//     touches four 72-byte pieces of four rows costs 190 clocks of the CU's request path, a contiguous one 58).
// Ring positions are runtime offsets (two additions per stage), so there is one stage body for all tiles.
#pragma once
#include "direct16.hpp"

namespace wino {

// DIL: the tensors are [C][H][W][N] (CHWN).  A channel plane row of such a tensor is W * N contiguous elements in
// which the horizontal neighbours of a pixel lie N elements away: the layer is a convolution of ONE image of width
// W * N with the tap columns N elements apart and N * pad zeros on either side of a row, and that is how the kernel
// runs it -- the same loads (neighbouring elements of a row in pairs: two images), the same stores, the tap columns
// of a fragment g.ds pixel slots apart instead of one.  The halo of a block's rows is 2 N slots wide, so an input
// stage is larger (6 rows x (128 + 2 N) slots with 128-filter tiles) and the filter ring is two deep instead of three.
template <int WF, bool DIL = false> struct D16R {
    static constexpr int KT = 64 * WF;                       // filters per tile
    static constexpr int WP = 8 / WF;                        // waves along the rows of a block
    static constexpr int FB = 9 * 2 * KT * 16;               // bytes of a filter stage: [tap][channel vector][KT] vectors
    static constexpr int XPLANE = DIL ? (WF == 2 ? 1152 : 1920) : (WF == 2 ? 704 : 1360);   // pixel slots per channel-vector plane (LR * PW must fit)
    static constexpr int XB = 2 * XPLANE * 16;               // bytes of an input stage
    static constexpr int NFR = DIL ? 2 : 3;                  // filter stages in the ring
    static constexpr int LDS = NFR * FB + 2 * XB;
    static constexpr int FROWS = 18 * WF;                    // 1 KB rows of a filter stage
    static constexpr int NF = (FROWS + 7) / 8;               // filter requests per wave and stage (some rows twice)
    static constexpr int NTASK = DIL ? (WF == 2 ? 3 : 4) : (WF == 2 ? 2 : 3);   // input tasks per thread and stage
};
static_assert(D16R<1, true>::LDS <= 160 * 1024 && D16R<2, true>::LDS <= 160 * 1024, "LDS of the CHWN instantiations");

// XN: x is [N][H][W][C].  The 8 channels of a pixel's vector are 16 contiguous bytes of x: an input task is one pixel
// slot of one channel vector (a 16-byte load, a 16-byte LDS write, zeros where the slot lies outside the image), the
// two vectors of a pixel on neighbouring lanes.  YN: y is [N][Ho][Wo][K].  The multiplies take the pixel fragment as
// the first operand, so a lane holds one FILTER and its registers the pixels: the 32 filters of a wave's half are 64
// contiguous bytes of a pixel of y.  The two are independent: a layer may read one layout and write the other.
template <typename T, int WF, bool XN = false, bool YN = XN, bool DIL = false>
__global__ __launch_bounds__(512, 1) void direct16_rows_kernel(const T* __restrict__ x, const T* __restrict__ W9,
                                                               T* __restrict__ y, D16Geom g, Epilogue ep) {
    typedef typename Mma<T>::vec vec;
    typedef D16R<WF, DIL> P;
    static_assert(!DIL || (!XN && !YN), "CHWN tensors on both sides");
    constexpr int NTASK = XN ? (2 * P::XPLANE + 511) / 512 : P::NTASK;   // input tasks per thread and stage
    constexpr int NX = XN ? NTASK : 8 * NTASK;                           // and the requests they make
    extern __shared__ __attribute__((aligned(16))) unsigned char d16r_smem[];     // [NFR][FB] filters, [2][XB] input
    unsigned char* const xsm = d16r_smem + P::NFR * P::FB;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wf = wave / P::WP, wp = wave % P::WP;          // filter half; position in the block: g.WC waves side by side
    const int wr = wp / g.WC, wc = wp - wr * g.WC;
    const int l32 = lane & 31, lh = lane >> 5;
    const int HW = g.H * g.W, Hp = g.Ho + 2;
    const int nst = g.CQ / 2;                                // stages of 16 channels per tile

    // ---- this workgroup's tiles: sequence items s = s0, s0 + sstep, ... < send of its XCD ------------------
    const int xcd = blockIdx.x & 7;
    const int sstep = gridDim.x >> 3;
    const int npb = g.colBlocks * g.rowBlocks;               // pixel blocks; block pbx*8 + xcd belongs to this XCD
    const int send = ((npb - xcd + 7) >> 3) * g.kTiles;
    const int s0 = (int)(blockIdx.x >> 3);
    if (s0 >= send) return;
    struct Tile {
        int k0, c0, n0, oh0, R;                              // R: output rows per wave, 4 or 3
    };
    // Row blocks: runs of BR = 4 S rows (S waves stacked) over the N * Ho rows of the batch; or, with g.b3 > 0, every
    // image cut into g.a4 blocks whose waves own 4 rows and g.b3 blocks whose waves own 3 (Ho = S (4 a4 + 3 b3)), all
    // the 4-row blocks first in the sequence: the host mixes the two so that the layer's tiles fill their rounds of the
    // chip evenly (a 3-row tile is the same stage loop less the multiplies of the fourth row).
    auto decode = [&](int s) {
        const int pbx = s / g.kTiles, kt = s - pbx * g.kTiles;
        const int pb = pbx * 8 + xcd;
        const int rb = pb / g.colBlocks, cb = pb - rb * g.colBlocks;
        if (g.b3 > 0) {
            const int n4 = g.N * g.a4;
            if (rb < n4) {
                const int n0 = rb / g.a4;
                return Tile{kt * P::KT, cb * g.BC, n0, (rb - n0 * g.a4) * g.BR, 4};
            }
            const int q = rb - n4, n0 = q / g.b3;
            return Tile{kt * P::KT, cb * g.BC, n0, g.a4 * g.BR + (q - n0 * g.b3) * (g.BR / 4 * 3), 3};
        }
        const long g0 = (long)rb * g.BR;
        const int n0 = (int)(g0 / g.Ho);
        return Tile{kt * P::KT, cb * g.BC, n0, (int)(g0 - (long)n0 * g.Ho), 4};
    };

    // ---- input tasks of this thread: (channel vector v, LDS row, column pair); what does not depend on the tile ----
    const int ntask = XN ? 2 * g.LR * g.PW : 2 * g.LR * g.PP;
    int tpk[NTASK];                                          // LDS row | (first column of the pair relative to c0, + 8) << 8 | v << 20
    int ldsw[NTASK];                                         // byte offset of the pair's first slot inside an input stage (a multiple of
                                                             // 16, -16 for the pair left of a row) | bit 0 / 1: slot 0 / 1 exists;
                                                             // neither: no task
#pragma unroll
    for (int q = 0; q < NTASK; ++q) {
        const int t = tid + 512 * q;
        if constexpr (XN) {
            // task t: channel vector t & 1 of pixel slot t >> 1 (row-major over the LR x PW slots of a plane)
            // (tid + 512 q: the vector is the same for all tasks of a thread; row and column are recomputed per tile)
            tpk[q] = 0;
            ldsw[q] = t < ntask ? ((((t & 1) * P::XPLANE + (t >> 1)) * 16) | 1) : 0;
            continue;
        }
        const int m = t % g.PP, rr = t / g.PP;
        const int lr = rr % g.LR, v = min(rr / g.LR, 1);
        // padw zero columns left of a row (pad, or N * pad for CHWN); pairs start at even columns of the image:
        // the pair (c0 + 2m - 2 ceil(padw / 2), + 1) sits in slots (2m - padw % 2, + 1)
        const int padw = g.pad * g.ds, hp = (padw + 1) >> 1;
        const int slot0 = 2 * m - (padw & 1);
        tpk[q] = lr | (2 * m - 2 * hp + 64) << 8 | v << 20;
        const int wbits = (slot0 >= 0 && slot0 < g.PW ? 1 : 0) | (slot0 + 1 >= 0 && slot0 + 1 < g.PW ? 2 : 0);
        ldsw[q] = t < ntask ? (((v * P::XPLANE + lr * g.PW + slot0) * 16) | wbits) : 0;
    }

    // ---- request cursors: the stage whose input is requested next, and the stage whose filters are ----------------
    struct Cursor {
        int s, cs;
        bool valid;
    };
    auto advance = [&](Cursor& c) {
        if (++c.cs == nst) {
            c.cs = 0;
            c.s += sstep;
            c.valid = c.s < send;
        }
    };
    Cursor cx{s0, 0, true}, cf{s0, 0, true};
    unsigned xoff[NTASK];                                    // byte offset from (image n0, the stage's first channel), a multiple
                                                             // of 4 | bit 0: the pair lies inside the image
    const char* xs = nullptr;                                // image n0, first channel of the stage to request
    const unsigned hw2 = (unsigned)(HW * 2);
    auto prep_x = [&](const Tile& t) {
#pragma unroll
        for (int q = 0; q < NTASK; ++q) {
            const int sl = min((tid + 512 * q) >> 1, g.LR * g.PW - 1);           // NHWC source: the task's pixel slot
            const int lr = XN ? sl / g.PW : tpk[q] & 0xFF, v = XN ? tid & 1 : tpk[q] >> 20;
            const int qq = t.oh0 + lr;                       // padded row index counted from image n0
            int dn = 0;
            for (int k = 1; k <= g.maxcross; ++k) dn += qq >= k * Hp ? 1 : 0;
            const int ih = qq - dn * Hp - g.pad;
            if constexpr (XN) {
                const int iw = t.c0 + (sl - lr * g.PW) - g.pad;
                const bool in = (ldsw[q] & 3) != 0 && t.n0 + dn < g.N && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
                const int ihc = min(max(ih, 0), g.H - 1), iwc = min(max(iw, 0), g.W - 1);
                const int dnc = max(min(dn, g.N - 1 - t.n0), 0);
                xoff[q] = ((unsigned)(((dnc * g.H + ihc) * g.W + iwc) * g.C + v * 8) * 2u) | (in ? 1u : 0u);   // a multiple of 16
                continue;
            }
            const int iw = t.c0 + ((tpk[q] >> 8) & 0xFFF) - 64;
            const bool in = (ldsw[q] & 3) != 0 && t.n0 + dn < g.N && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
            const int ihc = min(max(ih, 0), g.H - 1), iwc = min(max(iw, 0), g.W - 2);
            const int dnc = min(dn, g.N - 1 - t.n0);
            xoff[q] = ((unsigned)((dnc * g.C * g.H + ihc) * g.W + iwc) * 2u + (unsigned)v * 8u * hw2) | (in ? 1u : 0u);
        }
        xs = reinterpret_cast<const char*>(x) + (size_t)t.n0 * g.C * HW * 2;
    };
    // filter rows: request q of this wave moves row (wave + 8q) % FROWS = (tap*2 + v)*WF + half of the stage
    const unsigned lane_off = lane * 16;
    unsigned frow_src[P::NF];                                // byte offset of the row inside W9, relative to (k0, stage 0)
    int frow_dst[P::NF];                                     // and inside a filter stage of LDS
#pragma unroll
    for (int q = 0; q < P::NF; ++q) {
        const int r = (wave + 8 * q) % P::FROWS;
        const int tap = r / (2 * WF), v = (r / WF) & 1, half = r % WF;
        frow_src[q] = (unsigned)(((tap * g.CQ + v) * g.Kp + half * 64) * 16);
        frow_dst[q] = r * 1024;
    }
    const char* const w9b = reinterpret_cast<const char*>(W9);
    const unsigned fstep = (unsigned)(2 * g.Kp * 16);
    auto f_request = [&](const Cursor& c, int slot) {        // the filter rows of stage c into ring slot `slot`
        const int pbx = c.s / g.kTiles, kt = c.s - pbx * g.kTiles;
        const uint64_t base = reinterpret_cast<uint64_t>(w9b) + (uint64_t)kt * P::KT * 16 + (uint64_t)c.cs * fstep;
#pragma unroll
        for (int q = 0; q < P::NF; ++q) dma_row(base + frow_src[q], lane_off, d16r_smem + slot * P::FB + frow_dst[q]);
    };
    uint32_t raw[XN ? 1 : NTASK][8];
    uint4 rawn[XN ? NTASK : 1];                            // NHWC source: the 8 channels of a task's pixel
    unsigned poff[NTASK];
    int req_cs = 0;                                          // the stage (inside its tile) whose input was requested last
    // piece 8q + e of a stage's input requests: channel e of task q.  A stage's second channel vector may lie past
    // C: the first one is loaded instead, and masked when it is written
    auto x_piece = [&](int idx) {
        if (idx == 0) req_cs = cx.cs;
        if constexpr (XN) {
            const int v = tid & 1;
            const bool vok = cx.cs * 16 + v * 8 < g.C;
            rawn[XN ? idx : 0] = *reinterpret_cast<const uint4*>(xs + ((xoff[idx] & ~15u) - (vok ? 0u : (unsigned)v * 16u)));
            return;
        }
        const int q = idx >> 3, e = idx & 7;
        if (e == 0) {
            const int v = tpk[q] >> 20;
            const bool vok = cx.cs * 16 + v * 8 < g.C;
            poff[q] = (xoff[q] & ~3u) - (vok ? 0u : (unsigned)v * 8u * hw2);
        }
        raw[XN ? 0 : q][e] = *reinterpret_cast<const uint32_t*>(xs + poff[q]);
        poff[q] += hw2;
    };
    auto x_commit = [&](int xslot) {                         // the stage requested through x_piece into input slot xslot
#pragma unroll
        for (int q = 0; q < NTASK; ++q) {
            if ((ldsw[q] & 3) == 0) continue;
            const bool keep = (xoff[q] & 1u) && req_cs * 16 + (XN ? tid & 1 : tpk[q] >> 20) * 8 < g.C;
            const uint32_t km = keep ? 0xFFFFFFFFu : 0u;
            if constexpr (XN) {
                const uint4 r = rawn[XN ? q : 0];
                *reinterpret_cast<uint4*>(xsm + xslot * P::XB + (ldsw[q] & ~15)) = make_uint4(r.x & km, r.y & km, r.z & km, r.w & km);
                continue;
            }
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t a = raw[XN ? 0 : q][2 * e] & km, b = raw[XN ? 0 : q][2 * e + 1] & km;
                lo[e] = __builtin_amdgcn_perm(b, a, 0x05040100u);     // (a.lo16, b.lo16): the pair's first pixel
                hi[e] = __builtin_amdgcn_perm(b, a, 0x07060302u);     // (a.hi16, b.hi16): its second pixel
            }
            unsigned char* dst = xsm + xslot * P::XB + (ldsw[q] & ~15);
            if (ldsw[q] & 1) *reinterpret_cast<uint4*>(dst) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            if (ldsw[q] & 2) *reinterpret_cast<uint4*>(dst + 16) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        }
    };

    // ---- the tile being multiplied ------------------------------------------------------------------------------
    int xw_off = 0;                                          // the wave's first input row, this lane's column: byte offset in an input stage
    int yoff[4];                                             // element offset of (n, k0, oh, ow) in y per row of the wave, < 0: no pixel
    int k0c = 0;                                             // first filter of this wave
    int pc0 = 0;                                             // NHWC: first output column of this wave
    bool r4 = true;                                          // the waves of the tile own 4 rows (else 3: row 3 of a wave is not computed, not stored)
    auto prep_pix = [&](const Tile& t) {
        k0c = t.k0 + wf * 64;
        r4 = t.R == 4;
        const long g0 = (long)t.n0 * g.Ho + t.oh0;
        // DIL with pooling (32 images: a column group of 32 is one pixel column): a wave takes 16 images of TWO
        // neighbouring pixel columns, lanes 0-15 the even one, so that a pooling window's columns are lanes 16 apart;
        // the two waves of a pair take the two halves of the images
        const int col = DIL && ep.pool ? ((wc & ~1) + ((l32 >> 4) & 1)) * 32 + 16 * (wc & 1) + (l32 & 15) : 32 * wc + l32;
        const bool colok = t.c0 + col < g.Wo;
        const int ohp = t.oh0 + t.R * wr;                    // the wave's rows lie in one image: Ho is a multiple of 4 (of a block's rows, with 3-row blocks mixed in)
        int dn = 0;
        for (int k = 1; k <= g.maxcross; ++k) dn += ohp >= k * g.Ho ? 1 : 0;
        const int oh = ohp - dn * g.Ho;
        const bool rowok = g0 + t.R * wr < g.G;
        const int L = rowok ? dn * Hp + oh - t.oh0 : 0;
        xw_off = ((lh * P::XPLANE) + L * g.PW + (colok ? col : 0)) * 16;
        if constexpr (YN) {
            // element offset of (n, oh + j, the wave's first column, the wave's first filter); the lane's filter and
            // the register's column are added at the stores
            pc0 = t.c0 + 32 * wc;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                yoff[j] = rowok ? (int)((((long)(t.n0 + dn) * g.Ho + oh + j) * g.Wo + pc0) * g.K + k0c) : -1;
            if (ep.pool && rowok) {                          // the two pooled rows of the wave, its first pooled column
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    yoff[j] = (int)((((long)(t.n0 + dn) * (g.Ho >> 1) + (oh >> 1) + j) * (g.Wo >> 1) + (pc0 >> 1)) * g.K + k0c);
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            yoff[j] = (rowok && colok) ? (int)((((long)(t.n0 + dn) * g.K + k0c) * g.Ho + oh + j) * g.Wo + t.c0 + col) : -1;
        if (ep.pool && rowok && colok) {
            // 2x2 pooling: the wave's rows are two pooling rows (Ho is a multiple of 4), a lane pair is one pooling
            // column (Wo is even); yoff[0], yoff[1]: the two pooled rows, this pair's column
            const int Hq = g.Ho >> 1, Wq = g.Wo >> 1;
            // (DIL: column = 32 pixel column + image; the pooled row holds 32 (pixel column / 2) + image)
            const int pcol = DIL ? (((t.c0 + col) >> 6) << 5) + ((t.c0 + col) & 31) : (t.c0 + col) >> 1;
#pragma unroll
            for (int j = 0; j < 2; ++j)
                yoff[j] = (int)((((long)(t.n0 + dn) * g.K + k0c) * Hq + (oh >> 1) + j) * Wq + pcol);
        }
    };

    floatx16 acc[2][4];
    // ---- one stage of multiplies: 18 steps (filter column s, input row rho), each one pixel fragment and 2 to 6
    // multiplies.  The order is pinned: the pixel fragment of step t+2 and the filter fragments that the following
    // steps need are requested before the multiplies of step t, filter row r of the next column as soon as its last
    // use has issued.  service() -- everything else this wave does in a stage -- runs before step 0, 5, 9 or 14.
    auto compute = [&](int fslot, int xslot, int site, auto&& service) {
        const unsigned char* fs = d16r_smem + fslot * P::FB + (lh * P::KT + wf * 64 + l32) * 16;
        const unsigned char* xrow[6];                        // the wave's six input rows, this lane's column
#pragma unroll
        for (int r = 0; r < 6; ++r) xrow[r] = xsm + xslot * P::XB + xw_off + r * g.PW * 16;
        vec a[3][2], b[3];
        auto lda = [&](int r, int s) {
#pragma unroll
            for (int i = 0; i < 2; ++i) a[r][i] = *reinterpret_cast<const vec*>(fs + (3 * r + s) * (2 * P::KT * 16) + i * 512);
        };
        const int dsb = g.ds * 16;                           // bytes between the tap columns of a fragment
        auto ldb = [&](int t) { b[t % 3] = *reinterpret_cast<const vec*>(xrow[t % 6] + (DIL ? (t / 6) * dsb : (t / 6) * 16)); };
        lda(0, 0);
        ldb(0);
        lda(1, 0);
        ldb(1);
        lda(2, 0);
        auto step = [&](int t) {
            const int s = t / 6, rho = t % 6;
            if (t + 2 < 18) ldb(t + 2);
            if (rho == 4 && s < 2) lda(0, s + 1);
            if (rho == 5 && s < 2) lda(1, s + 1);
            if (rho == 0 && s > 0) lda(2, s);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int r = rho - j;
                if (r < 0 || r > 2) continue;
                if (j == 3 && !r4) continue;                 // (uniform)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    if constexpr (YN) Mma<T>::run(b[t % 3], a[r][i], acc[i][j]);
                    else Mma<T>::run(a[r][i], b[t % 3], acc[i][j]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        // (four short loops: one loop of 18 steps around the service code is more than the compiler unrolls)
        constexpr int SITE_STEP[5] = {0, 5, 9, 14, 18};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if (site == k) service();
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = SITE_STEP[k]; t < SITE_STEP[k + 1]; ++t) step(t);
        }
    };

    // ---- stores: register r of acc[i][j] is filter k0c + 32*i + 8*(r/4) + 4*lh + r%4, the lane's pixel of row j ----
    // Offsets into y are 32-bit element offsets (the host checks the tensor size) that run along with the filter
    // index: from one register pair to the next the filter advances by 2 or by 6.  Rows of y have an even length and
    // y is 4-byte aligned (the host checks): two neighbouring lanes hold neighbouring columns and exchange values, so
    // that each stores one 4-byte pair -- the even lane for filter r, the odd lane for filter r+1.
    // K is a multiple of 64 (the host checks), so a wave's 64 filters exist or the wave has none.  The four rows of
    // a wave exist together, so a lane stores all its values or none.
    const unsigned kstride2 = (ep.pool ? (unsigned)((g.Ho >> 1) * (g.Wo >> 1)) : (unsigned)(g.Ho * g.Wo)) * 2u;   // bytes between the planes of two filters
    const bool odd = lane & 1;
    const unsigned psel = odd ? 0x03020706u : 0x05040100u;   // (own pair, neighbour's pair) -> even lanes: both lanes' first value; odd lanes: both lanes' second
    auto stores = [&]() {
        if (k0c >= g.K || yoff[0] < 0) return;
        // (opaque to the optimiser: called from inside the stage loop, the 64 store addresses of a tile would be
        // loop invariants, computed ahead of the loop and kept in registers)
        unsigned ks = kstride2;
        asm volatile("" : "+s"(ks));
        char* const yb = reinterpret_cast<char*>(y);
        if constexpr (YN) {
            // register r of acc[i][j]: pixel column pc0 + 8*(r/4) + 4*lh + r%4 of row j, the lane's filter
            // k0c + 32*i + l32.  Two neighbouring lanes hold neighbouring filters and exchange values, so that each
            // stores one 4-byte pair of filters -- the even lane for the pixel of register r, the odd lane for that of
            // register r+1: per instruction the 16 even (odd) lanes of a half write 64 contiguous bytes of one pixel.
            unsigned kp = (unsigned)g.K * 2u;                // bytes between two pixels of y
            asm volatile("" : "+s"(kp));
            // (the two filter halves of a pixel, 64 + 64 bytes of one 128-byte line, are stored one right after the other)
            float bk[2] = {0.f, 0.f};
            if (ep.bias) {
                bk[0] = bias_of<T>(ep, k0c + l32);
                bk[1] = bias_of<T>(ep, k0c + 32 + l32);
            }
            if (ep.pool) {
                // a 2x2 window is two rows of the wave and two neighbouring registers of a lane: the maximum is taken in
                // registers and the lane stores its filter's pooled value (2 bytes; 32 lanes: 64 contiguous bytes)
                unsigned q[2];
#pragma unroll
                for (int j = 0; j < 2; ++j) q[j] = ((unsigned)yoff[j] + (unsigned)l32) * 2u + (unsigned)(2 * lh) * kp;
#pragma unroll
                for (int r2 = 0; r2 < 16; r2 += 2) {
                    const bool pok = pc0 + 8 * (r2 >> 2) + 4 * lh + (r2 & 3) < g.Wo;
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
#pragma unroll
                        for (int i = 0; i < 2; ++i) {
                            float v = fmaxf(fmaxf(acc[i][2 * j][r2], acc[i][2 * j][r2 + 1]), fmaxf(acc[i][2 * j + 1][r2], acc[i][2 * j + 1][r2 + 1])) + bk[i];
                            if (ep.relu) v = fmaxf(v, 0.f);
                            if (pok) *reinterpret_cast<T*>(yb + q[j] + (unsigned)(i * 64)) = from_f32<T>(v);
                        }
                        q[j] += ((r2 & 2) ? 3u : 1u) * kp;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                return;
            }
            unsigned o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = ((unsigned)yoff[j] + (unsigned)(l32 - (odd ? 1 : 0))) * 2u + (unsigned)(4 * lh + (odd ? 1 : 0)) * kp;
#pragma unroll
            for (int r2 = 0; r2 < 16; r2 += 2) {
                const bool pok = pc0 + 8 * (r2 >> 2) + 4 * lh + (r2 & 3) < g.Wo;    // (Wo is even: the pair's pixels exist together)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (j == 3 && !r4) continue;             // (uniform: a 3-row tile)
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        float v0 = acc[i][j][r2] + bk[i], v1 = acc[i][j][r2 + 1] + bk[i];
                        if (ep.relu) { v0 = fmaxf(v0, 0.f); v1 = fmaxf(v1, 0.f); }
                        // (rounded and packed first; the neighbour's pair by one DPP move, the lane's two by one byte permute)
                        const unsigned own = pack2<T>(v0, v1);
                        const unsigned nb = (unsigned)__builtin_amdgcn_mov_dpp((int)own, 0xB1, 0xF, 0xF, true);
                        if (pok) *reinterpret_cast<unsigned*>(yb + o[j] + (unsigned)(i * 64)) = __builtin_amdgcn_perm(nb, own, psel);
                    }
                    o[j] += ((r2 & 2) ? 6u : 2u) * kp;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            return;
        }
        if (ep.pool) {
            // with pooling: the maximum over the two rows in registers, over the two columns with the neighbouring lane;
            // the even lane stores the pooled value of filter r, the odd lane that of filter r+1 (2 bytes each)
            // (DIL: the window's other column is 16 lanes away; lanes 0-15 store filter r, lanes 16-31 filter r+1)
            const bool second = DIL ? (l32 & 16) != 0 : odd;
            unsigned q[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) q[j] = (unsigned)yoff[j] * 2u + (unsigned)(4 * lh + (second ? 1 : 0)) * ks;
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int r2 = 0; r2 < 16; r2 += 2) {
                    const int kk = 32 * i + 8 * (r2 >> 2) + 4 * lh + (r2 & 3);
                    float b0 = 0.f, b1 = 0.f;
                    if (ep.bias) {
                        b0 = bias_of<T>(ep, k0c + kk);
                        b1 = bias_of<T>(ep, k0c + kk + 1);
                    }
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        float v0 = fmaxf(acc[i][2 * j][r2], acc[i][2 * j + 1][r2]) + b0;
                        float v1 = fmaxf(acc[i][2 * j][r2 + 1], acc[i][2 * j + 1][r2 + 1]) + b1;
                        if (ep.relu) { v0 = fmaxf(v0, 0.f); v1 = fmaxf(v1, 0.f); }
                        if constexpr (DIL) {
                            v0 = fmaxf(v0, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v0), 0x401F)));   // lane ^ 16
                            v1 = fmaxf(v1, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v1), 0x401F)));
                        } else {
                            v0 = fmaxf(v0, swap_lane_pairs(v0));
                            v1 = fmaxf(v1, swap_lane_pairs(v1));
                        }
                        *reinterpret_cast<T*>(yb + q[j]) = from_f32<T>(second ? v1 : v0);
                        q[j] += ((r2 & 2) ? 6u : 2u) * ks;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            return;
        }
        unsigned o[4];                                       // byte offsets: a scalar base and a 32-bit offset per store
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = ((unsigned)yoff[j] - (odd ? 1u : 0u)) * 2u + (unsigned)(4 * lh + (odd ? 1 : 0)) * ks;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r2 = 0; r2 < 16; r2 += 2) {
                const int kk = 32 * i + 8 * (r2 >> 2) + 4 * lh + (r2 & 3);     // filter of register r2; r2 + 1: the next one
                float b0 = 0.f, b1 = 0.f;
                if (ep.bias) {
                    b0 = bias_of<T>(ep, k0c + kk);
                    b1 = bias_of<T>(ep, k0c + kk + 1);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (j == 3 && !r4) continue;             // (uniform: a 3-row tile)
                    float v0 = acc[i][j][r2] + b0, v1 = acc[i][j][r2 + 1] + b1;
                    if (ep.relu) { v0 = fmaxf(v0, 0.f); v1 = fmaxf(v1, 0.f); }
                    const unsigned own = pack2<T>(v0, v1);
                    const unsigned nb = (unsigned)__builtin_amdgcn_mov_dpp((int)own, 0xB1, 0xF, 0xF, true);
                    *reinterpret_cast<unsigned*>(yb + o[j]) = __builtin_amdgcn_perm(nb, own, psel);
                    o[j] += ((r2 & 2) ? 6u : 2u) * ks;
                }
                __builtin_amdgcn_sched_barrier(0);           // one register pair at a time
            }
    };

    // the filters of the stage after the next, into the ring slot that was read last in the previous stage (a ring of
    // two: the next stage's, into the other slot)
    auto f_next = [&](int fslot) {
        if (!cf.valid) return false;
        f_request(cf, P::NFR == 2 ? fslot ^ 1 : (fslot == 0 ? 2 : fslot - 1));
        advance(cf);
        return true;
    };
    auto zero_acc = [&]() {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
    };
    // wait until at most `newest` of this wave's memory requests are outstanding (loads return in order, so those
    // are the ones issued last), and for its LDS writes; then the workgroup's barrier
    auto wait_only = [&](int newest) {
        if (newest == 0) __builtin_amdgcn_s_waitcnt(0x0070);
        else if (newest == P::NF) __builtin_amdgcn_s_waitcnt(0x0070 | P::NF);
        else if (newest == NX) __builtin_amdgcn_s_waitcnt(0x0070 | (NX & 0xF) | ((NX >> 4) << 14));
        else __builtin_amdgcn_s_waitcnt(0x0070 | ((NX + P::NF) & 0xF) | (((NX + P::NF) >> 4) << 14));
        asm volatile("" ::: "memory");
    };
    auto wait_barrier = [&](int newest) {
        wait_only(newest);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    // ---- prologue: filters of the first two stages, input of the first, requests for the second ----------------------
    // A stage is one pass of all 8 waves over its 18 steps and one barrier.  Each wave interrupts its multiplies once
    // per stage, at a step that differs between the two waves of a SIMD and between the SIMDs, to do everything
    // else: write the input it requested one stage earlier to LDS (stage s+1), request its share of the input of
    // stage s+2 and of the filters of stage s+2.  While it does, the other wave of its SIMD multiplies, and only two
    // waves of the CU issue requests at a time (8 waves that issue together wait for each other in the CU's
    // request path for longer than the requests take).  The hardware issues the older wave of a SIMD first, so waves
    // 0-3 run ahead of waves 4-7 inside a stage: the younger ones take the two early points (they would wait for the
    // pipe there anyway), the older ones the two late ones (measured against the mixed assignment: 4-8 % on the
    // layers with C >= 128 and K >= 256, 2-4 % slower on the 64-channel ones).
    const int site = (wave >> 2) == 0 ? 2 + (wave & 1) : (wave & 1);
    f_request(cf, 0);
    advance(cf);
    if (P::NFR > 2 && cf.valid) {
        f_request(cf, 1);
        advance(cf);
    }
    bool pending = false;                                    // a requested stage waits in registers
    bool need_prep = true;                                   // the stage to request next opens a tile
    auto x_request = [&]() {
        if (need_prep) {
            prep_x(decode(cx.s));
            need_prep = false;
        }
#pragma unroll
        for (int i = 0; i < NX; ++i) x_piece(i);
        pending = true;
        xs += XN ? (size_t)32 : (size_t)16 * HW * 2;                           // the next 16 channels
        advance(cx);
        need_prep = cx.cs == 0;
    };
    x_request();
    x_commit(0);
    pending = false;
    if (cx.valid) x_request();
    wait_barrier(pending ? NX : 0);

    int fslot = 0, xslot = 0;
    const int ntiles = (send - s0 + sstep - 1) / sstep;
    int s = s0, cs = 0;
    const int total = ntiles * nst;
#pragma unroll 1
    for (int it = 0; it < total; ++it) {
        if (cs == 0) {
            prep_pix(decode(s));
            zero_acc();
        }
        bool xreq = false, freq = false;
        compute(fslot, xslot, site, [&]() {
            if (pending) {
                x_commit(xslot ^ 1);
                pending = false;
            }
            // (a filter ring of two: the filters requested now are read in the next stage, so they go first and
            // only the input requests may still be on their way at the stage's end)
            if (P::NFR == 2) f_next(fslot);
            if (cx.valid) {
                x_request();
                xreq = true;
            }
            if (P::NFR > 2) freq = f_next(fslot);
        });
        const int newest = (xreq ? NX : 0) + (freq ? P::NF : 0);
        if (cs == nst - 1) {
            wait_only(newest);                               // before the stores: they would count as the newest requests
            stores();
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else {
            wait_barrier(newest);
        }
        fslot = fslot == P::NFR - 1 ? 0 : fslot + 1;
        xslot ^= 1;
        if (++cs == nst) {
            cs = 0;
            s += sstep;
        }
    }
}

}  // namespace wino
