// Direct 3x3 convolution for layers with at most 4 input channels (the first layer of a VGG-style
// network: C = 3).  The reference sends that layer through the same Winograd wrappers as every other one
// (comparison/layoutCompare.cu:38-46, layer 1: 3 -> 64 channels at 224x224); here AUTO takes it out of
// the Winograd path, because with C <= 4 the channel reduction of a Winograd coordinate is shorter
// than one MFMA's k-depth pair, the transforms and the per-patch fold and stores dominate, and the
// layer is bound by writing y anyway.
//
// The whole reduction is one short GEMM per output pixel: y[k][q] = sum_kk W[k][kk] * X[kk][q],
// kk = (c, r, s) < 9*C <= 36, as NE = ceil(9*C/2) v_mfma_f32_32x32x2_f32 per 32 filters x 32 pixels
// (2-byte tensors are converted on load and multiplied in fp32 as well).  Lanes run along the
// pixels in the order in which y is contiguous (w for NCHW, n for CHWN), filters along registers, so
// a store instruction writes 128 contiguous bytes per filter; for NHWC destinations the two MFMA operands
// swap roles (SWAP: filters along lanes, pixels along registers; y offset = pixel index * K + k).  The filter bank is staged once per
// workgroup in LDS in MFMA operand order; the pixel operand is gathered from x with clamped
// addresses and masked (zero padding) -- neighbouring lanes read neighbouring elements.
#pragma once
#include "common.hpp"
#include "gemm.hpp"

namespace wino {

constexpr int DIRECT_MAX_GROUPS = 8;       // 32-pixel groups per wave: the host picks 1..8 so that the grid fills the chip

// bytes of LDS the kernel needs for a layer, or 0 when the layer does not qualify
__host__ inline size_t direct_lds_bytes(int C, int K) {
    if (C < 1 || C > 4) return 0;
    const size_t ne = (9 * C + 1) / 2, kt = (K + 31) / 32;
    return kt * ne * 64 * sizeof(float) + kt * 32 * sizeof(float);
}

template <typename T, int NE, bool SWAP>
__global__ __launch_bounds__(256) void direct_small_c_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                             T* __restrict__ y, ActStrides xs, FltStrides ws,
                                                             ActStrides ys, int N, int C, int K, int H, int W, int pad,
                                                             int Ho, int Wo, int batch_minor, long Q, int groups,
                                                             Epilogue ep) {
    extern __shared__ float smem[];
    const int KT = (K + 31) / 32;
    float* sW = smem;                         // [KT][NE][64]: lane (lh, l32) holds W[kt*32 + l32][2e + lh]
    float* sB = smem + (size_t)KT * NE * 64;  // [KT*32] bias
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int nk = 9 * C;

    for (int i = tid; i < KT * NE * 64; i += 256) {
        const int ln = i & 63, e = (i >> 6) % NE, kt = (i >> 6) / NE;
        const int k = kt * 32 + (ln & 31), kk = 2 * e + (ln >> 5);
        const bool ok = k < K && kk < nk;
        const int c = kk / 9, r = (kk % 9) / 3, s = kk % 3;
        const float v = to_f32(w[ok ? k * ws.k + c * ws.c + r * ws.r + s * ws.s : 0]);
        sW[i] = ok ? v : 0.f;
    }
    for (int i = tid; i < KT * 32; i += 256) sB[i] = i < K ? bias_of<T>(ep, i) : 0.f;

    // this lane's share of the reduction index: kk = 2e + lh -> (c, r, s); element offset of that tap
    // relative to the pixel's top-left tap, and the tap's row / column for the padding test
    int off[NE];
    unsigned rs[NE];                          // r | s << 2 | (kk real) << 4
#pragma unroll
    for (int e = 0; e < NE; ++e) {
        const int kk = 2 * e + lh;
        const int c = kk / 9, r = (kk % 9) / 3, s = kk % 3;
        const bool real = kk < nk;
        off[e] = real ? (int)(c * xs.c + r * xs.h + s * xs.w) : 0;
        rs[e] = (unsigned)r | (unsigned)s << 2 | (real ? 16u : 0u);
    }
    __syncthreads();

#pragma unroll 1
    for (int gi = 0; gi < groups; ++gi) {
        const long q0 = ((long)blockIdx.x * 4 + wave) * (groups * 32) + gi * 32;
        if (q0 >= Q) break;                   // wave-uniform
        const long q = q0 + l32;
        const bool qok = q < Q;
        const unsigned qu = (unsigned)(qok ? q : Q - 1);      // Q < 2^31 (checked by the host)
        int n, oh, ow;
        if (batch_minor) {
            const unsigned t = qu / (unsigned)N;
            n = (int)(qu - t * (unsigned)N);
            oh = (int)(t / (unsigned)Wo);
            ow = (int)(t - (unsigned)oh * (unsigned)Wo);
        } else {
            const unsigned t = qu / (unsigned)Wo;
            ow = (int)(qu - t * (unsigned)Wo);
            n = (int)(t / (unsigned)Ho);
            oh = (int)(t - (unsigned)n * (unsigned)Ho);
        }
        // taps (r, s) of this pixel read x[oh + r - pad][ow + s - pad]; bit r of rmask / bit s of cmask: inside
        unsigned rmask = 0, cmask = 0;
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            rmask |= (oh + t - pad >= 0 && oh + t - pad < H) ? 1u << t : 0u;
            cmask |= (ow + t - pad >= 0 && ow + t - pad < W) ? 1u << t : 0u;
        }
        // element offsets fit 32 bits (the host checks the tensor sizes): the loads and stores then take the
        // tensor's base from scalar registers and a 32-bit offset from the lane, with no 64-bit vector arithmetic
        const int base = (int)(n * xs.n + (long)(oh - pad) * xs.h + (long)(ow - pad) * xs.w);   // top-left tap, channel 0
        const int safe = (int)(n * xs.n + (long)oh * xs.h + (long)ow * xs.w);                  // always inside x
        T raw[NE];
        float b[NE];
        // wave-uniform: every tap of every pixel of the group lies inside its image (all groups but those on
        // the image's border): no masks, no address selects (taps past 9*C read channel 0 and meet a zero weight)
        if (__ballot(rmask != 7u || cmask != 7u) == 0) {
#pragma unroll
            for (int e = 0; e < NE; ++e) raw[e] = x[(unsigned)(base + off[e])];
#pragma unroll
            for (int e = 0; e < NE; ++e) b[e] = to_f32(raw[e]);
        } else {
            unsigned keep[NE];
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                const bool in = ((rmask >> (rs[e] & 3u)) & (cmask >> ((rs[e] >> 2) & 3u)) & (rs[e] >> 4) & 1u) != 0;
                keep[e] = in ? 0xFFFFFFFFu : 0u;
                raw[e] = x[(unsigned)(in ? base + off[e] : safe)];
            }
#pragma unroll
            for (int e = 0; e < NE; ++e) b[e] = mask_keep(to_f32(raw[e]), keep[e]);
        }

        const unsigned yq = (unsigned)(n * ys.n + oh * ys.h + ow * ys.w + 4 * lh * ys.c);   // this lane's pixel, filter 4*lh
#pragma unroll 1
        for (int kt = 0; kt < KT; ++kt) {
            floatx16 acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
            const float* wk = sW + (size_t)kt * NE * 64 + lane;
            float a[NE];
#pragma unroll
            for (int e = 0; e < NE; ++e) a[e] = wk[e * 64];
#pragma unroll
            for (int e = 0; e < NE; ++e)
                acc = SWAP ? __builtin_amdgcn_mfma_f32_32x32x2f32(b[e], a[e], acc, 0, 0, 0)
                           : __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], acc, 0, 0, 0);
            if (SWAP) {
                // rows = the group's pixels, columns = filters: the lane's filter is kt*32 + l32 (batch-major pixels)
                const int k = kt * 32 + l32;
                const float bk = sB[k];
                if (k < K) {
                    // element offsets fit 32 bits (the host checks the tensor sizes): one scalar base, a running offset
                    unsigned o = ((unsigned)q0 + 4u * lh) * (unsigned)K + (unsigned)k;
                    const bool whole = q0 + 32 <= Q;                              // wave-uniform: all 32 pixels of the group exist
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        float v = acc[r] + bk;
                        if (ep.relu) v = fmaxf(v, 0.f);
                        if (whole || q0 + 8 * (r >> 2) + 4 * lh + (r & 3) < Q) y[o] = from_f32<T>(v);
                        o += ((r & 3) == 3 ? 5u : 1u) * (unsigned)K;
                    }
                }
                continue;
            }
            float bv[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) bv[r] = sB[kt * 32 + 8 * (r >> 2) + (r & 3) + 4 * lh];
            const T* yk = y + (size_t)kt * 32 * ys.c;                        // wave-uniform
            auto put = [&](int r) {
                float v = acc[r] + bv[r];
                if (ep.relu) v = fmaxf(v, 0.f);
                const_cast<T*>(yk + (size_t)(8 * (r >> 2) + (r & 3)) * ys.c)[yq] = from_f32<T>(v);
            };
            if (!qok) continue;
            if (kt * 32 + 32 <= K) {                                         // wave-uniform: all 32 filters of the tile exist
#pragma unroll
                for (int r = 0; r < 16; ++r) put(r);
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (kt * 32 + 8 * (r >> 2) + (r & 3) + 4 * lh < K) put(r);
            }
        }
    }
}

// The same for fp32 NCHW tensors on both sides with an even width, as tiles: the kernel above gathers a pixel's taps
// with NE loads of one element per 32 pixels and filter tile -- 27 loads next to 32 stores for C = 3, K = 64, and a
// CU takes about one memory instruction per 16 clocks whatever its width.  Here every WAVE takes tiles of 4 rows x 32
// columns, one after the other, on its own: a tile's input, C x 6 rows x 36 columns, comes in as aligned 8-byte
// pairs (6 loads per lane for C = 3, zeros where the padding is) and goes to LDS of the wave's own, the next tile's
// requested before the current tile's multiplies (no workgroup barrier in the loop); a lane then reads its taps
// from LDS.  The stores are those of the kernel above (a lane's 32 pixels of a filter are 128 contiguous bytes).
// Same products in the same multiply slots, bias after the sum: the same bits as above.  (N = 32, 224 x 224, K = 64:
// 125 -> 115 us; 411 MB of y, and store instructions and multiplies of a wave add up rather than overlap.  CHWN
// tensors as one image of width W * N, which pays in 16 bits, were slower here than the kernel above: 130 against 117.)
constexpr int DSF_WR = 4;                           // output rows of a wave's tile
constexpr int DSF_PR = DSF_WR + 2;                  // input rows
constexpr int DSF_PP = 18;                          // 8-byte pairs of an input row: 34 columns from an even one
// loads per lane of a tile's input (pairs of [C][6][18]) by NE = ceil(9 C / 2)
constexpr int dsf_loads(int ne) { return ne == 5 ? 2 : ne == 9 ? 4 : ne == 14 ? 6 : 7; }
__host__ inline size_t direct_tiles_lds_bytes(int C, int K) {
    const size_t base = direct_lds_bytes(C, K);
    return base ? base + 4 * (size_t)C * DSF_PR * DSF_PP * 8 : 0;
}

template <int NE>
__global__ __launch_bounds__(256) void direct_small_c_tiles_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                   float* __restrict__ y, int N, int C, int K, int H, int W,
                                                                   int pad, int Ho, int Wo, int tiles_y, int tiles_x,
                                                                   int ntiles, Epilogue ep) {
    extern __shared__ __attribute__((aligned(16))) float smemt[];
    const int KT = (K + 31) / 32;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int nk = 9 * C;
    constexpr int PP = DSF_PP;
    const int npairs = C * DSF_PR * PP;
    float* sW = smemt;                                                           // [KT][NE][64]: lane (lh, l32) holds W[kt*32 + l32][2e + lh]
    float* sB = smemt + (size_t)KT * NE * 64;                                    // [KT*32] bias
    float* sP = sB + KT * 32 + wave * npairs * 2;                                // this wave's [C][6][2 PP] elements

    for (int i = tid; i < KT * NE * 64; i += 256) {
        const int ln = i & 63, e = (i >> 6) % NE, kt = (i >> 6) / NE;
        const int k = kt * 32 + (ln & 31), kk = 2 * e + (ln >> 5);
        const bool ok = k < K && kk < nk;
        const float v = w[ok ? k * nk + kk : 0];                                   // [K][C][3][3]: tap kk of filter k
        sW[i] = ok ? v : 0.f;
    }
    for (int i = tid; i < KT * 32; i += 256) sB[i] = i < K ? bias_of<float>(ep, i) : 0.f;
    __syncthreads();

    // a lane's taps in the tile's patch: element offset of (channel, row r, column s) relative to its pixel's first
    // column; a tap past 9 C reads the pixel itself and is masked
    int off[NE];
    unsigned tapmask = 0;
#pragma unroll
    for (int e = 0; e < NE; ++e) {
        const int kk = 2 * e + lh;
        const int c = kk / 9, r = (kk % 9) / 3, q = kk % 3;
        off[e] = kk < nk ? (c * DSF_PR + r) * PP * 2 + q : 0;
        tapmask |= kk < nk ? 1u << e : 0u;
    }
    // the patch as loaded: pair 64 j + lane of [C][6][PP], as channel | row << 4 | pair of the row << 8 (row 15,
    // never inside the image, past the patch)
    constexpr int NL = dsf_loads(NE);
    unsigned pd[NL];
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        const int t = 64 * j + lane;
        const int c = t / (DSF_PR * PP), rem = t - c * (DSF_PR * PP);
        const int rr = rem / PP, pp = rem - rr * PP;
        pd[j] = t < npairs ? (unsigned)(c | rr << 4 | pp << 8) : 0xF0u;
    }
    const int rounds = (npairs + 63) / 64;                                       // wave-uniform
    const char* xb = reinterpret_cast<const char*>(x);
    char* yb = reinterpret_cast<char*>(y);
    const unsigned plane_y = (unsigned)Ho * (unsigned)Wo * 4u;                    // bytes of a filter's plane of y

    const int wstride = (int)gridDim.x * 4;
    int tile = (int)blockIdx.x * 4 + wave;
    int n = 0, oh0 = 0, ow0 = 0;                                                  // of the tile whose input is on its way
    uint2 v[NL];
    unsigned inside = 0;                                                          // bit j: pair j lies inside the image
    auto request = [&](int t) __attribute__((always_inline)) {
        n = t / (tiles_y * tiles_x);
        const int trem = t - n * tiles_y * tiles_x;
        oh0 = (trem / tiles_x) * DSF_WR;
        ow0 = (trem - (trem / tiles_x) * tiles_x) * 32;
        const int ic0 = ow0 - pad - ((ow0 - pad) & 1);                           // first column of the patch: even, <= ow0 - pad
        const int base = (n * C * H + oh0 - pad) * W + ic0;
        inside = 0;
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            if (j < rounds) {                                                     // (uniform)
                const int c = pd[j] & 15, rr = (pd[j] >> 4) & 15, pp = pd[j] >> 8;
                const int ih = oh0 - pad + rr, iw = ic0 + 2 * pp;
                const bool in = ih >= 0 && ih < H && iw >= 0 && iw < W;           // (W even: both elements or neither)
                v[j] = *reinterpret_cast<const uint2*>(xb + (in ? (unsigned)(base + (c * H + rr) * W + 2 * pp) * 4u : 0u));
                inside |= in ? 1u << j : 0u;
            }
        }
    };
    if (tile < ntiles) request(tile);
#pragma unroll 1
    while (tile < ntiles) {
        const int cn = n, coh0 = oh0, cow0 = ow0;                                 // the tile to compute
        const int shift = (cow0 - pad) & 1;
#pragma unroll
        for (int j = 0; j < NL; ++j)
            if (j < rounds && 64 * j + lane < npairs) {
                const unsigned m = 0u - ((inside >> j) & 1u);
                reinterpret_cast<uint2*>(sP)[64 * j + lane] = make_uint2(v[j].x & m, v[j].y & m);
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        tile += wstride;
        if (tile < ntiles) request(tile);

        const int ow = cow0 + l32;
        const bool pok = ow < Wo;
#pragma unroll 1
        for (int g = 0; g < DSF_WR; ++g) {
            const int oh = coh0 + g;
            if (oh >= Ho) break;                                                  // wave-uniform
            const float* pb = sP + g * PP * 2 + l32 + shift;
            float b[NE];
#pragma unroll
            for (int e = 0; e < NE; ++e) b[e] = __uint_as_float(__float_as_uint(pb[off[e]]) & (0u - ((tapmask >> e) & 1u)));
            // this lane's pixel, filter 4 lh
            unsigned yq = (unsigned)(((cn * K + 4 * lh) * Ho + oh) * Wo + ow) * 4u;
#pragma unroll 1
            for (int kt = 0; kt < KT; ++kt) {
                floatx16 acc;
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[r] = 0.f;
                const float* wk = sW + (size_t)kt * NE * 64 + lane;
#pragma unroll
                for (int e = 0; e < NE; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wk[e * 64], b[e], acc, 0, 0, 0);
                // register r: filter 8 (r / 4) + 4 lh + r % 4 of the tile
                const float* bk = sB + kt * 32 + 4 * lh;
                unsigned o = yq;
                auto put = [&](int r, bool check) __attribute__((always_inline)) {
                    float val = acc[r] + bk[8 * (r >> 2) + (r & 3)];
                    if (ep.relu) val = fmaxf(val, 0.f);
                    if (pok && (!check || kt * 32 + 8 * (r >> 2) + (r & 3) + 4 * lh < K)) *reinterpret_cast<float*>(yb + o) = val;
                    o += ((r & 3) == 3 ? 5u : 1u) * plane_y;
                };
                if (kt * 32 + 32 <= K) {                                          // wave-uniform: all 32 filters of the tile exist
#pragma unroll
                    for (int r = 0; r < 16; ++r) put(r, false);
                } else {
#pragma unroll
                    for (int r = 0; r < 16; ++r) put(r, true);
                }
                yq += 32u * plane_y;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                   // (the tile's LDS reads before the next tile's writes)
        __builtin_amdgcn_wave_barrier();
    }
}

// The same for fp32 NHWC tensors on both sides (W * C even): an input row of a tile is ONE contiguous run of
// (32 + 2) x C elements, 17 C + 1 aligned 8-byte pairs (the run may start at an odd element; a row of the image starts
// and ends at an even one, so no pair straddles its edge); the pixels are the multiply's first operand, so a lane holds
// one filter and its registers the pixels; two filter tiles are multiplied at a time and exchange register halves, so
// that a store instruction writes 64 filters of one pixel, 256 contiguous bytes when K = 64.
// Same products in the same multiply slots as the gathering kernel, bias after the sum: the same bits.
constexpr int dsf_nhwc_loads(int ne) { return ne == 5 ? 2 : ne == 9 ? 4 : ne == 14 ? 5 : 7; }   // pairs of [6][17 C + 1] over 64 lanes
__host__ inline size_t direct_tiles_nhwc_lds_bytes(int C, int K) {
    const size_t base = direct_lds_bytes(C, K);
    return base ? base + 4 * (size_t)DSF_PR * (17 * C + 1) * 8 : 0;
}

template <int NE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void direct_small_c_tiles_nhwc_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                        float* __restrict__ y, int N, int C, int K, int H, int W,
                                                                        int pad, int Ho, int Wo, int tiles_y, int tiles_x,
                                                                        int ntiles, Epilogue ep) {
    extern __shared__ __attribute__((aligned(16))) float smemn[];
    const int KT = (K + 31) / 32;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int nk = 9 * C;
    const int PPN = 17 * C + 1;                                                  // pairs of an input row of a tile
    const int npairs = DSF_PR * PPN;
    float* sW = smemn;                                                           // [KT][NE][64]: lane (lh, l32) holds W[kt*32 + l32][2e + lh]
    float* sB = smemn + (size_t)KT * NE * 64;                                    // [KT*32] bias
    float* sP = sB + KT * 32 + wave * npairs * 2;                                // this wave's [6][2 PPN] elements

    for (int i = tid; i < KT * NE * 64; i += 256) {
        const int ln = i & 63, e = (i >> 6) % NE, kt = (i >> 6) / NE;
        const int k = kt * 32 + (ln & 31), kk = 2 * e + (ln >> 5);
        const bool ok = k < K && kk < nk;
        const float v = w[ok ? k * nk + (kk % 9) * C + kk / 9 : 0];                // [K][3][3][C]: tap kk = 9 c + 3 r + s of filter k
        sW[i] = ok ? v : 0.f;
    }
    for (int i = tid; i < KT * 32; i += 256) sB[i] = i < K ? bias_of<float>(ep, i) : 0.f;
    __syncthreads();

    // a lane's taps in the tile's patch: tap kk = 9 c + 3 r + s meets the input at row r, element s C + c past the
    // pixel's first; a tap past 9 C reads the pixel itself and is masked
    int off[NE];
    unsigned tapmask = 0;
#pragma unroll
    for (int e = 0; e < NE; ++e) {
        const int kk = 2 * e + lh;
        const int c = kk / 9, r = (kk % 9) / 3, q = kk % 3;
        off[e] = kk < nk ? r * PPN * 2 + q * C + c : 0;
        tapmask |= kk < nk ? 1u << e : 0u;
    }
    // the patch as loaded: pair 64 j + lane of [6][PPN], as row | pair of the row << 8 (row 255, never inside, past it)
    constexpr int NL = dsf_nhwc_loads(NE);
    unsigned prp[NL];
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        const int t = 64 * j + lane;
        const int rr = t / PPN, pp = t - rr * PPN;
        prp[j] = t < npairs ? (unsigned)(rr | pp << 8) : 0xFFu;
    }
    const int rounds = (npairs + 63) / 64;                                       // wave-uniform
    const char* xb = reinterpret_cast<const char*>(x);
    const int WC = W * C;                                                         // elements of an image row (even)

    const int wstride = (int)gridDim.x * 4;
    int tile = (int)blockIdx.x * 4 + wave;
    int n = 0, oh0 = 0, ow0 = 0;                                                  // of the tile whose input is on its way
    uint2 v[NL];
    unsigned inside = 0;                                                          // bit j: pair j lies inside the image
    auto request = [&](int t) __attribute__((always_inline)) {
        n = t / (tiles_y * tiles_x);
        const int trem = t - n * tiles_y * tiles_x;
        oh0 = (trem / tiles_x) * DSF_WR;
        ow0 = (trem - (trem / tiles_x) * tiles_x) * 32;
        const int e0 = (ow0 - pad) * C - (((ow0 - pad) * C) & 1);                // first element of the patch's rows: even
        const int base = (n * H + oh0 - pad) * WC + e0;
        inside = 0;
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            if (j < rounds) {                                                     // (uniform)
                const int rr = prp[j] & 0xFF, pp = prp[j] >> 8;
                const int ih = oh0 - pad + rr, ie = e0 + 2 * pp;
                const bool in = ih >= 0 && ih < H && ie >= 0 && ie < WC;          // (a row starts and ends at an even element)
                v[j] = *reinterpret_cast<const uint2*>(xb + (in ? (unsigned)(base + rr * WC + 2 * pp) * 4u : 0u));
                inside |= in ? 1u << j : 0u;
            }
        }
    };
    if (tile < ntiles) request(tile);
#pragma unroll 1
    while (tile < ntiles) {
        const int cn = n, coh0 = oh0, cow0 = ow0;                                 // the tile to compute
        const int shift = ((cow0 - pad) * C) & 1;
#pragma unroll
        for (int j = 0; j < NL; ++j)
            if (j < rounds && 64 * j + lane < npairs) {
                const unsigned m = 0u - ((inside >> j) & 1u);
                reinterpret_cast<uint2*>(sP)[64 * j + lane] = make_uint2(v[j].x & m, v[j].y & m);
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        tile += wstride;
        if (tile < ntiles) request(tile);

#pragma unroll 1
        for (int g = 0; g < DSF_WR; ++g) {
            const int oh = coh0 + g;
            if (oh >= Ho) break;                                                  // wave-uniform
            const float* pb = sP + g * PPN * 2 + l32 * C + shift;
            float b[NE];
#pragma unroll
            for (int e = 0; e < NE; ++e) b[e] = __uint_as_float(__float_as_uint(pb[off[e]]) & (0u - ((tapmask >> e) & 1u)));
            // two filter tiles at a time; register r of a lane: pixel 8 (r / 4) + 4 lh + r % 4 of the row's 32 for the
            // lane's filter of each tile; the upper half of the first tile's register and the lower half of the second's
            // change places (v_permlane32_swap), and a register holds ONE pixel for 64 filters: a store instruction
            // writes 256 contiguous bytes when K = 64
            const unsigned yrow = (unsigned)((cn * Ho + oh) * Wo + cow0) * (unsigned)K;
#pragma unroll 1
            for (int kp = 0; kp < KT; kp += 2) {
                floatx16 acc0, acc1;
#pragma unroll
                for (int r = 0; r < 16; ++r) acc0[r] = 0.f, acc1[r] = 0.f;
                const float* wk = sW + (size_t)kp * NE * 64 + lane;
                const bool two = kp + 1 < KT;                                     // (uniform)
#pragma unroll
                for (int e = 0; e < NE; ++e) acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(b[e], wk[e * 64], acc0, 0, 0, 0);
                if (two) {
#pragma unroll
                    for (int e = 0; e < NE; ++e) acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(b[e], wk[(NE + e) * 64], acc1, 0, 0, 0);
                }
                const int k = kp * 32 + lane;
                const float bk = k < KT * 32 ? sB[k] : 0.f;
                const bool kok = k < K;
                unsigned o = yrow + (unsigned)k;                                  // element offsets fit 32 bits (the host checks the sizes)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc0[r]), __float_as_uint(acc1[r]), false, false);
#pragma unroll
                    for (int u = 0; u < 2; ++u) {                                 // pixel 8 (r / 4) + 4 u + r % 4
                        float val = __uint_as_float(sw[u]) + bk;
                        if (ep.relu) val = fmaxf(val, 0.f);
                        if (kok && cow0 + 8 * (r >> 2) + 4 * u + (r & 3) < Wo) y[o + (unsigned)(4 * u) * (unsigned)K] = val;
                    }
                    o += ((r & 3) == 3 ? 5u : 1u) * (unsigned)K;
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                   // (the tile's LDS reads before the next tile's writes)
        __builtin_amdgcn_wave_barrier();
    }
}

// Direct 3x3 convolution for layers with FEW OUTPUT PIXELS and a reduction of any length (a batch of one image: the
// reference's sweep starts at layer 1-2 with batch 1, comparison/layoutCompare.cu:38-46).  Such a layer is a few
// microseconds of arithmetic; through the Winograd pipelines it is three dependent launches, each of which starts,
// fills and drains a pipeline, and whose 64- and 128-wide patches occupy a fraction of the chip.  Here it is ONE
// launch with the smallest unit the matrix instruction has: a workgroup computes a tile of 4 x 8 pixels for 32
// filters, and its eight waves share the REDUCTION -- wave v takes channels 4v .. 4v+3, then 32 further on, 18
// v_mfma_f32_32x32x2_f32 per group of 4 channels, the next group's operands on their way meanwhile -- so that a
// layer with C = 64 is one chain of 36 multiplies per wave.  What binds such a kernel is the number of memory
// instructions a CU can take (about one per 16 clocks, whatever its width), so a wave fetches a group with as few
// as the layout allows and hands the elements to the lanes that multiply them through LDS of its own:
//   * the input patch of a group, 4 channels x 6 x 10 elements (zeros where the padding is), is 4 loads per lane;
//     where the channels are the contiguous axis (XW: NHWC) a pixel's 4 channels are one load of 16 bytes, one
//     load per lane;
//   * the filter block, 32 filters x 36 elements, in 16-byte pieces, 5 loads per lane: a [K][C][3][3] bank holds a
//     filter's 36 elements of a group contiguously (FM = 1), a [K][3][3][C] bank the 4 channels of a (filter, tap)
//     (FM = 2), a [C][3][3][K] bank 4 filters of a (channel, tap) (FM = 3); any other order, or C (FM = 3: C or
//     K) not a multiple of 4: 18 loads of one element (FM = 0);
//   * the waves' partial sums meet in LDS and each wave stores two of the 16 filter rows of the sum (bias, ReLU).
// Any layout on either side (element strides), any padding; the partial sums are added in wave order, so results do
// not depend on the launch.  The order in which a group's 36 products enter the sum follows the bank (FM = 2: tap
// major), so results of different layouts agree to rounding, not bit for bit.
constexpr int DFP_NE = 18;                  // multiplies per group of 4 channels
constexpr int DFP_ROW = 37;                 // floats per filter in the wave's strip of LDS (36 + 1: the 32 lanes of a read hit 32 banks)
constexpr int DFP_PATCH = 4 * 6 * 10;       // a group's input patch: 4 channels x (4 + 2) rows x (8 + 2) columns

template <typename T, int FM, bool XW>
__global__ __launch_bounds__(512) void direct_few_pixels_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                T* __restrict__ y, ActStrides xs, FltStrides ws,
                                                                ActStrides ys, int N, int C, int K, int H, int W, int pad,
                                                                int Ho, int Wo, int tiles_y, int tiles_x, int PT,
                                                                Epilogue ep) {
    constexpr int NE = DFP_NE;
    __shared__ float red[8][16][64];                          // the partial sums
    __shared__ float strip[8][32 * DFP_ROW];                  // per wave, a group's filter block: [filter][channel * 9 + tap]
    __shared__ float patch[8][DFP_PATCH];                     // per wave, a group's input patch: [channel][row][column]
    __shared__ int tabw[36];                                  // byte offset of (channel, tap) 0 .. 35 of a group in w
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int pt = (int)(blockIdx.x % (unsigned)PT), kt = (int)(blockIdx.x / (unsigned)PT);
    if (tid < 36) tabw[tid] = (int)((tid / 9) * ws.c + ((tid % 9) / 3) * ws.r + (tid % 3) * ws.s) * (int)sizeof(T);

    // the workgroup's pixels: tile (n, ty, tx) of 4 rows x 8 columns; lane l32: row l32 / 8, column l32 % 8
    const int n = pt / (tiles_y * tiles_x), trem = pt - n * tiles_y * tiles_x;
    const int oh0 = (trem / tiles_x) * 4, ow0 = (trem % tiles_x) * 8;
    const int py = l32 >> 3, px = l32 & 7;
    // byte offsets fit 32 bits (the host checks the tensor sizes)

    // Input patch as loaded: element 64 j + lane of [4][6][10], j < 4: byte offset in x relative to the group's
    // first channel (0 and a zero mask where the element lies in the padding or past the patch).
    // XW: lane p < 60 loads the 4 channels of pixel p of [6][10] as one piece.
    constexpr int NX = XW ? 1 : 4;
    unsigned offx[NX], mx[NX];
#pragma unroll
    for (int j = 0; j < NX; ++j) {
        const int p = 64 * j + lane;
        const int c = XW ? 0 : (p * 1093) >> 16, rem = p - 60 * c;            // p / 60, p % 60 (p < 256)
        const int rr = (rem * 205) >> 11, cc = rem - 10 * rr;                 // rem / 10, rem % 10 (rem < 64)
        const int ih = oh0 - pad + rr, iw = ow0 - pad + cc;
        const bool in = p < (XW ? 60 : DFP_PATCH) && ih >= 0 && ih < H && iw >= 0 && iw < W;
        offx[j] = in ? (unsigned)((int)(n * xs.n + c * xs.c + ih * xs.h + iw * xs.w) * (int)sizeof(T)) : 0u;
        mx[j] = in ? 0xFFFFFFFFu : 0u;
    }
    __syncthreads();
    // Filter block as loaded.  FM = 1, 2: 16-byte piece 64 j + lane of the [32 filters][9] pieces of a group, j < 5
    // (FM = 1: elements 4 part .. 4 part + 3 of the filter's 36; FM = 2: the 4 channels of tap `part`).  FM = 3:
    // piece 64 j + lane of [36 (channel, tap)][8]: filters 4 piece .. 4 piece + 3.  FM = 0: element 64 j + lane of
    // [32][36], j < 18.  Byte offset in w relative to the group's first channel, mask (filters past K), place in
    // the strip: a filter's row holds position 9 c + tap (FM = 2: 4 tap + c) of the group.
    constexpr bool wide = FM != 0;
    constexpr int NW = wide ? 5 : NE;
    unsigned offw[NW], mw[NW];
    int sidx[NW];
#pragma unroll
    for (int j = 0; j < NW; ++j) {
        const int idx = 64 * j + lane;
        if (FM == 1 || FM == 2) {
            const int fk = (idx * 7282) >> 16, part = idx - 9 * fk;           // idx / 9, idx % 9 (idx < 320)
            const bool fok = fk < 32 && kt * 32 + fk < K;
            const int at = FM == 1 ? 4 * part : (part / 3) * (int)ws.r + (part % 3) * (int)ws.s;
            offw[j] = fok ? (unsigned)(((kt * 32 + fk) * (int)ws.k + at) * (int)sizeof(T)) : 0u;
            mw[j] = fok ? 0xFFFFFFFFu : 0u;
            sidx[j] = fk < 32 ? fk * DFP_ROW + 4 * part : 0;
        } else if (FM == 3) {
            const int row = idx >> 3, piece = idx & 7;                         // (channel, tap) 9 c + tap, filters 4 piece ..
            const bool fok = row < 36 && kt * 32 + 4 * piece < K;              // (K a multiple of 4)
            const int c = (row * 57) >> 9, tap = row - 9 * c;                  // row / 9 (row < 40)
            offw[j] = fok ? (unsigned)((c * (int)ws.c + (tap / 3) * (int)ws.r + (tap % 3) * (int)ws.s + kt * 32 + 4 * piece) * (int)sizeof(T)) : 0u;
            mw[j] = fok ? 0xFFFFFFFFu : 0u;
            sidx[j] = row < 36 ? 4 * piece * DFP_ROW + row : 0;
        } else {
            const int fk = (idx * 1821) >> 16, fkk = idx - 36 * fk;           // idx / 36, idx % 36 (idx < 1152)
            const bool fok = kt * 32 + fk < K;
            offw[j] = fok ? (unsigned)(((kt * 32 + fk) * (int)ws.k) * (int)sizeof(T) + tabw[fkk]) : 0u;
            mw[j] = fok ? 0xFFFFFFFFu : 0u;
            sidx[j] = idx + fk;                                               // [fk][fkk] in rows of 37
        }
    }
    const char* xg = reinterpret_cast<const char*>(x) + (size_t)(wave * 4) * xs.c * sizeof(T);   // this wave's group: first channel
    const char* wg = reinterpret_cast<const char*>(w) + (size_t)(wave * 4) * ws.c * sizeof(T);
    const size_t xstep = (size_t)32 * xs.c * sizeof(T), wstep = (size_t)32 * ws.c * sizeof(T);

    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    // the group on its way: 4 patch elements; 5 filter pieces of 4 elements (wide) or 18 elements
    struct alignas(4) T4 { T v[4]; };
    T rb[4];
    T4 rb4;
    T4 rw4[5];
    T rw[NW];
    int cleft = 0;                                            // channels of that group that exist, counted from the wave's first
    int crem = C - wave * 4;
    auto load = [&]() __attribute__((always_inline)) {        // the group at xg, wg; the pointers move on
        cleft = crem;
        if (XW) {
            rb4 = *reinterpret_cast<const T4*>(xg + offx[0]);                 // (C a multiple of 4: the group's channels exist)
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // (a channel past C: the first element of the group's first channel is read instead, and masked)
                const int c = ((64 * j + lane) * 1093) >> 16;
                rb[j] = *reinterpret_cast<const T*>(xg + (c < crem ? offx[j] : 0u));
            }
        }
        if (wide) {
#pragma unroll
            for (int j = 0; j < 5; ++j) rw4[j] = *reinterpret_cast<const T4*>(wg + offw[j]);
        } else {
#pragma unroll
            for (int j = 0; j < NE; ++j) {
                const int idx = 64 * j + lane, fkk = idx - 36 * ((idx * 1821) >> 16);
                rw[j] = *reinterpret_cast<const T*>(wg + (fkk < 9 * crem ? offw[j] : 0u));
            }
        }
        xg += xstep;
        wg += wstep;
        crem -= 32;
    };
    float* const mine = strip[wave];
    float* const mypatch = patch[wave];
    float a[NE], b[NE];
    // the group that has arrived -> the wave's strip and patch -> a, b: multiply e of a lane takes (channel
    // 2 lh + e / 9, tap e % 9) of the group (FM = 2: channel 2 lh + e % 2, tap e / 2)
    auto stage = [&]() __attribute__((always_inline)) {
        if (XW) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (lane < 60) mypatch[60 * i + lane] = __uint_as_float(__float_as_uint(to_f32(rb4.v[i])) & mx[0]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int p = 64 * j + lane, c = (p * 1093) >> 16;
                if (p < DFP_PATCH) mypatch[p] = __uint_as_float(__float_as_uint(to_f32(rb[j])) & (c < cleft ? mx[j] : 0u));
            }
        }
        if (FM == 3) {
#pragma unroll
            for (int j = 0; j < 5; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (j < 4 || lane < 32) mine[sidx[j] + i * DFP_ROW] = __uint_as_float(__float_as_uint(to_f32(rw4[j].v[i])) & mw[j]);
        } else if (wide) {
#pragma unroll
            for (int j = 0; j < 5; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (j < 4 || lane < 32) mine[sidx[j] + i] = __uint_as_float(__float_as_uint(to_f32(rw4[j].v[i])) & mw[j]);
        } else {
#pragma unroll
            for (int j = 0; j < NE; ++j) {
                const int idx = 64 * j + lane, fkk = idx - 36 * ((idx * 1821) >> 16);
                mine[sidx[j]] = __uint_as_float(__float_as_uint(to_f32(rw[j])) & (fkk < 9 * cleft ? mw[j] : 0u));
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const float* ar = mine + l32 * DFP_ROW + (FM == 2 ? 2 : 18) * lh;
        const float* br = mypatch + 120 * lh + py * 10 + px;
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            const int ec = FM == 2 ? e % 2 : e / 9, et = FM == 2 ? e / 2 : e % 9;       // channel (of the half's two), tap
            a[e] = ar[FM == 2 ? 4 * et + ec : e];
            b[e] = br[ec * 60 + (et / 3) * 10 + et % 3];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };
    // groups of this wave: channels 4 wave + 32 i
    const int ng = C > wave * 4 ? (C - wave * 4 + 31) / 32 : 0;
    if (ng > 0) load();
#pragma unroll 1
    for (int i = 0; i < ng; ++i) {
        stage();
        if (i + 1 < ng) load();
#pragma unroll
        for (int e = 0; e < NE; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], acc, 0, 0, 0);
    }

    // the eight partial sums meet in LDS; wave v adds and stores registers 2v and 2v + 1 of the sum: register r of a
    // lane is filter 8 * (r / 4) + 4 * lh + r % 4 of the tile, the lane's pixel
#pragma unroll
    for (int r = 0; r < 16; ++r) red[wave][r][lane] = acc[r];
    __syncthreads();
    const int oh = oh0 + py, ow = ow0 + px;
    const long yq = n * ys.n + oh * ys.h + ow * ys.w;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int r = 2 * wave + j;
        float v = 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) v += red[u][r][lane];
        const int kk = kt * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (oh < Ho && ow < Wo && kk < K) {
            v += bias_of<T>(ep, kk);
            if (ep.relu) v = fmaxf(v, 0.f);
            y[yq + kk * ys.c] = from_f32<T>(v);
        }
    }
}

// The same for 2-byte tensors on the 16-bit matrix instruction: the 9*C <= 36 taps of an output are NE =
// ceil(9*C/16) v_mfma_f32_32x32x16 (2 for C = 3) instead of 14 fp32 ones -- a fourteenth of the matrix time.
// The products are the same (two 2-byte values multiply exactly in fp32 either way), only the order in which
// an instruction sums its 16 of them is the hardware's.  A lane holds 8 consecutive taps per instruction:
// kk = 16e + 8*lh + i.
__host__ inline size_t direct16_lds_bytes(int C, int K) {
    if (C < 1 || C > 4) return 0;
    const size_t ne = (9 * C + 15) / 16, kt = (K + 31) / 32;
    return kt * ne * 64 * 16 + kt * 32 * sizeof(float);
}

template <typename T, int NE, bool SWAP>
__global__ __launch_bounds__(256) void direct_small_c16_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                               T* __restrict__ y, ActStrides xs, FltStrides ws,
                                                               ActStrides ys, int N, int C, int K, int H, int W,
                                                               int pad, int Ho, int Wo, int batch_minor, long Q,
                                                               int groups, Epilogue ep) {
    static_assert(sizeof(T) == 2, "2-byte tensors");
    typedef typename Mma<T>::vec vec;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem16[];
    const int KT = (K + 31) / 32;
    vec* sW = reinterpret_cast<vec*>(smem16);                              // [KT][NE][64]
    float* sB = reinterpret_cast<float*>(smem16 + (size_t)KT * NE * 64 * 16);   // [KT*32] bias
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int nk = 9 * C;

    for (int i = tid; i < KT * NE * 64; i += 256) {
        const int ln = i & 63, e = (i >> 6) % NE, kt = (i >> 6) / NE;
        const int k = kt * 32 + (ln & 31);
        T v8[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int kk = 16 * e + 8 * (ln >> 5) + j;
            const bool ok = k < K && kk < nk;
            const int c = kk / 9, r = (kk % 9) / 3, q = kk % 3;
            const T v = w[ok ? k * ws.k + c * ws.c + r * ws.r + q * ws.s : 0];
            v8[j] = ok ? v : from_f32<T>(0.f);
        }
        vec pk;
        __builtin_memcpy(&pk, v8, 16);
        sW[i] = pk;
    }
    for (int i = tid; i < KT * 32; i += 256) sB[i] = i < K ? bias_of<T>(ep, i) : 0.f;

    int off[NE][8];
    unsigned rs[NE];                          // per tap j: bits 4j..4j+3 = r | s << 2; taps past 9*C: r = s = 3 (never inside)
#pragma unroll
    for (int e = 0; e < NE; ++e) {
        rs[e] = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int kk = 16 * e + 8 * lh + j;
            const int c = kk / 9, r = (kk % 9) / 3, q = kk % 3;
            const bool real = kk < nk;
            off[e][j] = real ? (int)(c * xs.c + r * xs.h + q * xs.w) : 0;
            rs[e] |= (real ? ((unsigned)r | (unsigned)q << 2) : 15u) << (4 * j);
        }
    }
    __syncthreads();

#pragma unroll 1
    for (int gi = 0; gi < groups; ++gi) {
        const long q0 = ((long)blockIdx.x * 4 + wave) * (groups * 32) + gi * 32;
        if (q0 >= Q) break;                   // wave-uniform
        const long q = q0 + l32;
        const bool qok = q < Q;
        const unsigned qu = (unsigned)(qok ? q : Q - 1);
        int n, oh, ow;
        if (batch_minor) {
            const unsigned t = qu / (unsigned)N;
            n = (int)(qu - t * (unsigned)N);
            oh = (int)(t / (unsigned)Wo);
            ow = (int)(t - (unsigned)oh * (unsigned)Wo);
        } else {
            const unsigned t = qu / (unsigned)Wo;
            ow = (int)(qu - t * (unsigned)Wo);
            n = (int)(t / (unsigned)Ho);
            oh = (int)(t - (unsigned)n * (unsigned)Ho);
        }
        unsigned rmask = 0, cmask = 0;        // bit t: tap row / column t of this pixel lies inside the image (bit 3 never)
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            rmask |= (oh + t - pad >= 0 && oh + t - pad < H) ? 1u << t : 0u;
            cmask |= (ow + t - pad >= 0 && ow + t - pad < W) ? 1u << t : 0u;
        }
        const int base = (int)(n * xs.n + (long)(oh - pad) * xs.h + (long)(ow - pad) * xs.w);
        const int safe = (int)(n * xs.n + (long)oh * xs.h + (long)ow * xs.w);
        vec b[NE];
        if (__ballot(rmask != 7u || cmask != 7u) == 0) {
            // every tap of every pixel of the group inside its image (taps past 9*C read channel 0 and meet a zero weight)
            T raw[NE][8];
#pragma unroll
            for (int e = 0; e < NE; ++e)
#pragma unroll
                for (int j = 0; j < 8; ++j) raw[e][j] = x[(unsigned)(base + off[e][j])];
#pragma unroll
            for (int e = 0; e < NE; ++e) __builtin_memcpy(&b[e], raw[e], 16);
        } else {
            T raw[NE][8];
#pragma unroll
            for (int e = 0; e < NE; ++e)
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const unsigned t = rs[e] >> (4 * j);
                    const bool in = ((rmask >> (t & 3u)) & (cmask >> ((t >> 2) & 3u)) & 1u) != 0;
                    const T v = x[(unsigned)(in ? base + off[e][j] : safe)];
                    raw[e][j] = in ? v : from_f32<T>(0.f);
                }
#pragma unroll
            for (int e = 0; e < NE; ++e) __builtin_memcpy(&b[e], raw[e], 16);
        }

        const unsigned yq = (unsigned)(n * ys.n + oh * ys.h + ow * ys.w + 4 * lh * ys.c);
#pragma unroll 1
        for (int kt = 0; kt < KT; ++kt) {
            // the sum starts at the bias (SWAP: a lane holds one filter; else register r is filter 8 (r / 4) + 4 lh + r % 4)
            floatx16 acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = SWAP ? sB[kt * 32 + l32] : sB[kt * 32 + 8 * (r >> 2) + (r & 3) + 4 * lh];
            const vec* wk = sW + (size_t)kt * NE * 64 + lane;
            vec a[NE];
#pragma unroll
            for (int e = 0; e < NE; ++e) a[e] = wk[e * 64];
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                if (SWAP) Mma<T>::run(b[e], a[e], acc);
                else Mma<T>::run(a[e], b[e], acc);
            }
            if (SWAP) {
                const int k = kt * 32 + l32;
                if (k < K) {
                    unsigned o = ((unsigned)q0 + 4u * lh) * (unsigned)K + (unsigned)k;   // (element offsets fit 32 bits)
                    const bool whole = q0 + 32 <= Q;                              // wave-uniform: all 32 pixels of the group exist
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        float v = acc[r];
                        if (ep.relu) v = fmaxf(v, 0.f);
                        if (whole || q0 + 8 * (r >> 2) + 4 * lh + (r & 3) < Q) y[o] = from_f32<T>(v);
                        o += ((r & 3) == 3 ? 5u : 1u) * (unsigned)K;
                    }
                }
                continue;
            }
            const T* yk = y + (size_t)kt * 32 * ys.c;
            auto put = [&](int r) {
                float v = acc[r];
                if (ep.relu) v = fmaxf(v, 0.f);
                const_cast<T*>(yk + (size_t)(8 * (r >> 2) + (r & 3)) * ys.c)[yq] = from_f32<T>(v);
            };
            if (!qok) continue;
            if (kt * 32 + 32 <= K) {
#pragma unroll
                for (int r = 0; r < 16; ++r) put(r);
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (kt * 32 + 8 * (r >> 2) + (r & 3) + 4 * lh < K) put(r);
            }
        }
    }
}

// The same for NCHW tensors on both sides with an even width, as tiles.  The kernel above is bound by its memory
// instructions twice over: it gathers a pixel's taps with sixteen 2-byte loads and stores its sums 2 bytes at a time
// (48 memory instructions per 32 pixels x 64 filters; a CU takes about one per 16 clocks whatever its width), and the
// 64-byte runs a wave writes per filter are half cache lines whose other half arrives from another wave: written as
// stores and nothing else (cli/store_pattern.hip), that pattern moves 3.9 TB/s, whole 128-byte lines 4.4 (N = 32,
// 224 x 224, K = 64, 205 MB of y: 53 against 46 us).  Here every WAVE takes tiles of 4 rows x 64 columns, one after the
// other, on its own:
//   * a tile's input, C x 6 rows x 68 columns, comes in as aligned 4-byte pairs (10 loads per lane for C = 3, zeros
//     where the padding is) and goes to LDS of the wave's own; a lane then gathers its taps with 2-byte LDS reads.
//     The next tile's pairs are requested before the current tile's multiplies, so no wave waits for memory, and
//     there is no workgroup barrier in the loop;
//   * a row of the tile is two multiplies of 32 columns; the upper half of the first result and the lower half of
//     the second change places (v_permlane32_swap), so that a register holds ONE filter for the row's 64 columns;
//     neighbouring lanes then swap one of two sums (rounded and packed first: one DPP move, one byte permute) and
//     every lane stores a 4-byte pair: an instruction writes two filters x 128 contiguous bytes;
//   * the sum starts at the bias (the matrix instruction's third operand), ReLU is one instruction per value.
// The filter bank is staged once per workgroup, as above.  Same products and the same bits as above.
// DIL: CHWN tensors ([C][H][W][N], filters [C][3][3][K]) as ONE image of width W * N whose taps are N columns apart:
// the batch is the contiguous axis of both tensors, so a row of 64 "columns" is two pixels x 32 images (N = 32), the
// zero padding is pad * N columns wide, and everything else is the NCHW kernel.
constexpr int DSC_WR = 4;                           // output rows of a wave's tile
constexpr int DSC_WC = 64;                          // output columns
constexpr int DSC_PR = DSC_WR + 2;                  // input rows
constexpr int DSC_PP = 34;                          // 4-byte pairs of an input row: 66 columns from an even one
constexpr int DSC_DS = 32;                          // DIL: columns between taps, at most
// loads per lane of a tile's input: C = 1 (204 pairs), 2 or 3 (612), 4 (816); DIL: rows of up to 33 + 32 pairs
constexpr int dsc_loads(int ne, bool dil) { return dil ? (ne == 1 ? 7 : ne == 2 ? 19 : 25) : (ne == 1 ? 4 : ne == 2 ? 10 : 13); }
__host__ inline size_t direct16_tiles_lds_bytes(int C, int K, int ds = 1) {
    const size_t base = direct16_lds_bytes(C, K);
    return base ? base + 4 * (size_t)C * DSC_PR * (33 + ds) * 4 : 0;
}

template <typename T, int NE, bool DIL>
__global__ __launch_bounds__(256) void direct_small_c16_tiles_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                     T* __restrict__ y, int N, int C, int K, int H, int W,
                                                                     int pad, int ds, int Ho, int Wo, int tiles_y,
                                                                     int tiles_x, int ntiles, Epilogue ep) {
    static_assert(sizeof(T) == 2, "2-byte tensors");
    typedef typename Mma<T>::vec vec;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem16t[];
    const int KT = (K + 31) / 32;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int nk = 9 * C;
    const int PP = DIL ? 33 + ds : DSC_PP;                                       // pairs of an input row of a tile: 64 + 2 ds columns from an even one
    const int padw = pad * ds;                                                   // zero columns left of a row
    const int npairs = C * DSC_PR * PP;
    vec* sW = reinterpret_cast<vec*>(smem16t);                                   // [KT][NE][64]
    float* sB = reinterpret_cast<float*>(smem16t + (size_t)KT * NE * 64 * 16);  // [KT * 32] bias
    unsigned* sP = reinterpret_cast<unsigned*>(sB + KT * 32) + wave * npairs;    // this wave's [C][6][34] pairs

    for (int i = tid; i < KT * NE * 64; i += 256) {
        const int ln = i & 63, e = (i >> 6) % NE, kt = (i >> 6) / NE;
        const int k = kt * 32 + (ln & 31);
        T v8[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int kk = 16 * e + 8 * (ln >> 5) + j;
            const bool ok = k < K && kk < nk;
            const T v = w[ok ? (DIL ? kk * K + k : k * nk + kk) : 0];              // [K][C][3][3] (DIL: [C][3][3][K]): tap kk of filter k
            v8[j] = ok ? v : from_f32<T>(0.f);
        }
        vec pk;
        __builtin_memcpy(&pk, v8, 16);
        sW[i] = pk;
    }
    for (int i = tid; i < KT * 32; i += 256) sB[i] = i < K ? bias_of<T>(ep, i) : 0.f;
    __syncthreads();

    // a lane's taps in the tile's patch: byte offset of (channel, row r, column s) relative to its pixel's first
    // column; taps past 9 C read the pixel itself and are masked (bit 8 e + j of tapmask: a real tap)
    int off[NE][8];
    unsigned tapmask = 0;
#pragma unroll
    for (int e = 0; e < NE; ++e)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int kk = 16 * e + 8 * lh + j;
            const int c = kk / 9, r = (kk % 9) / 3, q = kk % 3;
            off[e][j] = kk < nk ? ((c * DSC_PR + r) * PP * 2 + q * ds) * 2 : 0;
            tapmask |= kk < nk ? 1u << (8 * e + j) : 0u;
        }
    constexpr int DSC_NL = dsc_loads(NE, DIL);
    // DIL: the patch as loaded, pair 64 j + lane of [C][6][PP], as channel | row << 4 | pair of the row << 8 (row 15,
    // never inside the image, past the patch)
    unsigned pd[DIL ? DSC_NL : 1];
    if (DIL) {
#pragma unroll
        for (int j = 0; j < DSC_NL; ++j) {
            const int t = 64 * j + lane;
            const int c = t / (DSC_PR * PP), rem = t - c * (DSC_PR * PP);
            const int rr = rem / PP, pp = rem - rr * PP;
            pd[j] = t < npairs ? (unsigned)(c | rr << 4 | pp << 8) : 0xF0u;
        }
    }
    const int rounds = (npairs + 63) / 64;                                       // wave-uniform
    const char* xb = reinterpret_cast<const char*>(x);
    char* yb = reinterpret_cast<char*>(y);
    const unsigned plane_y = (unsigned)Ho * (unsigned)Wo * 2u;                    // bytes of a filter's plane of y
    const unsigned psel = (lane & 1) ? 0x03020706u : 0x05040100u;                 // (own pair, neighbour's pair) -> what the lane stores

    // the wave's tiles: every (4 x workgroups)-th, columns fastest
    const int wstride = (int)gridDim.x * 4;
    int tile = (int)blockIdx.x * 4 + wave;
    int n = 0, oh0 = 0, ow0 = 0;                                                  // of the tile whose input is on its way
    unsigned v[DSC_NL], inside = 0;                                               // bit j: pair j lies inside the image
    auto request = [&](int t) __attribute__((always_inline)) {
        n = t / (tiles_y * tiles_x);
        const int trem = t - n * tiles_y * tiles_x;
        oh0 = (trem / tiles_x) * DSC_WR;
        ow0 = (trem - (trem / tiles_x) * tiles_x) * DSC_WC;
        const int ic0 = ow0 - padw - ((ow0 - padw) & 1);                         // first column of the patch: even, <= ow0 - padw
        const int base = (n * C * H + oh0 - pad) * W + ic0;
        inside = 0;
#pragma unroll
        for (int j = 0; j < DSC_NL; ++j) {
            if (j < rounds) {                                                     // (uniform)
                // pair 64 j + lane of [C][6][34]: channel, row, pair of the row (t < 1024)
                const int t = 64 * j + lane;
                int c = (t * 1286) >> 18, rem = t - c * (DSC_PR * DSC_PP);        // t / 204
                int rr = (rem * 1928) >> 16, pp = rem - rr * DSC_PP;               // rem / 34 (rem < 204)
                if (DIL) {
                    c = pd[j] & 15;
                    rr = (pd[j] >> 4) & 15;
                    pp = pd[j] >> 8;
                }
                const int ih = oh0 - pad + rr, iw = ic0 + 2 * pp;
                const bool in = t < npairs && ih >= 0 && ih < H && iw >= 0 && iw < W;   // (W even: both elements or neither)
                v[j] = *reinterpret_cast<const unsigned*>(xb + (in ? (unsigned)(base + (c * H + rr) * W + 2 * pp) * 2u : 0u));
                inside |= in ? 1u << j : 0u;
            }
        }
    };
    if (tile < ntiles) request(tile);
#pragma unroll 1
    while (tile < ntiles) {
        const int cn = n, coh0 = oh0, cow0 = ow0;                                 // the tile to compute
        const int shift = (cow0 - padw) & 1;
#pragma unroll
        for (int j = 0; j < DSC_NL; ++j)
            if (j < rounds && 64 * j + lane < npairs) sP[64 * j + lane] = v[j] & (0u - ((inside >> j) & 1u));
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        tile += wstride;
        if (tile < ntiles) request(tile);

        const int ow = cow0 + lane;                                               // the lane's column once a register holds one filter
        const bool pok = ow < Wo;                                                 // (Wo even, ow0 even: a pair is in or out)
#pragma unroll 1
        for (int g = 0; g < DSC_WR; ++g) {
            const int oh = coh0 + g;
            if (oh >= Ho) break;                                                  // wave-uniform
            const unsigned char* pb = reinterpret_cast<const unsigned char*>(sP) + (g * PP * 2 + l32 + shift) * 2;
            vec b[2][NE];                                                         // columns 0 .. 31 and 32 .. 63
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int e = 0; e < NE; ++e) {
                    unsigned short raw[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        raw[j] = (unsigned short)(*reinterpret_cast<const unsigned short*>(pb + 64 * h + off[e][j]) & (0u - ((tapmask >> (8 * e + j)) & 1u)));
                    __builtin_memcpy(&b[h][e], raw, 16);
                }
            // the lane's pair: columns ow & ~1 and the next one, of the filter it keeps (even lanes the first of two)
            const unsigned yq = (unsigned)(((cn * K + (lane & 1)) * Ho + oh) * Wo + (ow & ~1)) * 2u;
#pragma unroll 1
            for (int kt = 0; kt < KT; ++kt) {
                // register r of a lane: filter 8 (r / 4) + 4 lh + r % 4 of the tile; the sum starts at the bias
                floatx16 acc[2];
                const float* bk = sB + kt * 32 + 4 * lh;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const floatx4 bq = *reinterpret_cast<const floatx4*>(bk + 8 * q);
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[0][4 * q + r] = acc[1][4 * q + r] = bq[r];
                }
                const vec* wk = sW + (size_t)kt * NE * 64 + lane;
#pragma unroll
                for (int e = 0; e < NE; ++e) {
                    const vec a = wk[e * 64];
                    Mma<T>::run(a, b[0][e], acc[0]);
                    Mma<T>::run(a, b[1][e], acc[1]);
                }
                // registers 2i and 2i + 1 of half u (after the exchange of halves) are filters f and f + 1,
                // f = 8 (i / 2) + 4 u + 2 (i % 2), for the row's 64 columns: rounded, packed, swapped with the
                // neighbouring lane, and each lane keeps the two columns of one filter
                auto put = [&](int i, bool check, bool relu) __attribute__((always_inline)) {
                    const auto s0 = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[0][2 * i]), __float_as_uint(acc[1][2 * i]), false, false);
                    const auto s1 = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[0][2 * i + 1]), __float_as_uint(acc[1][2 * i + 1]), false, false);
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        float a0 = __uint_as_float(s0[u]), a1 = __uint_as_float(s1[u]);
                        if (relu) {                                                // max(a, 0), 0 for a NaN (as fmaxf)
                            asm("v_max_f32_e32 %0, 0, %1" : "=v"(a0) : "v"(a0));
                            asm("v_max_f32_e32 %0, 0, %1" : "=v"(a1) : "v"(a1));
                        }
                        const unsigned own = pack2<T>(a0, a1);
                        const unsigned nb = (unsigned)__builtin_amdgcn_mov_dpp((int)own, 0xB1, 0xF, 0xF, true);
                        const unsigned out = __builtin_amdgcn_perm(nb, own, psel);
                        const int f = kt * 32 + 8 * (i >> 1) + 4 * u + 2 * (i & 1);
                        if (pok && (!check || f + (lane & 1) < K)) *reinterpret_cast<unsigned*>(yb + (yq + (unsigned)f * plane_y)) = out;
                    }
                };
                // (every lane takes part in the exchanges; only the stores are conditional)
                if (kt * 32 + 32 > K) {                                           // (wave-uniform: the bank's last, partial tile)
#pragma unroll
                    for (int i = 0; i < 8; ++i) put(i, true, ep.relu != 0);
                } else if (ep.relu) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) put(i, false, true);
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) put(i, false, false);
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                   // (the tile's LDS reads before the next tile's writes)
        __builtin_amdgcn_wave_barrier();
    }
}

// The same for NHWC tensors on both sides (K even): y is then a matrix [pixel][filter] whose rows are K contiguous
// elements, and the gathering kernel writes it two bytes per lane, 64 bytes per pixel and instruction.  Per wave and
// tile of 4 rows x 32 columns, as above; the differences:
//   * an input row of a tile is ONE contiguous run of (32 + 2) x C elements: C x 17 + 1 aligned pairs a row (the run
//     may start at an odd element; a row of the image starts and ends at an even one, so no pair straddles its edge);
//   * the pixels are the first operand of a multiply, so a lane holds one filter and its registers the pixels;
//   * two filter tiles are multiplied at a time; the upper half of the first result and the lower half of the second
//     change places (v_permlane32_swap), so that a register holds ONE pixel for 64 filters; neighbouring lanes then
//     swap one of two sums and every lane stores a 4-byte pair: an instruction writes the 64 filters of two
//     neighbouring pixels, 256 contiguous bytes when K = 64.
// The sums start at the bias, as in the gathering kernel: same bits.
constexpr int dsc_nhwc_loads(int ne) { return ne == 1 ? 2 : ne == 2 ? 5 : 7; }   // loads per lane of a tile's input: C = 1 (108 pairs), 2 or 3 (312), 4 (414)
__host__ inline size_t direct16_tiles_nhwc_lds_bytes(int C, int K) {
    const size_t base = direct16_lds_bytes(C, K + 32);                           // (filter tiles in pairs: one more when their number is odd)
    return base ? base + 4 * (size_t)DSC_PR * (17 * C + 1) * 4 : 0;
}

template <typename T, int NE>
__global__ __launch_bounds__(256) void direct_small_c16_tiles_nhwc_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                          T* __restrict__ y, int N, int C, int K, int H,
                                                                          int W, int pad, int Ho, int Wo, int tiles_y,
                                                                          int tiles_x, int ntiles, Epilogue ep) {
    static_assert(sizeof(T) == 2, "2-byte tensors");
    typedef typename Mma<T>::vec vec;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem16n[];
    const int KT2 = (K + 63) / 64;                                               // pairs of filter tiles
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int nk = 9 * C;
    const int PPN = 17 * C + 1;                                                  // pairs of an input row of a tile
    const int npairs = DSC_PR * PPN;
    vec* sW = reinterpret_cast<vec*>(smem16n);                                   // [2 KT2][NE][64]
    float* sB = reinterpret_cast<float*>(smem16n + (size_t)2 * KT2 * NE * 64 * 16);   // [64 KT2] bias
    unsigned* sP = reinterpret_cast<unsigned*>(sB + KT2 * 64) + wave * npairs;   // this wave's [6][PPN] pairs

    for (int i = tid; i < 2 * KT2 * NE * 64; i += 256) {
        const int ln = i & 63, e = (i >> 6) % NE, kt = (i >> 6) / NE;
        const int k = kt * 32 + (ln & 31);
        T v8[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int kk = 16 * e + 8 * (ln >> 5) + j;
            const bool ok = k < K && kk < nk;
            const T v = w[ok ? k * nk + (kk % 9) * C + kk / 9 : 0];                 // [K][3][3][C]: tap kk = 9 c + 3 r + s of filter k
            v8[j] = ok ? v : from_f32<T>(0.f);
        }
        vec pk;
        __builtin_memcpy(&pk, v8, 16);
        sW[i] = pk;
    }
    for (int i = tid; i < KT2 * 64; i += 256) sB[i] = i < K ? bias_of<T>(ep, i) : 0.f;
    __syncthreads();

    // a lane's taps in the tile's patch, in the gathering kernel's order: tap kk = 9 c + 3 r + s meets the input at
    // row r, element s C + c past the pixel's first: byte offset relative to that; taps past 9 C read the pixel itself
    // and are masked
    int off[NE][8];
    unsigned tapmask = 0;
#pragma unroll
    for (int e = 0; e < NE; ++e)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int kk = 16 * e + 8 * lh + j;
            const int c = kk / 9, r = (kk % 9) / 3, q = kk % 3;
            off[e][j] = kk < nk ? (r * PPN * 2 + q * C + c) * 2 : 0;
            tapmask |= kk < nk ? 1u << (8 * e + j) : 0u;
        }
    // the patch as loaded: pair 64 j + lane of [6][PPN], as row | pair of the row << 8 (row 255, never inside, past it)
    constexpr int NL = dsc_nhwc_loads(NE);
    unsigned prp[NL];
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        const int t = 64 * j + lane;
        const int rr = t / PPN, pp = t - rr * PPN;
        prp[j] = t < npairs ? (unsigned)(rr | pp << 8) : 0xFFu;
    }
    const int rounds = (npairs + 63) / 64;                                       // wave-uniform
    const char* xb = reinterpret_cast<const char*>(x);
    char* yb = reinterpret_cast<char*>(y);
    const unsigned psel = (lane & 1) ? 0x03020706u : 0x05040100u;                 // (own pair, neighbour's pair) -> what the lane stores
    const int WC = W * C;                                                         // elements of an image row (even)

    const int wstride = (int)gridDim.x * 4;
    int tile = (int)blockIdx.x * 4 + wave;
    int n = 0, oh0 = 0, ow0 = 0;                                                  // of the tile whose input is on its way
    unsigned v[NL], inside = 0;                                                   // bit j: pair j lies inside the image
    auto request = [&](int t) __attribute__((always_inline)) {
        n = t / (tiles_y * tiles_x);
        const int trem = t - n * tiles_y * tiles_x;
        oh0 = (trem / tiles_x) * DSC_WR;
        ow0 = (trem - (trem / tiles_x) * tiles_x) * 32;
        const int e0 = (ow0 - pad) * C - (((ow0 - pad) * C) & 1);                // first element of the patch's rows: even
        const int base = (n * H + oh0 - pad) * WC + e0;
        inside = 0;
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            if (j < rounds) {                                                     // (uniform)
                const int rr = prp[j] & 0xFF, pp = prp[j] >> 8;
                const int ih = oh0 - pad + rr, ie = e0 + 2 * pp;
                const bool in = ih >= 0 && ih < H && ie >= 0 && ie < WC;          // (a row starts and ends at an even element)
                v[j] = *reinterpret_cast<const unsigned*>(xb + (in ? (unsigned)(base + rr * WC + 2 * pp) * 2u : 0u));
                inside |= in ? 1u << j : 0u;
            }
        }
    };
    if (tile < ntiles) request(tile);
#pragma unroll 1
    while (tile < ntiles) {
        const int cn = n, coh0 = oh0, cow0 = ow0;                                 // the tile to compute
        const int shift = ((cow0 - pad) * C) & 1;
#pragma unroll
        for (int j = 0; j < NL; ++j)
            if (j < rounds && 64 * j + lane < npairs) sP[64 * j + lane] = v[j] & (0u - ((inside >> j) & 1u));
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        tile += wstride;
        if (tile < ntiles) request(tile);

#pragma unroll 1
        for (int g = 0; g < DSC_WR; ++g) {
            const int oh = coh0 + g;
            if (oh >= Ho) break;                                                  // wave-uniform
            const unsigned char* pb = reinterpret_cast<const unsigned char*>(sP) + (g * PPN * 2 + l32 * C + shift) * 2;
            vec a[NE];                                                            // the pixels' taps
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                unsigned short raw[8];
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    raw[j] = (unsigned short)(*reinterpret_cast<const unsigned short*>(pb + off[e][j]) & (0u - ((tapmask >> (8 * e + j)) & 1u)));
                __builtin_memcpy(&a[e], raw, 16);
            }
            // after the exchanges a lane keeps filters (lane & ~1, + 1) of one pixel: even lanes the pixel of the
            // even register, odd lanes the next one
            const unsigned yrow = (unsigned)((cn * Ho + oh) * Wo + cow0) * (unsigned)K * 2u + (unsigned)(lane & ~1) * 2u;
#pragma unroll 1
            for (int kp = 0; kp < KT2; ++kp) {
                // register r of a lane: pixel 8 (r / 4) + 4 lh + r % 4 of the row's 32, filter 32 (2 kp + u) + l32
                // (the sums start at the bias of the lane's filter)
                floatx16 acc[2];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    acc[0][r] = sB[kp * 64 + l32];
                    acc[1][r] = sB[kp * 64 + 32 + l32];
                }
                const vec* wk = sW + (size_t)(2 * kp) * NE * 64 + lane;
#pragma unroll
                for (int e = 0; e < NE; ++e) {
                    Mma<T>::run(a[e], wk[e * 64], acc[0]);
                    Mma<T>::run(a[e], wk[(NE + e) * 64], acc[1]);
                }
                const bool kok = kp * 64 + (lane | 1) < K;                          // (K even: the lane's two filters exist together)
                // registers 2i and 2i + 1 of half u (after the exchange of halves) are pixels p and p + 1,
                // p = 8 (i / 2) + 4 u + 2 (i % 2), for 64 filters
                auto put = [&](int i, bool relu) __attribute__((always_inline)) {
                    const auto s0 = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[0][2 * i]), __float_as_uint(acc[1][2 * i]), false, false);
                    const auto s1 = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[0][2 * i + 1]), __float_as_uint(acc[1][2 * i + 1]), false, false);
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        float a0 = __uint_as_float(s0[u]), a1 = __uint_as_float(s1[u]);
                        if (relu) {                                                // max(a, 0), 0 for a NaN (as fmaxf)
                            asm("v_max_f32_e32 %0, 0, %1" : "=v"(a0) : "v"(a0));
                            asm("v_max_f32_e32 %0, 0, %1" : "=v"(a1) : "v"(a1));
                        }
                        const unsigned own = pack2<T>(a0, a1);
                        const unsigned nb = (unsigned)__builtin_amdgcn_mov_dpp((int)own, 0xB1, 0xF, 0xF, true);
                        const unsigned out = __builtin_amdgcn_perm(nb, own, psel);
                        const int p = 8 * (i >> 1) + 4 * u + 2 * (i & 1);           // (Wo even: pixels p and p + 1 exist together)
                        if (kok && cow0 + p < Wo)
                            *reinterpret_cast<unsigned*>(yb + (yrow + (unsigned)(p + (lane & 1)) * (unsigned)K * 2u + (unsigned)(kp * 128))) = out;
                    }
                };
                // (every lane takes part in the exchanges; only the stores are conditional)
                if (ep.relu) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) put(i, true);
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) put(i, false);
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                   // (the tile's LDS reads before the next tile's writes)
        __builtin_amdgcn_wave_barrier();
    }
}

}  // namespace wino
