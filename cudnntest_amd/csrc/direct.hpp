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
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const long pq = q0 + 8 * (r >> 2) + 4 * lh + (r & 3);
                        float v = acc[r] + bk;
                        if (ep.relu) v = fmaxf(v, 0.f);
                        if (pq < Q) y[pq * K + k] = from_f32<T>(v);
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
            floatx16 acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
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
                const float bk = sB[k];
                if (k < K) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const long pq = q0 + 8 * (r >> 2) + 4 * lh + (r & 3);
                        float v = acc[r] + bk;
                        if (ep.relu) v = fmaxf(v, 0.f);
                        if (pq < Q) y[pq * K + k] = from_f32<T>(v);
                    }
                }
                continue;
            }
            float bv[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) bv[r] = sB[kt * 32 + 8 * (r >> 2) + (r & 3) + 4 * lh];
            const T* yk = y + (size_t)kt * 32 * ys.c;
            auto put = [&](int r) {
                float v = acc[r] + bv[r];
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

}  // namespace wino
