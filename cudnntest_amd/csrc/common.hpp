// Shared definitions of the gfx950 Winograd F(2x2,3x3) library: layouts, strides,
// storage-type conversion, padded operand geometry.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/wino_amd.h"

namespace wino {

// element strides of an activation tensor in the order (n, c, h, w)
struct ActStrides {
    long n, c, h, w;
};

__host__ __device__ inline ActStrides act_strides(int layout, long N, long C, long H, long W) {
    switch (layout) {
    case WINO_NHWC: return {H * W * C, 1, W * C, C};
    case WINO_CHWN: return {1, H * W * N, W * N, N};
    default: return {C * H * W, H * W, W, 1};
    }
}

// element strides of a filter bank in the order (k, c, r, s)
struct FltStrides {
    long k, c, r, s;
};

__host__ __device__ inline FltStrides flt_strides(int layout, long K, long C) {
    switch (layout) {
    case WINO_NHWC: return {9 * C, 1, 3 * C, C};
    case WINO_CHWN: return {1, 9 * K, 3 * K, K};
    default: return {9 * C, 9, 3, 1};
    }
}

// ---- storage types ---------------------------------------------------------
struct bf16_t {
    uint16_t bits;
};
typedef _Float16 f16_t;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(f16_t v) { return (float)v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float((uint32_t)v.bits << 16); }

template <typename T> __device__ __forceinline__ T from_f32(float f);
template <> __device__ __forceinline__ float from_f32<float>(float f) { return f; }
template <> __device__ __forceinline__ f16_t from_f32<f16_t>(float f) { return (f16_t)f; }
// round to nearest even; gfx950 has the conversion in hardware (v_cvt_pk_bf16_f32)
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float f) {
    return bf16_t{__builtin_bit_cast(uint16_t, (__bf16)f)};
}

// two values rounded to T (nearest even), a in the low half of the result
template <typename T> __device__ __forceinline__ unsigned pack2(float a, float b);
template <> __device__ __forceinline__ unsigned pack2<bf16_t>(float a, float b) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(unsigned, __builtin_convertvector((f32x2){a, b}, bf16x2));
}
template <> __device__ __forceinline__ unsigned pack2<f16_t>(float a, float b) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(unsigned, __builtin_convertvector((f32x2){a, b}, f16x2));
}

// What the output stage applies to the 2x2 outputs of a tile before storing them:
//     y = pool2x2( relu( conv + bias[k] ) )        (each step optional)
// bias holds K elements of the tensor's element type.  With pool the destination has
// floor(Ho/2) x floor(Wo/2) outputs per image and filter: the 2x2 outputs of an F(2x2,3x3) tile are
// exactly one pooling window (the reference applies addBias_CHWN, relu_CHWN and maxPool_CHWN as
// separate passes over y: netTest/cudnn_test_0124/VGG_Batched/CHWN_support.cuh:107,512,248).
struct Epilogue {
    const void* bias;
    int relu, pool;
};
template <typename T> __device__ __forceinline__ float bias_of(const Epilogue& ep, int k) {
    return ep.bias ? to_f32(static_cast<const T*>(ep.bias)[k]) : 0.f;
}

// v with its lanes swapped pairwise (0 <-> 1, 2 <-> 3, ...)
__device__ __forceinline__ float swap_lane_pairs(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));
}

// v with its bits ANDed by m (m is all ones or zero).  Opaque to the optimiser on purpose:
// written as a select, the compiler moves the load that produced v under a branch on the mask and
// waits for every load separately, instead of issuing a batch of loads and masking afterwards.
__device__ __forceinline__ float mask_keep(float v, unsigned m) {
    unsigned r;
    asm("v_and_b32 %0, %1, %2" : "=v"(r) : "v"(__float_as_uint(v)), "v"(m));
    return __uint_as_float(r);
}

__host__ inline size_t dtype_size(int dtype) { return dtype == WINO_F32 ? 4 : 2; }

// ---- channel vectors ------------------------------------------------------------
// The transformed operands keep CV consecutive channels of one (coordinate, tile)
// or (coordinate, filter) together in a 16-byte vector:
//     U[xi][Cp/CV][Kp][CV]     V[xi][Cp/CV][Pp][CV]      CV = 16 / sizeof(T)
// so every HBM and LDS access of the GEMM side is a 16-byte access, and a lane
// of an MFMA fetches the channels it multiplies with one LDS read.
template <typename T> struct ChanVec {
    static constexpr int n = 16 / (int)sizeof(T);
};
__host__ inline int chan_vec(int dtype) { return dtype == WINO_F32 ? 4 : 8; }

template <typename T> struct alignas(16) Pack16 {
    T e[16 / sizeof(T)];
};

// dst[0..CV) = v[0..CV) as one 16-byte store
template <typename T> __device__ __forceinline__ void store_chan_vec(T* dst, const float* v) {
    Pack16<T> pk;
#pragma unroll
    for (int i = 0; i < ChanVec<T>::n; ++i) pk.e[i] = from_f32<T>(v[i]);
    *reinterpret_cast<Pack16<T>*>(dst) = pk;
}

// ---- padded geometry ---------------------------------------------------------
// the reduction (channel) dimension of U and V is padded to 4 channel vectors (two k-groups)
__host__ inline int c_pad(int dtype) { return 4 * chan_vec(dtype); }   // 16 (fp32) or 32 (f16/bf16)
constexpr int kKPad = 128;   // filter dimension of U / Mo
constexpr int kPPad = 128;   // tile dimension of V / Mo

struct Geometry {
    int m;          // outputs per tile side: 2 for F(2x2,3x3), 4 for F(4x4,3x3)
    int N, C, K, H, W, pad;
    int Ho, Wo, th, tw;
    long P;
    int Cp, Kp;
    long Pp;
};

__host__ inline long round_up(long v, long m) { return (v + m - 1) / m * m; }

// Zero padding beyond one row/column is honoured arithmetically, like the reference does
// (comparison/wrapedConv_NCHW.cuh:346-362), by the layout-generic transforms of the staged pipelines.
constexpr int kMaxPad = 1024;
__host__ inline bool make_geometry(int dtype, int N, int C, int K, int H, int W, int pad, Geometry* g, int m = 2) {
    g->m = m;
    if (N <= 0 || C <= 0 || K <= 0 || H <= 0 || W <= 0 || pad < 0 || pad > kMaxPad) return false;
    g->N = N; g->C = C; g->K = K; g->H = H; g->W = W; g->pad = pad;
    g->Ho = H + 2 * pad - 2;
    g->Wo = W + 2 * pad - 2;
    if (g->Ho <= 0 || g->Wo <= 0) return false;
    g->th = (g->Ho + m - 1) / m;
    g->tw = (g->Wo + m - 1) / m;
    g->P = (long)N * g->th * g->tw;
    if (g->P >= (1L << 31)) return false;          // the kernels decode tile indices with 32-bit arithmetic
    g->Cp = (int)round_up(C, c_pad(dtype));
    g->Kp = (int)round_up(K, kKPad);
    g->Pp = round_up(g->P, kPPad);
    return true;
}

// tile index -> (n, ty, tx); p < 2^31 (make_geometry), so 32-bit unsigned divisions (a quarter of the
// instructions of 64-bit ones: the stores of the GEMM epilogues decode up to 16 tiles per lane)
__device__ __forceinline__ void decode_tile(long p, int order, int N, int th, int tw, int& n, int& ty, int& tx) {
    const unsigned pu = (unsigned)p;
    if (order == WINO_TILES_BATCH_MAJOR) {
        const unsigned q = pu / (unsigned)tw;
        tx = (int)(pu - q * (unsigned)tw);
        const unsigned nn = q / (unsigned)th;
        ty = (int)(q - nn * (unsigned)th);
        n = (int)nn;
    } else {
        const unsigned q = pu / (unsigned)N;
        n = (int)(pu - q * (unsigned)N);
        const unsigned yy = q / (unsigned)tw;
        tx = (int)(q - yy * (unsigned)tw);
        ty = (int)yy;
    }
}

}  // namespace wino
