// Drop-in C++ shim: the reference's wrapped-convolution call surface, same
// names, same argument order and meaning, over the C ABI in wino_amd.h.
//
//   wrapedConv_NCHW / wrapedConv_NHWC / wrapedConv_CHWN
//       comparison/wrapedConv_NCHW.cuh:335, wrapedConv_NHWC.cuh:24, wrapedConv_CHWN.cuh:16
//   convLayoutTrans_{CHWN_to_NCHW, CHWN_to_NHWC, NHWC_to_NCHW, NHWC_to_CHWN, NCHW_to_NHWC, NCHW_to_CHWN}
//       comparison/DataLayoutTrans.cuh:9,101,192,309,418,502
//   enum class DataLayout, layoutManager
//       comparison/DataLayoutTrans.cuh:587-651
//
// Conventions kept from the reference: all pointers are device pointers owned
// by the caller; `chn` is overwritten with numOfFilter (wrapedConv_NCHW.cuh:479);
// only *output is used and it is never reallocated; the call returns after the
// work has finished (the reference ends with a device synchronisation, :482);
// work goes to the null stream; nothing is returned.  A failure, which the
// reference would let pass silently, is reported on stderr.
//
// Difference: inputTran_gpu / filterTran_gpu / gemmOutput_gpu are accepted and
// ignored.  The library picks its pipeline per layer -- F(4x4,3x3) like the
// reference for fp32 layers with C, K >= 128, F(2x2,3x3) or a direct kernel
// otherwise -- and pads its operands to its own tile sizes, so its scratch is
// not what a reference caller sizes (36*MSize*KSize ...): it draws scratch from
// its own per-device arena (or from wino_set_workspace).
#pragma once
#include <cstdio>

#include "wino_amd.h"

enum class DataLayout { NCHW, NHWC, CHWN };

namespace wino_dropin_detail {
inline void run(int src, int dst, int bat4Conv, int inside, int& chn, int numOfFilter, int padding, float* m1,
                float* m2, float** output) {
    int rc = output ? wino_conv(src, dst, WINO_F32, WINO_ALGO_AUTO, 0u, bat4Conv, chn, numOfFilter, inside, inside,
                                padding, m1, m2, *output, nullptr)
                    : WINO_ERR_INVALID;
    if (rc == WINO_OK) rc = wino_sync(nullptr);
    if (rc != WINO_OK) std::fprintf(stderr, "wino_amd: convolution failed (%d): %s\n", rc, wino_last_error());
    chn = numOfFilter;
}
}  // namespace wino_dropin_detail

#define WINO_DROPIN_ARGS                                                                                        \
    int bat4Conv, int inside, int &chn, int numOfFilter, int padding, float *m1, float *m2, float *inputTran_gpu, \
        float *filterTran_gpu, float *gemmOutput_gpu, float **output
#define WINO_DROPIN_UNUSED (void)inputTran_gpu, (void)filterTran_gpu, (void)gemmOutput_gpu

inline void wrapedConv_NCHW(WINO_DROPIN_ARGS) {
    WINO_DROPIN_UNUSED;
    wino_dropin_detail::run(WINO_NCHW, WINO_NCHW, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output);
}
inline void wrapedConv_NHWC(WINO_DROPIN_ARGS) {
    WINO_DROPIN_UNUSED;
    wino_dropin_detail::run(WINO_NHWC, WINO_NHWC, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output);
}
inline void wrapedConv_CHWN(WINO_DROPIN_ARGS) {
    WINO_DROPIN_UNUSED;
    wino_dropin_detail::run(WINO_CHWN, WINO_CHWN, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output);
}
inline void convLayoutTrans_CHWN_to_NCHW(WINO_DROPIN_ARGS) {
    WINO_DROPIN_UNUSED;
    wino_dropin_detail::run(WINO_CHWN, WINO_NCHW, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output);
}
inline void convLayoutTrans_CHWN_to_NHWC(WINO_DROPIN_ARGS) {
    WINO_DROPIN_UNUSED;
    wino_dropin_detail::run(WINO_CHWN, WINO_NHWC, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output);
}
inline void convLayoutTrans_NHWC_to_NCHW(WINO_DROPIN_ARGS) {
    WINO_DROPIN_UNUSED;
    wino_dropin_detail::run(WINO_NHWC, WINO_NCHW, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output);
}
inline void convLayoutTrans_NHWC_to_CHWN(WINO_DROPIN_ARGS) {
    WINO_DROPIN_UNUSED;
    wino_dropin_detail::run(WINO_NHWC, WINO_CHWN, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output);
}
inline void convLayoutTrans_NCHW_to_NHWC(WINO_DROPIN_ARGS) {
    WINO_DROPIN_UNUSED;
    wino_dropin_detail::run(WINO_NCHW, WINO_NHWC, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output);
}
inline void convLayoutTrans_NCHW_to_CHWN(WINO_DROPIN_ARGS) {
    WINO_DROPIN_UNUSED;
    wino_dropin_detail::run(WINO_NCHW, WINO_CHWN, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output);
}

// Dispatch on (source layout, destination layout), as comparison/DataLayoutTrans.cuh:594-651.
inline void layoutManager(DataLayout srcLayout, DataLayout dstLayout, int bat4Conv, int inside, int& chn,
                          int numOfFilter, int padding, float* input, float* weights, float* inputTran_gpu,
                          float* filterTran_gpu, float* gemmOutput_gpu, float** output) {
    WINO_DROPIN_UNUSED;
    wino_dropin_detail::run(static_cast<int>(srcLayout), static_cast<int>(dstLayout), bat4Conv, inside, chn,
                            numOfFilter, padding, input, weights, output);
}

#undef WINO_DROPIN_ARGS
#undef WINO_DROPIN_UNUSED
