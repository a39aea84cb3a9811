// Host-side C++ check of the drop-in shim (include/wino_dropin.hpp): a caller
// written against the reference's headers, as comparison/layoutCompare.cu:143-205
// is -- device buffers from hipMalloc, one call per (source, destination) layout
// pair, results copied back and compared with a direct convolution computed
// here.  Small integers make every value exact, so the comparison is ==.
// Prints "DROPIN OK" and exits 0 on success.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#include "wino_dropin.hpp"

static void strides(DataLayout l, long N, long C, long H, long W, long s[4]) {
    switch (l) {
    case DataLayout::NCHW: s[0] = C * H * W; s[1] = H * W; s[2] = W; s[3] = 1; break;
    case DataLayout::NHWC: s[0] = H * W * C; s[1] = 1; s[2] = W * C; s[3] = C; break;
    case DataLayout::CHWN: s[0] = 1; s[1] = H * W * N; s[2] = W * N; s[3] = N; break;
    }
}
static void fstrides(DataLayout l, long K, long C, long s[4]) {
    switch (l) {
    case DataLayout::NCHW: s[0] = 9 * C; s[1] = 9; s[2] = 3; s[3] = 1; break;
    case DataLayout::NHWC: s[0] = 9 * C; s[1] = 1; s[2] = 3 * C; s[3] = C; break;
    case DataLayout::CHWN: s[0] = 1; s[1] = 9 * K; s[2] = 3 * K; s[3] = K; break;
    }
}
#define CK(e)                                                                      \
    do {                                                                           \
        hipError_t r_ = (e);                                                       \
        if (r_ != hipSuccess) { std::printf("%s: %s\n", #e, hipGetErrorString(r_)); return 1; } \
    } while (0)

int main() {
    const int N = 3, C = 5, K = 7, H = 10, pad = 1;
    const DataLayout layouts[3] = {DataLayout::NCHW, DataLayout::NHWC, DataLayout::CHWN};
    unsigned seed = 12345u;
    auto rnd = [&](int lo, int hi) { seed = seed * 1664525u + 1013904223u; return (float)(lo + (int)((seed >> 16) % (unsigned)(hi - lo + 1))); };
    std::vector<float> xl((size_t)N * C * H * H), wl((size_t)K * C * 9);   // logical NCHW / KCRS
    for (auto& v : xl) v = rnd(-3, 3);
    for (auto& v : wl) v = rnd(-2, 2);
    wino_warmup();
    int bad = 0;
    for (DataLayout src : layouts)
        for (DataLayout dst : layouts) {
            long sx[4], sw[4], sy[4];
            strides(src, N, C, H, H, sx); fstrides(src, K, C, sw); strides(dst, N, K, H, H, sy);
            std::vector<float> x(xl.size()), w(wl.size()), y((size_t)N * K * H * H, -777.f), want(y.size());
            for (int n = 0; n < N; ++n) for (int c = 0; c < C; ++c) for (int h = 0; h < H; ++h) for (int v = 0; v < H; ++v)
                x[n * sx[0] + c * sx[1] + h * sx[2] + v * sx[3]] = xl[((size_t)(n * C + c) * H + h) * H + v];
            for (int k = 0; k < K; ++k) for (int c = 0; c < C; ++c) for (int r = 0; r < 3; ++r) for (int s = 0; s < 3; ++s)
                w[k * sw[0] + c * sw[1] + r * sw[2] + s * sw[3]] = wl[((size_t)(k * C + c) * 3 + r) * 3 + s];
            for (int n = 0; n < N; ++n) for (int k = 0; k < K; ++k) for (int i = 0; i < H; ++i) for (int j = 0; j < H; ++j) {
                float acc = 0;
                for (int c = 0; c < C; ++c) for (int r = 0; r < 3; ++r) for (int s = 0; s < 3; ++s) {
                    int ih = i + r - pad, iw = j + s - pad;
                    if (ih < 0 || ih >= H || iw < 0 || iw >= H) continue;
                    acc += xl[((size_t)(n * C + c) * H + ih) * H + iw] * wl[((size_t)(k * C + c) * 3 + r) * 3 + s];
                }
                want[n * sy[0] + k * sy[1] + i * sy[2] + j * sy[3]] = acc;
            }
            float *dx, *dw, *dy;
            CK(hipMalloc(&dx, x.size() * 4)); CK(hipMalloc(&dw, w.size() * 4)); CK(hipMalloc(&dy, y.size() * 4));
            CK(hipMemcpy(dx, x.data(), x.size() * 4, hipMemcpyHostToDevice));
            CK(hipMemcpy(dw, w.data(), w.size() * 4, hipMemcpyHostToDevice));
            CK(hipMemcpy(dy, y.data(), y.size() * 4, hipMemcpyHostToDevice));
            int chn = C;
            if (src == dst && src == DataLayout::NCHW) wrapedConv_NCHW(N, H, chn, K, pad, dx, dw, nullptr, nullptr, nullptr, &dy);
            else if (src == dst && src == DataLayout::NHWC) wrapedConv_NHWC(N, H, chn, K, pad, dx, dw, nullptr, nullptr, nullptr, &dy);
            else if (src == dst) wrapedConv_CHWN(N, H, chn, K, pad, dx, dw, nullptr, nullptr, nullptr, &dy);
            else layoutManager(src, dst, N, H, chn, K, pad, dx, dw, nullptr, nullptr, nullptr, &dy);
            CK(hipMemcpy(y.data(), dy, y.size() * 4, hipMemcpyDeviceToHost));   // no sync needed: the call is blocking
            size_t diff = 0;
            for (size_t i = 0; i < y.size(); ++i) diff += y[i] != want[i];
            if (chn != K) { std::printf("chn not updated: %d\n", chn); ++bad; }
            if (diff) { std::printf("layout %d -> %d: %zu mismatches\n", (int)src, (int)dst, diff); ++bad; }
            CK(hipFree(dx)); CK(hipFree(dw)); CK(hipFree(dy));
        }
    if (bad) { std::printf("DROPIN FAILED (%d)\n", bad); return 1; }
    std::printf("DROPIN OK\n");
    return 0;
}
