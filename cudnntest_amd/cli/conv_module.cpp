// Stand-alone single-layer driver with the reference's per-layout interface
// (layoutTest/NHWC/convModule_NHWC_padding.cu:8-121 and its NCHW / CHWN siblings, built there as
// ./NCHW/a.out, ./NHWC/a.out, ./CHWN/a.out by layoutTest/make.sh):
//
//     conv_module <bat4Conv> <inside> <chn> <numOfFilter> [layout=<NCHW|NHWC|CHWN|0|1|2>] [data=<dir>]
//                 [padding=<p>] [runs=<n>] [algo=<auto|staged|epilogue|fused|f4>]
//
// The reference has one program per layout; here the layout is an option (default NHWC, the program its
// only committed latencies come from: layoutTest/NHWC/test.sh:3-8 -> result.num).  Like the reference it reads
// raw float32 files <data>/data/input.bin and <data>/data/filter.bin (:11-15,53-54) in the layout's own
// element order, runs the layer `runs` times (10, :88-90) between two events with the filter transform and
// a device synchronisation in every call, and prints
//     inside: <H>, oside:<Ho>
//     time:<us> us TFLOPS:<rate>
//     convOutput_cpu[0]:<value>
// with the reference's own rate formula ((9*chn*chn + chn) * inside^2 * bat4Conv operations, :101 -- one per
// multiply-add, filters counted as chn), so layoutTest/NHWC/test.sh's `grep -Eo '[0-9]+(\.[0-9]+) us'` keeps
// working; a second line gives the direct-convolution rate 2*9*N*K*C*Ho*Wo / t.  The output is saved as
// <data>/data/ConvModule_<LAYOUT>.bin (:113-118).  A missing input file is replaced by seeded synthetic data
// of the same size, and said so; a missing data directory only loses the saved output.
#include <hip/hip_runtime.h>

#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "wino_dropin.hpp"

static std::string opt_str(int argc, char** argv, const char* key, const char* dflt) {
    const size_t n = std::strlen(key);
    for (int i = 5; i < argc; ++i)
        if (!std::strncmp(argv[i], key, n) && argv[i][n] == '=') return std::string(argv[i] + n + 1);
    return dflt;
}
static bool read_floats(const std::string& path, size_t count, std::vector<float>& out) {
    FILE* f = std::fopen(path.c_str(), "rb");
    if (!f) return false;
    std::vector<float> buf(count);
    const size_t got = std::fread(buf.data(), sizeof(float), count, f);
    std::fclose(f);
    if (got != count) return false;
    out.swap(buf);
    return true;
}
static void synthetic(std::vector<float>& v, size_t count, unsigned long long seed, float scale) {
    v.resize(count);
    for (size_t i = 0; i < count; ++i) {
        unsigned long long z = seed + 0x9E3779B97F4A7C15ull * (i + 1);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        v[i] = ((float)(z >> 40) * (1.0f / 8388608.0f) - 1.0f) * scale;
    }
}
#define CK(e)                                                                                    \
    do {                                                                                         \
        hipError_t r_ = (e);                                                                     \
        if (r_ != hipSuccess) { std::printf("%s: %s\n", #e, hipGetErrorString(r_)); return 1; } \
    } while (0)

int main(int argc, char** argv) {
    if (argc < 5) {
        std::printf("usage: %s <bat4Conv> <inside> <chn> <numOfFilter> [layout=NCHW|NHWC|CHWN] [data=<dir>] "
                    "[padding=<p>] [runs=<n>] [algo=auto|staged|epilogue|fused|f4]\n", argv[0]);
        return 2;
    }
    const int n = std::atoi(argv[1]), inside = std::atoi(argv[2]), chn = std::atoi(argv[3]), filters = std::atoi(argv[4]);
    const int padding = std::atoi(opt_str(argc, argv, "padding", "1").c_str());
    const int runs = std::atoi(opt_str(argc, argv, "runs", "10").c_str());
    const std::string data = opt_str(argc, argv, "data", ".");
    const std::string lname = opt_str(argc, argv, "layout", "NHWC"), aname = opt_str(argc, argv, "algo", "auto");
    int lay = -1, algo = -1;
    const char* lnames[3] = {"NCHW", "NHWC", "CHWN"};
    for (int i = 0; i < 3; ++i)
        if (lname == lnames[i] || lname == std::to_string(i)) lay = i;
    const struct { const char* name; int algo; } algos[5] = {{"auto", WINO_ALGO_AUTO}, {"staged", WINO_ALGO_STAGED},
        {"epilogue", WINO_ALGO_EPILOGUE}, {"fused", WINO_ALGO_FUSED}, {"f4", WINO_ALGO_STAGED_F4}};
    for (const auto& a : algos)
        if (aname == a.name) algo = a.algo;
    const int oside = inside - 2 + 2 * padding;
    if (n < 1 || inside < 1 || chn < 1 || filters < 1 || runs < 1 || lay < 0 || algo < 0 || oside < 1) {
        std::printf("bad argument\n");
        return 2;
    }
    const size_t nInput = (size_t)n * inside * inside * chn, nFilter = (size_t)9 * filters * chn;
    const size_t nOutput = (size_t)n * oside * oside * filters;
    std::vector<float> x_h, w_h, y_h(nOutput);
    if (!read_floats(data + "/data/input.bin", nInput, x_h)) {
        std::printf("no %s/data/input.bin (%zu floats): synthetic input\n", data.c_str(), nInput);
        synthetic(x_h, nInput, 0x1A6Eull, 0.5f);
    }
    if (!read_floats(data + "/data/filter.bin", nFilter, w_h)) {
        std::printf("no %s/data/filter.bin (%zu floats): synthetic filters\n", data.c_str(), nFilter);
        synthetic(w_h, nFilter, 0xF11Full, 0.5f);
    }
    float *x_d = nullptr, *w_d = nullptr, *y_d = nullptr;
    CK(hipMalloc(&x_d, nInput * sizeof(float)));
    CK(hipMalloc(&w_d, nFilter * sizeof(float)));
    CK(hipMalloc(&y_d, nOutput * sizeof(float)));
    CK(hipMemcpy(x_d, x_h.data(), nInput * sizeof(float), hipMemcpyHostToDevice));
    CK(hipMemcpy(w_d, w_h.data(), nFilter * sizeof(float), hipMemcpyHostToDevice));
    std::printf("inside: %d, oside:%d\n", inside, oside);
    wino_warmup();

    hipEvent_t t0, t1;
    CK(hipEventCreate(&t0));
    CK(hipEventCreate(&t1));
    CK(hipEventRecord(t0, nullptr));
    for (int i = 0; i < runs; ++i) {
        if (algo == WINO_ALGO_AUTO) {            // the reference's call, through the drop-in header
            int c = chn;
            const DataLayout L = (DataLayout)lay;
            layoutManager(L, L, n, inside, c, filters, padding, x_d, w_d, nullptr, nullptr, nullptr, &y_d);
        } else {                                 // a pipeline by name: the same call through the C ABI, synchronous like it
            const int rc = wino_conv(lay, lay, WINO_F32, algo, 0, n, chn, filters, inside, inside, padding, x_d, w_d, y_d, nullptr);
            if (rc) {
                std::printf("wino_conv: %s\n", wino_last_error());
                return 1;
            }
            CK(hipDeviceSynchronize());
        }
    }
    CK(hipEventRecord(t1, nullptr));
    CK(hipEventSynchronize(t1));
    float ms = 0.f;
    CK(hipEventElapsedTime(&ms, t0, t1));
    ms /= (float)runs;
    CK(hipMemcpy(y_h.data(), y_d, nOutput * sizeof(float), hipMemcpyDeviceToHost));
    const double ref_ops = ((9.0 * chn) * chn + chn) * 1.0e-9 * inside * inside * n;   // the reference's count
    std::printf("time:%lf us TFLOPS:%lf\n", (double)ms * 1000.0, ref_ops / ms);
    std::printf("direct-convolution rate: %lf TFLOP/s\n", 2.0 * 9.0 * n * filters * chn * oside * oside * 1.0e-9 / ms);
    std::printf("convOutput_cpu[0]:%lf\n", (double)y_h[0]);
    if (y_h[0] == 0.0f) std::printf("moduleConv error\n");

    const std::string out = data + "/data/ConvModule_" + lnames[lay] + ".bin";
    FILE* f = std::fopen(out.c_str(), "wb");
    if (!f) {
        std::printf("Bad file path: %s, %s\n", std::strerror(errno), out.c_str());
    } else {
        const size_t put = std::fwrite(y_h.data(), sizeof(float), nOutput, f);
        std::fclose(f);
        if (put != nOutput) return 1;
    }
    (void)hipFree(x_d);
    (void)hipFree(w_d);
    (void)hipFree(y_d);
    return 0;
}
