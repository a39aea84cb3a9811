// Command-line driver with the reference's interface (comparison/layoutCompare.cu:32-148):
//
//     layout_compare batch=<N> opt=<0|1|2> layer=<1..9> [data=<dir>] [runs=<n>] [save=<file.bin>]
//
// opt selects the layout of input, filters and output (0 NCHW, 1 NHWC, 2 CHWN, as :189-203; the
// reference's opt 3..6 are its cuDNN baselines and do not exist here), layer one of the nine distinct
// VGG-16 3x3 shapes of its table (:41-80).  Like the reference it reads raw float32 files --
// <data>/vggData/conv<k>.bin for the filter bank and <data>/binImage/file_<i>.bin for run i
// (get_parameter, comparison/util.h:99-113) -- runs the layer through layoutManager once per file
// inside an event bracket and prints "time:<ms> ms" and the first output value, so the reference's
// shell loops (comparison/test.sh greps "[0-9.]+ ms") can drive it.  A missing file is replaced by
// seeded synthetic data of the same size, and said so.  save= writes the last output as raw float32
// (save_parameter, util.h:115-127).
#include <hip/hip_runtime.h>

#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "wino_dropin.hpp"

static int arg_int(int argc, char** argv, const char* key, int dflt) {
    const size_t n = std::strlen(key);
    for (int i = 1; i < argc; ++i)
        if (!std::strncmp(argv[i], key, n) && argv[i][n] == '=') return std::atoi(argv[i] + n + 1);
    return dflt;
}
static std::string arg_str(int argc, char** argv, const char* key, const char* dflt) {
    const size_t n = std::strlen(key);
    for (int i = 1; i < argc; ++i)
        if (!std::strncmp(argv[i], key, n) && argv[i][n] == '=') return std::string(argv[i] + n + 1);
    return dflt;
}

// `count` float32 values of a raw file; false (and `out` untouched) if it cannot be read in full
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
static bool write_floats(const std::string& path, const std::vector<float>& v) {
    FILE* f = std::fopen(path.c_str(), "wb");
    if (!f) {
        std::printf("Bad file path: %s, %s\n", std::strerror(errno), path.c_str());
        return false;
    }
    const size_t put = std::fwrite(v.data(), sizeof(float), v.size(), f);
    std::fclose(f);
    return put == v.size();
}
// seeded stand-in for a missing file: uniform in [-scale, scale)
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
    const int n = arg_int(argc, argv, "batch", 1);
    const int opt = arg_int(argc, argv, "opt", 0);
    const int layer = arg_int(argc, argv, "layer", 0);
    const int runs = arg_int(argc, argv, "runs", 20);
    const std::string data = arg_str(argc, argv, "data", ".");
    const std::string save = arg_str(argc, argv, "save", "");
    // the reference's table: layer -> (side, channels, filters, filter file)
    static const struct { int h, c, k; const char* file; } table[10] = {
        {0, 0, 0, ""},           {224, 3, 64, "conv1.bin"},    {224, 64, 64, "conv2.bin"},   {112, 64, 128, "conv3.bin"},
        {112, 128, 128, "conv4.bin"}, {56, 128, 256, "conv5.bin"}, {56, 256, 256, "conv7.bin"},  {28, 256, 512, "conv8.bin"},
        {28, 512, 512, "conv10.bin"}, {14, 512, 512, "conv13.bin"}};
    if (layer < 1 || layer > 9 || n < 1 || runs < 1) {
        std::printf("The layer is not right\n");
        std::printf("usage: %s batch=<N> opt=<0 NCHW|1 NHWC|2 CHWN> layer=<1..9> [data=<dir>] [runs=<n>] [save=<file>]\n", argv[0]);
        return 2;
    }
    std::printf("opt:%d\n", opt);
    if (opt < 0 || opt > 2) {
        std::printf("The option is not right\n");   // 3..6 are the reference's cuDNN baselines
        return 2;
    }
    const DataLayout lay = opt == 0 ? DataLayout::NCHW : (opt == 1 ? DataLayout::NHWC : DataLayout::CHWN);
    const char* names[3] = {"Conv_NCHW", "Conv_NHWC", "Conv_CHWN"};
    const int side = table[layer].h, chn = table[layer].c, filters = table[layer].k;
    const size_t nFilter = (size_t)9 * filters * chn, nInput = (size_t)side * side * chn * n;
    const size_t nOutput = (size_t)side * side * filters * n;

    std::vector<float> w_h, x_h, y_h(nOutput);
    const std::string wpath = data + "/vggData/" + table[layer].file;
    if (!read_floats(wpath, nFilter, w_h)) {
        std::printf("no %s (%zu floats): synthetic filters\n", wpath.c_str(), nFilter);
        synthetic(w_h, nFilter, 0xF11Full + layer, 0.05f);
    }
    float *w_d = nullptr, *x_d = nullptr, *y_d = nullptr;
    CK(hipMalloc(&w_d, nFilter * sizeof(float)));
    CK(hipMalloc(&x_d, nInput * sizeof(float)));
    CK(hipMalloc(&y_d, nOutput * sizeof(float)));
    CK(hipMemcpy(w_d, w_h.data(), nFilter * sizeof(float), hipMemcpyHostToDevice));
    wino_warmup();

    for (int i = 0; i < runs; ++i) {
        const std::string xpath = data + "/binImage/file_" + std::to_string(i) + ".bin";
        if (!read_floats(xpath, nInput, x_h)) {
            if (i == 0) std::printf("no %s (%zu floats): synthetic images\n", xpath.c_str(), nInput);
            synthetic(x_h, nInput, 0x1A6Eull + i, 1.0f);
        }
        CK(hipMemcpy(x_d, x_h.data(), nInput * sizeof(float), hipMemcpyHostToDevice));
        hipEvent_t t0, t1;
        CK(hipEventCreate(&t0));
        CK(hipEventCreate(&t1));
        CK(hipEventRecord(t0, nullptr));
        std::printf("%s\n", names[opt]);
        int c = chn;
        layoutManager(lay, lay, n, side, c, filters, 1, x_d, w_d, nullptr, nullptr, nullptr, &y_d);
        CK(hipEventRecord(t1, nullptr));
        CK(hipEventSynchronize(t1));
        float ms = 0.f;
        CK(hipEventElapsedTime(&ms, t0, t1));
        CK(hipEventDestroy(t0));
        CK(hipEventDestroy(t1));
        CK(hipMemcpy(y_h.data(), y_d, nOutput * sizeof(float), hipMemcpyDeviceToHost));
        std::printf("time:%lf ms\n", (double)ms);
        std::printf("convOutput_cpu[0]:%lf\n", (double)y_h[0]);
        if (y_h[0] == 0.0f) std::printf("moduleConv error\n");
    }
    if (!save.empty() && !write_floats(save, y_h)) return 1;
    (void)hipFree(w_d);
    (void)hipFree(x_d);
    (void)hipFree(y_d);
    return 0;
}
