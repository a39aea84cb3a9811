// What a stream of stores reaches on this machine, by the shape of a store instruction (stand-alone microbenchmark).
//
// The first layer of a network writes a large NCHW tensor from matrix-instruction results: a wave holds 32 pixels x 32
// filters, and what one store instruction covers is a choice -- 2-byte elements of 32 consecutive pixels are 64 bytes
// of one filter's plane.  The kernels here store and do nothing else: y is [32][64][224][224] in 2-byte elements
// (205 MB), every wave takes tiles of 4 rows of an image, one after the other, and writes all 64 planes of it:
//   fill                   16 bytes per lane, the tensor front to back
//   4 filters x  64 bytes  tiles of 4 rows x 32 columns: a lane pair stores two columns of one filter
//   2 filters x 128 bytes  tiles of 4 rows x 64 columns: a register holds one filter for 64 columns
//   1 filter  x 256 bytes  tiles of 2 rows x 128 columns
// Four output tensors are written in turn, so that every launch finds its lines out of the last-level cache.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <vector>

#define CHECK(x)                                                                      \
    do {                                                                              \
        hipError_t e_ = (x);                                                          \
        if (e_ != hipSuccess) {                                                       \
            std::printf("%s failed: %s\n", #x, hipGetErrorString(e_));                \
            return 1;                                                                 \
        }                                                                             \
    } while (0)

namespace {
constexpr int N = 32, K = 64, H = 224, W = 224;
constexpr unsigned PLANE = (unsigned)H * W * 2;          // bytes of a filter's plane

__global__ void fill_kernel(uint4* y, long n) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = make_uint4(1, 2, 3, 4);
}

// COLS columns x ROWS rows per tile; a store instruction covers 256 / COLS filters x 2 COLS bytes
template <int COLS, int ROWS>
__global__ __launch_bounds__(256) void tile_kernel(char* y, int ntiles) {
    constexpr int TX = (W + COLS - 1) / COLS, TY = H / ROWS, FPI = 128 / COLS;   // tiles across and down, filters per instruction
    const int lane = threadIdx.x & 63;
    const int col = (lane % (COLS / 2)) * 2, f0 = lane / (COLS / 2);          // the lane's column pair and filter within an instruction
    for (int t = blockIdx.x * 4 + (threadIdx.x >> 6); t < ntiles; t += gridDim.x * 4) {
        const int n = t / (TY * TX), rem = t % (TY * TX), oh0 = (rem / TX) * ROWS, ow = (rem % TX) * COLS + col;
        if (ow >= W) continue;
        for (int g = 0; g < ROWS; ++g) {
            const unsigned at = (unsigned)(((n * K + f0) * H + oh0 + g) * W + ow) * 2u;
#pragma unroll 8
            for (int f = 0; f < K; f += FPI) *reinterpret_cast<unsigned*>(y + at + (unsigned)f * PLANE) = (unsigned)t;
        }
    }
}
}  // namespace

int main() {
    const long bytes = (long)N * K * PLANE;
    std::vector<char*> out(4);
    for (auto& p : out) CHECK(hipMalloc(&p, bytes));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    std::printf("%s, %d CUs; %.1f MB per launch\n", prop.gcnArchName, prop.multiProcessorCount, bytes / 1e6);
    auto timed = [&](const char* what, auto launch) -> int {
        for (int i = 0; i < 4; ++i) launch(out[i & 3]);
        CHECK(hipEventRecord(e0, 0));
        const int reps = 16;
        for (int i = 0; i < reps; ++i) launch(out[i & 3]);
        CHECK(hipEventRecord(e1, 0));
        CHECK(hipEventSynchronize(e1));
        float ms = 0;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        std::printf("%-46s %6.1f us  %5.2f TB/s\n", what, ms / reps * 1e3, bytes / (ms / reps * 1e-3) / 1e12);
        return 0;
    };
    const int cus = prop.multiProcessorCount;
    auto grid_for = [&](int ntiles, int wg_per_cu) {
        const long waves = 4L * wg_per_cu * cus, per = (ntiles + waves - 1) / waves;
        return (unsigned)((ntiles + 4 * per - 1) / (4 * per));
    };
    if (timed("fill, 16 bytes per lane", [&](char* y) { fill_kernel<<<(unsigned)((bytes / 16 + 255) / 256), 256>>>((uint4*)y, bytes / 16); })) return 1;
    for (int wg : {2, 4}) {
        char what[96];
        std::snprintf(what, sizeof what, "4 filters x  64 bytes, %d workgroups per CU", wg);
        const int t32 = N * (H / 4) * ((W + 31) / 32), t64 = N * (H / 4) * ((W + 63) / 64), t128 = N * (H / 2) * ((W + 127) / 128);
        if (timed(what, [&](char* y) { tile_kernel<32, 4><<<grid_for(t32, wg), 256>>>(y, t32); })) return 1;
        std::snprintf(what, sizeof what, "2 filters x 128 bytes, %d workgroups per CU", wg);
        if (timed(what, [&](char* y) { tile_kernel<64, 4><<<grid_for(t64, wg), 256>>>(y, t64); })) return 1;
        std::snprintf(what, sizeof what, "1 filter  x 256 bytes, %d workgroups per CU", wg);
        if (timed(what, [&](char* y) { tile_kernel<128, 2><<<grid_for(t128, wg), 256>>>(y, t128); })) return 1;
    }
    return 0;
}
