// mfma_rate: what the matrix pipe of this machine sustains, measured -- the practical roof the direct convolution
// kernels (16-bit) and the batched GEMMs (fp32) are read against.  Four loops on one workgroup per CU:
//   0. v_mfma_f32_32x32x2_f32 back to back, 8 accumulators per wave, operands in registers (against 157.3 TFLOP/s:
//      one multiply per 64 clocks and SIMD at 2.4 GHz);
// and, all operands resident in LDS,
//   1. v_mfma_f32_32x32x16_bf16 back to back, 8 accumulators per wave, no memory traffic;
//   2. the same with R ds_read_b128 per 8 multiplies (operand fetch from LDS, one step ahead);
//   3. the 18-step stage of the 8-wave direct kernel (direct16_rows.hpp): 36 fragment reads and 72 multiplies per
//      wave and stage, fragments requested two steps ahead.
// Each with 1 and 2 waves per SIMD, and with two kinds of operand data: "trivial" (tiny integers read as bf16:
// denormals, almost no bits toggle) and "real" (random sign and mantissa, exponents of 0.125 .. 2).  The chip's
// clock follows its power draw, and the multipliers' draw follows the data: with real operands the pipe sustains
// markedly less than with trivial ones.  Rates are printed against the nominal peak (one 32x32x16 multiply per 32
// clocks and SIMD at 2.4 GHz = 2.5 PFLOP/s over 256 CUs).
//
// usage: mfma_rate            (takes about a second)
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

#define CHECK(e)                                                                              \
    do {                                                                                      \
        hipError_t err_ = (e);                                                                \
        if (err_ != hipSuccess) {                                                             \
            fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(err_));      \
            exit(1);                                                                          \
        }                                                                                     \
    } while (0)

constexpr int KT = 128, FB = 9 * 2 * KT * 16, XPLANE = 704, XB = 2 * XPLANE * 16, LDS_BYTES = 3 * FB + 2 * XB;

__device__ void fill_lds(unsigned char* smem, int tid, int nthreads, int real) {
    for (int i = tid; i < LDS_BYTES / 4; i += nthreads) {
        unsigned h = i * 2654435761u;
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
        const unsigned lo = (h & 0x807Fu) | ((124u + ((h >> 8) & 3u)) << 7), hi = ((h >> 16) & 0x807Fu) | ((124u + ((h >> 28) & 3u)) << 7);
        reinterpret_cast<unsigned*>(smem)[i] = real ? (lo | (hi << 16)) : (i * 2654435761u >> 20);
    }
    __syncthreads();
}

// loops 1 and 2: NR reads per 8 multiplies
template <int NR>
__global__ __launch_bounds__(512, 1) void plain_kernel(float* out, int iters, int real) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    fill_lds(smem, tid, blockDim.x, real);
    floatx16 acc[8];
    for (int j = 0; j < 8; ++j)
        for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
    const unsigned char* base = smem + lane * 16 + (tid >> 6) * 2048;
    bf16x8 f[2][6];
    for (int q = 0; q < 6; ++q) f[0][q] = f[1][q] = *reinterpret_cast<const bf16x8*>(base + q * 1024);
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int t = 0; t < 8; ++t) {
#pragma unroll
            for (int q = 0; q < NR; ++q) f[(t + 1) & 1][q] = *reinterpret_cast<const bf16x8*>(base + ((t * 6 + q) & 31) * 1024 + (it & 1) * 16);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int m = 0; m < 8; ++m) acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[t & 1][m % 2], f[t & 1][2 + m % 4], acc[m], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if ((it & 15) == 15)                                 // keep the sums finite
            for (int j = 0; j < 8; ++j)
                for (int r = 0; r < 16; ++r) acc[j][r] *= 1e-3f;
    }
    float s = 0;
    for (int j = 0; j < 8; ++j)
        for (int r = 0; r < 16; ++r) s += acc[j][r];
    if (s == 12345.678f) out[tid] = s;                       // never true: keeps the multiplies
}

// loop 0: v_mfma_f32_32x32x2_f32 back to back (64 clocks each), 8 accumulators per wave, operands in registers
__global__ __launch_bounds__(512, 1) void plain32_kernel(float* out, int iters, int real) {
    const int tid = threadIdx.x;
    floatx16 acc[8];
    for (int j = 0; j < 8; ++j)
        for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
    float f[8];
    for (int q = 0; q < 8; ++q) {
        unsigned h = (tid * 8 + q) * 2654435761u;
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
        // real: random sign and mantissa, exponents of 0.125 .. 2; trivial: tiny integers read as floats (denormals)
        f[q] = real ? __uint_as_float((h & 0x807FFFFFu) | ((124u + ((h >> 8) & 3u)) << 23)) : __uint_as_float(h >> 28);
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int t = 0; t < 8; ++t) {
#pragma unroll
            for (int m = 0; m < 8; ++m) acc[m] = __builtin_amdgcn_mfma_f32_32x32x2f32(f[(t + m) & 7], f[(t + 3 * m + 1) & 7], acc[m], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if ((it & 15) == 15)
            for (int j = 0; j < 8; ++j)
                for (int r = 0; r < 16; ++r) acc[j][r] *= 1e-3f;
    }
    float s = 0;
    for (int j = 0; j < 8; ++j)
        for (int r = 0; r < 16; ++r) s += acc[j][r];
    if (s == 12345.678f) out[tid] = s;
}

// loop 3: the stage schedule of direct16_rows_kernel (filter rows r, input rows rho, columns s; see there)
__global__ __launch_bounds__(512, 1) void stage_kernel(float* out, int iters, int real, int PW) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    fill_lds(smem, tid, blockDim.x, real);
    const int wf = wave / 4, wp = wave % 4, l32 = lane & 31, lh = lane >> 5;
    unsigned char* const xsm = smem + 3 * FB;
    floatx16 acc[2][4];
    for (int i = 0; i < 2; ++i)
        for (int j = 0; j < 4; ++j)
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    const int xw_off = (lh * XPLANE + (4 * (wp / 2)) * PW + 32 * (wp & 1) + l32) * 16;
    int fslot = 0, xslot = 0;
    for (int it = 0; it < iters; ++it) {
        const unsigned char* fs = smem + fslot * FB + (lh * KT + wf * 64 + l32) * 16;
        const unsigned char* xrow[6];
#pragma unroll
        for (int r = 0; r < 6; ++r) xrow[r] = xsm + xslot * XB + xw_off + r * PW * 16;
        bf16x8 a[3][2], b[3];
        auto lda = [&](int r, int s) {
#pragma unroll
            for (int i = 0; i < 2; ++i) a[r][i] = *reinterpret_cast<const bf16x8*>(fs + (3 * r + s) * (2 * KT * 16) + i * 512);
        };
        auto ldb = [&](int t) { b[t % 3] = *reinterpret_cast<const bf16x8*>(xrow[t % 6] + (t / 6) * 16); };
        lda(0, 0); ldb(0); lda(1, 0); ldb(1); lda(2, 0);
#pragma unroll
        for (int t = 0; t < 18; ++t) {
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
#pragma unroll
                for (int i = 0; i < 2; ++i) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r][i], b[t % 3], acc[i][j], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_barrier();
        fslot = fslot == 2 ? 0 : fslot + 1;
        xslot ^= 1;
        if ((it & 15) == 15)
            for (int i = 0; i < 2; ++i)
                for (int j = 0; j < 4; ++j)
                    for (int r = 0; r < 16; ++r) acc[i][j][r] *= 1e-3f;
    }
    float s = 0;
    for (int i = 0; i < 2; ++i)
        for (int j = 0; j < 4; ++j)
            for (int r = 0; r < 16; ++r) s += acc[i][j][r];
    if (s == 12345.678f) out[tid] = s;
}

static int g_cus = 0;
template <typename F> static void report(const char* name, int waves, int real, double mfma_per_simd, F launch, int clocks = 32,
                                          double peak = 2500.0) {
    hipEvent_t a, b;
    CHECK(hipEventCreate(&a));
    CHECK(hipEventCreate(&b));
    float ms = 0;
    for (int rep = 0; rep < 3; ++rep) {                      // the last of three runs counts
        CHECK(hipEventRecord(a));
        launch();
        CHECK(hipGetLastError());
        CHECK(hipEventRecord(b));
        CHECK(hipEventSynchronize(b));
        CHECK(hipEventElapsedTime(&ms, a, b));
    }
    const double frac = mfma_per_simd * clocks / 2.4e9 / (ms * 1e-3);
    printf("%-34s %-8s data, %d waves/SIMD: %7.3f ms  %5.1f ns per multiply and SIMD  %.2f of nominal peak (%.0f TFLOP/s over %d CUs)\n", name,
           real ? "real" : "trivial", waves / 4, ms, ms * 1e6 / mfma_per_simd, frac, frac * peak * g_cus / 256, g_cus);
}

int main() {
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    g_cus = prop.multiProcessorCount;
    printf("%s, %d CUs\n", prop.gcnArchName, g_cus);
    float* out;
    CHECK(hipMalloc(&out, 4096));
    CHECK(hipFuncSetAttribute((const void*)plain_kernel<0>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
    CHECK(hipFuncSetAttribute((const void*)plain_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
    CHECK(hipFuncSetAttribute((const void*)stage_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
    const int iters = 2000;
    for (int real = 0; real < 2; ++real)
        for (int waves = 4; waves <= 8; waves += 4) {
            const double per_simd = (double)iters * 64 * waves / 4;
            report("fp32 multiplies only (32x32x2)", waves, real, (double)(iters / 2) * 64 * waves / 4,
                   [&] { hipLaunchKernelGGL(plain32_kernel, dim3(g_cus), dim3(64 * waves), 0, 0, out, iters / 2, real); }, 64, 157.3);
            report("multiplies only", waves, real, per_simd,
                   [&] { hipLaunchKernelGGL(plain_kernel<0>, dim3(g_cus), dim3(64 * waves), LDS_BYTES, 0, out, iters, real); });
            report("4 LDS reads per 8 multiplies", waves, real, per_simd,
                   [&] { hipLaunchKernelGGL(plain_kernel<4>, dim3(g_cus), dim3(64 * waves), LDS_BYTES, 0, out, iters, real); });
            report("direct kernel's stage (36 : 72)", waves, real, (double)(iters / 2) * 72 * waves / 4,
                   [&] { hipLaunchKernelGGL(stage_kernel, dim3(g_cus), dim3(64 * waves), LDS_BYTES, 0, out, iters / 2, real, 58); });
        }
    CHECK(hipFree(out));
    return 0;
}
