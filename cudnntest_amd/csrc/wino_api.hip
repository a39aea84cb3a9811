// C ABI of the gfx950 Winograd F(2x2,3x3) convolution library (see include/wino_amd.h).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <memory>
#include <vector>

#include "common.hpp"
#include "fused.hpp"
#include "direct.hpp"
#include "direct16.hpp"
#include "direct16_rows.hpp"
#include "gemm.hpp"
#include "gemm_rows_f4.hpp"
#include "transforms.hpp"
#include "transforms_f4.hpp"

using namespace wino;

// Scratch of wino_conv_noalloc: a fixed buffer in the library's own device image, one copy per GPU, held until the
// process ends.  In host code this name is only a handle for hipGetSymbolAddress (see noalloc_scratch below).
static __device__ __align__(256) unsigned char scratch[WINO_NOALLOC_SCRATCH_BYTES];

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

#define HIP_TRY(expr)                                                                            \
    do {                                                                                         \
        hipError_t e_ = (expr);                                                                  \
        if (e_ != hipSuccess) return fail(WINO_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

#define LAUNCH_CHECK(name)                                                                        \
    do {                                                                                          \
        hipError_t e_ = hipGetLastError();                                                        \
        if (e_ != hipSuccess) return fail(WINO_ERR_HIP, "launch %s: %s", name, hipGetErrorString(e_)); \
    } while (0)

bool valid_layout(int l) { return l == WINO_NCHW || l == WINO_NHWC || l == WINO_CHWN; }
bool valid_dtype(int d) { return d == WINO_F32 || d == WINO_F16 || d == WINO_BF16; }
bool valid_porder(int o) { return o == WINO_PRODUCT_KP || o == WINO_PRODUCT_PK; }
// Winograd-domain operands (U, V, M) move as 16-byte vectors, partly by direct-to-LDS loads: their addresses
// must be 16-byte aligned (every hipMalloc'ed buffer is); plain tensors need their element's alignment only.
bool misaligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }
size_t elem_bytes(int dtype) { return dtype == WINO_F32 ? 4 : 2; }
bool valid_order(int o) { return o == WINO_TILES_BATCH_MAJOR || o == WINO_TILES_BATCH_MINOR; }

constexpr int kMaxDevices = 16;

// Compute units of the current device, asked once per device.  The launch heuristics below (how many workgroups
// are resident at once, when a reduction is cut so that every CU has work) are derived from it; an MI355X has 256
// in 8 XCDs of 32, which is also what is assumed if the runtime cannot tell.
int device_cus() {
    static int cus[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    if (cus[dev] == 0) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
        cus[dev] = v;
    }
    return cus[dev];
}
// workgroups of the row-at-a-time GEMM resident at once: 2 per CU (64 KB of LDS, fp32) or 3 (48 KB, 2-byte operands)
long rows_slots(int dtype) { return (long)device_cus() * (dtype == WINO_F32 ? 2 : 3); }

// ---- scratch arena: one grow-only allocation per device ------------------------
struct Arena {
    void* own = nullptr;
    size_t own_bytes = 0;
    void* ext = nullptr;
    size_t ext_bytes = 0;
    unsigned long generation = 0;          // bumped whenever the arena's address may have changed
};
constexpr size_t kCounterBytes = 4096;     // 1024 arrival counters at the head of every arena
Arena g_arena[kMaxDevices];
std::mutex g_arena_mu;

int arena_get(size_t bytes, void** out) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(WINO_ERR_UNSUPPORTED, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lk(g_arena_mu);
    Arena& a = g_arena[dev];
    if (a.ext) {
        if (a.ext_bytes < bytes)
            return fail(WINO_ERR_WORKSPACE, "workspace of %zu bytes installed, %zu needed", a.ext_bytes, bytes);
        *out = a.ext;
        return WINO_OK;
    }
    if (a.own_bytes < bytes) {
        if (a.own) {
            HIP_TRY(hipDeviceSynchronize());
            HIP_TRY(hipFree(a.own));
            a.own = nullptr;
            a.own_bytes = 0;
        }
        HIP_TRY(hipMalloc(&a.own, bytes));
        a.own_bytes = bytes;
        ++a.generation;
        HIP_TRY(hipMemset(a.own, 0, kCounterBytes));       // arrival counters: zero between launches
    }
    *out = a.own;
    return WINO_OK;
}

// Where a whole-layer call takes its scratch from: the device's arena (grown on demand), or a fixed buffer that
// is never grown (the entry point that allocates nothing).
struct ScratchSource {
    void* fixed = nullptr;
    size_t fixed_bytes = 0;
    int get(size_t bytes, void** out) const {
        if (!fixed) return arena_get(bytes, out);
        if (bytes > fixed_bytes)
            return fail(WINO_ERR_WORKSPACE, "this problem needs %zu bytes of scratch, the built-in buffer holds %zu",
                        bytes, fixed_bytes);
        *out = fixed;
        return WINO_OK;
    }
};

unsigned long arena_generation(int dev) {
    std::lock_guard<std::mutex> lk(g_arena_mu);
    return g_arena[dev].generation;
}

// ---- optional per-stage timing: HIP events recorded on the launch stream ---------
struct StageSpan {
    int stage;
    hipEvent_t a, b;
};
bool g_timing = false;
thread_local bool t_no_timing = false;       // set while a call that must not create events is running
std::vector<StageSpan> g_spans;
std::mutex g_spans_mu;

struct StageScope {
    bool on;
    int stage;
    hipStream_t st;
    hipEvent_t a = nullptr, b = nullptr;
    StageScope(int stage_, hipStream_t st_) : on(g_timing && !t_no_timing), stage(stage_), st(st_) {
        if (on) {
            on = hipEventCreate(&a) == hipSuccess && hipEventCreate(&b) == hipSuccess &&
                 hipEventRecord(a, st) == hipSuccess;
        }
    }
    ~StageScope() {
        if (on && hipEventRecord(b, st) == hipSuccess) {
            std::lock_guard<std::mutex> lk(g_spans_mu);
            g_spans.push_back({stage, a, b});
        }
    }
};

struct Scratch {
    size_t u_off, v_off, m_off, total;
};

// The arena opens with the arrival counters of the epilogue GEMM's tail workgroups (zero whenever no
// kernel is running); U, V and the product follow.  The product region doubles as the tail workgroups'
// partial sums: the epilogue path has no product tensor.
// Whether a launch orders its workgroup ids by XCD (8 tile patches side by side, one per XCD): only if that keeps
// the XCDs evenly loaded.  With pTiles tile patches the padded order has ceil(pTiles/8)*8 slots; it is used when
// at most an eighth of them is empty, otherwise ids walk the patches in plain order and the hardware's round-robin
// spreads them (a layer with one tile patch would otherwise run on one XCD: 32 of 256 CUs).
bool xcd_map_ok(int pTiles) {
    const int padded = (pTiles + 7) / 8 * 8;
    return pTiles >= 8 && (padded - pTiles) * 8 <= padded;
}

// How many runs the staged GEMM's channel reduction is cut into.  A layer with fewer 128x128 workgroups than CUs
// leaves CUs idle while each workgroup walks the whole reduction, so the reduction is cut until there is one
// workgroup per CU (more than one per CU measured slower again: N=1, C=K=512, H=14 in fp32 takes 37 us uncut,
// 22 us in 2 runs, 16 us in 4, 23 us in 6, 20 us in 8), each run at least 4 stages long.  The partial products
// are summed by the output transform in a fixed order.
int gemm_splits(int dtype, int Cp, int Kp, long Pp) {
    const long wgs = 16L * (Kp / GEMM_BM) * (Pp / GEMM_BN);
    const int chunks = Cp / c_pad(dtype);          // stages of the reduction: 4 channel vectors each
    const long s = std::min<long>(device_cus() / std::max<long>(wgs, 1), chunks / 4);
    if (s <= 1) return 1;
    const int per = (int)((chunks + s - 1) / s);
    return (chunks + per - 1) / per;
}

// The epilogue GEMM's cut-up last round.  Workgroups resident at once: 2 per CU (64 KB of LDS, fp32) or 3 (48 KB,
// 2-byte operands).  If the last round of 64x64 patches would occupy at most 60 % of them, its patches are cut
// into TAIL workgroups, one Winograd row each (measured: a last round of 272 of 512 gains 8 %, one of 424 loses
// 4 %).  fp32 only: with 2-byte operands a patch is short and the cut costs more than the idle CUs (measured).
// Returns the number of groups of 8 tile patches (x all filter tiles) that are cut, 0 for none; each cut patch
// needs an arrival counter and four rows of 64 x 256 partial sums.
int rows_tail_groups(int dtype, const Geometry& g) {
    if (dtype != WINO_F32) return 0;
    const int kTiles = (g.K + GO_T - 1) / GO_T;
    const int pTiles = (int)((g.P + GO_T - 1) / GO_T);
    const int pGroups = (pTiles + 7) / 8, group = 8 * kTiles;
    const long slots = rows_slots(dtype), real = (long)pTiles * kTiles;
    if (!(real > slots && real % slots != 0 && 5 * (real % slots) <= 3 * slots)) return 0;
    const int tail_groups = (int)((real % slots + group - 1) / group);
    if (tail_groups >= pGroups || (long)tail_groups * group > (long)(kCounterBytes / sizeof(int))) return 0;
    return tail_groups;
}
inline size_t tail_part_bytes(int dtype, const Geometry& g) {
    return (size_t)rows_tail_groups(dtype, g) * 8 * ((g.K + GO_T - 1) / GO_T) * 4 * 64 * 256 * sizeof(float);
}

// The F(4x4) GEMM with the output transform in its epilogue (gemm_rows_f4.hpp): 64 x 64 patches dealt to the 8 XCDs
// (to as many as there are patches), one persistent workgroup per CU (fewer when that would leave a workgroup less
// than 4 stages), each with room for one patch's partial outputs and an arrival counter.  fp32 only.
struct F4RowsPlan {
    int kTiles, pTiles, nparts, grid;
    size_t part_bytes;
};
bool f4_rows_plan(int dtype, const Geometry& g, F4RowsPlan* p) {
    if (dtype != WINO_F32 || g.m != 4) return false;
    p->kTiles = (g.K + GF4_T - 1) / GF4_T;
    p->pTiles = (int)((g.P + GF4_T - 1) / GF4_T);
    const long patches = (long)p->kTiles * p->pTiles;
    p->nparts = (int)std::min<long>(8, patches);
    const long per_part = patches / p->nparts * 6 * (g.Cp / 16);                 // stages of the XCD with the fewest patches
    const long sx = std::max<long>(1, std::min<long>(std::min<long>(device_cus() / 8, (long)(kCounterBytes / sizeof(int)) / 8), per_part / 4));
    p->grid = (int)sx * 8;
    p->part_bytes = (size_t)p->grid * GF4_PART * sizeof(float);
    return true;
}

// What a pipeline keeps in scratch: STAGED (and the F(4x4) mode) U, V and the product; EPILOGUE U, V and the
// partial sums of its cut-up workgroups (EPILOGUE_F4: of the workgroups that share a patch); FUSED U only.
// The default is the largest of them.
Scratch scratch_layout(const Geometry& g, int dtype, int algo = WINO_ALGO_STAGED) {
    const size_t es = dtype_size(dtype);
    const size_t nxi = (size_t)(g.m + 2) * (g.m + 2);
    auto al = [](size_t v) { return (v + 255) / 256 * 256; };
    Scratch s;
    s.u_off = kCounterBytes;
    s.v_off = s.u_off + al(nxi * (size_t)g.Cp * g.Kp * es);
    if (algo == WINO_ALGO_FUSED) {
        s.m_off = s.total = s.v_off;
        return s;
    }
    s.m_off = s.v_off + al(nxi * (size_t)g.Cp * g.Pp * es);
    const size_t copies = g.m == 2 ? (size_t)gemm_splits(dtype, g.Cp, g.Kp, g.Pp) : 1;
    const size_t product = copies * nxi * (size_t)g.Kp * g.Pp * sizeof(float);
    F4RowsPlan fp;
    if (algo == WINO_ALGO_EPILOGUE_F4 && f4_rows_plan(dtype, g, &fp)) s.total = s.m_off + al(fp.part_bytes);
    else s.total = s.m_off + al(algo == WINO_ALGO_EPILOGUE ? tail_part_bytes(dtype, g) : product);
    return s;
}

// ---- stage launchers (typed) -------------------------------------------------------
template <typename T>
int launch_filter_transform(int layout, int K, int C, int Kp, int Cp, const void* w, void* U, hipStream_t st) {
    // one wave per workgroup: the kernel is all latency, and K*C/CV threads in workgroups of 256 would leave
    // most CUs of the chip without a wave
    dim3 grid((Kp + 63) / 64, Cp / ChanVec<T>::n), block(64);
    hipLaunchKernelGGL(filter_transform_kernel<T>, grid, block, 0, st, (const T*)w, (T*)U, flt_strides(layout, K, C),
                       K, C, Kp, Cp);
    LAUNCH_CHECK("filter_transform");
    return WINO_OK;
}

// whether the input transform of this problem runs as the tiled NCHW kernel, which can carry a filter job
inline bool input_is_nchw_tiled(int layout, int order, const Geometry& g) {
    return layout == WINO_NCHW && order == WINO_TILES_BATCH_MAJOR && g.th * g.tw >= 64;
}

template <typename T>
int launch_input_transform(int layout, int order, const Geometry& g, const void* x, void* V, hipStream_t st,
                           const FilterJob& fj = FilterJob{}) {
    constexpr int CV = ChanVec<T>::n;
    const int CQ = g.Cp / CV;
    if (layout == WINO_NCHW && order == WINO_TILES_BATCH_MAJOR && g.th * g.tw <= 256) {
        // small images: one image and NQ channel vectors per workgroup, thread per (channel vector, tile)
        const int tiles = g.th * g.tw;
        const int NQ = std::min(std::min(256 / tiles, 32), CQ);
        const int groups = (CQ + NQ - 1) / NQ;
        const long in_blocks = (long)g.N * groups;
        const long extra = fj.w ? ((long)fj.Kp * CQ + 255) / 256 : 0;
        if (in_blocks + extra >= (1L << 31)) return fail(WINO_ERR_UNSUPPORTED, "input transform: too many workgroups");
        // 2-byte types move pairs (4 bytes per lane) when every channel plane starts 4-byte aligned
        const bool vec2 = sizeof(T) == 2 && g.W % 2 == 0 && !misaligned(x, 4);
        const int Ww = vec2 ? g.W / 2 : g.W;
        const int stepC = 256 / (g.H * Ww), stepH = (256 - stepC * g.H * Ww) / Ww,
                  stepW = 256 - stepC * g.H * Ww - stepH * Ww;
        const size_t lds = (size_t)NQ * CV * (2 * g.th + 2) * (2 * g.tw + 2) * sizeof(T);
        dim3 grid((unsigned)(in_blocks + extra)), block(256);
        if (vec2)
            hipLaunchKernelGGL((input_transform_nchw_small_kernel<T, (sizeof(T) == 2 ? 2 : 1)>), grid, block, lds, st,
                               (const T*)x, (T*)V, g.C, g.H, g.W, g.pad, g.th, g.tw, g.Pp, g.Cp, NQ, groups,
                               (int)in_blocks, stepC, stepH, stepW, fj);
        else
            hipLaunchKernelGGL((input_transform_nchw_small_kernel<T, 1>), grid, block, lds, st, (const T*)x, (T*)V,
                               g.C, g.H, g.W, g.pad, g.th, g.tw, g.Pp, g.Cp, NQ, groups, (int)in_blocks, stepC, stepH,
                               stepW, fj);
        LAUNCH_CHECK("input_transform_nchw_small");
        return WINO_OK;
    }
    if (input_is_nchw_tiled(layout, order, g)) {
        // TR x TC tiles per workgroup, TR*TC <= 256, halo of CV channels in LDS (<= 60 KB).
        // TR is kept a multiple of 8 when it can be, so a workgroup's run of V (TR*tw
        // 16-byte vectors per coordinate) starts and ends on a 128-byte boundary.
        const int TC = g.tw < 128 ? g.tw : 128;
        int TR = 256 / TC;
        if (TR >= g.th) TR = g.th;                        // a whole image per workgroup
        else if (TR > 8) TR &= ~7;
        const int colBlocks = (g.tw + TC - 1) / TC, rowBlocks = (g.th + TR - 1) / TR;
        const int ldsW = 2 * TC + 2;
        // 2-byte types move image-aligned column pairs (4 bytes per lane) when every row starts 4-byte aligned
        const bool vec2 = sizeof(T) == 2 && g.W % 2 == 0 && !misaligned(x, 4);
        const int span = vec2 ? ldsW + 2 : ldsW;          // loaded columns per row (one extra pair on the left)
        const int perUnit = vec2 ? 128 : 64;
        int chunkLog2 = 0;
        while ((perUnit << chunkLog2) < span) ++chunkLog2;
        const size_t lds = (size_t)CV * (2 * TR + 2) * ldsW * sizeof(T);
        dim3 grid(rowBlocks * colBlocks, CQ, g.N + (fj.w ? 1 : 0)), block(256);   // z-slice 0: the filter job
        if (vec2)
            hipLaunchKernelGGL((input_transform_nchw_kernel<T, (sizeof(T) == 2 ? 2 : 1)>), grid, block, lds, st,
                               (const T*)x, (T*)V, g.N, g.C, g.H, g.W, g.pad, g.th, g.tw, g.Pp, g.Cp, TR, TC,
                               colBlocks, chunkLog2, fj);
        else
            hipLaunchKernelGGL((input_transform_nchw_kernel<T, 1>), grid, block, lds, st, (const T*)x, (T*)V, g.N,
                               g.C, g.H, g.W, g.pad, g.th, g.tw, g.Pp, g.Cp, TR, TC, colBlocks, chunkLog2, fj);
        LAUNCH_CHECK("input_transform_nchw");
        return WINO_OK;
    }
    if (layout == WINO_NHWC && order == WINO_TILES_BATCH_MAJOR && g.C % CV == 0 &&
        (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
        // 256 threads = TC tile columns x NQ channel vectors.  Narrow images take narrow blocks (a 7-tile row in a
        // 32-wide block leaves three threads in four without a tile) as long as the layer has the channel vectors
        // to fill the other axis.
        auto launch = [&](auto tc_c) -> int {
            constexpr int TC = decltype(tc_c)::value, NQ = 256 / TC, TR = 2;
            const int colBlocks = (g.tw + TC - 1) / TC, rowBlocks = (g.th + TR - 1) / TR;
            const long in_blocks = (long)g.N * rowBlocks * colBlocks;
            const int gy = (CQ + NQ - 1) / NQ;
            // a filter job gets workgroups appended along x: enough, over all y, for one thread per (filter, channel vector)
            const long extra = fj.w ? ((long)fj.Kp * CQ + (long)TC * NQ * gy - 1) / ((long)TC * NQ * gy) : 0;
            if (in_blocks + extra >= (1L << 31))
                return fail(WINO_ERR_UNSUPPORTED, "input transform: too many workgroups");
            dim3 grid((unsigned)(in_blocks + extra), gy), block(TC * NQ);
            hipLaunchKernelGGL((input_transform_nhwc_kernel<T, TC, NQ, TR>), grid, block, 0, st, (const T*)x, (T*)V,
                               g.N, g.C, g.H, g.W, g.pad, g.th, g.tw, g.Pp, g.Cp, colBlocks, rowBlocks, fj,
                               (int)in_blocks);
            LAUNCH_CHECK("input_transform_nhwc");
            return WINO_OK;
        };
        if (g.tw <= 8 && CQ >= 32) return launch(std::integral_constant<int, 8>{});
        if (g.tw <= 16 && CQ >= 16 && sizeof(T) == 2) return launch(std::integral_constant<int, 16>{});
        return launch(std::integral_constant<int, 32>{});
    }
    const long in_blocks = (g.P + 255) / 256;
    const long extra = fj.w ? (fj.Kp + 255) / 256 : 0;          // x all CQ rows of the grid
    if (in_blocks + extra >= (1L << 31)) return fail(WINO_ERR_UNSUPPORTED, "input transform: too many workgroups");
    dim3 grid((unsigned)(in_blocks + extra), CQ), block(256);
    // channel vectors fastest while the transform's tensors fit the 256 MB last-level cache (N=32, C=256, H=56 from
    // CHWN: bf16, 257 MB, 54 -> 45 us; fp32, 514 MB, 103 -> 113 us)
    const double bytes = ((double)g.N * g.C * g.H * g.W + 16.0 * g.P * g.C) * sizeof(T);
    const int cq_fast = bytes <= 300e6 ? 1 : 0;
    hipLaunchKernelGGL(input_transform_generic_kernel<T>, grid, block, 0, st, (const T*)x, (T*)V,
                       act_strides(layout, g.N, g.C, g.H, g.W), g.N, g.C, g.H, g.W, g.pad, g.th, g.tw, g.P, g.Pp,
                       g.Cp, order, fj, (int)in_blocks, cq_fast);
    LAUNCH_CHECK("input_transform");
    return WINO_OK;
}

// the epilogue a call asks for, and the strides of the tensor it writes (pooled or not)
inline Epilogue make_epilogue(unsigned flags, const void* bias) {
    return Epilogue{bias, (flags & WINO_FLAG_RELU) ? 1 : 0, (flags & WINO_FLAG_POOL2) ? 1 : 0};
}
inline ActStrides out_strides(int layout, unsigned flags, int N, int K, int Ho, int Wo) {
    return (flags & WINO_FLAG_POOL2) ? act_strides(layout, N, K, Ho / 2, Wo / 2) : act_strides(layout, N, K, Ho, Wo);
}

template <typename T>
int launch_output_transform(int layout, int order, int porder, unsigned flags, const void* bias, int N, int K, int Ho,
                            int Wo, int Kp, long P, long Pp, const float* Mo, void* y, hipStream_t st,
                            int splits = 1) {
    const int th = (Ho + 1) / 2, tw = (Wo + 1) / 2;
    const Epilogue ep = make_epilogue(flags, bias);
    if (porder == WINO_PRODUCT_PK) {
        int bx = 64;
        while (bx < K && bx < 256) bx *= 2;
        dim3 block(bx, 256 / bx), grid((K + bx - 1) / bx, (unsigned)((P + block.y - 1) / block.y));
        hipLaunchKernelGGL(output_transform_pk_kernel<T>, grid, block, 0, st, Mo, (T*)y,
                           out_strides(layout, flags, N, K, Ho, Wo), N, K, Ho, Wo, th, tw, P, Pp, Kp, order, ep, splits);
    } else {
        dim3 grid((unsigned)((P + 255) / 256), K), block(256);
        hipLaunchKernelGGL(output_transform_generic_kernel<T>, grid, block, 0, st, Mo, (T*)y,
                           out_strides(layout, flags, N, K, Ho, Wo), N, K, Ho, Wo, th, tw, P, Pp, Kp, order, ep, splits);
    }
    LAUNCH_CHECK("output_transform");
    return WINO_OK;
}

template <typename T, int NV, bool PK>
int launch_gemm_t(int nxi, int Cp, int Kp, long Pp, const void* U, const void* V, float* Mo, int splits,
                  hipStream_t st) {
    const int kTiles = Kp / GEMM_BM, pTiles = (int)(Pp / GEMM_BN);
    const int chunks = Cp / (NV * ChanVec<T>::n), per = (chunks + splits - 1) / splits;
    if (splits < 1 || (long)per * (splits - 1) >= chunks)
        return fail(WINO_ERR_INVALID, "reduction of %d stages cannot be cut into %d runs", chunks, splits);
    constexpr int RING = sizeof(T) == 4 ? 4 : 3;     // from measurements, see gemm.hpp
    // the walking kernel: an uncut reduction of at most 24 stages (beyond, the starts and ends it saves weigh less
    // than its 3 % slower loop: C = 512 in fp32 measured 488 against 470 us, C = 256 242 against 256 us), and
    // work for three rounds of the resident set
    const int slots = 2 * device_cus(), per_xcd = slots / 8 / std::max(kTiles, 1);
    // (fp32 reductions of a multiple of four stages run the variant that spreads a pair's stores over the next
    // pair's first stages: C = 512 measured 456 against 466 us, C = 256 226 against 242 us)
    const int walk_max = sizeof(T) == 4 && NV == 4 && chunks % RING == 0 ? 32 : 24;
    // (and from two pairs to a group: N = 64, C = K = 512 at 14 x 14, 2.25 pairs to a group, 157 against 163 us)
    const long walk_min = sizeof(T) == 4 && NV == 4 && chunks % RING == 0 ? 2 : 3;
    if (splits == 1 && chunks <= walk_max && per_xcd >= 1 && (long)pTiles * nxi >= walk_min * per_xcd * 8) {
        const int groups = per_xcd * 8;
        if constexpr (sizeof(T) == 4 && NV == 4) {
            if (chunks % RING == 0) {
                hipLaunchKernelGGL((gemm_128x128_walk_spread_kernel<T, NV, PK, RING>), dim3((unsigned)(groups * kTiles)), dim3(256), 0, st,
                                   (const T*)U, (const T*)V, Mo, Cp, Kp, Pp, kTiles, pTiles, nxi, groups);
                LAUNCH_CHECK("batched_gemm_walk_spread");
                return WINO_OK;
            }
        }
        hipLaunchKernelGGL((gemm_128x128_walk_kernel<T, NV, PK, RING>), dim3((unsigned)(groups * kTiles)), dim3(256), 0, st,
                           (const T*)U, (const T*)V, Mo, Cp, Kp, Pp, kTiles, pTiles, nxi, groups);
        LAUNCH_CHECK("batched_gemm_walk");
        return WINO_OK;
    }
    const bool xm = xcd_map_ok(pTiles);
    dim3 grid((unsigned)((xm ? (pTiles + 7) / 8 * 8 : pTiles) * kTiles), nxi, splits), block(256);
    hipLaunchKernelGGL((gemm_128x128_kernel<T, NV, PK, RING>), grid, block, 0, st, (const T*)U, (const T*)V, Mo, Cp,
                       Kp, Pp, kTiles, pTiles, per, xm ? 1 : 0);
    LAUNCH_CHECK("batched_gemm");
    return WINO_OK;
}

int launch_gemm(int nxi, int dtype, int porder, int Cp, int Kp, long Pp, const void* U, const void* V, float* Mo,
                hipStream_t st, int splits = 1) {
    // slab per barrier: 4 channel vectors = 16 channels (fp32) or 32 (16-bit); Cp is a multiple of that
    const bool pk = porder == WINO_PRODUCT_PK;
    switch (dtype) {
    case WINO_F32:
        return pk ? launch_gemm_t<float, 4, true>(nxi, Cp, Kp, Pp, U, V, Mo, splits, st)
                  : launch_gemm_t<float, 4, false>(nxi, Cp, Kp, Pp, U, V, Mo, splits, st);
    case WINO_F16:
        return pk ? launch_gemm_t<f16_t, 4, true>(nxi, Cp, Kp, Pp, U, V, Mo, splits, st)
                  : launch_gemm_t<f16_t, 4, false>(nxi, Cp, Kp, Pp, U, V, Mo, splits, st);
    case WINO_BF16:
        return pk ? launch_gemm_t<bf16_t, 4, true>(nxi, Cp, Kp, Pp, U, V, Mo, splits, st)
                  : launch_gemm_t<bf16_t, 4, false>(nxi, Cp, Kp, Pp, U, V, Mo, splits, st);
    }
    return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
}

// tail: scratch for the cut-up last round (partial sums, arrival counters), or null to launch every patch whole
struct TailScratch {
    float* part = nullptr;
    size_t part_bytes = 0;
    int* cnt = nullptr;
};

template <typename T, bool SWAP, int NVG, int RING>
int launch_gemm_rows_t(int order, unsigned flags, const void* bias, const Geometry& g, const void* U,
                       const void* V, void* y, int dst, const TailScratch& ts, hipStream_t st) {
    const int kTiles = (g.K + GO_T - 1) / GO_T;
    const int pTiles = (int)((g.P + GO_T - 1) / GO_T);
    const int pGroups = (pTiles + 7) / 8;
    const int group = 8 * kTiles;                         // workgroup ids per group of 8 tile patches
    const ActStrides ys = out_strides(dst, flags, g.N, g.K, g.Ho, g.Wo);
    const Epilogue ep = make_epilogue(flags, bias);
    // a small last round is cut into TAIL workgroups (rows_tail_groups) when the caller brought scratch for it
    int tail_groups = ts.part ? rows_tail_groups(sizeof(T) == 4 ? WINO_F32 : WINO_F16, g) : 0;
    if (tail_part_bytes(sizeof(T) == 4 ? WINO_F32 : WINO_F16, g) > ts.part_bytes) tail_groups = 0;
    const bool xm = tail_groups > 0 || xcd_map_ok(pTiles);      // (a cut-up last round implies hundreds of patches)
    const int main_ids = xm ? (pGroups - tail_groups) * group : pTiles * kTiles;
    hipLaunchKernelGGL((gemm_rows_kernel<T, SWAP, NVG, RING>), dim3((unsigned)(main_ids + tail_groups * group * 4)),
                       dim3(256), 0, st, (const T*)U, (const T*)V, (T*)y, ys, g.N, g.K, g.Ho, g.Wo, g.th, g.tw, g.P,
                       g.Cp, g.Kp, g.Pp, order, ep, kTiles, pTiles, main_ids, tail_groups ? ts.part : nullptr,
                       tail_groups ? ts.cnt : nullptr, xm ? 1 : 0);
    LAUNCH_CHECK("gemm_rows");
    return WINO_OK;
}

template <typename T>
int launch_gemm_rows_d(int dst, int order, unsigned flags, const void* bias, const Geometry& g, const void* U,
                       const void* V, void* y, const TailScratch& ts, hipStream_t st) {
    // one k-group per stage; ring depth from measurements: 3 for 2-byte operands, 4 for fp32
    constexpr int RING = sizeof(T) == 2 ? 3 : 4;
    if (dst == WINO_NHWC) return launch_gemm_rows_t<T, true, 1, RING>(order, flags, bias, g, U, V, y, dst, ts, st);
    return launch_gemm_rows_t<T, false, 1, RING>(order, flags, bias, g, U, V, y, dst, ts, st);
}

int launch_gemm_out(int dst, int dtype, int order, unsigned flags, const void* bias, const Geometry& g, const void* U,
                    const void* V, void* y, const TailScratch& ts, hipStream_t st) {
    switch (dtype) {
    case WINO_F32: return launch_gemm_rows_d<float>(dst, order, flags, bias, g, U, V, y, ts, st);
    case WINO_F16: return launch_gemm_rows_d<f16_t>(dst, order, flags, bias, g, U, V, y, ts, st);
    case WINO_BF16: return launch_gemm_rows_d<bf16_t>(dst, order, flags, bias, g, U, V, y, ts, st);
    }
    return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
}

template <typename T, bool SWAP, int XM, int NVG>
int launch_fused_rows_t(int src, int dst, int order, unsigned flags, const void* bias, const Geometry& g, const void* x,
                        const void* U, void* y, hipStream_t st) {
    const int kTiles = (g.K + GO_T - 1) / GO_T;
    const int pTiles = (int)((g.P + GO_T - 1) / GO_T);
    const int pGroups = (pTiles + 7) / 8;
    const bool xm = xcd_map_ok(pTiles);
    dim3 grid((unsigned)((xm ? pGroups * 8 : pTiles) * kTiles)), block(256);
    hipLaunchKernelGGL((fused_rows_kernel<T, SWAP, XM, NVG>), grid, block, 0, st, (const T*)x, (const T*)U, (T*)y,
                       act_strides(src, g.N, g.C, g.H, g.W), out_strides(dst, flags, g.N, g.K, g.Ho, g.Wo), g.N, g.C, g.K,
                       g.H, g.W, g.pad, g.Ho, g.Wo, g.th, g.tw, g.P, g.Cp, g.Kp, order, make_epilogue(flags, bias),
                       kTiles, pTiles, xm ? 1 : 0);
    LAUNCH_CHECK("fused_rows");
    return WINO_OK;
}

template <typename T>
int launch_fused_d(int src, int dst, int order, unsigned flags, const void* bias, const Geometry& g, const void* x,
                   const void* U, void* y, hipStream_t st) {
    if ((long)g.N * g.C * g.H * g.W * (long)sizeof(T) >= (1L << 32))
        return fail(WINO_ERR_UNSUPPORTED, "fused kernel: input tensor too large for 32-bit byte offsets");
    constexpr int CV = ChanVec<T>::n;
    const bool swap = dst == WINO_NHWC, chan_contig = src == WINO_NHWC;
    // two k-groups per stage when Cp allows an even stage count; a 2-byte source without
    // channel-vector loads would then hold 64 raw values per thread (spills): one k-group there
    bool two = (g.Cp / CV) % 8 == 0;
    if (sizeof(T) == 2 && !(chan_contig && g.C % CV == 0)) two = false;
    const int un = (two ? 2 : 1) * CV / 2;     // channels per thread
    const int xm = (chan_contig && g.C % un == 0) ? XM_CHANVEC : ((src == WINO_NCHW && g.W >= 4) ? XM_ROW : XM_SCALAR);
#define FR(SW, XM, NG) return launch_fused_rows_t<T, SW, XM, NG>(src, dst, order, flags, bias, g, x, U, y, st)
#define FR2(SW, NG)                               \
    if (xm == XM_CHANVEC) FR(SW, XM_CHANVEC, NG); \
    if (xm == XM_ROW) FR(SW, XM_ROW, NG);         \
    FR(SW, XM_SCALAR, NG)
    if (two) {
        if constexpr (sizeof(T) == 2) {        // here two implies channel-vector loads
            if (swap) FR(true, XM_CHANVEC, 2);
            FR(false, XM_CHANVEC, 2);
        } else {
            if (swap) { FR2(true, 2); }
            FR2(false, 2);
        }
    }
    if (swap) { FR2(true, 1); }
    FR2(false, 1);
#undef FR2
#undef FR
}

int launch_fused(int src, int dst, int dtype, int order, unsigned flags, const void* bias, const Geometry& g,
                 const void* x, const void* U, void* y, hipStream_t st) {
    switch (dtype) {
    case WINO_F32: return launch_fused_d<float>(src, dst, order, flags, bias, g, x, U, y, st);
    case WINO_F16: return launch_fused_d<f16_t>(src, dst, order, flags, bias, g, x, U, y, st);
    case WINO_BF16: return launch_fused_d<bf16_t>(src, dst, order, flags, bias, g, x, U, y, st);
    }
    return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
}

// ---- F(4x4,3x3) stage launchers -----------------------------------------------------------------
template <typename T>
int launch_f4_filter(int layout, int K, int C, int Kp, int Cp, const void* w, void* U, hipStream_t st) {
    dim3 grid((Kp + 63) / 64, Cp / ChanVec<T>::n), block(64);
    hipLaunchKernelGGL(filter_transform_f4_kernel<T>, grid, block, 0, st, (const T*)w, (T*)U,
                       flt_strides(layout, K, C), K, C, Kp, Cp);
    LAUNCH_CHECK("f4_filter_transform");
    return WINO_OK;
}

// fj: a filter job to ride in the launch (its w is null for none).  Its threads are Kp x Cp/CV; the extra z-slice of
// the grid has at least that many (the input side has P x Cp/CV x CV or more), or the job gets a launch of its own.
template <typename T>
int launch_f4_input(int layout, int order, const Geometry& g, const void* x, void* V, hipStream_t st,
                    const FilterJob& fj = FilterJob{}) {
    constexpr int CV = ChanVec<T>::n;
    const long job = fj.w ? (long)fj.Kp * (fj.Cp / CV) : 0;
    if (layout == WINO_NHWC && order == WINO_TILES_BATCH_MAJOR && sizeof(T) == 4 && g.N < 65535 && g.Cp / F4N_CC < 65535 &&
        (long)g.H * g.W * g.C * 4 < (1L << 32) && (long)g.Cp * g.Pp * 4 < (1L << 32)) {   // (32-bit byte offsets inside an image and a plane of V)
        const int colBlocks = (g.tw + F4N_TCB - 1) / F4N_TCB;
        dim3 grid((unsigned)(g.th * colBlocks), (g.Cp + F4N_CC - 1) / F4N_CC, g.N);
        const bool ride = job > 0 && (long)grid.x * grid.y * 256 >= job;
        if (job > 0 && !ride) {
            const int rc = launch_f4_filter<T>(layout, fj.K, fj.C, fj.Kp, fj.Cp, fj.w, fj.U, st);
            if (rc) return rc;
        }
        if (ride) grid.z += 1;
        hipLaunchKernelGGL(input_transform_f4_nhwc_kernel<F4N_CC>, grid, dim3(256), 0, st, (const float*)x, (float*)V, g.N, g.C, g.H,
                           g.W, g.pad, g.th, g.tw, g.Pp, g.Cp, colBlocks, ride ? fj : FilterJob{});
        LAUNCH_CHECK("f4_input_transform_nhwc");
        return WINO_OK;
    }
    if constexpr (sizeof(T) == 4) {
        // NCHW rows with at least 128 tiles to an image: TR x TC tiles per workgroup through an LDS halo of 4 channels
        // (<= 64 KB), the tiled kernel of the F(2x2) pipeline with 6x6 tiles every 4 pixels
        if (layout == WINO_NCHW && order == WINO_TILES_BATCH_MAJOR && g.th * g.tw >= 128 && g.tw <= 252 && g.N < 65535) {
            const int TC = g.tw < 64 ? g.tw : 64;
            int TR = std::min(256 / TC, g.th);
            while (TR > 1 && (size_t)CV * (4 * TR + 2) * (4 * TC + 2) * 4 > 65536) --TR;
            const int colBlocks = (g.tw + TC - 1) / TC, rowBlocks = (g.th + TR - 1) / TR;
            const int ldsW = 4 * TC + 2;
            int chunkLog2 = 0;
            while ((64 << chunkLog2) < ldsW) ++chunkLog2;
            const size_t lds = (size_t)CV * (4 * TR + 2) * ldsW * 4;
            dim3 grid(rowBlocks * colBlocks, g.Cp / CV, g.N + (job ? 1 : 0));
            hipLaunchKernelGGL((input_transform_nchw_kernel<float, 1, 4>), grid, dim3(256), lds, st, (const float*)x, (float*)V,
                               g.N, g.C, g.H, g.W, g.pad, g.th, g.tw, g.Pp, g.Cp, TR, TC, colBlocks, chunkLog2, fj);
            LAUNCH_CHECK("f4_input_transform_nchw");
            return WINO_OK;
        }
        // smaller images: one image and NQ channel vectors per workgroup (LDS planes of 4 NQ channels, <= 64 KB)
        if (layout == WINO_NCHW && order == WINO_TILES_BATCH_MAJOR && g.th * g.tw < 128) {
            const int tiles = g.th * g.tw, CQ = g.Cp / CV;
            const int plane = (4 * g.th + 2) * (4 * g.tw + 2) * CV * 4;          // bytes of a channel vector's planes
            // (at most 4: more, smaller workgroups fill the chip more evenly -- N = 64, C = 512 at 14 x 14: 23.7 us with 4
            // channel vectors to a workgroup, 25.2 with 8, 27.0 with the 12 that fit)
            const int NQ = std::max(1, std::min(std::min(std::min(256 / tiles, 65536 / plane), CQ), 4));
            const int groups = (CQ + NQ - 1) / NQ;
            const long in_blocks = (long)g.N * groups, extra = (job + 255) / 256;
            if (in_blocks + extra < (1L << 31) && (size_t)NQ * plane <= 65536) {
                const int stepC = 256 / (g.H * g.W), stepH = (256 - stepC * g.H * g.W) / g.W,
                          stepW = 256 - stepC * g.H * g.W - stepH * g.W;
                // rows in 16-byte pieces where they consist of them and a thread's share is at most 16
                const bool quad = g.W % 4 == 0 && !misaligned(x, 16) && (long)NQ * CV * g.H * (g.W / 4) <= 16 * 256;
                if (quad)
                    hipLaunchKernelGGL((input_transform_nchw_small_kernel<float, 1, 4, true>), dim3((unsigned)(in_blocks + extra)), dim3(256),
                                       (size_t)NQ * plane, st, (const float*)x, (float*)V, g.C, g.H, g.W, g.pad, g.th, g.tw, g.Pp, g.Cp,
                                       NQ, groups, (int)in_blocks, stepC, stepH, stepW, fj);
                else
                    hipLaunchKernelGGL((input_transform_nchw_small_kernel<float, 1, 4>), dim3((unsigned)(in_blocks + extra)), dim3(256),
                                       (size_t)NQ * plane, st, (const float*)x, (float*)V, g.C, g.H, g.W, g.pad, g.th, g.tw, g.Pp, g.Cp,
                                       NQ, groups, (int)in_blocks, stepC, stepH, stepW, fj);
                LAUNCH_CHECK("f4_input_transform_nchw_small");
                return WINO_OK;
            }
        }
    }
    if constexpr (sizeof(T) == 4) {
        // batch-minor tiles of a CHWN source: a thread per (tile, channel vector)
        if (layout == WINO_CHWN && order == WINO_TILES_BATCH_MINOR && g.P < (1L << 28) && (long)g.N * g.H * g.W * 4 < (1L << 32) &&
            (long)g.Cp * g.Pp * 4 < (1L << 32)) {
            dim3 grid((unsigned)((g.P + 255) / 256), g.Cp / CV), block(256);
            const bool ride = job > 0 && (long)grid.x * grid.y * 256 >= job;
            if (job > 0 && !ride) {
                const int rc = launch_f4_filter<T>(layout, fj.K, fj.C, fj.Kp, fj.Cp, fj.w, fj.U, st);
                if (rc) return rc;
            }
            if (ride) grid.z = 2;
            hipLaunchKernelGGL(input_transform_f4_vec_kernel, grid, block, 0, st, (const float*)x, (float*)V,
                               act_strides(layout, g.N, g.C, g.H, g.W), g.N, g.C, g.H, g.W, g.pad, g.th, g.tw, g.P, g.Pp, g.Cp, order,
                               ride ? fj : FilterJob{});
            LAUNCH_CHECK("f4_input_transform_vec");
            return WINO_OK;
        }
    }
    dim3 grid((unsigned)((g.P * CV + 255) / 256), g.Cp / CV), block(256);
    const bool ride = job > 0 && (long)grid.x * grid.y * 256 >= job;
    if (job > 0 && !ride) {
        const int rc = launch_f4_filter<T>(layout, fj.K, fj.C, fj.Kp, fj.Cp, fj.w, fj.U, st);
        if (rc) return rc;
    }
    if (ride) grid.z = 2;
    hipLaunchKernelGGL(input_transform_f4_generic_kernel<T>, grid, block, 0, st, (const T*)x, (T*)V,
                       act_strides(layout, g.N, g.C, g.H, g.W), g.N, g.C, g.H, g.W, g.pad, g.th, g.tw, g.P, g.Pp,
                       g.Cp, order, ride ? fj : FilterJob{});
    LAUNCH_CHECK("f4_input_transform");
    return WINO_OK;
}

template <typename T>
int launch_f4_output(int layout, int order, int porder, unsigned flags, const void* bias, int N, int K, int Ho, int Wo,
                     int Kp, long P, long Pp, const float* Mo, void* y, hipStream_t st) {
    const int th = (Ho + 3) / 4, tw = (Wo + 3) / 4;
    const Epilogue ep = make_epilogue(flags, bias);
    const ActStrides ys = out_strides(layout, flags, N, K, Ho, Wo);
    if (porder == WINO_PRODUCT_PK) {
        int bx = 64;
        while (bx < K && bx < 256) bx *= 2;
        dim3 block(bx, 256 / bx), grid((K + bx - 1) / bx, (unsigned)((P + block.y - 1) / block.y));
        hipLaunchKernelGGL((output_transform_f4_kernel<T, true>), grid, block, 0, st, Mo, (T*)y, ys, N, K, Ho, Wo, th, tw, P,
                           Pp, Kp, order, ep);
    } else {
        dim3 grid((unsigned)((P + 255) / 256), K), block(256);
        hipLaunchKernelGGL((output_transform_f4_kernel<T, false>), grid, block, 0, st, Mo, (T*)y, ys, N, K, Ho, Wo, th, tw, P,
                           Pp, Kp, order, ep);
    }
    LAUNCH_CHECK("f4_output_transform");
    return WINO_OK;
}

// part: room for plan.part_bytes; cnt: the arena's arrival counters (zero between launches)
int launch_f4_gemm_rows(int dst, int order, unsigned flags, const void* bias, const Geometry& g, const F4RowsPlan& plan,
                        const void* U, const void* V, void* y, float* part, int* cnt, hipStream_t st) {
    static std::atomic<bool> attr_set{false};
    if (!attr_set.load(std::memory_order_acquire)) {
        HIP_TRY(hipFuncSetAttribute((const void*)gemm_rows_f4_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, GF4_LDS));
        HIP_TRY(hipFuncSetAttribute((const void*)gemm_rows_f4_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, GF4_LDS));
        attr_set.store(true, std::memory_order_release);
    }
    const ActStrides ys = out_strides(dst, flags, g.N, g.K, g.Ho, g.Wo);
    const Epilogue ep = make_epilogue(flags, bias);
    const int spin_limit = 1 << 22;                       // x ~1 us: seconds, against a wait that is normally over before it starts
    if (dst == WINO_NHWC)
        hipLaunchKernelGGL((gemm_rows_f4_kernel<true>), dim3((unsigned)plan.grid), dim3(512), GF4_LDS, st, (const float*)U,
                           (const float*)V, (float*)y, ys, g.N, g.K, g.Ho, g.Wo, g.th, g.tw, g.P, g.Cp, g.Kp, g.Pp, order, ep,
                           plan.kTiles, plan.pTiles, plan.nparts, part, cnt, spin_limit);
    else
        hipLaunchKernelGGL((gemm_rows_f4_kernel<false>), dim3((unsigned)plan.grid), dim3(512), GF4_LDS, st, (const float*)U,
                           (const float*)V, (float*)y, ys, g.N, g.K, g.Ho, g.Wo, g.th, g.tw, g.P, g.Cp, g.Kp, g.Pp, order, ep,
                           plan.kTiles, plan.pTiles, plan.nparts, part, cnt, spin_limit);
    LAUNCH_CHECK("f4_gemm_rows");
    return WINO_OK;
}

#define DISPATCH_DTYPE(dtype, CALL)                          \
    switch (dtype) {                                         \
    case WINO_F32: { typedef float T; return CALL; }         \
    case WINO_F16: { typedef f16_t T; return CALL; }         \
    case WINO_BF16: { typedef bf16_t T; return CALL; }       \
    default: return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype); \
    }

#define DISPATCH_DTYPE_RC(rc, dtype, CALL)                   \
    switch (dtype) {                                         \
    case WINO_F32: { typedef float T; rc = CALL; break; }    \
    case WINO_F16: { typedef f16_t T; rc = CALL; break; }    \
    case WINO_BF16: { typedef bf16_t T; rc = CALL; break; }  \
    default: rc = fail(WINO_ERR_INVALID, "unknown dtype %d", dtype); \
    }

int tile_order_for(int src, int /*dst*/) {
    // The tile order follows the source: batch-minor keeps CHWN reads (and CHWN
    // writes, when the destination is CHWN too) contiguous along n.
    return src == WINO_CHWN ? WINO_TILES_BATCH_MINOR : WINO_TILES_BATCH_MAJOR;
}

// Measured on MI355X over the VGG-16 layer shapes: the fewer the channels, the more
// the transformed tensors cost relative to the multiplies, and the more fusion pays.
// Chosen from sweeps of the VGG-16 shapes over the three algorithms, per layout and element type.
// ---- direct convolution of layers with C <= 4 ----------------------------------------
// lanes along the contiguous axis of y (w for NCHW, n for CHWN, k for NHWC); the kernels do not pool: a pooled layer
// runs unpooled into scratch and a pooling kernel follows (direct_pooled_ok)
bool direct_ok(int dst, unsigned flags, const Geometry& g) {
    const size_t lds = direct_lds_bytes(g.C, g.K);
    return lds != 0 && lds <= 64 * 1024 && !(flags & WINO_FLAG_POOL2) && g.pad <= 1 &&
           (long)g.N * g.C * g.H * g.W < (1L << 30) && (long)g.N * g.K * g.Ho * g.Wo < (1L << 30);   // 32-bit byte offsets
}

template <typename T>
int launch_direct_t(int src, int dst, unsigned flags, const void* bias, const Geometry& g, const void* x, const void* w,
                    void* y, hipStream_t st) {
    const long Q = (long)g.N * g.Ho * g.Wo;
    // 32-pixel groups per wave: as many as leave about eight workgroups for every CU (the filter bank is staged
    // per workgroup, so more pixels per workgroup are cheaper, fewer workgroups fill the chip worse)
    int groups = (int)std::min<long>(DIRECT_MAX_GROUPS, std::max<long>(1, Q / (128L * 2048)));
    const long per_wg = 128L * groups;
    const dim3 grid((unsigned)((Q + per_wg - 1) / per_wg)), block(256);
    const size_t lds = direct_lds_bytes(g.C, g.K);
    const ActStrides xs = act_strides(src, g.N, g.C, g.H, g.W), ys = act_strides(dst, g.N, g.K, g.Ho, g.Wo);
    const FltStrides fs = flt_strides(src, g.K, g.C);
    const Epilogue ep = make_epilogue(flags, bias);
    const int minor = dst == WINO_CHWN;
#define DIRECT_LAUNCH(NE)                                                                                           \
    if (dst == WINO_NHWC)                                                                                           \
        hipLaunchKernelGGL((direct_small_c_kernel<T, NE, true>), grid, block, lds, st, (const T*)x, (const T*)w, (T*)y, \
                           xs, fs, ys, g.N, g.C, g.K, g.H, g.W, g.pad, g.Ho, g.Wo, minor, Q, groups, ep);            \
    else                                                                                                            \
        hipLaunchKernelGGL((direct_small_c_kernel<T, NE, false>), grid, block, lds, st, (const T*)x, (const T*)w, (T*)y, \
                           xs, fs, ys, g.N, g.C, g.K, g.H, g.W, g.pad, g.Ho, g.Wo, minor, Q, groups, ep)
    if constexpr (sizeof(T) == 2) {
        // 2-byte tensors: the 16-bit matrix instruction, 16 taps each
        const size_t lds16 = direct16_lds_bytes(g.C, g.K);
        const bool chwn_tiles = src == WINO_CHWN && dst == WINO_CHWN && g.N <= DSC_DS && ((long)g.W * g.N) % 2 == 0;
        if (((src == WINO_NCHW && dst == WINO_NCHW && g.W % 2 == 0) || chwn_tiles) && !misaligned(x, 4) && !misaligned(y, 4) &&
            direct16_tiles_lds_bytes(g.C, g.K, chwn_tiles ? g.N : 1) <= 64 * 1024) {
            // NCHW on both sides, rows of whole 4-byte pairs: tiles of 4 rows x 64 columns per wave, input through LDS,
            // whole cache lines stored; the tiles are dealt evenly to two workgroups per CU (the kernel's registers
            // leave room for two waves a SIMD).  CHWN on both sides: one image of width W * N, taps N columns apart.
            const int ds = chwn_tiles ? g.N : 1, n1 = chwn_tiles ? 1 : g.N, w1 = g.W * ds, wo1 = g.Wo * ds;
            const int tiles_y = (g.Ho + DSC_WR - 1) / DSC_WR, tiles_x = (wo1 + DSC_WC - 1) / DSC_WC;
            const long ntiles = (long)n1 * tiles_y * tiles_x, resident = 8L * device_cus();
            const long per = (ntiles + resident - 1) / resident;                 // tiles per wave
            const dim3 tgrid((unsigned)((ntiles + 4 * per - 1) / (4 * per)));
            const size_t ldst = direct16_tiles_lds_bytes(g.C, g.K, ds);
#define DIRECT16_TILES(NE)                                                                                                 \
    if (chwn_tiles)                                                                                                        \
        hipLaunchKernelGGL((direct_small_c16_tiles_kernel<T, NE, true>), tgrid, block, ldst, st, (const T*)x, (const T*)w,  \
                           (T*)y, n1, g.C, g.K, g.H, w1, g.pad, ds, g.Ho, wo1, tiles_y, tiles_x, (int)ntiles, ep);          \
    else                                                                                                                   \
        hipLaunchKernelGGL((direct_small_c16_tiles_kernel<T, NE, false>), tgrid, block, ldst, st, (const T*)x, (const T*)w, \
                           (T*)y, n1, g.C, g.K, g.H, w1, g.pad, ds, g.Ho, wo1, tiles_y, tiles_x, (int)ntiles, ep)
            switch (g.C) {
            case 1: DIRECT16_TILES(1); break;
            case 4: DIRECT16_TILES(3); break;
            default: DIRECT16_TILES(2); break;
            }
#undef DIRECT16_TILES
            LAUNCH_CHECK("direct_small_c16_tiles");
            return WINO_OK;
        }
        if (src == WINO_NHWC && dst == WINO_NHWC && g.W % 2 == 0 && g.K % 2 == 0 && !misaligned(x, 4) && !misaligned(y, 4) &&
            direct16_tiles_nhwc_lds_bytes(g.C, g.K) <= 64 * 1024) {
            // NHWC on both sides, rows and pixels of whole 4-byte pairs: tiles of 4 rows x 32 columns per wave, input
            // through LDS, the 64 filters of two neighbouring pixels stored per instruction
            const int tiles_y = (g.Ho + DSC_WR - 1) / DSC_WR, tiles_x = (g.Wo + 31) / 32;
            const long ntiles = (long)g.N * tiles_y * tiles_x, resident = 8L * device_cus();
            const long per = (ntiles + resident - 1) / resident;                 // tiles per wave
            const dim3 tgrid((unsigned)((ntiles + 4 * per - 1) / (4 * per)));
            const size_t ldst = direct16_tiles_nhwc_lds_bytes(g.C, g.K);
#define DIRECT16_TILES(NE)                                                                                                   \
    hipLaunchKernelGGL((direct_small_c16_tiles_nhwc_kernel<T, NE>), tgrid, block, ldst, st, (const T*)x, (const T*)w, (T*)y, g.N, \
                       g.C, g.K, g.H, g.W, g.pad, g.Ho, g.Wo, tiles_y, tiles_x, (int)ntiles, ep)
            switch (g.C) {
            case 1: DIRECT16_TILES(1); break;
            case 4: DIRECT16_TILES(3); break;
            default: DIRECT16_TILES(2); break;
            }
#undef DIRECT16_TILES
            LAUNCH_CHECK("direct_small_c16_tiles_nhwc");
            return WINO_OK;
        }
#define DIRECT16_LAUNCH(NE)                                                                                          \
    if (dst == WINO_NHWC)                                                                                           \
        hipLaunchKernelGGL((direct_small_c16_kernel<T, NE, true>), grid, block, lds16, st, (const T*)x, (const T*)w, \
                           (T*)y, xs, fs, ys, g.N, g.C, g.K, g.H, g.W, g.pad, g.Ho, g.Wo, minor, Q, groups, ep);     \
    else                                                                                                            \
        hipLaunchKernelGGL((direct_small_c16_kernel<T, NE, false>), grid, block, lds16, st, (const T*)x, (const T*)w, \
                           (T*)y, xs, fs, ys, g.N, g.C, g.K, g.H, g.W, g.pad, g.Ho, g.Wo, minor, Q, groups, ep)
        switch (g.C) {
        case 1: DIRECT16_LAUNCH(1); break;
        case 4: DIRECT16_LAUNCH(3); break;
        default: DIRECT16_LAUNCH(2); break;
        }
#undef DIRECT16_LAUNCH
    } else {
        if (src == WINO_NCHW && dst == WINO_NCHW && g.W % 2 == 0 && !misaligned(x, 8) && direct_tiles_lds_bytes(g.C, g.K) <= 64 * 1024) {
            // NCHW on both sides, rows of whole 8-byte pairs: tiles of 4 rows x 32 columns per wave, input through LDS;
            // the tiles are dealt evenly to the waves the kernel's registers leave room for (four a SIMD)
            const int tiles_y = (g.Ho + DSF_WR - 1) / DSF_WR, tiles_x = (g.Wo + 31) / 32;
            const long ntiles = (long)g.N * tiles_y * tiles_x, resident = 16L * device_cus();
            const long per = (ntiles + resident - 1) / resident;                 // tiles per wave
            const dim3 tgrid((unsigned)((ntiles + 4 * per - 1) / (4 * per)));
            const size_t ldst = direct_tiles_lds_bytes(g.C, g.K);
#define DIRECT_TILES(NE)                                                                                                  \
    hipLaunchKernelGGL((direct_small_c_tiles_kernel<NE>), tgrid, block, ldst, st, (const float*)x, (const float*)w, (float*)y, \
                       g.N, g.C, g.K, g.H, g.W, g.pad, g.Ho, g.Wo, tiles_y, tiles_x, (int)ntiles, ep)
            switch (g.C) {
            case 1: DIRECT_TILES(5); break;
            case 2: DIRECT_TILES(9); break;
            case 3: DIRECT_TILES(14); break;
            default: DIRECT_TILES(18); break;
            }
#undef DIRECT_TILES
            LAUNCH_CHECK("direct_small_c_tiles");
            return WINO_OK;
        }
        if (src == WINO_NHWC && dst == WINO_NHWC && ((long)g.W * g.C) % 2 == 0 && !misaligned(x, 8) &&
            direct_tiles_nhwc_lds_bytes(g.C, g.K) <= 64 * 1024) {
            // NHWC on both sides, rows of whole 8-byte pairs: tiles of 4 rows x 32 columns per wave, input through LDS
            const int tiles_y = (g.Ho + DSF_WR - 1) / DSF_WR, tiles_x = (g.Wo + 31) / 32;
            const long ntiles = (long)g.N * tiles_y * tiles_x, resident = 16L * device_cus();
            const long per = (ntiles + resident - 1) / resident;                 // tiles per wave
            const dim3 tgrid((unsigned)((ntiles + 4 * per - 1) / (4 * per)));
            const size_t ldst = direct_tiles_nhwc_lds_bytes(g.C, g.K);
#define DIRECT_TILES_N(NE)                                                                                                     \
    hipLaunchKernelGGL((direct_small_c_tiles_nhwc_kernel<NE>), tgrid, block, ldst, st, (const float*)x, (const float*)w, (float*)y, \
                       g.N, g.C, g.K, g.H, g.W, g.pad, g.Ho, g.Wo, tiles_y, tiles_x, (int)ntiles, ep)
            switch (g.C) {
            case 1: DIRECT_TILES_N(5); break;
            case 2: DIRECT_TILES_N(9); break;
            case 3: DIRECT_TILES_N(14); break;
            default: DIRECT_TILES_N(18); break;
            }
#undef DIRECT_TILES_N
            LAUNCH_CHECK("direct_small_c_tiles_nhwc");
            return WINO_OK;
        }
        switch (g.C) {
        case 1: DIRECT_LAUNCH(5); break;
        case 2: DIRECT_LAUNCH(9); break;
        case 3: DIRECT_LAUNCH(14); break;
        default: DIRECT_LAUNCH(18); break;
        }
    }
#undef DIRECT_LAUNCH
    LAUNCH_CHECK("direct_small_c");
    return WINO_OK;
}

int launch_direct(int src, int dst, int dtype, unsigned flags, const void* bias, const Geometry& g, const void* x,
                  const void* w, void* y, hipStream_t st) {
    DISPATCH_DTYPE(dtype, launch_direct_t<T>(src, dst, flags, bias, g, x, w, y, st));
}

// The one-launch kernel for fp32 layers with few output pixels (direct_few_pixels_kernel): offered while its units of
// 4 x 8 pixels x 32 filters fit four rounds of the chip; pooled outputs stay on the Winograd path.
long direct_few_units(const Geometry& g) { return (long)g.N * ((g.Ho + 3) / 4) * ((g.Wo + 7) / 8) * ((g.K + 31) / 32); }
bool direct_few_ok(int dtype, unsigned flags, const Geometry& g) {
    return dtype == WINO_F32 && !(flags & WINO_FLAG_POOL2) && direct_few_units(g) <= 4L * device_cus() &&
           (long)g.N * g.C * g.H * g.W < (1L << 29) && (long)g.N * g.K * g.Ho * g.Wo < (1L << 29) &&
           (long)g.K * g.C * 9 < (1L << 29);                                                 // 32-bit byte offsets
}
// Which 16-byte pieces the filter bank offers (FM of the kernel): a [K][C][3][3] bank 1, [K][3][3][C] 2, [C][3][3][K] 3,
// when the pieces are whole (C, for the last order also K, a multiple of 4); otherwise 0, one element per load.
int direct_few_filter_mode(int src, const Geometry& g) {
    if (g.C % 4) return 0;
    if (src == WINO_NCHW) return 1;
    if (src == WINO_NHWC) return 2;
    return g.K % 4 ? 0 : 3;
}
int launch_direct_few(int src, int dst, unsigned flags, const void* bias, const Geometry& g, const void* x, const void* w,
                      void* y, hipStream_t st) {
    const int tiles_y = (g.Ho + 3) / 4, tiles_x = (g.Wo + 7) / 8, PT = g.N * tiles_y * tiles_x;
    const ActStrides xs = act_strides(src, g.N, g.C, g.H, g.W), ys = act_strides(dst, g.N, g.K, g.Ho, g.Wo);
    const FltStrides fs = flt_strides(src, g.K, g.C);
    const dim3 grid((unsigned)direct_few_units(g));
    const Epilogue ep = make_epilogue(flags, bias);
#define WINO_DFP(FM, XW)                                                                                                     \
    hipLaunchKernelGGL((direct_few_pixels_kernel<float, FM, XW>), grid, dim3(512), 0, st, (const float*)x, (const float*)w, \
                       (float*)y, xs, fs, ys, g.N, g.C, g.K, g.H, g.W, g.pad, g.Ho, g.Wo, tiles_y, tiles_x, PT, ep)
    switch (direct_few_filter_mode(src, g)) {
        case 1: WINO_DFP(1, false); break;
        case 2: WINO_DFP(2, true); break;                  // (NHWC with C a multiple of 4: a pixel's channels in pieces as well)
        case 3: WINO_DFP(3, false); break;
        default: WINO_DFP(0, false); break;
    }
#undef WINO_DFP
    LAUNCH_CHECK("direct_few_pixels");
    return WINO_OK;
}

// ---- direct convolution of 2-byte NCHW tensors on the 16-bit matrix instruction (direct16.hpp) ----------------
// Block shape for a layer: BC columns (even, at most 32: the one that wastes the fewest lanes on the image's width,
// the widest among equals), BR = pixels per workgroup / BC rows, shrunk until the block's input rows fit a buffer
// (LR * PW <= D16_PLANE pixel slots) and its load tasks fit three rounds of the 256 threads.
// rows: blocks of 16 rows x 32 columns whose waves own 4 consecutive rows of one image (Ho a multiple of 4).
bool direct16_plan(const Geometry& g, int npg, bool rows, D16Geom* d) {
    const int PB = 128 * npg;
    int BC = 0;
    long best = 0;
    for (int bc = 32; bc >= 8; bc -= 2) {
        const long padded = (long)((g.Wo + bc - 1) / bc) * bc;
        if (BC == 0 || padded < best) { BC = bc; best = padded; }
    }
    const long G = (long)g.N * g.Ho;
    if (rows) {
        if (npg != 4 || g.Ho % 4 != 0 || G < 16) return false;
        BC = 32;
    }
    int BR = (int)std::min<long>(PB / BC, G);
    auto lr_of = [&](int br) { return br + 2 + 2 * ((g.Ho + br - 2) / g.Ho); };
    const int PW = BC + 2, PP = BC / 2 + 1 + g.pad;
    if (!rows)
        while (BR > 1 && (lr_of(BR) * PW > D16_PLANE || 2 * lr_of(BR) * PP > 768)) --BR;
    if (lr_of(BR) * PW > D16_PLANE || 2 * lr_of(BR) * PP > 768) return false;
    d->N = g.N; d->C = g.C; d->K = g.K; d->H = g.H; d->W = g.W; d->pad = g.pad; d->Ho = g.Ho; d->Wo = g.Wo;
    d->BR = BR; d->BC = BC; d->PW = PW; d->LR = lr_of(BR); d->PP = PP; d->WC = 1; d->ds = 1;
    d->colBlocks = (g.Wo + BC - 1) / BC;
    d->rowBlocks = (int)((G + BR - 1) / BR);
    d->maxcross = (g.Ho + BR - 2) / g.Ho;
    d->a4 = 0; d->b3 = 0;
    d->kTiles = (g.K + D16_KT - 1) / D16_KT;
    d->CQ = (int)round_up(g.C, 32) / 8;
    d->Kp = (int)round_up(g.K, D16_KT);
    d->G = G;
    return true;
}

// The 8-wave kernel of direct16_rows.hpp: blocks of 32/WF rows x 32 columns whose waves own 4 consecutive rows of one
// image.  WF = 2 (128 filters per tile) when that wastes no filters, else 1.
// DIL: a CHWN layer taken as ONE image of width W * N whose tap columns lie N elements apart (direct16_rows.hpp).
// xn: the source is NHWC.  With 64-filter tiles its blocks stay 128 columns wide and 8 rows high on wider images: a stage
// takes 32 of a pixel's bytes, and the taller block reads 10 input rows for 8 instead of 6 for 4 (C = K = 64, 224 x 224
// at N = 32 in bf16: 210 -> 178 us; from NCHW, where a row of a block is one contiguous run, the wide block stays: 195 against 199).
template <int WF, bool DIL = false>
bool direct16_rows_plan(const Geometry& gl, D16Geom* d, bool xn = false) {
    typedef D16R<WF, DIL> P;
    Geometry g = gl;
    int ds = 1;
    if (DIL) {
        // (pairs of neighbouring elements are two images; the zero columns of a row must fit the task encoding)
        if (gl.N % 2 != 0 || (long)gl.pad * gl.N > 64 || (long)gl.W * gl.N >= (1L << 24)) return false;
        ds = gl.N;
        g.N = 1;
        g.W = gl.W * gl.N;
        g.Wo = gl.Wo * gl.N;
    }
    const long G = (long)g.N * g.Ho;
    if (g.Ho % 4 != 0 || g.K % 64 != 0 || g.Wo % 2 != 0) return false;
    // the block's waves (4 rows x 32 columns each) side by side until they span the image, the rest stacked
    int WC = 0, BR = 0, BC = 0, maxcross = 0, PW = 0, LR = 0, PP = 0;
    const int padw = g.pad * ds;                              // zero columns left of a row; pairs start at even columns
    for (int wc_cap : {xn && WF == 1 ? 4 : P::WP, P::WP}) {   // (the narrower block first where it is preferred; the wide one if its rows do not fit)
        WC = 1;
        while (WC < wc_cap && 32 * WC < g.Wo) WC *= 2;
        BR = 4 * (P::WP / WC);
        BC = 32 * WC;
        if (G < BR) return false;
        maxcross = g.Ho % BR == 0 ? 0 : (g.Ho + BR - 2) / g.Ho;           // images a block's rows can span beyond the first
        PW = std::min(BC, (g.Wo + 1) / 2 * 2) + 2 * ds;     // slots of an LDS row: the block's columns (or the image's) + the two tap columns
        LR = BR + 2 + 2 * maxcross;
        PP = (PW + (padw & 1) + 1) / 2;
        if (!(LR * PW > P::XPLANE || 2 * LR * PP > P::NTASK * 512 || LR > 255 || PW > 2048)) break;
        if (wc_cap == P::WP) return false;
    }
    d->N = g.N; d->C = g.C; d->K = g.K; d->H = g.H; d->W = g.W; d->pad = g.pad; d->Ho = g.Ho; d->Wo = g.Wo;
    d->BR = BR; d->BC = BC; d->WC = WC; d->PW = PW; d->LR = LR; d->PP = PP; d->ds = ds;
    d->colBlocks = (g.Wo + BC - 1) / BC;
    d->rowBlocks = (int)((G + BR - 1) / BR);
    d->maxcross = maxcross;
    d->a4 = 0; d->b3 = 0;
    d->kTiles = (g.K + P::KT - 1) / P::KT;
    d->CQ = (int)round_up(g.C, 16) / 8;
    d->Kp = (int)round_up(g.K, P::KT);
    d->G = G;
    return (long)d->rowBlocks * d->colBlocks < (1L << 28);
}
inline int direct16_rows_wf(const Geometry& g) { return (g.K % 128 == 0 || g.K > 256) ? 2 : 1; }

// Blocks whose waves own 3 rows mixed in with the 4-row ones.  A layer is a handful of tiles per CU, and rounds of
// whole tiles leave a good part of the chip idle in the last one (N = 32, C = K = 256, 56 x 56: 448 tiles on 256 CUs, two
// rounds for 1.75 rounds of work).  A 3-row tile is three quarters of the multiplies: cut every image into a4 blocks of
// 4-row waves and b3 of 3-row waves, 4-row blocks first, and the same layer is 512 tiles, one of each kind to a CU:
// 7 units instead of 8.  The cost of a cut is taken as the largest sum of rows-per-wave over a workgroup's tiles,
// dealt round-robin; a cut is taken when it saves at least 6 %.  (Pooling needs whole row pairs in a wave: no cut.)
long direct16_deal_cost(long t4, long t3, long wgs) {
    long worst = 0;
    const long total = t4 + t3;
    const long probe[5] = {0, t4 % wgs, (t4 % wgs + wgs - 1) % wgs, total % wgs, (total % wgs + wgs - 1) % wgs};
    for (long j : probe) {
        if (j >= total) continue;
        const long n = (total - j + wgs - 1) / wgs, n4 = j < t4 ? (t4 - j + wgs - 1) / wgs : 0;
        worst = std::max(worst, 4 * n4 + 3 * (n - n4));
    }
    return worst;
}
void direct16_row_mix(D16Geom* d, bool pool) {
    const int S = d->BR / 4;
    if (pool || d->Ho % S != 0) return;
    const long per = (long)d->colBlocks * d->kTiles, cus = std::max(8, device_cus() / 8 * 8);
    const long plain_tiles = (long)d->rowBlocks * per;
    const long plain = direct16_deal_cost(plain_tiles, 0, std::min(cus, (plain_tiles + 7) / 8 * 8));
    long best = plain;
    int best_b = 0;
    const int units = d->Ho / S;                             // = 4 a4 + 3 b3
    for (int b = 1; 3 * b <= units; ++b) {
        if ((units - 3 * b) % 4 != 0) continue;
        const int a = (units - 3 * b) / 4;
        const long t4 = (long)d->N * a * per, t3 = (long)d->N * b * per;
        if ((t4 + t3) / per >= (1L << 28) / d->colBlocks) break;
        const long cost = direct16_deal_cost(t4, t3, std::min(cus, (t4 + t3 + 7) / 8 * 8));
        if (cost < best) {
            best = cost;
            best_b = b;
        }
    }
    if (best_b == 0 || best * 100 > plain * 94) return;
    d->b3 = best_b;
    d->a4 = (units - 3 * best_b) / 4;
    d->rowBlocks = d->N * (d->a4 + d->b3);
    d->maxcross = 0;
}

template <typename T, int WF, bool XN = false, bool YN = XN, bool DIL = false>
int launch_direct16_rows_t(const D16Geom& planned, const Epilogue& ep, const void* x, const void* W9, void* y, hipStream_t st) {
    D16Geom d = planned;
    direct16_row_mix(&d, ep.pool != 0);
    static std::atomic<bool> attr_set{false};    // (per instantiation; setting it twice from two threads is harmless)
    if (!attr_set.load(std::memory_order_acquire)) {
        HIP_TRY(hipFuncSetAttribute((const void*)direct16_rows_kernel<T, WF, XN, YN, DIL>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    D16R<WF, DIL>::LDS));
        attr_set.store(true, std::memory_order_release);
    }
    // persistent grid: one workgroup of 8 waves per CU (or as many as there are tiles), a multiple of the 8 XCDs
    const long tiles = (long)d.rowBlocks * d.colBlocks * d.kTiles;
    const long blocks = std::max<long>(8, std::min<long>(device_cus(), (tiles + 7) / 8 * 8) / 8 * 8);
    constexpr int kLds = D16R<WF, DIL>::LDS;
    hipLaunchKernelGGL((direct16_rows_kernel<T, WF, XN, YN, DIL>), dim3((unsigned)blocks), dim3(512), kLds, st, (const T*)x,
                       (const T*)W9, (T*)y, d, ep);
    LAUNCH_CHECK("direct16_rows");
    return WINO_OK;
}

size_t direct16_bank_bytes(const Geometry& g) { return (size_t)9 * round_up(g.C, 32) * round_up(g.K, 128) * 2; }

// whether a layer runs on the 8-wave kernel (given 4-byte aligned tensors); chwn: as one image of width W * N
bool direct16_big(const Geometry& g, D16Geom* d, bool chwn = false, bool xn = false) {
    const bool plan = chwn ? (direct16_rows_wf(g) == 2 ? direct16_rows_plan<2, true>(g, d) : direct16_rows_plan<1, true>(g, d))
                           : (direct16_rows_wf(g) == 2 ? direct16_rows_plan<2>(g, d, xn) : direct16_rows_plan<1>(g, d, xn));
    return plan && (long)d->rowBlocks * d->colBlocks * d->kTiles >= device_cus() / 2;
}
// A pooled CHWN layer in the 8-wave kernel's own stores: with 32 images a column group of 32 is one pixel column, and a
// wave takes 16 images of two neighbouring pixel columns instead, so that a window's columns are lanes 16 apart.
inline bool direct16_chwn_pools(const Geometry& g) { return g.N == 32 && g.Wo % 2 == 0; }
bool direct16_ok(int src, int dst, int dtype, unsigned flags, const Geometry& g) {
    D16Geom d;
    if (dtype == WINO_F32 || g.C % 8 != 0 || g.pad > 1 || (long)g.N * g.K * g.Ho * g.Wo >= (1L << 31)) return false;
    if (src == WINO_CHWN || dst == WINO_CHWN) {
        // CHWN on both sides: the 8-wave kernel only, no pooling in its stores (a pooling window's columns are N elements
        // apart: direct16_chwn_pool_ok and a pooling kernel take such a layer);
        // 32-bit byte offsets inside a stage's 16 channel planes
        return src == dst && (!(flags & WINO_FLAG_POOL2) || direct16_chwn_pools(g)) && (long)g.H * g.W * g.N * 2 * 16 < (1L << 32) &&
               direct16_big(g, &d, true);
    }
    if (src == WINO_NHWC || dst == WINO_NHWC) {
        // an NHWC side: the 8-wave kernel only; offsets inside a block's images are 32-bit
        if (!direct16_big(g, &d, false, src == WINO_NHWC)) return false;
        return src == WINO_NHWC ? (long)(d.maxcross + 1) * g.C * g.H * g.W * 2 < (1L << 32)
                                : g.W % 2 == 0 && (long)g.C * g.H * g.W * 2 * 8 < (1L << 32);
    }
    if (!(g.W % 2 == 0 && (long)g.C * g.H * g.W * 2 * 8 < (1L << 32) && direct16_plan(g, 4, false, &d))) return false;
    // 2x2 pooling lives in the stores of the 8-wave kernel only
    return !(flags & WINO_FLAG_POOL2) || direct16_big(g, &d);
}

template <typename T, int NPG, bool ROWS>
int launch_direct16_t(const D16Geom& d, const Epilogue& ep, const void* x, const void* W9, void* y, hipStream_t st) {
    static std::atomic<bool> attr_set{false};    // (per instantiation; the attribute is a property of the kernel)
    if (!attr_set.load(std::memory_order_acquire)) {
        HIP_TRY(hipFuncSetAttribute((const void*)direct16_kernel<T, NPG, ROWS>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    2 * D16_BUF));
        attr_set.store(true, std::memory_order_release);
    }
    // persistent grid: two workgroups per CU (or as many as there are tiles), a multiple of the 8 XCDs
    const long tiles = (long)d.rowBlocks * d.colBlocks * d.kTiles;
    if ((long)d.rowBlocks * d.colBlocks >= (1L << 28)) return fail(WINO_ERR_UNSUPPORTED, "direct convolution: too many pixel blocks");
    const long blocks = std::min<long>(2L * device_cus(), (tiles + 7) / 8 * 8) / 8 * 8;
    hipLaunchKernelGGL((direct16_kernel<T, NPG, ROWS>), dim3((unsigned)std::max<long>(blocks, 8)), dim3(256), 2 * D16_BUF, st,
                       (const T*)x, (const T*)W9, (T*)y, d, ep);
    LAUNCH_CHECK("direct16");
    return WINO_OK;
}

// W9: room for direct16_bank_bytes(g), 16-byte aligned.  The order of the bank depends on the kernel that reads it,
// and that on the layer and on the alignment of x and y, so packing and running take the same arguments:
// D16_PACK_RUN both, D16_PACK only the bank (x and y are looked at, not touched), D16_RUN with a bank packed earlier
// for tensors of the same alignment.
enum { D16_PACK_RUN = 0, D16_PACK = 1, D16_RUN = 2 };
int launch_direct16(int layout, int dst, int dtype, unsigned flags, const void* bias, const Geometry& g, const void* x,
                    const void* w, void* W9, void* y, hipStream_t st, int mode = D16_PACK_RUN) {
    const bool nhwc = layout == WINO_NHWC, ynhwc = dst == WINO_NHWC, chwn = layout == WINO_CHWN;
    if (chwn != (dst == WINO_CHWN)) return fail(WINO_ERR_UNSUPPORTED, "direct convolution: CHWN tensors on both sides or on neither");
    if (misaligned(x, nhwc ? 16 : 4))
        return fail(WINO_ERR_UNSUPPORTED, "the 16-bit direct path loads column pairs (NHWC: channel vectors): x must be 4-byte (16-byte) aligned");
    D16Geom d;
    // large layers: the 8-wave kernel, one workgroup per CU; else tiles of 512 pixels, fewer pixels when that leaves
    // the chip short of tiles
    int npg = 4, wf = direct16_rows_wf(g);
    const bool pool = (flags & WINO_FLAG_POOL2) != 0;        // (pooled values are stored one by one: no alignment asked of y)
    const bool big = (pool || !misaligned(y, 4)) && !(chwn && pool && !direct16_chwn_pools(g)) && direct16_big(g, &d, chwn, nhwc);
    if (chwn && !big) return fail(WINO_ERR_UNSUPPORTED, "direct convolution of CHWN tensors: the 8-wave kernel's layer shapes, an even batch (pooling: 32 images, an even width), y 4-byte aligned");
    if ((nhwc || ynhwc) && !big) return fail(WINO_ERR_UNSUPPORTED, "direct convolution of NHWC tensors: the 8-wave kernel's layer shapes, y 4-byte aligned");
    if (pool && !big) return fail(WINO_ERR_UNSUPPORTED, "direct convolution: pooling needs the 8-wave kernel's layer shapes");
    const bool rows = !big && direct16_plan(g, 4, true, &d) && (long)d.rowBlocks * d.colBlocks * d.kTiles >= 2L * device_cus();
    if (!big && !rows) {
        for (; npg > 1; npg >>= 1) {
            if (!direct16_plan(g, npg, false, &d)) return fail(WINO_ERR_UNSUPPORTED, "direct convolution: no block shape for this layer");
            if ((long)d.rowBlocks * d.colBlocks * d.kTiles >= 2L * device_cus()) break;
        }
        if (!direct16_plan(g, npg, false, &d)) return fail(WINO_ERR_UNSUPPORTED, "direct convolution: no block shape for this layer");
    }
    const Epilogue ep = make_epilogue(flags, bias);
    const FltStrides fs = flt_strides(layout, g.K, g.C);
    dim3 pgrid((d.Kp + 63) / 64, d.CQ);
    const bool pvec = g.C % 8 == 0 && !misaligned(w, 16) && !chwn;          // ([C][3][3][K] banks: element by element)
#define D16_GO(T)                                                                                                  \
    if (mode != D16_RUN) {                                                                                         \
        if (pvec && nhwc) hipLaunchKernelGGL((direct16_pack_kernel<T, 2>), pgrid, dim3(64), 0, st, (const T*)w, (T*)W9, fs, g.K, g.C, d.Kp, d.CQ); \
        else if (pvec) hipLaunchKernelGGL((direct16_pack_kernel<T, 1>), pgrid, dim3(64), 0, st, (const T*)w, (T*)W9, fs, g.K, g.C, d.Kp, d.CQ); \
        else hipLaunchKernelGGL((direct16_pack_kernel<T, 0>), pgrid, dim3(64), 0, st, (const T*)w, (T*)W9, fs, g.K, g.C, d.Kp, d.CQ); \
        LAUNCH_CHECK("direct16_pack");                                                                             \
    }                                                                                                              \
    if (mode == D16_PACK) return WINO_OK;                                                                          \
    if (chwn) { if (wf == 2) return launch_direct16_rows_t<T, 2, false, false, true>(d, ep, x, W9, y, st);         \
                return launch_direct16_rows_t<T, 1, false, false, true>(d, ep, x, W9, y, st); }                    \
    if (nhwc && ynhwc) { if (wf == 2) return launch_direct16_rows_t<T, 2, true, true>(d, ep, x, W9, y, st);        \
                         return launch_direct16_rows_t<T, 1, true, true>(d, ep, x, W9, y, st); }                   \
    if (nhwc) { if (wf == 2) return launch_direct16_rows_t<T, 2, true, false>(d, ep, x, W9, y, st);                \
                return launch_direct16_rows_t<T, 1, true, false>(d, ep, x, W9, y, st); }                           \
    if (ynhwc) { if (wf == 2) return launch_direct16_rows_t<T, 2, false, true>(d, ep, x, W9, y, st);               \
                 return launch_direct16_rows_t<T, 1, false, true>(d, ep, x, W9, y, st); }                          \
    if (big && wf == 2) return launch_direct16_rows_t<T, 2>(d, ep, x, W9, y, st);                                  \
    if (big) return launch_direct16_rows_t<T, 1>(d, ep, x, W9, y, st);                                             \
    if (rows) return launch_direct16_t<T, 4, true>(d, ep, x, W9, y, st);                                           \
    if (npg == 4) return launch_direct16_t<T, 4, false>(d, ep, x, W9, y, st);                                      \
    if (npg == 2) return launch_direct16_t<T, 2, false>(d, ep, x, W9, y, st);                                      \
    return launch_direct16_t<T, 1, false>(d, ep, x, W9, y, st)
    if (dtype == WINO_F16) { D16_GO(f16_t); }
    D16_GO(bf16_t);
#undef D16_GO
}

// CHWN tensors with 2x2 pooling that the 8-wave kernel does not pool itself (batches other than 32): the layer unpooled
// into `tmp` (room for direct16_unpooled_bytes), then the pooling kernel
bool direct16_chwn_pool_ok(int src, int dst, int dtype, unsigned flags, const Geometry& g) {
    return src == WINO_CHWN && dst == WINO_CHWN && (flags & WINO_FLAG_POOL2) && !direct16_chwn_pools(g) &&
           direct16_ok(src, dst, dtype, flags & ~(unsigned)WINO_FLAG_POOL2, g);
}
size_t direct16_unpooled_bytes(int dtype, const Geometry& g) {
    return ((size_t)g.N * g.K * g.Ho * g.Wo * dtype_size(dtype) + 255) / 256 * 256;
}
// 2x2 pooling of an unpooled tensor in scratch (aligned) into y, [outer][Ho][Wo][inner] or, inner == 1, planes of rows
template <typename T>
int launch_pool2_t(int layout, const Geometry& g, const void* tmp, void* y, hipStream_t st) {
    const int Hp = g.Ho / 2, Wp = g.Wo / 2;
    if (layout == WINO_NCHW) {
        constexpr int V = 8 / (int)sizeof(T);                                // 16-byte loads, 8-byte stores
        const bool wide = g.Wo % (2 * V) == 0 && !misaligned(y, 8);
        const long total = (long)g.N * g.K * Hp * (wide ? Wp / V : Wp);
        const dim3 grid((unsigned)((total + 255) / 256));
        if (wide) hipLaunchKernelGGL((pool2_rows_kernel<T, V>), grid, dim3(256), 0, st, (const T*)tmp, (T*)y, g.Ho, g.Wo, total);
        else hipLaunchKernelGGL((pool2_rows_kernel<T, 1>), grid, dim3(256), 0, st, (const T*)tmp, (T*)y, g.Ho, g.Wo, total);
        LAUNCH_CHECK("pool2_rows");
        return WINO_OK;
    }
    const int inner = layout == WINO_CHWN ? g.N : g.K, outer = layout == WINO_CHWN ? g.K : g.N;
    constexpr int V = 16 / (int)sizeof(T);
    const int vec = inner % V == 0 && !misaligned(y, 16) ? V : inner % 2 == 0 && !misaligned(y, 2 * sizeof(T)) ? 2 : 1;
    const long total = (long)outer * Hp * Wp * (inner / vec);
    const dim3 grid((unsigned)((total + 255) / 256));
    if (vec == V) hipLaunchKernelGGL((pool2_inner_kernel<T, V>), grid, dim3(256), 0, st, (const T*)tmp, (T*)y, g.Ho, g.Wo, inner, total);
    else if (vec == 2) hipLaunchKernelGGL((pool2_inner_kernel<T, 2>), grid, dim3(256), 0, st, (const T*)tmp, (T*)y, g.Ho, g.Wo, inner, total);
    else hipLaunchKernelGGL((pool2_inner_kernel<T, 1>), grid, dim3(256), 0, st, (const T*)tmp, (T*)y, g.Ho, g.Wo, inner, total);
    LAUNCH_CHECK("pool2_inner");
    return WINO_OK;
}
int launch_direct16_chwn_pooled(int dtype, unsigned flags, const void* bias, const Geometry& g, const void* x, const void* w,
                                void* W9, void* tmp, void* y, hipStream_t st, int mode) {
    const int rc = launch_direct16(WINO_CHWN, WINO_CHWN, dtype, flags & ~(unsigned)WINO_FLAG_POOL2, bias, g, x, w, W9, tmp, st, mode);
    if (rc || mode == D16_PACK) return rc;
    if (dtype == WINO_F16) return launch_pool2_t<f16_t>(WINO_CHWN, g, tmp, y, st);
    return launch_pool2_t<bf16_t>(WINO_CHWN, g, tmp, y, st);
}
// pooled layers of at most four channels: the layer unpooled into `tmp` (room for direct16_unpooled_bytes), then pooling
bool direct_pooled_ok(int dst, unsigned flags, const Geometry& g) {
    return (flags & WINO_FLAG_POOL2) && direct_ok(dst, flags & ~(unsigned)WINO_FLAG_POOL2, g);
}
int launch_direct_pooled(int src, int dst, int dtype, unsigned flags, const void* bias, const Geometry& g, const void* x, const void* w,
                         void* tmp, void* y, hipStream_t st) {
    const int rc = launch_direct(src, dst, dtype, flags & ~(unsigned)WINO_FLAG_POOL2, bias, g, x, w, tmp, st);
    if (rc) return rc;
    DISPATCH_DTYPE(dtype, launch_pool2_t<T>(dst, g, tmp, y, st));
}

int pick_algo(int layout, int dtype, const Geometry& g) {
    const long patches = ((g.P + GO_T - 1) / GO_T) * ((g.K + GO_T - 1) / GO_T);
    const bool nhwc = layout == WINO_NHWC;
    // the single-kernel path addresses the input with 32-bit byte offsets
    const bool fused_ok = (long)g.N * g.C * g.H * g.W * (long)dtype_size(dtype) < (1L << 32);
    if (dtype == WINO_F32) {
        // (a short reduction into one filter tile runs best as the single kernel from 64 patches on:
        // N = 8, C = K = 64, H = 56, 98 patches: 0.038 against 0.044 ms)
        if (patches >= 64 && g.C <= 64 && g.K <= 64 && fused_ok) return WINO_ALGO_FUSED;
        if (patches < 128) return WINO_ALGO_STAGED;      // a 64x64 patch for every other CU at most
        // few channels: V would be 4x the input and is consumed by few filter tiles -- build it in the kernel.
        // With one filter tile (K <= 64) no tile is transformed twice, whatever C (C = 256, K = 64, H = 56:
        // 0.185 against 0.233 ms); with two, the single kernel needs many patches to win (C = K = 128: 196
        // patches 0.067 against 0.062 ms for EPILOGUE, 392 a tie, 12544 0.57 against 0.63)
        // (and past C = 256: C = 384, K = 64, N = 8, H = 112: 0.27 against 0.35 and 0.46 ms for the other two; C = 512,
        // K = 32, N = 32, H = 56: 0.35 against 0.47 and 0.59)
        if (fused_ok && g.K <= 64) return WINO_ALGO_FUSED;
        if (g.C <= 128 && g.K <= 128) return (fused_ok && patches >= 512) ? WINO_ALGO_FUSED : WINO_ALGO_EPILOGUE;
        if (patches < 256) return WINO_ALGO_STAGED;      // not even one 64x64 patch per CU
        if (g.C <= 256) return WINO_ALGO_EPILOGUE;
        // many channels: the 128x128 GEMM's lower L2 traffic per flop wins, unless there are few tiles or the
        // 64x64 patches fill their rounds of 512 resident workgroups (a small last round is cut up, see
        // launch_gemm_rows_t)
        const long slots = rows_slots(WINO_F32), rem = patches % slots;
        const bool full_rounds = patches > slots && (rem == 0 || 5 * rem <= 3 * slots);
        return (g.P <= 4096 || full_rounds) ? WINO_ALGO_EPILOGUE : WINO_ALGO_STAGED;
    }
    // 16-bit operands: the fp32 product tensor is the largest HBM stream, so STAGED only for tiny problems;
    // the in-kernel input transform is VALU work repeated per filter tile and pays only with few filter
    // tiles and cheap loads (channel vectors for NHWC, which need C % 8 == 0)
    // (the last of these with more than one filter tile only: C = 512, K = 16 .. 64, N = 16, H = 56, 196 patches: EPILOGUE
    // takes 92 to 107 us where STAGED takes 142 to 150)
    if (patches < 64 || (g.C >= 256 && patches < 128) || (g.C >= 512 && g.K > 64 && patches < 256)) return WINO_ALGO_STAGED;
    if (!fused_ok) return WINO_ALGO_EPILOGUE;
    if (nhwc) {
        // (one filter tile: any C up to 256; two: only with many patches -- C = K = 128 at 196 patches is 6 % behind EPILOGUE)
        // (a sweep of 720 bf16 NHWC layers: with one filter tile the single kernel wins at any C once there are some 400
        // patches -- C = 512, K = 32, N = 16, H = 80: 125 against 233 us -- and from C = 8 on; with fewer patches and more
        // than 64 channels it is 1.2 to 1.5 times behind -- C = 192, K = 16, N = 8, H = 48: 1.49)
        if (g.C >= 8 && g.K <= 64 && (g.C <= 64 || patches >= 384)) return WINO_ALGO_FUSED;
        if (g.C >= 16 && g.C <= 128 && g.K <= 128 && patches >= 1024) return WINO_ALGO_FUSED;
    } else if (g.C <= 64 && g.K <= 64 && patches >= 1536) {   // (fewer patches: measured behind EPILOGUE)
        return WINO_ALGO_FUSED;
    } else if (g.C >= 384 && g.K <= 64 && patches >= 384) {   // (CHWN, C = 384, K = 64, N = 32, H = 56: 1.35 times faster than EPILOGUE)
        return WINO_ALGO_FUSED;
    }
    return WINO_ALGO_EPILOGUE;
}

// Where AUTO leaves the Winograd kernels: layers with C <= 4 (direct.hpp), and 2-byte NCHW layers with large images
// and enough tiles for the whole chip (direct16.hpp, direct16_rows.hpp; measured on the VGG-16 shapes at N = 32 in
// bf16, direct against the fastest Winograd pipeline: 175 against 373 us at C = K = 64, H = 224; 138 against 245 us
// at C = K = 128, H = 112; 130 against 164 us at C = K = 256, H = 56; 75 against 79 and 127 against 135 us for the
// two 28 x 28 shapes, which only the 8-wave kernel wins; at 14 x 14 the Winograd pipelines are faster, 55 against
// 98 us; NHWC tensors, 8-wave kernel only: 236 against 462, 92 against 150, 143 against 257, 73 against 96, 122
// against 170, 68 against 79, 117 against 133 us).  x, y: the tensors if known (their alignment decides: with an NHWC
// side only the 8-wave kernel runs, and it stores 4-byte pairs unless it pools).
bool direct16_chwn_pool_ok(int src, int dst, int dtype, unsigned flags, const Geometry& g);
bool auto_direct16(int src, int dst, int dtype, unsigned flags, const Geometry& g, const void* x, const void* y) {
    // (a pooled CHWN layer runs unpooled into scratch, then a pooling kernel: N = 32 in bf16, direct + pooling against the
    // fastest Winograd pipeline with pooling in its output stage: 183 + 46 against 528 us at C = K = 64, H = 224)
    if (direct16_chwn_pool_ok(src, dst, dtype, flags, g)) return auto_direct16(src, dst, dtype, flags & ~(unsigned)WINO_FLAG_POOL2, g, x, nullptr);
    if (!direct16_ok(src, dst, dtype, flags, g) || misaligned(x, src == WINO_NHWC ? 16 : 4)) return false;
    if ((src == WINO_NHWC || dst == WINO_NHWC) && !(flags & WINO_FLAG_POOL2) && misaligned(y, 4)) return false;
    D16Geom d;
    if (src == WINO_CHWN) {                    // (both sides, direct16_ok has checked; the 8-wave kernel only)
        if (misaligned(y, 4)) return false;
        const bool planc = direct16_rows_wf(g) == 2 ? direct16_rows_plan<2, true>(g, &d) : direct16_rows_plan<1, true>(g, &d);
        // (measured at N = 32 in bf16, direct against the fastest Winograd pipeline: 177 against 532 us at C = K = 64,
        // H = 224; 140 against 307 at C = K = 128, H = 112; 73 against 91 and 130 against 183 at 56 x 56; at 28 x 28 the
        // 7 x 7 blocks of a filter tile leave a quarter of the chip idle: 121 against 72, 225 against 128 us)
        // (fewer than 64 channels, which the network does not have: C = 8 .. 32, K = 128 and 256, 56 x 56 to 112 x 112: 0.53
        // to 0.81 of the fastest Winograd pipeline's time)
        return planc && g.Ho >= 48 && g.Wo >= 48 && 4L * d.rowBlocks * d.colBlocks * d.kTiles >= 3L * device_cus();
    }
    const bool plan8 = direct16_rows_wf(g) == 2 ? direct16_rows_plan<2>(g, &d, src == WINO_NHWC) : direct16_rows_plan<1>(g, &d, src == WINO_NHWC);
    // (with an NHWC side and fewer than 64 channels, C = 8 .. 32: 0.45 to 0.83 of the fastest Winograd pipeline's time)
    if (plan8 && g.Ho >= 28 && g.Wo >= 28 && (g.C >= 64 || src == WINO_NHWC || dst == WINO_NHWC) &&
        4L * d.rowBlocks * d.colBlocks * d.kTiles >= 3L * device_cus())
        return true;
    // (the general kernel: a sweep of 780 bf16 NCHW layers, C = 8 .. 512, K = 16 .. 256, 28 x 28 to 224 x 224, N = 1 .. 32,
    // against the fastest Winograd pipeline: it wins on 85 % of them, by 1.28 in the geometric mean; it loses where few
    // tiles each carry a long reduction for two filter tiles one after the other -- N = 8, C = 512, K = 96, H = 48, 96
    // tiles: 94 against 53 us -- so: a tile for every CU, or one filter tile, or a short reduction)
    if (src == WINO_NHWC || dst == WINO_NHWC || g.Ho < 28 || g.Wo < 28) return false;
    const long tiles = ((long)g.N * g.Ho + 15) / 16 * ((g.Wo + 31) / 32) * ((g.K + D16_KT - 1) / D16_KT);
    // (N = 1, C = 128, K = 96, H = 56, 16 tiles: 30 against 21 us; N = 1, C = 512, K = 64, 8 tiles: 44 against 29)
    return tiles >= device_cus() || (g.K <= D16_KT && (tiles >= 32 || g.C <= 128)) || g.C <= 64 || (g.C <= 128 && tiles >= 64);
}
// Small fp32 layers go to the one-launch direct kernel while its cost stays small: a round of the chip costs a fixed
// part (the first group's trip to memory, the sum over the waves, the stores) and a part per group of 32 channels.
// Measured against the fastest Winograd pipeline with the bank read in 16-byte pieces (times of calls issued one
// by one from Python, about 5 us above back-to-back launches; (rounds, groups)): N = 1, C = K = 64, H = 56 (1, 2):
// 13.5 against 19.8 us, from NHWC 12.1 against 19.9; N = 2 (2, 2): 16.8 against 23.1; N = 4 (4, 2): 29.6 against
// 29.9, NHWC 25.3 against 26.8; N = 1, C = K = 128, H = 22 (1, 4): 13.2 against 18.6; N = 4 (2, 4): 23.5 against
// 23.4; N = 8 (3, 4): 33.5 against 28.0; N = 4, C = K = 256, H = 14 (1, 8): 22.4 against 27.0, NHWC 26.0 against
// 25.5; N = 8 (2, 8): 41.0 against 30.7; N = 1, C = K = 512, H = 7 (1, 16): 33.1 against 29.4; N = 8, C = K = 32,
// H = 56 (4, 1): 22.1 against 27.8.  With one element per load (C not a multiple of 4) the kernel takes about twice
// as long per group: N = 2, C = K = 64, H = 56 (2, 2): 32 against 22; N = 1, C = K = 128, H = 22: 26 against 19.
bool auto_direct_few(int src, int dtype, unsigned flags, const Geometry& g) {
    if (!direct_few_ok(dtype, flags, g) || g.C <= 4) return false;          // (at most four channels: the kernels above, or none)
    const long rounds = (direct_few_units(g) + device_cus() - 1) / device_cus(), groups = (g.C + 31) / 32;
    // (a sweep of 560 shapes, NCHW, against the fastest pipeline: at rounds x (1 + groups) = 12 the kernel takes 0.59 to
    // 0.98 of its time, at 14 and 16 with at most 64 filters 0.60 to 0.99; at 17 and more, or 15 with 128 filters, it loses)
    const long cost = rounds * (1 + groups);
    // (one tile of 32 filters: up to 34 -- N = 64, C = 512, K = 16, H = 14: 66 against 94 us -- with 1.07 the worst ratio.
    // The two wider offers hold for NCHW tensors only: from NHWC and CHWN the kernel is slower and F(4x4) wins there --
    // NHWC, N = 4, C = 96, K = 64, H = 56, cost 16: 35 against 28 us; CHWN, N = 32, C = 192, K = 32, H = 28, cost 28: 72 against 51)
    const int mode = direct_few_filter_mode(src, g);
    if (mode == 0) return rounds * groups <= 2;
    return cost <= 12 || (mode == 1 && ((cost <= 16 && g.K <= 64) || (cost <= 34 && g.K <= 32)));
}
// fp32 layers with a long reduction and enough 4x4 tiles run faster through the F(4x4,3x3) pipeline, product tensor
// and all: 2.25 multiplies per output instead of 4, and a transformed input of 2.25x the tensor instead of 4x.
// Measured at N = 32, NCHW, against the fastest F(2x2) pipeline: C = K = 256, H = 56: 0.37 against 0.54 ms;
// C = 256, K = 512, H = 28: 0.19 against 0.28; C = K = 512, H = 28: 0.34 against 0.52; C = K = 512, H = 14 (512
// tiles): 0.13 against 0.17; C = 128, K = 256, H = 56: 0.24 against 0.28; C = K = 128, H = 112: 0.52 against 0.57
// (the single-kernel path); C = K = 128, H = 56: 0.14 against 0.18; C = 64, K = 128, H = 112: 0.36 against 0.31.
// (NHWC: 0.40 against 0.53 on the first of these, CHWN 0.38 against 0.52.)  Its rounding error is about four times
// that of F(2x2) (3e-6 to 5e-6 relative L2 on these layers).
// Beyond those shapes (sweeps of 680 layers with C = 8 .. 512, K = 16 .. 512, 7 x 7 to 160 x 160, N = 1 .. 64, NCHW,
// every pipeline by name; F(4x4) against the fastest F(2x2) pipeline):
//   * more than one filter tile (K > 64) and C >= 96: F(4x4) takes 0.69 to 0.95 of the time at every size measured
//     (C = 128, K = 96, N = 32, H = 112: 0.47 against 0.55 ms; C = 192, K = 96, N = 16, H = 80: 0.18 against 0.26);
//   * K > 64 and 48 <= C < 96: it wins while V and the product together stay inside the 256 MB last-level cache
//     (C = 64, K = 128, N = 32, H = 56, 177 MB: 0.085 against 0.107 ms) and loses beyond (N = 32, H = 112, 694 MB:
//     0.36 against 0.31);
//   * one filter tile (K <= 64): the single kernel transforms no tile twice and wins from about 400 patches on
//     whatever C (C = 192, K = 64, N = 32, H = 80: 0.26 against 0.31 ms); with fewer patches it leaves the chip half
//     empty and F(4x4) wins from C = 96 (C = 192, K = 64, N = 4, H = 80: 0.056 against 0.082).
bool auto_f4(int dtype, const Geometry& g) {
    if (dtype != WINO_F32) return false;
    const long tiles4 = (long)g.N * ((g.Ho + 3) / 4) * ((g.Wo + 3) / 4);
    if (tiles4 < 512) return false;
    // (14 x 14 images fill 16 x 16 outputs of 4x4 tiles, 1.31 times the work: below C = 192 the F(2x2) pipelines keep such
    // layers -- N = 64, C = K = 128, H = 14: 45 against 42 us; C = 64, K = 128: 39 against 34)
    if (16L * ((g.Ho + 3) / 4) * ((g.Wo + 3) / 4) * 4 > 5L * g.Ho * g.Wo && g.C < 192) return false;
    if (g.C >= 128 && g.K >= 128) return true;
    if (g.K > 64) return g.C >= 96 || (g.C >= 48 && 36.0 * (double)tiles4 * (g.C + g.K) * 4 <= 256e6);
    const long patches = (g.P + GO_T - 1) / GO_T;                            // (one filter tile)
    return g.C >= 96 && patches <= 256;
}
int resolve_auto(int src, int dst, int dtype, unsigned flags, const Geometry& g, const void* x, const void* y, bool have_w) {
    // (a pooled layer of at most four channels: direct into scratch, then pooling -- the network's first layer shape with
    // pooling, N = 32: bf16 NCHW 59 + 31 us against 242 for the Winograd pipeline that pools in its output stage)
    // (its workgroups take 128 pixels and every filter tile in turn: with a workgroup for every other CU at most and many filters the
    // Winograd pipelines spread the work better -- N = 1, C = 3, K = 256, H = 112: 45 against 24 us; N = 8, K = 128, H = 20: 28
    // against 19; K = 96: a tie)
    const bool few_wide = (long)g.N * g.Ho * g.Wo < 64L * device_cus() && g.K >= 128;
    if (have_w && !few_wide && (direct_ok(dst, flags, g) || direct_pooled_ok(dst, flags, g))) return WINO_ALGO_DIRECT;
    if (have_w && auto_direct16(src, dst, dtype, flags, g, x, y)) return WINO_ALGO_DIRECT;
    if (have_w && auto_direct_few(src, dtype, flags, g)) return WINO_ALGO_DIRECT;
    if (have_w && auto_f4(dtype, g)) return WINO_ALGO_STAGED_F4;
    const int algo = pick_algo(src, dtype, g);
    return algo == WINO_ALGO_FUSED && g.pad > 1 ? WINO_ALGO_EPILOGUE : algo;   // the single kernel masks one ring of padding
}

int conv_f4_impl(const ScratchSource& ss, int src, int dst, int dtype, int algo, unsigned flags, const void* bias, int N, int C,
                 int K, int H, int W, int pad, const void* x, const void* w, const void* Upre, void* y, void* stream) {
    Geometry g;
    if (!make_geometry(dtype, N, C, K, H, W, pad, &g, 4))
        return fail(WINO_ERR_INVALID, "bad shape N=%d C=%d K=%d H=%d W=%d pad=%d", N, C, K, H, W, pad);
    hipStream_t st = (hipStream_t)stream;
    F4RowsPlan plan;
    if (algo == WINO_ALGO_EPILOGUE_F4 && !f4_rows_plan(dtype, g, &plan))
        return fail(WINO_ERR_UNSUPPORTED, "the F(4x4) pipeline with the output transform in the GEMM is built for fp32 tensors");
    const Scratch sc = scratch_layout(g, dtype, algo);
    void* base = nullptr;
    int rc = ss.get(sc.total, &base);
    if (rc) return rc;
    char* b = (char*)base;
    void* U = b + sc.u_off;
    void* V = b + sc.v_off;
    float* Mo = (float*)(b + sc.m_off);
    const int order = tile_order_for(src, dst);
    const int porder = dst == WINO_NHWC ? WINO_PRODUCT_PK : WINO_PRODUCT_KP;
    // the filter transform rides in the input transform's launch, unless the stages are being timed one by one
    const bool ride = !Upre && !g_timing;
    if (Upre) {
        U = const_cast<void*>(Upre);
    } else if (!ride) {
        StageScope t(WINO_STAGE_FILTER, st);
        rc = wino_f4_filter_transform(src, dtype, K, C, w, U, stream);
        if (rc) return rc;
    }
    {
        StageScope t(WINO_STAGE_INPUT, st);
        const FilterJob fj = ride ? FilterJob{w, U, flt_strides(src, K, C), K, C, g.Kp, g.Cp} : FilterJob{};
        DISPATCH_DTYPE_RC(rc, dtype, launch_f4_input<T>(src, order, g, x, V, st, fj));
        if (rc) return rc;
    }
    if (algo == WINO_ALGO_EPILOGUE_F4) {
        StageScope t(WINO_STAGE_GEMM, st);
        return launch_f4_gemm_rows(dst, order, flags, bias, g, plan, U, V, y, Mo, (int*)base, st);   // (the product region holds the partial outputs)
    }
    {
        StageScope t(WINO_STAGE_GEMM, st);
        rc = launch_gemm(36, dtype, porder, g.Cp, g.Kp, g.Pp, U, V, Mo, st);
        if (rc) return rc;
    }
    StageScope t(WINO_STAGE_OUTPUT, st);
    DISPATCH_DTYPE(dtype, launch_f4_output<T>(dst, order, porder, flags, bias, N, K, g.Ho, g.Wo, g.Kp, g.P, g.Pp, Mo, y, st));
}

// Images per pass of a pooled layer of at most four channels (0: no room).  The unpooled tensor of a pass stays under
// 224 MB, so that the last-level cache still holds it when the pooling kernel reads it (fp32, N = 32, 64 filters at
// 224 x 224, 411 MB unpooled: 236 us in one pass, 179 in two; NHWC 256 and 204), and inside a fixed scratch buffer.
// CHWN tensors are not cut: their images are the contiguous axis.
int direct_pooled_images(const ScratchSource& ss, int src, int dst, int dtype, const Geometry& g) {
    if (src == WINO_CHWN || dst == WINO_CHWN)
        return !ss.fixed || kCounterBytes + direct16_unpooled_bytes(dtype, g) <= ss.fixed_bytes ? g.N : 0;
    const size_t img = (size_t)g.K * g.Ho * g.Wo * dtype_size(dtype);
    size_t lim = (size_t)224 << 20;
    if (ss.fixed) lim = std::min(lim, ss.fixed_bytes > kCounterBytes + 256 ? ss.fixed_bytes - kCounterBytes - 256 : 0);
    long fit = (long)(lim / img);
    if (fit < 1 && !ss.fixed) fit = 1;
    if (fit < 1) return 0;
    const long passes = (g.N + fit - 1) / fit;
    return (int)((g.N + passes - 1) / passes);
}

// What the automatic choice runs when its first choice does not fit a fixed scratch buffer: a pooled CHWN layer and a
// pooled layer of at most four channels on the direct path keep the unpooled tensor in scratch, the F(4x4) pipeline its
// transformed input and product; without room for them the F(2x2) pipelines take the layer, the single kernel last.
int auto_within(const ScratchSource& ss, int algo, int src, int dst, int dtype, unsigned flags, const Geometry& g) {
    if (!ss.fixed) return algo;
    bool refit = false;
    if (algo == WINO_ALGO_DIRECT)
        refit = (direct16_chwn_pool_ok(src, dst, dtype, flags, g) &&
                 kCounterBytes + (direct16_bank_bytes(g) + 255) / 256 * 256 + direct16_unpooled_bytes(dtype, g) > ss.fixed_bytes) ||
                (direct_pooled_ok(dst, flags, g) && direct_pooled_images(ss, src, dst, dtype, g) == 0);
    if (algo == WINO_ALGO_STAGED_F4) {                                        // (V and the product of the 36 coordinates)
        Geometry g4;
        refit = !make_geometry(dtype, g.N, g.C, g.K, g.H, g.W, g.pad, &g4, 4) || scratch_layout(g4, dtype, algo).total > ss.fixed_bytes;
    }
    if (refit) {
        algo = pick_algo(src, dtype, g);
        // (the single kernel keeps only the transformed filters in scratch: it runs where the others' tensors do not fit)
        if (algo != WINO_ALGO_FUSED && g.pad <= 1 && scratch_layout(g, dtype, algo).total > ss.fixed_bytes &&
            (long)g.N * g.C * g.H * g.W * (long)dtype_size(dtype) < (1L << 32))
            algo = WINO_ALGO_FUSED;
        if (algo == WINO_ALGO_FUSED && g.pad > 1) algo = WINO_ALGO_EPILOGUE;
    }
    return algo;
}

int conv_pass(const ScratchSource& ss, int src, int dst, int dtype, int algo, unsigned flags, int N, int C, int K, int H,
              int W, int pad, const void* x, const void* w, const void* Upre, const void* bias, void* y, void* stream) {
    if (!valid_layout(src) || !valid_layout(dst)) return fail(WINO_ERR_INVALID, "unknown layout %d -> %d", src, dst);
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    if (algo < WINO_ALGO_AUTO || algo > WINO_ALGO_EPILOGUE_F4) return fail(WINO_ERR_INVALID, "unknown algo %d", algo);
    if (!x || (!w && !Upre) || !y) return fail(WINO_ERR_INVALID, "null tensor pointer");
    if (misaligned(x, elem_bytes(dtype)) || misaligned(w, elem_bytes(dtype)) || misaligned(y, elem_bytes(dtype)) ||
        misaligned(bias, elem_bytes(dtype)))
        return fail(WINO_ERR_INVALID, "tensor pointer not aligned to its element size");
    if (misaligned(Upre, 16)) return fail(WINO_ERR_INVALID, "transformed filters must be 16-byte aligned");
    Geometry g;
    if (!make_geometry(dtype, N, C, K, H, W, pad, &g))
        return fail(WINO_ERR_INVALID, "bad shape N=%d C=%d K=%d H=%d W=%d pad=%d", N, C, K, H, W, pad);
    if (flags & ~(unsigned)(WINO_FLAG_RELU | WINO_FLAG_POOL2)) return fail(WINO_ERR_INVALID, "unknown flags 0x%x", flags);
    if ((flags & WINO_FLAG_POOL2) && (g.Ho < 2 || g.Wo < 2))
        return fail(WINO_ERR_INVALID, "2x2 pooling of a %dx%d output", g.Ho, g.Wo);
    if (algo == WINO_ALGO_AUTO) {
        algo = resolve_auto(src, dst, dtype, flags, g, x, y, w != nullptr);
        if (algo == WINO_ALGO_STAGED_F4 || algo == WINO_ALGO_EPILOGUE_F4) Upre = nullptr;      // transformed filters handed in alongside w are F(2x2) ones
        algo = auto_within(ss, algo, src, dst, dtype, flags, g);
    }
    if (algo == WINO_ALGO_DIRECT) {
        if (!w) return fail(WINO_ERR_INVALID, "the direct path needs the filter bank, not its Winograd transform");
        if (direct_ok(dst, flags, g)) {
            StageScope t(WINO_STAGE_GEMM, (hipStream_t)stream);
            return launch_direct(src, dst, dtype, flags, bias, g, x, w, y, (hipStream_t)stream);
        }
        if (direct_pooled_ok(dst, flags, g)) {
            const int per = direct_pooled_images(ss, src, dst, dtype, g);
            if (per == 0) return fail(WINO_ERR_WORKSPACE, "an image of this layer unpooled does not fit the scratch buffer");
            Geometry gp;
            make_geometry(dtype, per, C, K, H, W, pad, &gp);
            void* base = nullptr;
            const int rcb = ss.get(kCounterBytes + direct16_unpooled_bytes(dtype, gp), &base);
            if (rcb) return rcb;
            StageScope t(WINO_STAGE_GEMM, (hipStream_t)stream);
            const size_t es = dtype_size(dtype), x_img = (size_t)C * H * W * es, y_img = (size_t)K * (g.Ho / 2) * (g.Wo / 2) * es;
            for (int n0 = 0; n0 < g.N; n0 += per) {
                make_geometry(dtype, std::min(per, g.N - n0), C, K, H, W, pad, &gp);
                const int rc = launch_direct_pooled(src, dst, dtype, flags, bias, gp, (const char*)x + n0 * x_img, w, (char*)base + kCounterBytes,
                                                    (char*)y + n0 * y_img, (hipStream_t)stream);
                if (rc) return rc;
            }
            return WINO_OK;
        }
        if (direct_few_ok(dtype, flags, g)) {
            StageScope t(WINO_STAGE_GEMM, (hipStream_t)stream);
            return launch_direct_few(src, dst, flags, bias, g, x, w, y, (hipStream_t)stream);
        }
        if (direct16_chwn_pool_ok(src, dst, dtype, flags, g)) {
            const size_t bank = (direct16_bank_bytes(g) + 255) / 256 * 256;
            void* base = nullptr;
            const int rcb = ss.get(kCounterBytes + bank + direct16_unpooled_bytes(dtype, g), &base);
            if (rcb) return rcb;
            StageScope t(WINO_STAGE_GEMM, (hipStream_t)stream);
            return launch_direct16_chwn_pooled(dtype, flags, bias, g, x, w, (char*)base + kCounterBytes, (char*)base + kCounterBytes + bank, y,
                                               (hipStream_t)stream, D16_PACK_RUN);
        }
        if (!direct16_ok(src, dst, dtype, flags, g))
            return fail(WINO_ERR_UNSUPPORTED, "the direct path is built for pad 0 and 1: for C <= 4, and for 2-byte NCHW tensors with "
                                              "C a multiple of 8 and an even width (pooling: output height a multiple of 4, K a multiple of 64, a large layer)");
        void* base = nullptr;
        const int rcb = ss.get(kCounterBytes + direct16_bank_bytes(g), &base);
        if (rcb) return rcb;
        StageScope t(WINO_STAGE_GEMM, (hipStream_t)stream);
        return launch_direct16(src, dst, dtype, flags, bias, g, x, w, (char*)base + kCounterBytes, y, (hipStream_t)stream);
    }
    if (algo == WINO_ALGO_STAGED_F4 || algo == WINO_ALGO_EPILOGUE_F4)
        return conv_f4_impl(ss, src, dst, dtype, algo, flags, bias, N, C, K, H, W, pad, x, w, Upre, y, stream);

    hipStream_t st = (hipStream_t)stream;
    const Scratch sc = scratch_layout(g, dtype, algo);
    void* base = nullptr;
    int rc = ss.get(sc.total, &base);
    if (rc) return rc;
    char* b = (char*)base;
    void* U = b + sc.u_off;
    void* V = b + sc.v_off;
    float* Mo = (float*)(b + sc.m_off);
    const int order = tile_order_for(src, dst);

    // The filter transform rides in the input transform's launch (a launch of its own costs as much as its few
    // microseconds of work); with stage timing on it stays a launch of its own, so that its span can be measured.
    const bool ride = !Upre && algo != WINO_ALGO_FUSED && !g_timing;
    if (Upre) {
        U = const_cast<void*>(Upre);
    } else if (!ride) {
        StageScope t(WINO_STAGE_FILTER, st);
        rc = wino_filter_transform(src, dtype, K, C, w, U, stream);
        if (rc) return rc;
    }
    if (algo == WINO_ALGO_FUSED) {
        if (g.pad > 1) return fail(WINO_ERR_UNSUPPORTED, "the single-kernel path is built for pad 0 and 1 (pad=%d)", g.pad);
        StageScope t(WINO_STAGE_GEMM, st);
        return launch_fused(src, dst, dtype, order, flags, bias, g, x, U, y, st);
    }
    {
        StageScope t(WINO_STAGE_INPUT, st);
        const FilterJob fj = ride ? FilterJob{w, U, flt_strides(src, K, C), K, C, g.Kp, g.Cp} : FilterJob{};
        DISPATCH_DTYPE_RC(rc, dtype, launch_input_transform<T>(src, order, g, x, V, st, fj));
        if (rc) return rc;
    }
    if (algo == WINO_ALGO_EPILOGUE) {
        StageScope t(WINO_STAGE_GEMM, st);
        TailScratch ts;
        ts.part = Mo;                                 // the product region is free in this pipeline
        ts.part_bytes = sc.total - sc.m_off;
        ts.cnt = (int*)base;
        return launch_gemm_out(dst, dtype, order, flags, bias, g, U, V, y, ts, st);
    }
    const int porder = dst == WINO_NHWC ? WINO_PRODUCT_PK : WINO_PRODUCT_KP;
    const int splits = gemm_splits(dtype, g.Cp, g.Kp, g.Pp);
    {
        StageScope t(WINO_STAGE_GEMM, st);
        rc = launch_gemm(16, dtype, porder, g.Cp, g.Kp, g.Pp, U, V, Mo, st, splits);
        if (rc) return rc;
    }
    StageScope t(WINO_STAGE_OUTPUT, st);
    DISPATCH_DTYPE(dtype, launch_output_transform<T>(dst, order, porder, flags, bias, N, K, g.Ho, g.Wo, g.Kp, g.P, g.Pp, Mo, y, st, splits));
}

__global__ void warmup_kernel() {}

// ---- scratch of the entry point that allocates nothing --------------------------------------------
// The file-scope array `scratch` is laid out like the arena: arrival counters first, then U, V and the product or
// partial sums.  Host code never uses the array's name as an address: each device's copy is looked up once
// (noalloc_scratch) and that pointer is what kernels and the fill below receive.
constexpr size_t kNoAllocBytes = WINO_NOALLOC_SCRATCH_BYTES;
void* g_noalloc_ptr[kMaxDevices] = {};
std::mutex g_noalloc_mu;

// The current device's copy of `scratch`.  Nothing is cleared here: the array is a zero-initialised object of the
// device image, the only part of it that must be zero when a kernel starts is the arrival counters at its head,
// and every kernel that counts arrivals returns its counters to zero before it ends.
int noalloc_scratch(void** out) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(WINO_ERR_UNSUPPORTED, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lk(g_noalloc_mu);
    if (!g_noalloc_ptr[dev]) {
        void* ptr = nullptr;
        HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr || misaligned(ptr, 256)) return fail(WINO_ERR_HIP, "built-in scratch buffer not found on device %d", dev);
        g_noalloc_ptr[dev] = ptr;
    }
    *out = g_noalloc_ptr[dev];
    return WINO_OK;
}

// How many passes over the batch a layer call makes.  The epilogue pipeline of a 2-byte layer is bound by memory
// on both sides of V (written by the input transform, read by the GEMM); when V is much larger than the 256 MB
// last-level cache, running the two kernels on one part of the batch after the other lets the GEMM find V still
// cached and the next pass overwrite the same addresses.  Batch-major tensors only (a part of the batch is then a
// contiguous slice of x, V and y).  Measured (bf16, N=32, NCHW): C=K=128, H=112 (V 411 MB) 280 us in one pass,
// 236 in two, 253 in three; C=64, K=128, H=112 (205 MB) 158 -> 143 in two; C=K=256, H=56 (205 MB, but only 1568
// workgroups) 166 -> 172 in two: a pass aims at 105 MB of V and keeps at least ~1500 GEMM workgroups (two rounds
// of the chip).
int batch_passes(int src, int dst, int dtype, int algo, const Geometry& g) {
    if (algo != WINO_ALGO_EPILOGUE || dtype == WINO_F32 || src == WINO_CHWN || dst == WINO_CHWN) return 1;
    const double v_bytes = 16.0 * (double)g.P * g.Cp * dtype_size(dtype);
    const long wgs = ((g.P + GO_T - 1) / GO_T) * ((g.K + GO_T - 1) / GO_T);
    const long by_cache = (long)(v_bytes / 105e6 + 0.5), by_work = wgs / 1500;
    return (int)std::max(1L, std::min<long>(g.N, std::min(by_cache, by_work)));
}

int conv_impl(const ScratchSource& ss, int src, int dst, int dtype, int algo, unsigned flags, int N, int C, int K, int H,
              int W, int pad, const void* x, const void* w, const void* Upre, const void* bias, void* y, void* stream) {
    Geometry g;
    int passes = 1;
    if (valid_layout(src) && valid_layout(dst) && valid_dtype(dtype) && x && y && (w || Upre) &&
        make_geometry(dtype, N, C, K, H, W, pad, &g) && algo >= WINO_ALGO_AUTO && algo <= WINO_ALGO_EPILOGUE_F4) {
        if (algo == WINO_ALGO_AUTO) {
            algo = resolve_auto(src, dst, dtype, flags, g, x, y, w != nullptr);
            if (algo == WINO_ALGO_STAGED_F4 || algo == WINO_ALGO_EPILOGUE_F4) Upre = nullptr;  // transformed filters handed in alongside w are F(2x2) ones
            algo = auto_within(ss, algo, src, dst, dtype, flags, g);
        }
        passes = batch_passes(src, dst, dtype, algo, g);
    }
    if (passes <= 1) return conv_pass(ss, src, dst, dtype, algo, flags, N, C, K, H, W, pad, x, w, Upre, bias, y, stream);
    const size_t es = dtype_size(dtype);
    const size_t x_img = (size_t)C * H * W * es;
    const size_t y_img = (size_t)K * ((flags & WINO_FLAG_POOL2) ? (size_t)(g.Ho / 2) * (g.Wo / 2) : (size_t)g.Ho * g.Wo) * es;
    const int per = (N + passes - 1) / passes;
    for (int n0 = 0; n0 < N; n0 += per) {
        const int nn = std::min(per, N - n0);
        const int rc = conv_pass(ss, src, dst, dtype, algo, flags, nn, C, K, H, W, pad, (const char*)x + n0 * x_img,
                                 Upre ? nullptr : w, Upre, bias, (char*)y + n0 * y_img, stream);
        if (rc) return rc;
        if (!Upre) {
            // the first pass left the transformed filters at the head of the arena; the later ones reuse them
            Geometry gp;
            make_geometry(dtype, nn, C, K, H, W, pad, &gp);
            void* base = nullptr;
            const Scratch scp = scratch_layout(gp, dtype, algo);
            const int rc2 = ss.get(scp.total, &base);
            if (rc2) return rc2;
            Upre = (char*)base + scp.u_off;
        }
    }
    return WINO_OK;
}

}  // namespace

extern "C" {
int wino_conv(int src, int dst, int dtype, int algo, unsigned flags, int N, int C, int K, int H, int W, int pad,
              const void* x, const void* w, void* y, void* stream) {
    if (!w) return fail(WINO_ERR_INVALID, "null filter pointer");
    return conv_impl(ScratchSource{}, src, dst, dtype, algo, flags, N, C, K, H, W, pad, x, w, nullptr, nullptr, y, stream);
}
int wino_conv_ex(int src, int dst, int dtype, int algo, unsigned flags, int N, int C, int K, int H, int W, int pad,
                 const void* x, const void* w, const void* bias, void* y, void* stream) {
    if (!w) return fail(WINO_ERR_INVALID, "null filter pointer");
    return conv_impl(ScratchSource{}, src, dst, dtype, algo, flags, N, C, K, H, W, pad, x, w, nullptr, bias, y, stream);
}

int wino_conv_prepared(int src, int dst, int dtype, int algo, unsigned flags, int N, int C, int K, int H, int W,
                       int pad, const void* x, const void* U, void* y, void* stream) {
    if (!U) return fail(WINO_ERR_INVALID, "null transformed-filter pointer");
    return conv_impl(ScratchSource{}, src, dst, dtype, algo, flags, N, C, K, H, W, pad, x, nullptr, U, nullptr, y, stream);
}
int wino_conv_prepared_ex(int src, int dst, int dtype, int algo, unsigned flags, int N, int C, int K, int H, int W,
                          int pad, const void* x, const void* U, const void* bias, void* y, void* stream) {
    if (!U) return fail(WINO_ERR_INVALID, "null transformed-filter pointer");
    return conv_impl(ScratchSource{}, src, dst, dtype, algo, flags, N, C, K, H, W, pad, x, nullptr, U, bias, y, stream);
}

int wino_conv_noalloc(int src, int dst, int dtype, int algo, unsigned flags, int N, int C, int K, int H, int W, int pad,
                      const void* x, const void* w, const void* bias, void* y, void* stream) {
    if (!w) return fail(WINO_ERR_INVALID, "null filter pointer");
    struct NoTiming {                          // stage timing creates events: not in this call
        NoTiming() { t_no_timing = true; }
        ~NoTiming() { t_no_timing = false; }
    } guard;
    ScratchSource ss;
    const int rc = noalloc_scratch(&ss.fixed);
    if (rc) return rc;
    ss.fixed_bytes = kNoAllocBytes;
    return conv_impl(ss, src, dst, dtype, algo, flags, N, C, K, H, W, pad, x, w, nullptr, bias, y, stream);
}

int wino_pick_algo(int layout, int dtype, int N, int C, int K, int H, int W, int pad) {
    if (!valid_layout(layout)) return fail(WINO_ERR_INVALID, "unknown layout %d", layout);
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    Geometry g;
    if (!make_geometry(dtype, N, C, K, H, W, pad, &g))
        return fail(WINO_ERR_INVALID, "bad shape N=%d C=%d K=%d H=%d W=%d pad=%d", N, C, K, H, W, pad);
    return resolve_auto(layout, layout, dtype, 0, g, nullptr, nullptr, true);
}

int wino_geometry(int dtype, int N, int C, int K, int H, int W, int pad, int* th, int* tw, long* P, int* Cp, int* Kp,
                  long* Pp) {
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    Geometry g;
    if (!make_geometry(dtype, N, C, K, H, W, pad, &g))
        return fail(WINO_ERR_INVALID, "bad shape N=%d C=%d K=%d H=%d W=%d pad=%d", N, C, K, H, W, pad);
    if (th) *th = g.th;
    if (tw) *tw = g.tw;
    if (P) *P = g.P;
    if (Cp) *Cp = g.Cp;
    if (Kp) *Kp = g.Kp;
    if (Pp) *Pp = g.Pp;
    return WINO_OK;
}

size_t wino_workspace_bytes(int dtype, int N, int C, int K, int H, int W, int pad) {
    Geometry g;
    if (!valid_dtype(dtype) || !make_geometry(dtype, N, C, K, H, W, pad, &g)) {
        fail(WINO_ERR_INVALID, "bad shape or dtype");
        return 0;
    }
    Geometry g4;
    size_t need = scratch_layout(g, dtype).total;
    if (make_geometry(dtype, N, C, K, H, W, pad, &g4, 4))
        need = std::max(need, std::max(scratch_layout(g4, dtype).total, scratch_layout(g4, dtype, WINO_ALGO_EPILOGUE_F4).total));
    return need;
}

int wino_set_workspace(void* ptr, size_t bytes) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(WINO_ERR_UNSUPPORTED, "device index %d out of range", dev);
    if (ptr && bytes == 0) return fail(WINO_ERR_INVALID, "workspace pointer with zero size");
    if (misaligned(ptr, 256)) return fail(WINO_ERR_INVALID, "workspace must be 256-byte aligned");
    if (ptr && bytes < kCounterBytes) return fail(WINO_ERR_WORKSPACE, "workspace smaller than %zu bytes", kCounterBytes);
    if (ptr) HIP_TRY(hipMemset(ptr, 0, kCounterBytes));   // arrival counters (blocking, like every allocation)
    std::lock_guard<std::mutex> lk(g_arena_mu);
    g_arena[dev].ext = ptr;
    g_arena[dev].ext_bytes = ptr ? bytes : 0;
    ++g_arena[dev].generation;
    return WINO_OK;
}

int wino_filter_transform(int layout, int dtype, int K, int C, const void* w, void* U, void* stream) {
    if (!valid_layout(layout)) return fail(WINO_ERR_INVALID, "unknown layout %d", layout);
    if (!w || !U) return fail(WINO_ERR_INVALID, "null pointer");
    if (misaligned(U, 16)) return fail(WINO_ERR_INVALID, "transformed filters must be 16-byte aligned");
    if (K <= 0 || C <= 0) return fail(WINO_ERR_INVALID, "bad filter bank K=%d C=%d", K, C);
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    const int Kp = (int)round_up(K, kKPad), Cp = (int)round_up(C, c_pad(dtype));
    DISPATCH_DTYPE(dtype, launch_filter_transform<T>(layout, K, C, Kp, Cp, w, U, (hipStream_t)stream));
}

int wino_input_transform(int layout, int dtype, int tile_order, int N, int C, int H, int W, int pad, const void* x,
                         void* V, void* stream) {
    if (!valid_layout(layout)) return fail(WINO_ERR_INVALID, "unknown layout %d", layout);
    if (!valid_order(tile_order)) return fail(WINO_ERR_INVALID, "unknown tile order %d", tile_order);
    if (!x || !V) return fail(WINO_ERR_INVALID, "null pointer");
    if (misaligned(V, 16)) return fail(WINO_ERR_INVALID, "transformed input must be 16-byte aligned");
    Geometry g;
    if (!make_geometry(dtype, N, C, 1, H, W, pad, &g))
        return fail(WINO_ERR_INVALID, "bad shape N=%d C=%d H=%d W=%d pad=%d", N, C, H, W, pad);
    DISPATCH_DTYPE(dtype, launch_input_transform<T>(layout, tile_order, g, x, V, (hipStream_t)stream));
}

int wino_batched_gemm(int dtype, int product_order, int C, int K, long P, const void* U, const void* V, float* Mo,
                      void* stream) {
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    if (!valid_porder(product_order)) return fail(WINO_ERR_INVALID, "unknown product order %d", product_order);
    if (!U || !V || !Mo) return fail(WINO_ERR_INVALID, "null pointer");
    if (misaligned(U, 16) || misaligned(V, 16) || misaligned(Mo, 16))
        return fail(WINO_ERR_INVALID, "GEMM operands must be 16-byte aligned");
    if (C <= 0 || K <= 0 || P <= 0) return fail(WINO_ERR_INVALID, "bad GEMM shape C=%d K=%d P=%ld", C, K, P);
    return launch_gemm(16, dtype, product_order, (int)round_up(C, c_pad(dtype)), (int)round_up(K, kKPad), round_up(P, kPPad), U, V, Mo,
                       (hipStream_t)stream);
}

int wino_output_transform(int layout, int dtype, int tile_order, int product_order, unsigned flags, int N, int K,
                          int Ho, int Wo, const float* Mo, void* y, void* stream) {
    if (!valid_layout(layout)) return fail(WINO_ERR_INVALID, "unknown layout %d", layout);
    if (!valid_porder(product_order)) return fail(WINO_ERR_INVALID, "unknown product order %d", product_order);
    if (!valid_order(tile_order)) return fail(WINO_ERR_INVALID, "unknown tile order %d", tile_order);
    if (!Mo || !y) return fail(WINO_ERR_INVALID, "null pointer");
    if (misaligned(Mo, 16)) return fail(WINO_ERR_INVALID, "the product tensor must be 16-byte aligned");
    if (N <= 0 || K <= 0 || Ho <= 0 || Wo <= 0)
        return fail(WINO_ERR_INVALID, "bad shape N=%d K=%d Ho=%d Wo=%d", N, K, Ho, Wo);
    const long P = (long)N * ((Ho + 1) / 2) * ((Wo + 1) / 2);
    const int Kp = (int)round_up(K, kKPad);
    const long Pp = round_up(P, kPPad);
    DISPATCH_DTYPE(dtype, launch_output_transform<T>(layout, tile_order, product_order, flags, nullptr, N, K, Ho, Wo, Kp, P, Pp, Mo, y,
                                                     (hipStream_t)stream));
}

int wino_gemm_output(int layout, int dtype, int tile_order, unsigned flags, int N, int C, int K, int Ho, int Wo,
                     const void* U, const void* V, void* y, void* stream) {
    if (!valid_layout(layout)) return fail(WINO_ERR_INVALID, "unknown layout %d", layout);
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    if (!valid_order(tile_order)) return fail(WINO_ERR_INVALID, "unknown tile order %d", tile_order);
    if (!U || !V || !y) return fail(WINO_ERR_INVALID, "null pointer");
    if (misaligned(U, 16) || misaligned(V, 16)) return fail(WINO_ERR_INVALID, "GEMM operands must be 16-byte aligned");
    Geometry g;
    // geometry from the output size: pad 1 keeps H == Ho
    if (!make_geometry(dtype, N, C, K, Ho, Wo, 1, &g))
        return fail(WINO_ERR_INVALID, "bad shape N=%d C=%d K=%d Ho=%d Wo=%d", N, C, K, Ho, Wo);
    return launch_gemm_out(layout, dtype, tile_order, flags, nullptr, g, U, V, y, TailScratch{}, (hipStream_t)stream);
}

int wino_layout_transform(int src, int dst, int dtype, int N, int C, int H, int W, const void* in, void* out,
                          void* stream) {
    if (!valid_layout(src) || !valid_layout(dst)) return fail(WINO_ERR_INVALID, "unknown layout %d -> %d", src, dst);
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    if (!in || !out) return fail(WINO_ERR_INVALID, "null pointer");
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0) return fail(WINO_ERR_INVALID, "bad shape");
    const long total = (long)N * C * H * W;
    hipStream_t st = (hipStream_t)stream;
    if (src != dst) {
        // [R][A][B]: A = the source's contiguous axis, B = the destination's (see permute_tiled_kernel)
        const long HW = (long)H * W;
        PermuteDims d;
        if (src == WINO_NCHW && dst == WINO_NHWC) d = {HW, C, N, HW, C * HW, C, HW * C};
        else if (src == WINO_NHWC && dst == WINO_NCHW) d = {C, HW, N, C, HW * C, HW, C * HW};
        else if (src == WINO_NCHW && dst == WINO_CHWN) d = {C * HW, N, 1, C * HW, 0, N, 0};
        else if (src == WINO_CHWN && dst == WINO_NCHW) d = {N, C * HW, 1, N, 0, C * HW, 0};
        else if (src == WINO_NHWC && dst == WINO_CHWN) d = {C, N, HW, HW * C, C, HW * N, N};
        else d = {N, C, HW, HW * N, N, HW * C, C};               // CHWN -> NHWC
        // 2-byte elements move in pairs when every pair is 4-byte aligned on both sides
        const bool pairs = dtype != WINO_F32 && d.nA % 2 == 0 && d.nB % 2 == 0 && d.sB % 2 == 0 && d.sR % 2 == 0 &&
                           d.dA % 2 == 0 && d.dR % 2 == 0 && !misaligned(in, 4) && !misaligned(out, 4);
        if (pairs) {
            const int TA = d.nA <= 32 ? 32 : (d.nB <= 32 ? 256 : (d.nA <= 64 ? 64 : 128)), TB = 8192 / TA;
            const long tilesA = (d.nA + TA - 1) / TA, tilesB = (d.nB + TB - 1) / TB;
            const long blocks = tilesA * tilesB * d.nR;
            if (blocks >= (1L << 31)) return fail(WINO_ERR_UNSUPPORTED, "layout transform: tensor too large");
#define PERMUTE2(A, B)                                                                                          \
    hipLaunchKernelGGL((permute_tiled_pairs_kernel<A, B>), dim3((unsigned)blocks), dim3(256), 0, st,              \
                       (const uint16_t*)in, (uint16_t*)out, d, (int)tilesA, (int)tilesB)
            if (TA == 32) PERMUTE2(32, 256); else if (TA == 256) PERMUTE2(256, 32);
            else if (TA == 64) PERMUTE2(64, 128); else PERMUTE2(128, 64);
#undef PERMUTE2
            LAUNCH_CHECK("layout_transform");
            return WINO_OK;
        }
        const int TA = d.nA <= 32 ? 32 : (d.nB <= 32 ? 128 : 64), TB = 4096 / TA;
        const long tilesA = (d.nA + TA - 1) / TA, tilesB = (d.nB + TB - 1) / TB;
        const long blocks = tilesA * tilesB * d.nR;
        if (blocks >= (1L << 31)) return fail(WINO_ERR_UNSUPPORTED, "layout transform: tensor too large");
#define PERMUTE(T, A, B)                                                                                      \
    hipLaunchKernelGGL((permute_tiled_kernel<T, A, B>), dim3((unsigned)blocks), dim3(256), 0, st, (const T*)in, \
                       (T*)out, d, (int)tilesA, (int)tilesB)
        if (dtype == WINO_F32) {
            if (TA == 32) PERMUTE(float, 32, 128); else if (TA == 128) PERMUTE(float, 128, 32); else PERMUTE(float, 64, 64);
        } else {
            if (TA == 32) PERMUTE(uint16_t, 32, 128); else if (TA == 128) PERMUTE(uint16_t, 128, 32); else PERMUTE(uint16_t, 64, 64);
        }
#undef PERMUTE
        LAUNCH_CHECK("layout_transform");
        return WINO_OK;
    }
    // same layout on both sides: a plain copy
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    const ActStrides a = act_strides(src, N, C, H, W);
    if (dtype == WINO_F32)
        hipLaunchKernelGGL(permute_gather_kernel<float>, grid, block, 0, st, (const float*)in, (float*)out, a, dst, N,
                           C, H, W);
    else
        hipLaunchKernelGGL(permute_gather_kernel<uint16_t>, grid, block, 0, st, (const uint16_t*)in, (uint16_t*)out,
                           a, dst, N, C, H, W);
    LAUNCH_CHECK("layout_transform");
    return WINO_OK;
}

int wino_f4_geometry(int dtype, int N, int C, int K, int H, int W, int pad, int* th, int* tw, long* P, int* Cp,
                     int* Kp, long* Pp) {
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    Geometry g;
    if (!make_geometry(dtype, N, C, K, H, W, pad, &g, 4))
        return fail(WINO_ERR_INVALID, "bad shape N=%d C=%d K=%d H=%d W=%d pad=%d", N, C, K, H, W, pad);
    if (th) *th = g.th;
    if (tw) *tw = g.tw;
    if (P) *P = g.P;
    if (Cp) *Cp = g.Cp;
    if (Kp) *Kp = g.Kp;
    if (Pp) *Pp = g.Pp;
    return WINO_OK;
}

int wino_f4_filter_transform(int layout, int dtype, int K, int C, const void* w, void* U, void* stream) {
    if (!valid_layout(layout)) return fail(WINO_ERR_INVALID, "unknown layout %d", layout);
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    if (!w || !U) return fail(WINO_ERR_INVALID, "null pointer");
    if (misaligned(U, 16)) return fail(WINO_ERR_INVALID, "transformed filters must be 16-byte aligned");
    if (K <= 0 || C <= 0) return fail(WINO_ERR_INVALID, "bad filter bank K=%d C=%d", K, C);
    const int Kp = (int)round_up(K, kKPad), Cp = (int)round_up(C, c_pad(dtype));
    DISPATCH_DTYPE(dtype, launch_f4_filter<T>(layout, K, C, Kp, Cp, w, U, (hipStream_t)stream));
}

int wino_f4_input_transform(int layout, int dtype, int tile_order, int N, int C, int H, int W, int pad, const void* x,
                            void* V, void* stream) {
    if (!valid_layout(layout)) return fail(WINO_ERR_INVALID, "unknown layout %d", layout);
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    if (!valid_order(tile_order)) return fail(WINO_ERR_INVALID, "unknown tile order %d", tile_order);
    if (!x || !V) return fail(WINO_ERR_INVALID, "null pointer");
    if (misaligned(V, 16)) return fail(WINO_ERR_INVALID, "transformed input must be 16-byte aligned");
    Geometry g;
    if (!make_geometry(dtype, N, C, 1, H, W, pad, &g, 4))
        return fail(WINO_ERR_INVALID, "bad shape N=%d C=%d H=%d W=%d pad=%d", N, C, H, W, pad);
    DISPATCH_DTYPE(dtype, launch_f4_input<T>(layout, tile_order, g, x, V, (hipStream_t)stream));
}

int wino_f4_batched_gemm(int dtype, int product_order, int C, int K, long P, const void* U, const void* V, float* Mo,
                         void* stream) {
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    if (!valid_porder(product_order)) return fail(WINO_ERR_INVALID, "unknown product order %d", product_order);
    if (!U || !V || !Mo) return fail(WINO_ERR_INVALID, "null pointer");
    if (misaligned(U, 16) || misaligned(V, 16) || misaligned(Mo, 16))
        return fail(WINO_ERR_INVALID, "GEMM operands must be 16-byte aligned");
    if (C <= 0 || K <= 0 || P <= 0) return fail(WINO_ERR_INVALID, "bad GEMM shape C=%d K=%d P=%ld", C, K, P);
    return launch_gemm(36, dtype, product_order, (int)round_up(C, c_pad(dtype)), (int)round_up(K, kKPad),
                       round_up(P, kPPad), U, V, Mo, (hipStream_t)stream);
}

int wino_f4_output_transform(int layout, int dtype, int tile_order, int product_order, unsigned flags, int N, int K,
                             int Ho, int Wo, const float* Mo, void* y, void* stream) {
    if (!valid_layout(layout)) return fail(WINO_ERR_INVALID, "unknown layout %d", layout);
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    if (!valid_porder(product_order)) return fail(WINO_ERR_INVALID, "unknown product order %d", product_order);
    if (!valid_order(tile_order)) return fail(WINO_ERR_INVALID, "unknown tile order %d", tile_order);
    if (!Mo || !y) return fail(WINO_ERR_INVALID, "null pointer");
    if (misaligned(Mo, 16)) return fail(WINO_ERR_INVALID, "the product tensor must be 16-byte aligned");
    if (N <= 0 || K <= 0 || Ho <= 0 || Wo <= 0)
        return fail(WINO_ERR_INVALID, "bad shape N=%d K=%d Ho=%d Wo=%d", N, K, Ho, Wo);
    const long P = (long)N * ((Ho + 3) / 4) * ((Wo + 3) / 4);
    const int Kp = (int)round_up(K, kKPad);
    const long Pp = round_up(P, kPPad);
    if (flags & ~(unsigned)(WINO_FLAG_RELU | WINO_FLAG_POOL2)) return fail(WINO_ERR_INVALID, "unknown flags 0x%x", flags);
    if ((flags & WINO_FLAG_POOL2) && (Ho < 2 || Wo < 2)) return fail(WINO_ERR_INVALID, "2x2 pooling of a %dx%d output", Ho, Wo);
    DISPATCH_DTYPE(dtype, launch_f4_output<T>(layout, tile_order, product_order, flags, nullptr, N, K, Ho, Wo, Kp, P, Pp, Mo,
                                              y, (hipStream_t)stream));
}

int wino_f4_gemm_output(int layout, int dtype, int tile_order, unsigned flags, int N, int C, int K, int Ho, int Wo,
                        const void* U, const void* V, void* y, void* stream) {
    if (!valid_layout(layout)) return fail(WINO_ERR_INVALID, "unknown layout %d", layout);
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    if (!valid_order(tile_order)) return fail(WINO_ERR_INVALID, "unknown tile order %d", tile_order);
    if (!U || !V || !y) return fail(WINO_ERR_INVALID, "null pointer");
    if (misaligned(U, 16) || misaligned(V, 16)) return fail(WINO_ERR_INVALID, "GEMM operands must be 16-byte aligned");
    if (flags & ~(unsigned)(WINO_FLAG_RELU | WINO_FLAG_POOL2)) return fail(WINO_ERR_INVALID, "unknown flags 0x%x", flags);
    Geometry g;
    // geometry from the output size: pad 1 keeps H == Ho
    if (!make_geometry(dtype, N, C, K, Ho, Wo, 1, &g, 4))
        return fail(WINO_ERR_INVALID, "bad shape N=%d C=%d K=%d Ho=%d Wo=%d", N, C, K, Ho, Wo);
    if ((flags & WINO_FLAG_POOL2) && (Ho < 2 || Wo < 2)) return fail(WINO_ERR_INVALID, "2x2 pooling of a %dx%d output", Ho, Wo);
    F4RowsPlan plan;
    if (!f4_rows_plan(dtype, g, &plan))
        return fail(WINO_ERR_UNSUPPORTED, "the F(4x4) GEMM with the output transform in its epilogue is built for fp32 operands");
    void* base = nullptr;                      // partial outputs and arrival counters: the arena (shared like a whole-layer call's)
    const int rc = arena_get(kCounterBytes + plan.part_bytes, &base);
    if (rc) return rc;
    return launch_f4_gemm_rows(layout, tile_order, flags, nullptr, g, plan, U, V, y, (float*)((char*)base + kCounterBytes),
                               (int*)base, (hipStream_t)stream);
}

int wino_stage_timing(int enable) {
    std::lock_guard<std::mutex> lk(g_spans_mu);
    g_timing = enable != 0;
    return WINO_OK;
}

int wino_stage_stats(float* sum_ms, float* min_ms, float* max_ms, long* calls) {
    if (!sum_ms || !calls) return fail(WINO_ERR_INVALID, "null pointer");
    std::vector<StageSpan> spans;
    {
        std::lock_guard<std::mutex> lk(g_spans_mu);
        spans.swap(g_spans);
    }
    for (int i = 0; i < WINO_NUM_STAGES; ++i) {
        sum_ms[i] = 0.f;
        calls[i] = 0;
        if (min_ms) min_ms[i] = 0.f;
        if (max_ms) max_ms[i] = 0.f;
    }
    int rc = WINO_OK;
    for (auto& sp : spans) {
        float t = 0.f;
        hipError_t e = hipEventSynchronize(sp.b);
        if (e == hipSuccess) e = hipEventElapsedTime(&t, sp.a, sp.b);
        if (e != hipSuccess) rc = fail(WINO_ERR_HIP, "stage timing: %s", hipGetErrorString(e));
        else {
            const int s = sp.stage;
            if (min_ms) min_ms[s] = calls[s] == 0 ? t : std::min(min_ms[s], t);
            if (max_ms) max_ms[s] = calls[s] == 0 ? t : std::max(max_ms[s], t);
            sum_ms[s] += t;
            calls[s] += 1;
        }
        (void)hipEventDestroy(sp.a);
        (void)hipEventDestroy(sp.b);
    }
    return rc;
}

int wino_stage_times(float* ms, long* calls) { return wino_stage_stats(ms, nullptr, nullptr, calls); }

// ---- conv stack ------------------------------------------------------------------------------------
struct wino_stack {
    int device = 0, dtype = 0, N = 0;
    struct Layer {
        int C, K, H, W;            // input of the layer
        int Ho, Wo;                // what it writes (after pooling)
        int layout_in, layout_out, algo;
        unsigned flags;
        void* U = nullptr;         // cached transformed filters
        void* wraw = nullptr;      // layers with C <= 4: a copy of the filter bank itself, for the direct path
        void* U4 = nullptr;        // fp32 layers AUTO runs through F(4x4): their filters transformed for it
        void* W9 = nullptr;        // 2-byte NCHW layers AUTO runs directly: the bank in the direct kernel's order
        void* bias = nullptr;
        bool set = false, has_bias = false;
    };
    std::vector<Layer> layers;
    void* act[2] = {nullptr, nullptr};   // activations between layers
    size_t act_bytes = 0;
    // the captured forward pass (wino_stack_forward_graph) and what it was captured for
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipStream_t capture_stream = nullptr;
    const void* gx = nullptr;
    void* gy = nullptr;
    unsigned long garena = 0;
};

static int stack_run(wino_stack* s, const void* x, void* y, void* stream) {
    const int n = (int)s->layers.size();
    const void* in = x;
    for (int l = 0; l < n; ++l) {
        const auto& L = s->layers[l];
        void* out = l + 1 == n ? y : s->act[l & 1];
        const void* bias = L.has_bias ? L.bias : nullptr;
        int rc;
        Geometry g, g4;
        make_geometry(s->dtype, s->N, L.C, L.K, L.H, L.W, 1, &g);
        make_geometry(s->dtype, s->N, L.C, L.K, L.H, L.W, 1, &g4, 4);
        if (L.U4) {
            rc = conv_impl(ScratchSource{}, L.layout_in, L.layout_out, s->dtype, WINO_ALGO_STAGED_F4, L.flags, s->N, L.C, L.K,
                           L.H, L.W, 1, in, nullptr, L.U4, bias, out, stream);
        } else if (L.W9 && !misaligned(in, 4) && (!misaligned(out, 4) || (L.flags & WINO_FLAG_POOL2)) &&
                   auto_direct16(L.layout_in, L.layout_out, s->dtype, L.flags, g, in, out)) {
            // (the bank was packed for 4-byte aligned tensors; a caller's tensor that is not takes the general call)
            StageScope t(WINO_STAGE_GEMM, (hipStream_t)stream);
            if (direct16_chwn_pool_ok(L.layout_in, L.layout_out, s->dtype, L.flags, g)) {
                void* tmp = nullptr;
                rc = arena_get(direct16_unpooled_bytes(s->dtype, g), &tmp);
                if (!rc) rc = launch_direct16_chwn_pooled(s->dtype, L.flags, bias, g, in, nullptr, L.W9, tmp, out, (hipStream_t)stream, D16_RUN);
            } else
                rc = launch_direct16(L.layout_in, L.layout_out, s->dtype, L.flags, bias, g, in, nullptr, L.W9, out, (hipStream_t)stream, D16_RUN);
        } else {
            rc = conv_impl(ScratchSource{}, L.layout_in, L.layout_out, s->dtype, L.algo, L.flags, s->N, L.C, L.K, L.H, L.W, 1, in,
                           L.wraw, L.U, bias, out, stream);
        }
        if (rc) return rc;
        in = out;
    }
    return WINO_OK;
}

static void stack_drop_graph(wino_stack* s) {
    if (s->exec) (void)hipGraphExecDestroy(s->exec);
    if (s->graph) (void)hipGraphDestroy(s->graph);
    s->exec = nullptr;
    s->graph = nullptr;
}

int wino_stack_create(int dtype, int N, int C, int H, int W, int nlayers, const wino_stack_layer_t* layers,
                      wino_stack_t** stack) {
    if (!stack || !layers) return fail(WINO_ERR_INVALID, "null pointer");
    *stack = nullptr;
    if (!valid_dtype(dtype)) return fail(WINO_ERR_INVALID, "unknown dtype %d", dtype);
    if (nlayers <= 0 || N <= 0 || C <= 0 || H <= 0 || W <= 0)
        return fail(WINO_ERR_INVALID, "bad stack shape N=%d C=%d H=%d W=%d layers=%d", N, C, H, W, nlayers);
    std::unique_ptr<wino_stack> s(new wino_stack);
    s->dtype = dtype;
    s->N = N;
    HIP_TRY(hipGetDevice(&s->device));
    const size_t es = dtype_size(dtype);
    int c = C, h = H, w = W;
    for (int l = 0; l < nlayers; ++l) {
        const wino_stack_layer_t& d = layers[l];
        if (d.K <= 0 || !valid_layout(d.layout_in) || !valid_layout(d.layout_out) ||
            d.algo < WINO_ALGO_AUTO || d.algo > WINO_ALGO_FUSED ||
            (d.flags & ~(unsigned)(WINO_FLAG_RELU | WINO_FLAG_POOL2)))
            return fail(WINO_ERR_INVALID, "layer %d: bad description", l);
        if (l > 0 && d.layout_in != layers[l - 1].layout_out)
            return fail(WINO_ERR_INVALID, "layer %d reads layout %d, layer %d writes %d", l, d.layout_in, l - 1,
                        layers[l - 1].layout_out);
        wino_stack::Layer L;
        L.C = c; L.K = d.K; L.H = h; L.W = w;
        L.layout_in = d.layout_in; L.layout_out = d.layout_out; L.algo = d.algo; L.flags = d.flags;
        const bool pool = d.flags & WINO_FLAG_POOL2;
        if (pool && (h < 2 || w < 2)) return fail(WINO_ERR_INVALID, "layer %d pools a %dx%d image", l, h, w);
        L.Ho = pool ? h / 2 : h;
        L.Wo = pool ? w / 2 : w;
        Geometry g;
        if (!make_geometry(dtype, N, c, d.K, h, w, 1, &g)) return fail(WINO_ERR_INVALID, "layer %d: bad shape", l);
        if (l + 1 < nlayers) s->act_bytes = std::max(s->act_bytes, (size_t)N * d.K * L.Ho * L.Wo * es);
        s->layers.push_back(L);
        c = d.K; h = L.Ho; w = L.Wo;
    }
    // device memory; on failure the destructor path below releases what was taken
    wino_stack* raw = s.release();
    auto bail = [&](hipError_t e) {
        wino_stack_destroy(raw);
        return fail(WINO_ERR_HIP, "stack allocation: %s", hipGetErrorString(e));
    };
    for (auto& L : raw->layers) {
        Geometry g;
        make_geometry(dtype, N, L.C, L.K, L.H, L.W, 1, &g);
        hipError_t e = hipMalloc(&L.U, (size_t)16 * g.Cp * g.Kp * es);
        if (e == hipSuccess) e = hipMalloc(&L.bias, (size_t)L.K * es);
        // a copy of the bank itself for the layers AUTO may run without Winograd (C <= 4; 2-byte layers; small fp32 layers)
        const bool direct16_layer = dtype != WINO_F32 && (L.layout_in == WINO_CHWN) == (L.layout_out == WINO_CHWN) && L.C % 8 == 0;
        if (e == hipSuccess && (L.C <= 4 || direct16_layer || auto_direct_few(L.layout_in, dtype, L.flags, g)))
            e = hipMalloc(&L.wraw, (size_t)9 * L.K * L.C * es);
        // what AUTO runs outside the F(2x2) kernels gets its filters prepared once as well
        if (e == hipSuccess && L.algo == WINO_ALGO_AUTO && auto_f4(dtype, g)) {
            Geometry g4;
            make_geometry(dtype, N, L.C, L.K, L.H, L.W, 1, &g4, 4);
            e = hipMalloc(&L.U4, (size_t)36 * g4.Cp * g4.Kp * es);
        }
        if (e == hipSuccess && L.algo == WINO_ALGO_AUTO && direct16_layer &&
            auto_direct16(L.layout_in, L.layout_out, dtype, L.flags, g, nullptr, nullptr))
            e = hipMalloc(&L.W9, direct16_bank_bytes(g));
        if (e != hipSuccess) return bail(e);
    }
    for (int i = 0; i < 2 && raw->act_bytes; ++i) {
        hipError_t e = hipMalloc(&raw->act[i], raw->act_bytes);
        if (e != hipSuccess) return bail(e);
    }
    *stack = raw;
    return WINO_OK;
}

int wino_stack_set_layer(wino_stack_t* s, int layer, const void* w, const void* bias, void* stream) {
    if (!s || !w) return fail(WINO_ERR_INVALID, "null pointer");
    if (layer < 0 || layer >= (int)s->layers.size()) return fail(WINO_ERR_INVALID, "no layer %d", layer);
    auto& L = s->layers[layer];
    // a recorded pass holds the layer's bias pointer (or its absence) in its kernel arguments
    stack_drop_graph(s);
    int rc = wino_filter_transform(L.layout_in, s->dtype, L.K, L.C, w, L.U, stream);
    if (rc) return rc;
    if (L.wraw)
        HIP_TRY(hipMemcpyAsync(L.wraw, w, (size_t)9 * L.K * L.C * dtype_size(s->dtype), hipMemcpyDeviceToDevice,
                               (hipStream_t)stream));
    if (L.U4) {
        rc = wino_f4_filter_transform(L.layout_in, s->dtype, L.K, L.C, w, L.U4, stream);
        if (rc) return rc;
    }
    if (L.W9) {
        Geometry g;
        make_geometry(s->dtype, s->N, L.C, L.K, L.H, L.W, 1, &g);
        const unsigned pflags = L.layout_in == WINO_CHWN ? L.flags & ~(unsigned)WINO_FLAG_POOL2 : L.flags;   // (a pooled CHWN layer runs unpooled)
        rc = launch_direct16(L.layout_in, L.layout_out, s->dtype, pflags, nullptr, g, L.W9, w, L.W9, L.W9, (hipStream_t)stream, D16_PACK);   // (x, y: any aligned address)
        if (rc) return rc;
    }
    L.has_bias = bias != nullptr;
    if (bias)
        HIP_TRY(hipMemcpyAsync(L.bias, bias, (size_t)L.K * dtype_size(s->dtype), hipMemcpyDeviceToDevice,
                               (hipStream_t)stream));
    L.set = true;
    return WINO_OK;
}

int wino_stack_output(const wino_stack_t* s, int* N, int* K, int* H, int* W, int* layout) {
    if (!s || !N || !K || !H || !W || !layout) return fail(WINO_ERR_INVALID, "null pointer");
    const auto& L = s->layers.back();
    *N = s->N; *K = L.K; *H = L.Ho; *W = L.Wo; *layout = L.layout_out;
    return WINO_OK;
}

int wino_stack_forward(wino_stack_t* s, const void* x, void* y, void* stream) {
    if (!s || !x || !y) return fail(WINO_ERR_INVALID, "null pointer");
    const int n = (int)s->layers.size();
    for (int l = 0; l < n; ++l)
        if (!s->layers[l].set) return fail(WINO_ERR_INVALID, "layer %d has no filters yet", l);
    return stack_run(s, x, y, stream);
}

int wino_stack_forward_graph(wino_stack_t* s, const void* x, void* y, void* stream) {
    if (!s || !x || !y) return fail(WINO_ERR_INVALID, "null pointer");
    for (size_t l = 0; l < s->layers.size(); ++l)
        if (!s->layers[l].set) return fail(WINO_ERR_INVALID, "layer %zu has no filters yet", l);
    if (g_timing) return stack_run(s, x, y, stream);          // stage timing brackets eager launches
    // the arena must not grow while the pass is being captured: size it for the largest layer first
    size_t need = 0;
    for (const auto& L : s->layers) {
        Geometry g;
        if (!make_geometry(s->dtype, s->N, L.C, L.K, L.H, L.W, 1, &g)) return fail(WINO_ERR_INVALID, "bad layer shape");
        need = std::max(need, scratch_layout(g, s->dtype).total);
        Geometry g4;
        if (L.U4 && make_geometry(s->dtype, s->N, L.C, L.K, L.H, L.W, 1, &g4, 4))
            need = std::max(need, scratch_layout(g4, s->dtype, WINO_ALGO_STAGED_F4).total);
    }
    void* base = nullptr;
    int rc = arena_get(need, &base);
    if (rc) return rc;
    const unsigned long gen = arena_generation(s->device);
    if (!s->exec || s->gx != x || s->gy != y || s->garena != gen) {
        stack_drop_graph(s);
        if (!s->capture_stream) HIP_TRY(hipStreamCreateWithFlags(&s->capture_stream, hipStreamNonBlocking));
        HIP_TRY(hipStreamBeginCapture(s->capture_stream, hipStreamCaptureModeThreadLocal));
        rc = stack_run(s, x, y, s->capture_stream);
        const hipError_t e = hipStreamEndCapture(s->capture_stream, &s->graph);
        if (rc || e != hipSuccess) {
            stack_drop_graph(s);
            return rc ? rc : fail(WINO_ERR_HIP, "hipStreamEndCapture: %s", hipGetErrorString(e));
        }
        const hipError_t ei = hipGraphInstantiate(&s->exec, s->graph, nullptr, nullptr, 0);
        if (ei != hipSuccess) {
            stack_drop_graph(s);
            return fail(WINO_ERR_HIP, "hipGraphInstantiate: %s", hipGetErrorString(ei));
        }
        s->gx = x;
        s->gy = y;
        s->garena = gen;
    }
    HIP_TRY(hipGraphLaunch(s->exec, (hipStream_t)stream));
    return WINO_OK;
}

int wino_stack_destroy(wino_stack_t* s) {
    if (!s) return WINO_OK;
    for (auto& L : s->layers) {
        if (L.U) (void)hipFree(L.U);
        if (L.wraw) (void)hipFree(L.wraw);
        if (L.U4) (void)hipFree(L.U4);
        if (L.W9) (void)hipFree(L.W9);
        if (L.bias) (void)hipFree(L.bias);
    }
    for (int i = 0; i < 2; ++i)
        if (s->act[i]) (void)hipFree(s->act[i]);
    stack_drop_graph(s);
    if (s->capture_stream) (void)hipStreamDestroy(s->capture_stream);
    delete s;
    return WINO_OK;
}

int wino_warmup(void) {
    hipLaunchKernelGGL(warmup_kernel, dim3(1), dim3(1), 0, 0);
    LAUNCH_CHECK("warmup");
    void* unused = nullptr;                    // also the set-up of wino_conv_noalloc's buffer on this device
    return noalloc_scratch(&unused);
}

int wino_sync(void* stream) {
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return WINO_OK;
}

const char* wino_last_error(void) { return g_err; }

const char* wino_version(void) { return "wino_amd 0.3 (gfx950; F(2x2,3x3), F(4x4,3x3), direct)"; }

}  // extern "C"
