/*
 * wino_amd.h -- C ABI of the MI355X (gfx950) Winograd 3x3 convolution library: F(2x2,3x3) and F(4x4,3x3)
 * pipelines in fp32, F(2x2,3x3) with f16 / bf16 storage, and direct MFMA convolutions where those are faster.
 * What a caller of the whole-layer entry points gets under WINO_ALGO_AUTO: fp32 layers with long reductions and
 * more than one tile of 64 filters (C >= 96 or so, at least 512 tiles of 4x4 outputs) run in F(4x4,3x3), the
 * reference's own tile size (relative L2 error against a direct convolution 3e-6 to 5e-6), other fp32 layers in
 * F(2x2,3x3) or directly (about 1e-6), 2-byte layers in F(2x2,3x3) or directly (about 2e-3 bf16, 3e-4 f16).
 *
 * Every entry point takes plain device pointers and sizes; `stream` is a
 * hipStream_t passed as void* (NULL = the null stream).  Calls are asynchronous
 * on that stream unless stated otherwise.  Return value: 0 on success, a
 * negative wino_status_t otherwise; wino_last_error() gives the text of the
 * calling thread's last failure.
 *
 * Tensor conventions (those of the reference's three wrappers):
 *   layout   activations x / y           3x3 filter bank w
 *   NCHW     [N][C][H][W]                [K][C][3][3]   comparison/wrapedConv_NCHW.cuh:869
 *   NHWC     [N][H][W][C]                [K][3][3][C]   comparison/wrapedConv_NHWC.cuh:341
 *   CHWN     [C][H][W][N]                [C][3][3][K]   comparison/wrapedConv_CHWN.cuh:288
 * The convolution is a stride-1 cross-correlation with `pad` rows/columns of
 * zeros on every side; the output is Ho x Wo = (H+2*pad-2) x (W+2*pad-2).
 * pad is 0 .. 1024 (the reference takes it arithmetically,
 * comparison/wrapedConv_NCHW.cuh:346-362, and its drivers pass 1).  The staged
 * and epilogue pipelines and WINO_ALGO_AUTO take any of these; WINO_ALGO_FUSED and
 * WINO_ALGO_DIRECT are built for 0 and 1 and answer WINO_ERR_UNSUPPORTED beyond
 * (but for the small-layer fp32 kernel of WINO_ALGO_DIRECT, which takes any).
 *
 * Alignment: x, w, bias and y need only the alignment of their element type (any
 * view of a device allocation works).  The Winograd-domain operands U, V and the
 * product tensor move as 16-byte vectors and must be 16-byte aligned, a caller's
 * workspace 256-byte aligned; anything else is refused with WINO_ERR_INVALID.
 *
 * Concurrency: the whole-layer calls (wino_conv*, wino_stack_forward*) of one
 * device share that device's scratch arena -- transformed operands, product
 * tensor, arrival counters -- as the calls of the reference's driver share the
 * three scratch buffers it allocates once and hands to every wrapper call
 * (comparison/layoutCompare.cu:124-126, wrapedConv_NCHW.cuh:335).  Issue them in order on one
 * stream, or serialise the streams yourself: two layers in flight at once on one
 * device overwrite each other's scratch.  The stage entry points touch only the
 * buffers they are given and may overlap freely.  Any entry point may be called
 * from several host threads (the error text is per thread, the arena's
 * bookkeeping is locked) under the same rule; growing the arena synchronises the
 * device.
 */
#ifndef WINO_AMD_H
#define WINO_AMD_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* same order as `enum class DataLayout` (comparison/DataLayoutTrans.cuh:587-591) */
typedef enum { WINO_NCHW = 0, WINO_NHWC = 1, WINO_CHWN = 2 } wino_layout_t;

/* storage type of x, w, y and of the transformed operands; accumulation is always fp32 */
typedef enum { WINO_F32 = 0, WINO_F16 = 1, WINO_BF16 = 2 } wino_dtype_t;

typedef enum {
    WINO_ALGO_AUTO = 0,     /* library picks per shape */
    WINO_ALGO_STAGED = 1,   /* four kernels: input/filter transform, 16-way GEMM, output transform
                               (the pipeline of comparison/wrapedConv_NCHW.cuh:408-452) */
    WINO_ALGO_EPILOGUE = 2, /* output transform applied in the GEMM epilogue (no product tensor in HBM) */
    WINO_ALGO_FUSED = 3,    /* one kernel: input transform, multiply-accumulate and output transform
                               (the structure of fusedTest/winotrans.cuh:1452 Winofuse4433) */
    WINO_ALGO_STAGED_F4 = 4, /* the staged pipeline in F(4x4,3x3) -- 6x6 tiles, 36 coordinates, the reference's
                               own tile size and matrices (wrapedConv_NCHW.cuh:836-855,879-899,1084-1101):
                               2.25 multiplies per output instead of 4, about four times the rounding error of
                               F(2x2) (3e-6 to 5e-6 relative L2 in fp32 on the VGG layers).  WINO_ALGO_AUTO takes it
                               for fp32 layers with at least 512 tiles and either C, K >= 128, or K > 64 and
                               C >= 96 (C >= 48 while its transformed tensors fit the 256 MB cache), or K <= 64,
                               C >= 96 and few patches, when it is given the filter bank itself; transformed
                               filters handed to this algorithm by name must come from wino_f4_filter_transform. */
    WINO_ALGO_DIRECT = 5,    /* no Winograd at all, the convolution itself on the matrix cores.  Three kinds of layer:
                               small fp32 layers -- at most four rounds of the chip in units of 4 x 8 pixels x 32
                               filters, e.g. the reference's sweep at batch 1 (comparison/layoutCompare.cu:38-46: N = 1,
                               C = K = 64, 56 x 56) -- run as ONE launch whose waves share the channel reduction,
                               any layout pair, any padding, bias and ReLU but no pooling;
                               layers with C <= 4 (the network's first layer, which the reference runs through
                               the same wrappers: comparison/layoutCompare.cu:38-46): the 9*C <= 36 products of an
                               output as one short MFMA reduction, any layout, fp32 or 2-byte; with 2x2 pooling the
                               layer runs unpooled into scratch, at most 224 MB of images at a time, and a pooling
                               kernel follows;
                               2-byte NCHW -> NCHW layers with C a multiple of 8, an even width and a 4-byte aligned
                               x: an implicit GEMM on the 16-bit instruction with fp32 accumulation -- with 2-byte
                               operands the Winograd pipelines are bound by the transformed input in memory, the
                               direct product by nothing but the multiplies (the stage it replaces is
                               comparison/GEMM.cuh:124-253; the reference's own direct kernel in tile geometry is
                               Conv_fuse, fusedTest/winotrans.cuh:1868).
                               2-byte layers with an NHWC side (NHWC -> NHWC, NCHW -> NHWC, NHWC -> NCHW; the filters in
                               the source's layout), C a multiple of 8 and, from NHWC, a 16-byte aligned x run on the
                               larger of its two kernels (the 8-wave one) when the layer has its shape: output height a multiple of 4, even output width, K a multiple of 64, at least a
                               tile for every other CU; other NHWC layers are refused (WINO_ERR_UNSUPPORTED).
                               2-byte CHWN -> CHWN layers (comparison/wrapedConv_CHWN.cuh:16-82) run on the same kernel, taken as one
                               image of width W * N whose tap columns lie N elements apart: the same shape conditions, an
                               even batch of at most 32 images (more where the rows are short), x and y 4-byte aligned; 2x2
                               pooling in the kernel's stores for 32 images and an even width, otherwise the layer runs
                               unpooled into scratch (N*K*Ho*Wo elements) and a pooling kernel follows; other CHWN
                               layers, and layers with CHWN on one side only, are refused.
                               Bias and ReLU; 2x2 pooling for C <= 4 and for the 2-byte layers that run on the
                               8-wave kernel (the shape just named); needs the filter bank itself (not
                               wino_conv_prepared).
                               What WINO_ALGO_AUTO picks for C <= 4 and for large 2-byte NCHW, NHWC and CHWN layers. */
    WINO_ALGO_EPILOGUE_F4 = 6 /* F(4x4,3x3) with the output transform A^T (.) A in the epilogue of the 36-way GEMM: no
                               product tensor in HBM.  The arrangement of the reference's fused F(4x4) kernels
                               (fusedTest/winotrans.cuh:1530-1574: 36 running products, A^T acc A in registers, 16
                               stores) for the matrix cores, one Winograd row resident at a time.  fp32, any layout
                               pair, bias / ReLU / pooling; transformed filters as for WINO_ALGO_STAGED_F4; 2-byte
                               tensors are refused (WINO_ERR_UNSUPPORTED). */
} wino_algo_t;

/* order of the tile index p inside the transformed operands */
typedef enum {
    WINO_TILES_BATCH_MAJOR = 0, /* p = (n*th + ty)*tw + tx */
    WINO_TILES_BATCH_MINOR = 1  /* p = (ty*tw + tx)*N + n  */
} wino_tile_order_t;

/* orientation of the GEMM product in HBM (staged algorithm only) */
typedef enum {
    WINO_PRODUCT_KP = 0, /* Mo[16][Kp][Pp]: tiles contiguous -- for NCHW / CHWN destinations */
    WINO_PRODUCT_PK = 1  /* Mo[16][Pp][Kp]: filters contiguous -- for NHWC destinations      */
} wino_product_order_t;

typedef enum {
    WINO_OK = 0,
    WINO_ERR_INVALID = -1,     /* null pointer, non-positive size, unknown enum */
    WINO_ERR_UNSUPPORTED = -2, /* valid request this build does not implement */
    WINO_ERR_HIP = -3,         /* a HIP runtime call failed */
    WINO_ERR_WORKSPACE = -4    /* caller-provided workspace too small */
} wino_status_t;

/* flags for wino_conv and the output-side stage functions */
#define WINO_FLAG_RELU 1u  /* clamp negatives in the output stage */
#define WINO_FLAG_POOL2 2u /* 2x2 / stride-2 max pooling in the output stage: y has floor(Ho/2) x floor(Wo/2)
                              outputs per image and filter (the 2x2 outputs of a tile are one window) */

/*
 * Whole layer: y = conv3x3(x, w).  x and w are in `src`'s conventions, y in
 * `dst`'s.  Replaces the body of
 *   wrapedConv_NCHW  comparison/wrapedConv_NCHW.cuh:335-492
 *   wrapedConv_NHWC  comparison/wrapedConv_NHWC.cuh:24-112
 *   wrapedConv_CHWN  comparison/wrapedConv_CHWN.cuh:16-82
 * and, for src != dst, the six convLayoutTrans_X_to_Y of
 * comparison/DataLayoutTrans.cuh:9,101,192,309,418,502 (dispatch :594-651).
 * Scratch comes from the library's per-device arena (grown on demand) unless
 * wino_set_workspace() installed a caller buffer.
 */
int wino_conv(int src, int dst, int dtype, int algo, unsigned flags, int N, int C, int K, int H,
              int W, int pad, const void *x, const void *w, void *y, void *stream);

/*
 * Same, with the filter bank already transformed by wino_filter_transform()
 * (the reference recomputes it on every call: wrapedConv_NCHW.cuh:423).
 */
int wino_conv_prepared(int src, int dst, int dtype, int algo, unsigned flags, int N, int C, int K,
                       int H, int W, int pad, const void *x, const void *U, void *y, void *stream);

/*
 * The two calls above with a per-filter bias (K elements of the tensor's element type, or NULL):
 *   y = pool2x2?( relu?( conv3x3(x, w) + bias[k] ) )
 * in the output stage of whichever algorithm runs, instead of the separate passes over y of
 *   addBias_CHWN / relu_CHWN / maxPool_CHWN
 *   netTest/cudnn_test_0124/VGG_Batched/CHWN_support.cuh:107,512,248
 * (the fused form is what fusedTest/winotrans.cuh:380-400 sketches).
 */
int wino_conv_ex(int src, int dst, int dtype, int algo, unsigned flags, int N, int C, int K, int H,
                 int W, int pad, const void *x, const void *w, const void *bias, void *y, void *stream);
int wino_conv_prepared_ex(int src, int dst, int dtype, int algo, unsigned flags, int N, int C, int K,
                          int H, int W, int pad, const void *x, const void *U, const void *bias, void *y,
                          void *stream);

/*
 * wino_conv_ex for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose callers allocate their three
 * scratch buffers themselves (comparison/layoutCompare.cu:124-126).  Same arguments, same kernels and the same
 * bits as wino_conv_ex; the scratch (transformed operands, product or partial sums, arrival counters) is a
 * fixed buffer of WINO_NOALLOC_SCRATCH_BYTES inside the library's device image, one per GPU, held until the
 * process ends, instead of the arena.  The call makes no hipMalloc / hipFree and creates no events (stage timing
 * does not see it).  A problem whose pipeline needs more scratch than the buffer holds is refused with
 * WINO_ERR_WORKSPACE and a message giving both sizes: ask for WINO_ALGO_FUSED (keeps only the transformed
 * filters, 16*Cp*Kp elements) or WINO_ALGO_DIRECT, or use a smaller batch.  Under WINO_ALGO_AUTO a first choice that
 * keeps large tensors in scratch (F(4x4); a direct kernel that pools through scratch) gives way to one that fits: the
 * pooled first layer in smaller passes, the F(2x2) pipelines, the single kernel last.  The first call on a device looks the
 * buffer's address up (wino_warmup() does the same ahead of time); nothing is cleared: the buffer is a
 * zero-initialised object of the device image, and the kernels that count arrivals in it leave their counters at zero.  Every call on a GPU shares that GPU's buffer: calls that overlap
 * on one GPU (two streams, two threads) race, exactly as whole-layer calls sharing the arena do.
 */
#define WINO_NOALLOC_SCRATCH_BYTES (64u << 20)
int wino_conv_noalloc(int src, int dst, int dtype, int algo, unsigned flags, int N, int C, int K, int H,
                      int W, int pad, const void *x, const void *w, const void *bias, void *y, void *stream);

/* the algorithm WINO_ALGO_AUTO resolves to for this problem (a wino_algo_t), or a negative status;
 * layout is that of the input tensor */
int wino_pick_algo(int layout, int dtype, int N, int C, int K, int H, int W, int pad);

/* ---- padded operand geometry ------------------------------------------------
 * With th = ceil(Ho/2), tw = ceil(Wo/2), P = N*th*tw and CV = 16/sizeof(element)
 * (4 channels per 16-byte vector for fp32, 8 for f16/bf16):
 *   U   [16][Cp/CV][Kp][CV]   transformed filters, channel vectors innermost
 *   V   [16][Cp/CV][Pp][CV]   transformed input tiles
 *   Mo  [16][Kp][Pp]          GEMM product, always fp32 ([16][Pp][Kp] with WINO_PRODUCT_PK)
 * Cp is C rounded up to 4 channel vectors (16 for fp32, 32 for f16/bf16); Kp and Pp are K
 * and P rounded up to 128.  The counterpart of
 * MSize/NSize/KSize at comparison/wrapedConv_NCHW.cuh:346-362. */
int wino_geometry(int dtype, int N, int C, int K, int H, int W, int pad, int *th, int *tw,
                  long *P, int *Cp, int *Kp, long *Pp);

/* bytes of scratch wino_conv needs for this problem (upper bound over algos) */
size_t wino_workspace_bytes(int dtype, int N, int C, int K, int H, int W, int pad);

/* install (ptr != NULL) or remove (ptr == NULL) a caller-owned workspace for the current device */
int wino_set_workspace(void *ptr, size_t bytes);

/* ---- the four stages on their own (stage parity tests, per-stage timing) -- */

/* U = G g G^T.  Replaces wino_kernel_trans_{nchw,nhwc,chwn}_suitFor128
 * (wrapedConv_NCHW.cuh:861, wrapedConv_NHWC.cuh:333, wrapedConv_CHWN.cuh:279).
 * Rows c >= C and columns k >= K of U are written as zeros. */
int wino_filter_transform(int layout, int dtype, int K, int C, const void *w, void *U, void *stream);

/* V = B^T d B.  Replaces wino_input_trans_{nchw,nhwc,chwn}_suitFor128*
 * (wrapedConv_NCHW.cuh:683,760, wrapedConv_NHWC.cuh:266, wrapedConv_CHWN.cuh:225).
 * Rows c >= C are written as zeros; columns p >= P are left untouched. */
int wino_input_transform(int layout, int dtype, int tile_order, int N, int C, int H, int W, int pad,
                         const void *x, void *V, void *stream);

/* Mo[xi][k][p] = sum_c U[xi][c][k] V[xi][c][p], xi = 0..15, fp32 accumulate on MFMA.
 * Replaces GEMM_batch_256_128x128_{KMKN,MKNK} (comparison/GEMM.cuh:124,4). */
int wino_batched_gemm(int dtype, int product_order, int C, int K, long P, const void *U, const void *V,
                      float *Mo, void *stream);

/* y = A^T Mo A.  Replaces wino_invers_{nchw,nhwc,chwn}_suitFor128*
 * (wrapedConv_NCHW.cuh:905,1034, wrapedConv_NHWC.cuh:376, wrapedConv_CHWN.cuh:379). */
int wino_output_transform(int layout, int dtype, int tile_order, int product_order, unsigned flags, int N,
                          int K, int Ho, int Wo, const float *Mo, void *y, void *stream);

/* GEMM with the output transform in its epilogue: y directly from U and V. */
int wino_gemm_output(int layout, int dtype, int tile_order, unsigned flags, int N, int C, int K,
                     int Ho, int Wo, const void *U, const void *V, void *y, void *stream);

/* ---- the same four stages in F(4x4,3x3): 36 coordinates, th = ceil(Ho/4), tw = ceil(Wo/4).
 * Operand layouts as above with 36 in place of 16; sizes from wino_f4_geometry. */
int wino_f4_geometry(int dtype, int N, int C, int K, int H, int W, int pad, int *th, int *tw, long *P,
                     int *Cp, int *Kp, long *Pp);
int wino_f4_filter_transform(int layout, int dtype, int K, int C, const void *w, void *U, void *stream);
int wino_f4_input_transform(int layout, int dtype, int tile_order, int N, int C, int H, int W, int pad,
                            const void *x, void *V, void *stream);
int wino_f4_batched_gemm(int dtype, int product_order, int C, int K, long P, const void *U, const void *V,
                         float *Mo, void *stream);
int wino_f4_output_transform(int layout, int dtype, int tile_order, int product_order, unsigned flags, int N,
                             int K, int Ho, int Wo, const float *Mo, void *y, void *stream);
/* The 36-way GEMM with the output transform in its epilogue: y directly from U and V (fp32; pad 1 geometry, as
 * wino_gemm_output).  The GEMM + inverse transform of the reference's fused kernel, fusedTest/winotrans.cuh:1530-1574.
 * Takes its partial-sum scratch from the device's arena, like a whole-layer call. */
int wino_f4_gemm_output(int layout, int dtype, int tile_order, unsigned flags, int N, int C, int K, int Ho, int Wo,
                        const void *U, const void *V, void *y, void *stream);

/* ---- plain layout permutation (bench harness; the reference has no such kernel) */
int wino_layout_transform(int src, int dst, int dtype, int N, int C, int H, int W, const void *in,
                          void *out, void *stream);

/* ---- per-stage timing (the commented-out event pairs of wrapedConv_NCHW.cuh:88-138, made usable)
 * While enabled, wino_conv / wino_conv_prepared bracket every stage they launch
 * with a pair of HIP events on the launch stream.  wino_stage_times() waits for
 * the recorded events, returns the accumulated milliseconds and number of spans
 * per stage (arrays of WINO_NUM_STAGES) and forgets them; wino_stage_stats() does
 * the same and also returns the shortest and longest span of every stage (the
 * average / minimum / maximum line that the reference's timing harness prints per
 * configuration, delayTest/testbench/src/M1/M1Test.h:100-151); min_ms and max_ms may be null. */
typedef enum {
    WINO_STAGE_FILTER = 0,
    WINO_STAGE_INPUT = 1,
    WINO_STAGE_GEMM = 2,   /* the batched GEMM, or the kernel that contains it (epilogue-fused / fused) */
    WINO_STAGE_OUTPUT = 3,
    WINO_NUM_STAGES = 4
} wino_stage_t;
int wino_stage_timing(int enable);
int wino_stage_times(float *ms, long *calls);
int wino_stage_stats(float *sum_ms, float *min_ms, float *max_ms, long *calls);

/* ---- a stack of 3x3 convolution layers with cached filter transforms -------------------------
 * The convolution part of the reference's network driver, classify_example_modified
 * (netTest/cudnn_test_0124/VGG_Batched/Network.h:603-669): per layer convMethodChoose (:456-519:
 * layoutManager with the layer's own layout_in / layout_out, then addBias), activationForward, and
 * poolForward after some layers -- here one wino_conv_prepared_ex call per layer, with bias, ReLU and
 * pooling in its output stage, the filter bank of every layer transformed once when it is set (the
 * reference transforms it again on every call), and the activations between layers in two buffers the
 * stack owns.  The fully connected layers and the softmax of the reference driver are cuBLAS/cuDNN
 * code and not part of this library.  Every layer is 3x3, stride 1, pad 1. */
typedef struct wino_stack wino_stack_t;
typedef struct {
    int K;                     /* filters of the layer; its channels are the previous layer's K */
    int layout_in, layout_out; /* wino_layout_t; layout_in must equal the previous layer's layout_out */
    unsigned flags;            /* WINO_FLAG_RELU | WINO_FLAG_POOL2 */
    int algo;                  /* wino_algo_t, normally WINO_ALGO_AUTO */
} wino_stack_layer_t;
/* the stack for inputs of N x C x H x W in layers[0].layout_in; allocates device memory */
int wino_stack_create(int dtype, int N, int C, int H, int W, int nlayers, const wino_stack_layer_t *layers,
                      wino_stack_t **stack);
/* filter bank (in the layer's layout_in convention) and bias (K elements or NULL) of one layer, both device
 * pointers; the bank is transformed and the bias copied before the call returns control to the stream */
int wino_stack_set_layer(wino_stack_t *stack, int layer, const void *w, const void *bias, void *stream);
/* shape and layout of what wino_stack_forward writes */
int wino_stack_output(const wino_stack_t *stack, int *N, int *K, int *H, int *W, int *layout);
/* all layers on `stream`; x and y are caller tensors; fails if a layer has not been set */
int wino_stack_forward(wino_stack_t *stack, const void *x, void *y, void *stream);
/* The same pass replayed from a HIP graph: the first call for a pair (x, y) records the launches of all layers
 * (on a stream of the stack's own) and instantiates the graph, later calls with the same pointers launch it on
 * `stream` -- one submission instead of two or three kernel launches per layer, which is what small batches are
 * bound by.  Recorded again by itself when x, y or the scratch arena's address change.  Not for concurrent use
 * with calls that may grow the arena from other threads.  The reference launches layer by layer
 * (VGG_Batched/Network.h:603-669) and has no counterpart. */
int wino_stack_forward_graph(wino_stack_t *stack, const void *x, void *y, void *stream);
int wino_stack_destroy(wino_stack_t *stack);

/* ---- housekeeping ----------------------------------------------------------- */
int wino_warmup(void);                 /* empty kernel; replaces warmup<<<1,1>>> (wrapedConv_NCHW.cuh:4-7) */
int wino_sync(void *stream);           /* hipStreamSynchronize; the reference ends each wrapper with a device sync (:482) */
const char *wino_last_error(void);
const char *wino_version(void);

#ifdef __cplusplus
}
#endif
#endif /* WINO_AMD_H */
