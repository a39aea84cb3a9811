"""MI355X-native Winograd F(2x2,3x3) convolution: host-side mirror of the
reference's wrapped-convolution call surface over the C ABI in
include/wino_amd.h.  torch supplies device memory and streams only."""
from .ops import (  # noqa: F401
    ALGO_AUTO, ALGO_EPILOGUE, ALGO_FUSED, ALGO_STAGED, ALGO_STAGED_F4, BF16, CHWN, F16, F32, NCHW, NHWC, PRODUCT_KP, PRODUCT_PK,
    TILES_BATCH_MAJOR, TILES_BATCH_MINOR, DataLayout, batched_gemm, conv, conv_prepared,
    convLayoutTrans_CHWN_to_NCHW, convLayoutTrans_CHWN_to_NHWC, convLayoutTrans_NCHW_to_CHWN,
    convLayoutTrans_NCHW_to_NHWC, convLayoutTrans_NHWC_to_CHWN, convLayoutTrans_NHWC_to_NCHW,
    filter_transform, gemm_output, geometry, input_transform, layoutManager, layout_transform,
    output_transform, warmup, workspace_bytes, wrapedConv_CHWN, wrapedConv_NCHW, wrapedConv_NHWC)
