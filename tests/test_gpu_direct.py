"""The direct path (WINO_ALGO_DIRECT) outside the 16-bit implicit GEMM: layers with at most four input channels
(what AUTO picks for the network's first layer, comparison/layoutCompare.cu:38-46: 3 -> 64 channels; 2-byte tensors
are multiplied in fp32 as well), and small fp32 layers of any channel count (the same sweep at batch 1).  Oracle: the
CPU direct convolution.  Bit-exact on small integers for all nine layout pairs, with bias and ReLU; within the layer
tolerance on floats."""
import itertools

import numpy as np
import pytest
import torch

from cudnntest_amd import _lib, ops, synth
from gpu_util import TOL, dev, host, rounded

pytestmark = pytest.mark.gpu
SRC = [ops.NCHW, ops.NHWC, ops.CHWN]
DST = [ops.NCHW, ops.NHWC, ops.CHWN]
SHAPES = [(2, 3, 64, 9, 11), (1, 1, 1, 3, 3), (3, 4, 70, 8, 5), (5, 2, 33, 7, 7), (2, 3, 130, 6, 13), (33, 3, 8, 4, 4)]


@pytest.mark.parametrize("dtype", [ops.F32, ops.F16, ops.BF16])
@pytest.mark.parametrize("shape", SHAPES)
def test_integers_bit_exact(oracle, shape, dtype):
    N, C, K, H, W = shape
    x = synth.small_ints(N * C * H * W, sum(shape), -2, 2).reshape(N, C, H, W)
    w = synth.small_ints(K * C * 9, 7 + sum(shape), -1, 1).reshape(K, C, 3, 3)
    bias = synth.small_ints(K, 3, -2, 2).astype(np.float32)
    for pad in (1, 0):
        for src, dst in itertools.product(SRC, DST):
            xs, ws = synth.act_to_layout(x, src), synth.flt_to_layout(w, src)
            want = synth.act_from_layout(oracle.direct_conv(xs, ws, pad, src, dst), dst) + bias[None, :, None, None]
            want = synth.act_to_layout(np.ascontiguousarray(np.maximum(want, 0).astype(np.float32)), dst)
            got = ops.conv(dev(xs, dtype), dev(ws, dtype), pad, src, dst, algo=ops.ALGO_DIRECT, relu=True,
                           bias=dev(bias, dtype))
            assert np.array_equal(host(got), want), (pad, src, dst)


TILE_SHAPES = [(2, 3, 64, 40, 70), (1, 4, 70, 18, 34), (3, 1, 33, 17, 32), (2, 2, 40, 33, 66), (5, 3, 64, 16, 2), (1, 3, 130, 9, 36), (32, 3, 64, 9, 6), (16, 4, 40, 5, 10)]


@pytest.mark.parametrize("layout", [ops.NCHW, ops.NHWC, ops.CHWN])
@pytest.mark.parametrize("dtype", [ops.F32, ops.F16, ops.BF16])
@pytest.mark.parametrize("shape", TILE_SHAPES)
def test_few_channel_layers_as_tiles_bit_exact(oracle, shape, dtype, layout):
    """fp32 NCHW tensors with an even width run as tiles of 4 rows x 32 columns per wave (input through LDS).
    2-byte NCHW (NHWC) tensors with an even width (and an even K) run as tiles of 4 rows x 64 (32) columns per wave
    (input through LDS, sums exchanged between lanes, 4-byte pairs stored), CHWN tensors of up to 32 images as one
    NCHW image of width W * N with taps N columns apart (batches of 1, 2, 3 and 5): several tiles each way with ragged
    last ones, one to four channels, filter counts off the tile of 32 (K = 33 from NHWC: the gathering kernel), pad 0 and 1
    (the patch starts at an even or an odd element), with and without bias and ReLU; a view that is only element
    aligned takes the gathering kernel and gives the same bits."""
    N, C, K, H, W = shape
    x = synth.small_ints(N * C * H * W, sum(shape), -2, 2).reshape(N, C, H, W)
    w = synth.small_ints(K * C * 9, 7 + sum(shape), -1, 1).reshape(K, C, 3, 3)
    bias = synth.small_ints(K, 3, -2, 2).astype(np.float32)
    xs, ws = synth.act_to_layout(x, layout), synth.flt_to_layout(w, layout)
    for pad in (1, 0):
        if H + 2 * pad < 3 or W + 2 * pad < 3:
            continue
        plain = oracle.direct_conv(xs, ws, pad, layout, layout)
        got = ops.conv(dev(xs, dtype), dev(ws, dtype), pad, layout, algo=ops.ALGO_DIRECT)
        assert np.array_equal(host(got), plain), pad
        want = np.maximum(synth.act_from_layout(plain, layout) + bias[None, :, None, None], 0).astype(np.float32)
        want = synth.act_to_layout(np.ascontiguousarray(want), layout)
        got = ops.conv(dev(xs, dtype), dev(ws, dtype), pad, layout, algo=ops.ALGO_DIRECT, relu=True, bias=dev(bias, dtype))
        assert np.array_equal(host(got), want), pad
        xd = dev(xs, dtype)
        shifted = torch.empty(xd.numel() + 1, dtype=xd.dtype, device="cuda")[1:].view(xd.shape)
        shifted.copy_(xd)
        got2 = ops.conv(shifted, dev(ws, dtype), pad, layout, algo=ops.ALGO_DIRECT, relu=True, bias=dev(bias, dtype))
        assert torch.equal(got2, got), pad


@pytest.mark.parametrize("dtype", [ops.F32, ops.BF16])
@pytest.mark.parametrize("layout", DST)
def test_floats_within_tolerance_and_auto_takes_the_path(oracle, layout, dtype):
    N, C, K, H = 4, 3, 64, 40
    x, w = synth.conv_inputs(N, C, K, H, H, seed=77, layout=layout)
    xr, wr = rounded(x, dtype, oracle), rounded(w, dtype, oracle)
    want = oracle.direct_conv(xr, wr, 1, layout)
    got = ops.conv(dev(xr, dtype), dev(wr, dtype), 1, layout, algo=ops.ALGO_DIRECT)
    assert oracle.rel_l2(host(got), want) <= (1e-6 if dtype == ops.F32 else TOL[dtype])
    assert ops.pick_algo(layout, dtype, N, C, K, H, H) == ops.ALGO_DIRECT
    assert torch.equal(ops.conv(dev(xr, dtype), dev(wr, dtype), 1, layout), got)
    # the Winograd paths agree with it within their own rounding
    fused = ops.conv(dev(xr, dtype), dev(wr, dtype), 1, layout, algo=ops.ALGO_FUSED)
    assert oracle.rel_l2(host(fused), host(got)) <= (1e-5 if dtype == ops.F32 else TOL[dtype])


POOLED_SHAPES = [(2, 3, 64, 40, 70), (1, 4, 70, 18, 34), (3, 1, 33, 17, 32), (2, 2, 40, 33, 66), (32, 3, 64, 9, 6), (8, 3, 16, 2, 3)]


@pytest.mark.parametrize("layout", [ops.NCHW, ops.NHWC, ops.CHWN])
@pytest.mark.parametrize("dtype", [ops.F32, ops.F16, ops.BF16])
@pytest.mark.parametrize("shape", POOLED_SHAPES)
def test_pooled_few_channel_layers_bit_exact(oracle, shape, dtype, layout):
    """Bias, ReLU and 2x2 pooling on a layer of at most four channels: the direct kernel writes the unpooled tensor into
    scratch and a pooling kernel follows (rows of planes for NCHW, 16-byte pieces where the width allows; vectors of the
    contiguous axis for NHWC and CHWN).  Odd output heights and widths drop their last row and column; pad 0 and 1.
    Integers: bit-exact against the pooled oracle; the automatic choice runs the same kernels."""
    N, C, K, H, W = shape
    x = synth.small_ints(N * C * H * W, sum(shape), -2, 2).reshape(N, C, H, W)
    w = synth.small_ints(K * C * 9, 7 + sum(shape), -1, 1).reshape(K, C, 3, 3)
    bias = synth.small_ints(K, 3, -2, 2).astype(np.float32)
    xs, ws = synth.act_to_layout(x, layout), synth.flt_to_layout(w, layout)
    for pad in (1, 0):
        Ho, Wo = H + 2 * pad - 2, W + 2 * pad - 2
        if Ho < 2 or Wo < 2:
            continue
        full = np.maximum(oracle.direct_conv(x, w, pad) + bias[None, :, None, None], 0).astype(np.float32)
        Hp, Wp = Ho // 2, Wo // 2
        want = full[:, :, :2 * Hp, :2 * Wp].reshape(N, K, Hp, 2, Wp, 2).max(axis=(3, 5))
        want = synth.act_to_layout(np.ascontiguousarray(want), layout)
        got = ops.conv(dev(xs, dtype), dev(ws, dtype), pad, layout, algo=ops.ALGO_DIRECT, relu=True, pool=True, bias=dev(bias, dtype))
        assert np.array_equal(host(got), want), pad
        auto = ops.conv(dev(xs, dtype), dev(ws, dtype), pad, layout, relu=True, pool=True, bias=dev(bias, dtype))
        assert torch.equal(auto, got), pad


def test_what_the_path_is_not_built_for():
    x = torch.zeros((1, 3, 8, 8), device="cuda")
    w = torch.zeros((4, 3, 3, 3), device="cuda")
    with pytest.raises(_lib.WinoError) as e:         # five channels and more output pixels than the small-layer kernel takes
        ops.conv(torch.zeros((64, 5, 58, 58), device="cuda"), torch.zeros((64, 5, 3, 3), device="cuda"), algo=ops.ALGO_DIRECT)
    assert e.value.code == -2
    U = ops.filter_transform(w)
    with pytest.raises(_lib.WinoError) as e:         # transformed filters only
        ops.conv_prepared(x, U, 4, algo=ops.ALGO_DIRECT)
    assert e.value.code == -1
    ops.conv_prepared(x, U, 4)


@pytest.mark.parametrize("dtype", [ops.F32, ops.BF16])
def test_direct_with_the_largest_filter_bank_that_fits_lds(oracle, dtype):
    """K = 544 at C = 3: 17 filter tiles, 63 KB of LDS in fp32 (the few-channel kernel is offered up to 64 KB); K = 576
    no longer fits: by name a 2-byte layer is refused, an fp32 one this small runs on the small-layer kernel.  The
    automatic choice keeps a layer of 90 pixels and this many filters on the Winograd kernels.  Integers: bit-exact
    every way."""
    from gpu_util import dev, host
    N, C, H, W = 1, 3, 9, 10
    for K in (544, 576):
        x, w = synth.conv_inputs(N, C, K, H, W, seed=K, integer=True)
        want = oracle.direct_conv(x, w, 1)
        assert ops.pick_algo(ops.NCHW, dtype, N, C, K, H, W) != ops.ALGO_DIRECT
        assert np.array_equal(host(ops.conv(dev(x, dtype), dev(w, dtype), 1, ops.NCHW)), want)
        if K == 544 or dtype == ops.F32:
            assert np.array_equal(host(ops.conv(dev(x, dtype), dev(w, dtype), 1, ops.NCHW, algo=ops.ALGO_DIRECT)), want)
        else:
            with pytest.raises(_lib.WinoError) as e:
                ops.conv(dev(x, dtype), dev(w, dtype), 1, ops.NCHW, algo=ops.ALGO_DIRECT)
            assert e.value.code == -2


FEW_SHAPES = [(1, 64, 64, 12, 16), (2, 7, 40, 6, 6), (1, 130, 70, 9, 11), (3, 36, 100, 13, 5), (1, 5, 33, 7, 20), (1, 8, 32, 3, 3), (2, 12, 30, 5, 9)]


@pytest.mark.parametrize("shape", FEW_SHAPES)
def test_fp32_layers_with_few_pixels_bit_exact_on_integers(oracle, shape):
    """direct_few_pixels_kernel: any number of channels in fp32 while the layer has few output pixels.  Channel counts
    that are and are not multiples of 4 (16-byte and element-wise filter loads; from CHWN the pieces run along the
    filters, so K = 30 takes the element-wise path there), of 32 (the waves' share of the reduction), filter counts off
    the tile of 32, images off the 4 x 8 pixel tile, all nine layout pairs, pad 0 to 3."""
    N, C, K, H, W = shape
    x = synth.small_ints(N * C * H * W, sum(shape), -2, 2).reshape(N, C, H, W)
    w = synth.small_ints(K * C * 9, 7 + sum(shape), -1, 1).reshape(K, C, 3, 3)
    bias = synth.small_ints(K, 3, -2, 2).astype(np.float32)
    for pad in (1, 0, 2, 3):
        if H + 2 * pad < 3 or W + 2 * pad < 3:
            continue
        for src, dst in itertools.product(SRC, DST):
            xs, ws = synth.act_to_layout(x, src), synth.flt_to_layout(w, src)
            want = synth.act_from_layout(oracle.direct_conv(xs, ws, pad, src, dst), dst) + bias[None, :, None, None]
            want = synth.act_to_layout(np.ascontiguousarray(np.maximum(want, 0).astype(np.float32)), dst)
            got = ops.conv(dev(xs), dev(ws), pad, src, dst, algo=ops.ALGO_DIRECT, relu=True, bias=dev(bias))
            assert np.array_equal(host(got), want), (pad, src, dst)
            plain = ops.conv(dev(xs), dev(ws), pad, src, dst, algo=ops.ALGO_DIRECT)
            assert np.array_equal(host(plain), oracle.direct_conv(xs, ws, pad, src, dst)), (pad, src, dst)


@pytest.mark.parametrize("layout", DST)
def test_the_first_layer_of_the_references_sweep_at_batch_one(oracle, layout):
    """N = 1, C = K = 64, 56 x 56 (comparison/layoutCompare.cu:38-46 at batch 1): AUTO runs it as one launch of the
    small-layer kernel; floats within the fp32 tolerance of the oracle, and the Winograd pipeline agrees."""
    N, C, K, H = 1, 64, 64, 56
    x, w = synth.conv_inputs(N, C, K, H, H, seed=5, layout=layout)
    want = oracle.direct_conv(x, w, 1, layout)
    got = ops.conv(dev(x), dev(w), 1, layout, algo=ops.ALGO_DIRECT)
    assert oracle.rel_l2(host(got), want) <= 1e-6
    assert ops.pick_algo(layout, ops.F32, N, C, K, H, H) == ops.ALGO_DIRECT
    assert torch.equal(ops.conv(dev(x), dev(w), 1, layout), got)
    staged = ops.conv(dev(x), dev(w), 1, layout, algo=ops.ALGO_STAGED)
    assert oracle.rel_l2(host(staged), host(got)) <= 1e-5
