"""Zero padding of more than one row and column.  The reference's wrapped convolutions take `padding` as an
argument and honour it arithmetically (comparison/wrapedConv_NCHW.cuh:346-362: the output is
inside + 2*padding - 2 wide, tiles start at 2*tile - padding), although its drivers only ever pass 1.  Here the
Winograd pipelines take any padding; the single-kernel and the direct paths are built for 0 and 1 and say so.
Oracle: the CPU direct convolution and the CPU input transforms, bit for bit on small integers."""
import itertools

import numpy as np
import pytest

from cudnntest_amd import ops, synth
from cudnntest_amd._lib import WinoError
from gpu_util import batch_minor_perm, dev, host, rounded, unpack_operand

pytestmark = pytest.mark.gpu
LAYOUTS = [ops.NCHW, ops.NHWC, ops.CHWN]

# shapes that reach every input-transform kernel: NCHW small-image and tiled (F(2x2): more than 256 tiles an image;
# F(4x4): 128 and more), NHWC with whole channel vectors, ragged channels, CHWN
STAGE_SHAPES = [((2, 5, 8, 7), 2), ((3, 16, 12, 12), 3), ((1, 24, 34, 34), 2), ((2, 8, 46, 44), 2), ((2, 40, 20, 30), 5),
                ((1, 3, 3, 3), 4)]


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("order", [ops.TILES_BATCH_MAJOR, ops.TILES_BATCH_MINOR])
@pytest.mark.parametrize("shape,pad", STAGE_SHAPES)
@pytest.mark.parametrize("m", [2, 4])
def test_input_transforms_with_wide_padding(oracle, layout, order, shape, pad, m):
    N, C, H, W = shape
    x = synth.small_ints(N * C * H * W, 5 + sum(shape) + pad, -8, 8).reshape(N, C, H, W)
    xl = synth.act_to_layout(x, layout)
    fn = ops.input_transform if m == 2 else ops.f4_input_transform
    V = unpack_operand(fn(dev(xl), pad, layout, order))
    want = oracle.wino_input_transform(xl, pad, layout, m=m)
    th, tw = oracle.wino_tiles(m, H, W, pad)
    P = N * th * tw
    got = V[:, :C, :P]
    if order == ops.TILES_BATCH_MINOR:
        got = got[:, :, np.argsort(batch_minor_perm(N, th, tw))]
    assert np.array_equal(got, want)
    assert not V[:, C:, :P].any(), "channel padding must be zero"


@pytest.mark.parametrize("dtype", [ops.F16, ops.BF16])
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("shape,pad", [((2, 16, 12, 12), 2), ((1, 24, 34, 34), 3), ((2, 9, 10, 8), 2)])
def test_two_byte_input_transforms_with_wide_padding(oracle, dtype, layout, shape, pad):
    N, C, H, W = shape
    x = synth.small_ints(N * C * H * W, 9 + sum(shape), -8, 8).reshape(N, C, H, W)
    xl = synth.act_to_layout(x, layout)
    V = unpack_operand(ops.input_transform(dev(xl, dtype), pad, layout, ops.TILES_BATCH_MAJOR), dtype)
    th, tw = oracle.wino_tiles(2, H, W, pad)
    assert np.array_equal(V[:, :C, :N * th * tw], oracle.wino_input_transform(xl, pad, layout))


@pytest.mark.parametrize("algo", [ops.ALGO_AUTO, ops.ALGO_STAGED, ops.ALGO_EPILOGUE])
@pytest.mark.parametrize("shape,pad", [((2, 3, 4, 5, 5), 2), ((2, 16, 130, 7, 10), 3), ((1, 64, 70, 8, 4), 2),
                                       ((3, 5, 7, 9, 9), 4), ((1, 1, 1, 1, 1), 1), ((1, 2, 3, 1, 2), 2)])
def test_whole_layer_all_layout_pairs(oracle, algo, shape, pad):
    N, C, K, H, W = shape
    x, w = synth.conv_inputs(N, C, K, H, W, seed=sum(shape) + pad, integer=True)
    for src, dst in itertools.product(LAYOUTS, LAYOUTS):
        xs, ws = synth.act_to_layout(x, src), synth.flt_to_layout(w, src)
        want = oracle.direct_conv(xs, ws, pad, src, dst)
        got = host(ops.conv(dev(xs), dev(ws), pad, src, dst, algo))
        assert got.shape == want.shape and np.array_equal(got, want), (src, dst)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_f4_pipeline_and_epilogue_flags(oracle, layout):
    N, C, K, H, W, pad = 2, 20, 24, 13, 11, 2
    x, w = synth.conv_inputs(N, C, K, H, W, seed=77, layout=layout)
    want = oracle.direct_conv(x, w, pad, layout)
    got = host(ops.conv(dev(x), dev(w), pad, layout, algo=ops.ALGO_STAGED_F4))
    assert oracle.rel_l2(got, want) <= 2e-5
    # bias, ReLU and 2x2 pooling after a padding of 2, on an F(2x2) pipeline (integers: exact)
    xi, wi = synth.conv_inputs(N, C, K, H, W, seed=78, layout=layout, integer=True)
    bi = synth.small_ints(K, 4, -5, 5).astype(np.float32)
    full = synth.act_from_layout(oracle.direct_conv(xi, wi, pad, layout), layout) + bi[None, :, None, None]
    full = np.maximum(full, 0)
    Ho, Wo = H + 2 * pad - 2, W + 2 * pad - 2
    pooled = full[:, :, :Ho // 2 * 2, :Wo // 2 * 2].reshape(N, K, Ho // 2, 2, Wo // 2, 2).max(axis=(3, 5))
    for algo in (ops.ALGO_STAGED, ops.ALGO_EPILOGUE, ops.ALGO_STAGED_F4):
        got = host(ops.conv(dev(xi), dev(wi), pad, layout, algo=algo, relu=True, bias=dev(bi), pool=True))
        got = synth.act_from_layout(got, layout)
        if algo == ops.ALGO_STAGED_F4:
            np.testing.assert_allclose(got, pooled, rtol=1e-5, atol=1e-3)
        else:
            assert np.array_equal(got, pooled), algo


@pytest.mark.parametrize("dtype", [ops.F16, ops.BF16])
def test_two_byte_layer_with_wide_padding(oracle, dtype):
    """A layer AUTO would hand to the 16-bit direct kernel at pad 1 stays on the Winograd kernels at pad 2."""
    N, C, K, H, W, pad = 2, 64, 64, 60, 60, 2
    x, w = synth.conv_inputs(N, C, K, H, W, seed=12, integer=True)
    want = rounded(oracle.direct_conv(x, w, pad), dtype, oracle)
    got = host(ops.conv(dev(x, dtype), dev(w, dtype), pad))
    assert np.array_equal(got, want)
    with pytest.raises(WinoError):
        ops.conv(dev(x, dtype), dev(w, dtype), pad, algo=ops.ALGO_DIRECT)


def test_paths_built_for_one_ring_of_padding_refuse(oracle):
    N, C, K, H, W = 16, 64, 64, 40, 40
    x, w = synth.conv_inputs(N, C, K, H, W, seed=5, integer=True)
    assert ops.pick_algo(ops.NCHW, ops.F32, N, C, K, H, W, 1) == ops.ALGO_FUSED   # what AUTO takes at pad 1
    with pytest.raises(WinoError):
        ops.conv(dev(x), dev(w), 2, algo=ops.ALGO_FUSED)
    got = host(ops.conv(dev(x), dev(w), 2))                                        # AUTO: a pipeline that can
    assert np.array_equal(got, oracle.direct_conv(x, w, 2))
    x3, w3 = synth.conv_inputs(2, 3, 16, 20, 20, seed=6, integer=True)             # C <= 4: the direct kernel at pad 1;
    with pytest.raises(WinoError):                                                 # 2-byte tensors: nothing direct at pad 2
        ops.conv(dev(x3, ops.BF16), dev(w3, ops.BF16), 2, algo=ops.ALGO_DIRECT)
    got = host(ops.conv(dev(x3), dev(w3), 2, algo=ops.ALGO_DIRECT))                # fp32: the small-layer kernel, any padding
    assert np.array_equal(got, oracle.direct_conv(x3, w3, 2))
    assert np.array_equal(host(ops.conv(dev(x3), dev(w3), 2)), oracle.direct_conv(x3, w3, 2))
    with pytest.raises(WinoError):
        ops.conv(dev(x3), dev(w3), 1025)
