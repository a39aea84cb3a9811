"""The direct path for layers with at most four input channels (WINO_ALGO_DIRECT; what AUTO picks for
the network's first layer, comparison/layoutCompare.cu:38-46: 3 -> 64 channels).  Oracle: the CPU
direct convolution.  Bit-exact on small integers for all nine layout pairs, with bias and ReLU; within the layer tolerance on floats; 2-byte tensors are
multiplied in fp32 as well."""
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


def test_what_the_path_is_not_built_for():
    x = torch.zeros((1, 3, 8, 8), device="cuda")
    w = torch.zeros((4, 3, 3, 3), device="cuda")
    for kwargs in (dict(pool=True),):
        with pytest.raises(_lib.WinoError) as e:
            ops.conv(x, w, algo=ops.ALGO_DIRECT, **kwargs)
        assert e.value.code == -2
        ops.conv(x, w, **kwargs)                     # AUTO falls back to the Winograd kernels
    with pytest.raises(_lib.WinoError) as e:         # five channels
        ops.conv(torch.zeros((1, 5, 8, 8), device="cuda"), torch.zeros((4, 5, 3, 3), device="cuda"), algo=ops.ALGO_DIRECT)
    assert e.value.code == -2
    U = ops.filter_transform(w)
    with pytest.raises(_lib.WinoError) as e:         # transformed filters only
        ops.conv_prepared(x, U, 4, algo=ops.ALGO_DIRECT)
    assert e.value.code == -1
    ops.conv_prepared(x, U, 4)


@pytest.mark.parametrize("dtype", [ops.F32, ops.BF16])
def test_direct_with_the_largest_filter_bank_that_fits_lds(oracle, dtype):
    """K = 544 at C = 3: 17 filter tiles, 63 KB of LDS in fp32 (the path is offered up to 64 KB); K = 576 no
    longer fits and AUTO goes back to the Winograd kernels.  Integers: bit-exact either way."""
    from gpu_util import dev, host
    N, C, H, W = 1, 3, 9, 10
    for K, want_algo in ((544, ops.ALGO_DIRECT), (576, None)):
        x, w = synth.conv_inputs(N, C, K, H, W, seed=K, integer=True)
        got_algo = ops.pick_algo(ops.NCHW, dtype, N, C, K, H, W)
        if want_algo is None:
            assert got_algo != ops.ALGO_DIRECT
        else:
            assert got_algo == want_algo
        y = host(ops.conv(dev(x, dtype), dev(w, dtype), 1, ops.NCHW))
        assert np.array_equal(y, oracle.direct_conv(x, w, 1))
