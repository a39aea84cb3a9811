"""Bias, ReLU and 2x2 max pooling applied in the output stage (wino_conv_ex), through the C ABI,
against the CPU oracle's direct convolution followed by the same three steps in NumPy.  The reference
runs them as separate passes over y (addBias_CHWN, relu_CHWN, maxPool_CHWN in
netTest/cudnn_test_0124/VGG_Batched/CHWN_support.cuh:107,512,248): bias per filter, then max(.,0), then
2x2 windows of stride 2 (a window cut by the border is dropped)."""
import itertools

import numpy as np
import pytest
import torch

from cudnntest_amd import _lib, ops, synth
from gpu_util import TOL, dev, host, rounded

pytestmark = pytest.mark.gpu
LAYOUTS = [ops.NCHW, ops.NHWC, ops.CHWN]
ALGOS = [ops.ALGO_STAGED, ops.ALGO_EPILOGUE, ops.ALGO_FUSED]


def expected(oracle, x, w, bias, pad, src, dst, relu, pool):
    """x, w in src's conventions -> y in dst's; all arithmetic in float64 after the oracle's convolution."""
    y = synth.act_from_layout(oracle.direct_conv(x, w, pad, src, dst), dst).astype(np.float64)   # NCHW
    if bias is not None:
        y = y + bias.astype(np.float64)[None, :, None, None]
    if relu:
        y = np.maximum(y, 0)
    if pool:
        N, K, Ho, Wo = y.shape
        y = y[:, :, :Ho // 2 * 2, :Wo // 2 * 2].reshape(N, K, Ho // 2, 2, Wo // 2, 2).max(axis=(3, 5))
    return synth.act_to_layout(np.ascontiguousarray(y.astype(np.float32)), dst)


@pytest.mark.parametrize("algo", ALGOS)
@pytest.mark.parametrize("shape", [(2, 5, 7, 8, 8), (1, 16, 70, 9, 7), (3, 32, 20, 6, 10), (2, 3, 4, 5, 5)])
def test_bias_relu_pool_bit_exact_on_integers(oracle, algo, shape):
    N, C, K, H, W = shape
    x, w = synth.conv_inputs(N, C, K, H, W, seed=77 + sum(shape), integer=True)
    bias = synth.small_ints(K, seed=5, lo=-4, hi=4).astype(np.float32)
    for src, dst in itertools.product(LAYOUTS, LAYOUTS):
        xs, ws = synth.act_to_layout(x, src), synth.flt_to_layout(w, src)
        for relu, pool, with_bias in [(True, True, True), (False, True, False), (True, False, True), (False, False, True)]:
            b = bias if with_bias else None
            want = expected(oracle, xs, ws, b, 1, src, dst, relu, pool)
            got = host(ops.conv(dev(xs), dev(ws), 1, src, dst, algo, relu=relu, pool=pool,
                                bias=dev(b) if with_bias else None))
            assert got.shape == want.shape, (src, dst, relu, pool)
            assert np.array_equal(got, want), (src, dst, relu, pool, with_bias)


@pytest.mark.parametrize("algo", ALGOS)
def test_pad0_odd_output_drops_the_cut_windows(oracle, algo):
    N, C, K, H, W = 2, 6, 5, 9, 8          # pad 0: 7 x 6 outputs -> 3 x 3 pooled
    x, w = synth.conv_inputs(N, C, K, H, W, seed=3, integer=True)
    bias = synth.small_ints(K, seed=9, lo=-2, hi=2).astype(np.float32)
    want = expected(oracle, x, w, bias, 0, ops.NCHW, ops.NCHW, True, True)
    got = host(ops.conv(dev(x), dev(w), 0, algo=algo, relu=True, pool=True, bias=dev(bias)))
    assert got.shape == (N, K, 3, 3)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", [ops.F32, ops.F16, ops.BF16])
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("algo", ALGOS)
def test_floats_within_tolerance(oracle, algo, layout, dtype):
    N, C, K, H, W = 2, 64, 48, 28, 28
    x, w = synth.conv_inputs(N, C, K, H, W, seed=404, layout=layout)
    bias = synth.normal(K, seed=11, std=0.5).astype(np.float32)
    xr, wr, br = rounded(x, dtype, oracle), rounded(w, dtype, oracle), rounded(bias, dtype, oracle)
    want = expected(oracle, xr, wr, br, 1, layout, layout, True, True)
    got = host(ops.conv(dev(xr, dtype), dev(wr, dtype), 1, layout, algo=algo, relu=True, pool=True,
                        bias=dev(br, dtype)))
    assert oracle.rel_l2(got, want) <= TOL[dtype]


@pytest.mark.parametrize("f4_algo", [ops.ALGO_STAGED_F4, ops.ALGO_EPILOGUE_F4])
@pytest.mark.parametrize("shape", [(2, 5, 7, 8, 8), (1, 16, 70, 9, 7), (3, 32, 20, 6, 10), (2, 24, 40, 13, 18)])
def test_f4_bias_relu_pool_every_layout_pair(oracle, shape, f4_algo):
    """The F(4x4,3x3) pipeline's output stage: the same three steps, 2x2 pooled values per 4x4 tile.  Its transforms
    hold sixths and twenty-fourths, so integers do not come out bit for bit: the layer tolerance (relative L2 1e-4 in
    fp32) applies, and the pooled and unpooled shapes are checked."""
    N, C, K, H, W = shape
    x, w = synth.conv_inputs(N, C, K, H, W, seed=177 + sum(shape))
    bias = synth.normal(K, seed=15, std=0.5).astype(np.float32)
    for src, dst in itertools.product(LAYOUTS, LAYOUTS):
        xs, ws = synth.act_to_layout(x, src), synth.flt_to_layout(w, src)
        for relu, pool, with_bias in [(True, True, True), (False, True, False), (True, False, True), (False, False, True)]:
            b = bias if with_bias else None
            want = expected(oracle, xs, ws, b, 1, src, dst, relu, pool)
            got = host(ops.conv(dev(xs), dev(ws), 1, src, dst, f4_algo, relu=relu, pool=pool,
                                bias=dev(b) if with_bias else None))
            assert got.shape == want.shape, (src, dst, relu, pool)
            assert oracle.rel_l2(got, want) <= TOL[ops.F32], (src, dst, relu, pool, with_bias)


@pytest.mark.parametrize("f4_algo", [ops.ALGO_STAGED_F4, ops.ALGO_EPILOGUE_F4])
def test_f4_pad0_odd_output_drops_the_cut_windows(oracle, f4_algo):
    N, C, K, H, W = 2, 6, 5, 9, 8          # pad 0: 7 x 6 outputs -> 3 x 3 pooled; the last tile row holds one pooled row
    x, w = synth.conv_inputs(N, C, K, H, W, seed=3)
    bias = synth.normal(K, seed=9, std=0.5).astype(np.float32)
    want = expected(oracle, x, w, bias, 0, ops.NCHW, ops.NCHW, True, True)
    got = host(ops.conv(dev(x), dev(w), 0, algo=f4_algo, relu=True, pool=True, bias=dev(bias)))
    assert got.shape == (N, K, 3, 3)
    assert oracle.rel_l2(got, want) <= TOL[ops.F32]
    # the stage function takes the pooling flag (no bias)
    g = ops.f4_geometry(ops.F32, N, C, K, H, W, 0)
    Mo = ops.f4_batched_gemm(ops.f4_filter_transform(dev(w)), ops.f4_input_transform(dev(x), 0), C, K, g["P"])
    want_nb = expected(oracle, x, w, None, 0, ops.NCHW, ops.NCHW, True, True)
    assert oracle.rel_l2(host(ops.f4_output_transform(Mo, N, K, 7, 6, relu=True, pool=True)), want_nb) <= TOL[ops.F32]


def test_prepared_filters_and_stage_functions(oracle):
    N, C, K, H = 2, 16, 24, 12
    x, w = synth.conv_inputs(N, C, K, H, H, seed=8, integer=True)
    bias = synth.small_ints(K, seed=2, lo=-3, hi=3).astype(np.float32)
    xd, wd, bd = dev(x), dev(w), dev(bias)
    U = ops.filter_transform(wd)
    want = expected(oracle, x, w, bias, 1, ops.NCHW, ops.NCHW, True, True)
    assert np.array_equal(host(ops.conv_prepared(xd, U, K, relu=True, pool=True, bias=bd)), want)
    # the stage functions take the pooling flag (no bias)
    V = ops.input_transform(xd)
    want_nb = expected(oracle, x, w, None, 1, ops.NCHW, ops.NCHW, True, True)
    assert np.array_equal(host(ops.gemm_output(U, V, N, C, K, H, H, relu=True, pool=True)), want_nb)
    g = ops.geometry(ops.F32, N, C, K, H, H, 1)
    Mo = ops.batched_gemm(U, V, C, K, g["P"])
    assert np.array_equal(host(ops.output_transform(Mo, N, K, H, H, relu=True, pool=True)), want_nb)


def test_rejected_requests():
    x = torch.zeros((1, 4, 8, 8), device="cuda")
    w = torch.zeros((4, 4, 3, 3), device="cuda")
    with pytest.raises(TypeError):
        ops.conv(x, w, bias=torch.zeros(5, device="cuda"))           # K = 4
    with pytest.raises(ValueError):
        ops.conv(x, w, pool=True, out=torch.zeros((1, 4, 8, 8), device="cuda"))
