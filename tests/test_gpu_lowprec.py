"""f16 / bf16 storage with fp32 accumulation (the reference has no such path:
its wrappers are float-only, comparison/wrapedConv_NCHW.cuh:335).  Oracle:
the fp32 direct convolution fed the same, already-rounded inputs and weights;
tolerance 2e-2 relative L2 for a whole layer.  On small integers every value
stays representable, so stages and whole layers must be bit-exact."""
import itertools

import numpy as np
import pytest
import torch

from cudnntest_amd import ops, synth
from gpu_util import TOL, batch_minor_perm, dev, host, pack_operand, rounded, unpack_operand

pytestmark = pytest.mark.gpu
LAYOUTS = [ops.NCHW, ops.NHWC, ops.CHWN]
DTYPES = [ops.F16, ops.BF16]
ALGOS = [ops.ALGO_STAGED, ops.ALGO_EPILOGUE, ops.ALGO_FUSED]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layout", LAYOUTS)
def test_filter_and_input_transform_exact_on_integers(oracle, dtype, layout):
    K, C, N, H, W = 20, 19, 2, 9, 7
    w = synth.small_ints(K * C * 9, 3, -2, 2).reshape(K, C, 3, 3)
    wl = synth.flt_to_layout(w, layout)
    U = unpack_operand(ops.filter_transform(dev(wl, dtype), layout))
    assert np.array_equal(U[:, :C, :K], oracle.wino_filter_transform(wl, layout))
    assert not U[:, C:, :].any() and not U[:, :, K:].any()
    x = synth.small_ints(N * C * H * W, 4, -4, 4).reshape(N, C, H, W)
    xl = synth.act_to_layout(x, layout)
    for order in (ops.TILES_BATCH_MAJOR, ops.TILES_BATCH_MINOR):
        V = unpack_operand(ops.input_transform(dev(xl, dtype), 1, layout, order))
        th, tw = oracle.wino_tiles(2, H, W, 1)
        got = V[:, :C, :N * th * tw]
        if order == ops.TILES_BATCH_MINOR:
            got = got[:, :, np.argsort(batch_minor_perm(N, th, tw))]
        assert np.array_equal(got, oracle.wino_input_transform(xl, 1, layout))
        assert not V[:, C:, :N * th * tw].any()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,K,P", [(16, 128, 128), (3, 5, 30), (48, 130, 300), (256, 64, 512)])
def test_batched_gemm_exact_on_integers(oracle, dtype, C, K, P):
    g = ops.geometry(dtype, 1, C, K, 4, 4, 1)
    Cp, Kp = g["Cp"], g["Kp"]
    Pp = (P + 127) // 128 * 128
    U = np.zeros((16, Cp, Kp), np.float32)
    V = np.zeros((16, Cp, Pp), np.float32)
    U[:, :C, :K] = synth.small_ints(16 * C * K, 3, -3, 3).reshape(16, C, K)
    V[:, :C, :P] = synth.small_ints(16 * C * P, 4, -5, 5).reshape(16, C, P)
    Mo = host(ops.batched_gemm(pack_operand(U, dtype), pack_operand(V, dtype), C, K, P))
    want = oracle.wino_gemm(np.ascontiguousarray(U[:, :C, :K]), np.ascontiguousarray(V[:, :C, :P]))
    assert np.array_equal(Mo[:, :K, :P], want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("algo", ALGOS)
def test_small_integer_layers_bit_exact(oracle, dtype, algo):
    # |y| <= 9*C*2*1 = 36 with C = 2: representable in bf16
    N, C, K, H, W = 3, 2, 70, 9, 6
    x = synth.small_ints(N * C * H * W, 5, -2, 2).reshape(N, C, H, W)
    w = synth.small_ints(K * C * 9, 6, -1, 1).reshape(K, C, 3, 3)
    for src, dst in itertools.product(LAYOUTS, LAYOUTS):
        xs, ws = synth.act_to_layout(x, src), synth.flt_to_layout(w, src)
        got = host(ops.conv(dev(xs, dtype), dev(ws, dtype), 1, src, dst, algo))
        assert np.array_equal(got, oracle.direct_conv(xs, ws, 1, src, dst)), (src, dst)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("algo", ALGOS)
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("shape", [(2, 64, 64, 28, 28), (1, 3, 64, 32, 32), (4, 256, 128, 14, 14), (2, 40, 24, 9, 11)])
def test_float_layers_within_tolerance(oracle, dtype, algo, layout, shape):
    N, C, K, H, W = shape
    x, w = synth.conv_inputs(N, C, K, H, W, seed=500 + sum(shape), layout=layout)
    xr, wr = rounded(x, dtype, oracle), rounded(w, dtype, oracle)
    want = oracle.direct_conv(xr, wr, 1, layout)
    got = host(ops.conv(dev(xr, dtype), dev(wr, dtype), 1, layout, algo=algo))
    err = oracle.rel_l2(got, want)
    assert err <= TOL[dtype], err
