"""Pins the oracle's direct convolution (oracle/wino_oracle.c) without the reference.

Checks: a float64 library cross-correlation, a pure-Python brute force, and the
closed-form cases (delta filter, all-ones, one hot pixel) -- each would fail
for a flipped filter, a transposed index, a wrong padding offset or a dropped
term.  Covers the three layouts and the six cross-layout pairs of
comparison/DataLayoutTrans.cuh:594-651.
"""
import itertools

import numpy as np
import pytest
import torch

from cudnntest_amd import synth

LAYOUTS = [0, 1, 2]
SHAPES = [(2, 3, 4, 5, 5), (1, 8, 8, 6, 6), (3, 5, 7, 9, 9), (1, 1, 1, 4, 4), (2, 4, 3, 7, 10)]


def torch_conv(x_nchw, w_kcrs, pad):
    y = torch.nn.functional.conv2d(torch.from_numpy(x_nchw).double(), torch.from_numpy(w_kcrs).double(),
                                   padding=pad)
    return y.numpy()


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("pad", [0, 1, 2, 3])
def test_direct_vs_library_all_layout_pairs(oracle, shape, pad):
    N, C, K, H, W = shape
    if pad == 0 and min(H, W) < 3:
        pytest.skip("no output")
    x, w = synth.conv_inputs(N, C, K, H, W, seed=sum(shape) + pad)
    want = torch_conv(x, w, pad)
    for src, dst in itertools.product(LAYOUTS, LAYOUTS):
        xs, ws = synth.act_to_layout(x, src), synth.flt_to_layout(w, src)
        y = oracle.direct_conv(xs, ws, pad, src, dst)
        got = synth.act_from_layout(y, dst)
        assert got.shape == want.shape
        np.testing.assert_allclose(got, want, rtol=2e-6, atol=2e-6)
        # the fp32 baseline variant computes the same function
        y32 = oracle.direct_conv_f32(xs, ws, pad, src, dst)
        np.testing.assert_allclose(synth.act_from_layout(y32, dst), want, rtol=1e-4, atol=1e-5)


def test_direct_vs_python_brute_force(oracle):
    N, C, K, H, W, pad = 1, 2, 2, 4, 5, 1
    x, w = synth.conv_inputs(N, C, K, H, W, seed=5, integer=True)
    want = np.zeros((N, K, H, W), np.float32)
    for n, k, i, j in itertools.product(range(N), range(K), range(H), range(W)):
        acc = 0.0
        for c, r, s in itertools.product(range(C), range(3), range(3)):
            ih, iw = i + r - pad, j + s - pad
            if 0 <= ih < H and 0 <= iw < W:
                acc += float(x[n, c, ih, iw]) * float(w[k, c, r, s])
        want[n, k, i, j] = acc
    assert np.array_equal(oracle.direct_conv(x, w, pad), want)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_delta_filter_is_identity(oracle, layout):
    N, C, H, W = 2, 5, 6, 7
    x, _ = synth.conv_inputs(N, C, C, H, W, seed=3)
    w = np.zeros((C, C, 3, 3), np.float32)
    for c in range(C):
        w[c, c, 1, 1] = 1.0
    y = oracle.direct_conv(synth.act_to_layout(x, layout), synth.flt_to_layout(w, layout), 1, layout)
    assert np.array_equal(synth.act_from_layout(y, layout), x)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_all_ones_counts_taps(oracle, layout):
    N, C, K, H, W = 1, 7, 3, 5, 6
    x = np.ones((N, C, H, W), np.float32)
    w = np.ones((K, C, 3, 3), np.float32)
    y = synth.act_from_layout(
        oracle.direct_conv(synth.act_to_layout(x, layout), synth.flt_to_layout(w, layout), 1, layout), layout)
    assert np.all(y[:, :, 1:-1, 1:-1] == 9 * C)
    assert np.all(y[:, :, 0, 1:-1] == 6 * C) and np.all(y[:, :, 1:-1, 0] == 6 * C)
    assert np.all(y[:, :, [0, 0, -1, -1], [0, -1, 0, -1]] == 4 * C)


def test_hot_pixel_stamps_flipped_filter(oracle):
    # correlation: a single 1 at (2,3) paints w rotated by 180 degrees around it
    H = W = 6
    x = np.zeros((1, 1, H, W), np.float32)
    x[0, 0, 2, 3] = 1.0
    w = np.arange(1, 10, dtype=np.float32).reshape(1, 1, 3, 3)
    y = oracle.direct_conv(x, w, 1)
    assert np.array_equal(y[0, 0, 1:4, 2:5], w[0, 0, ::-1, ::-1])
    assert y.sum() == w.sum()


def test_permutes_roundtrip(oracle):
    x, w = synth.conv_inputs(2, 3, 4, 5, 6, seed=9)
    for a, b in itertools.product(LAYOUTS, LAYOUTS):
        xa = synth.act_to_layout(x, a)
        assert np.array_equal(oracle.permute_act(a, b, xa), synth.act_to_layout(x, b))
        wa = synth.flt_to_layout(w, a)
        assert np.array_equal(oracle.permute_flt(a, b, wa), synth.flt_to_layout(w, b))


def test_rounding_helpers_match_torch(oracle):
    v = np.concatenate([synth.uniform_pm1(4096, 1) * 3.0, synth.normal(4096, 2, 1e-3),
                        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 6e-8, 3e-5, -7.3e-6], np.float32)])
    t = torch.from_numpy(v)
    assert np.array_equal(oracle.round_bf16(v), t.bfloat16().float().numpy())
    assert np.array_equal(oracle.round_f16(v), t.half().float().numpy())


def test_rel_l2(oracle):
    a = np.array([3.0, 4.0], np.float32)
    b = np.array([3.0, 0.0], np.float32)
    assert oracle.rel_l2(a, a) == 0.0
    assert abs(oracle.rel_l2(a, b) - 4.0 / 3.0) < 1e-12
