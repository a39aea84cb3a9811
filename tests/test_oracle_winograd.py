"""Pins the oracle's Winograd stage functions (oracle/wino_oracle.c).

The joint identity  A^T[(G g G^T) . (B^T d B)]A == valid correlation(d, g)  is
exact in rationals; for F(2x2,3x3) every constant is a power of two, so on small
integers it must hold bit-for-bit in fp32 -- a wrong sign, a transposed matrix
or a wrong tile origin breaks it.  Single-stage closed forms pin each stage on
its own, for F(2x2) and for F(4x4) (one-hot taps, pixels and products against outer products of the columns of
G, B^T and A^T), and the tile geometry is checked against the instances the
reference's notebooks print (layoutTest/NCHW/data/ConvTest_V3_NCHW-Mar18.ipynb
cell 2: inside=22 -> blockn=6, M=2304 at N=64).
"""
import itertools

import numpy as np
import pytest

from cudnntest_amd import synth

LAYOUTS = [0, 1, 2]


@pytest.mark.parametrize("shape", [(2, 3, 4, 5, 5), (1, 8, 8, 6, 6), (3, 5, 7, 9, 9), (1, 2, 3, 4, 7), (2, 1, 1, 3, 3)])
@pytest.mark.parametrize("pad", [0, 1])
def test_f2x2_bit_exact_on_integers_all_layout_pairs(oracle, shape, pad):
    N, C, K, H, W = shape
    if pad == 0 and min(H, W) < 3:
        pytest.skip("no output")
    x, w = synth.conv_inputs(N, C, K, H, W, seed=sum(shape), integer=True)
    for src, dst in itertools.product(LAYOUTS, LAYOUTS):
        xs, ws = synth.act_to_layout(x, src), synth.flt_to_layout(w, src)
        want = oracle.direct_conv(xs, ws, pad, src, dst)
        got = oracle.wino_conv(xs, ws, pad, src, dst, m=2)
        assert np.array_equal(got, want), (src, dst)


@pytest.mark.parametrize("m,tol", [(2, 2e-6), (4, 2e-5)])
def test_winograd_close_on_floats(oracle, m, tol):
    N, C, K, H, W = 2, 16, 8, 11, 11
    x, w = synth.conv_inputs(N, C, K, H, W, seed=77)
    want = oracle.direct_conv(x, w, 1)
    got = oracle.wino_conv(x, w, 1, m=m)
    assert oracle.rel_l2(got, want) < tol


def test_f4x4_exact_when_filter_divisible_by_24(oracle):
    # G of F(4x4) has denominators 4, 6, 12, 24: G g G^T is integral when g is a
    # multiple of 24*24 = 576, so the identity is exact again.
    N, C, K, H, W = 1, 3, 2, 8, 8
    x, w = synth.conv_inputs(N, C, K, H, W, seed=4, integer=True)
    w = w * 576.0
    assert np.array_equal(oracle.wino_conv(x, w, 1, m=4), oracle.direct_conv(x, w, 1))


def test_filter_transform_closed_forms(oracle):
    # centre tap only: U = G[:,1] G[:,1]^T ; for F(2x2) G[:,1] = (0, 1/2, -1/2, 0)
    w = np.zeros((1, 1, 3, 3), np.float32)
    w[0, 0, 1, 1] = 1.0
    U = oracle.wino_filter_transform(w, m=2).reshape(4, 4)
    g = np.array([0, .5, -.5, 0])
    assert np.array_equal(U, np.outer(g, g).astype(np.float32))
    # top-left tap only: G[:,0] = (1, 1/2, 1/2, 0)
    w[:] = 0
    w[0, 0, 0, 0] = 1.0
    U = oracle.wino_filter_transform(w, m=2).reshape(4, 4)
    g = np.array([1, .5, .5, 0])
    assert np.array_equal(U, np.outer(g, g).astype(np.float32))
    # row/col asymmetry: tap (0, 2) -> outer(G[:,0], G[:,2]), G[:,2] = (0, 1/2, 1/2, 1)
    w[:] = 0
    w[0, 0, 0, 2] = 1.0
    U = oracle.wino_filter_transform(w, m=2).reshape(4, 4)
    assert np.array_equal(U, np.outer([1, .5, .5, 0], [0, .5, .5, 1]).astype(np.float32))


def test_filter_transform_index_order(oracle):
    # U[xi][c][k]: the k-th filter's c-th channel lands at [:, c, k] in every layout
    K, C = 3, 2
    w = synth.small_ints(K * C * 9, 8).reshape(K, C, 3, 3)
    base = oracle.wino_filter_transform(w, 0, m=2)
    for k, c in itertools.product(range(K), range(C)):
        one = oracle.wino_filter_transform(w[k:k + 1, c:c + 1].copy(), 0, m=2)
        assert np.array_equal(base[:, c, k], one[:, 0, 0])
    for layout in LAYOUTS:
        assert np.array_equal(oracle.wino_filter_transform(synth.flt_to_layout(w, layout), layout, m=2), base)


def test_input_transform_closed_forms(oracle):
    # pad 0, one 4x4 tile of ones: row sums of B^T are (0, 2, 0, 0) -> only V[1][1] = 4
    x = np.ones((1, 1, 4, 4), np.float32)
    V = oracle.wino_input_transform(x, pad=0, m=2).reshape(4, 4)
    want = np.zeros((4, 4), np.float32)
    want[1, 1] = 4
    assert np.array_equal(V, want)
    # a single 1 at d[r][s] gives outer(B^T[:, r], B^T[:, s])
    BT = np.array([[1, 0, -1, 0], [0, 1, 1, 0], [0, -1, 1, 0], [0, 1, 0, -1]], np.float32)
    for r, s in [(0, 0), (1, 2), (3, 1), (2, 3)]:
        x = np.zeros((1, 1, 4, 4), np.float32)
        x[0, 0, r, s] = 1
        V = oracle.wino_input_transform(x, pad=0, m=2).reshape(4, 4)
        assert np.array_equal(V, np.outer(BT[:, r], BT[:, s]))


def test_input_transform_tiling_and_padding(oracle):
    # pad 1, H = W = 5 -> 3x3 tiles with origin (2ty-1, 2tx-1); tile (ty,tx) of
    # image n is column p = (n*3 + ty)*3 + tx and sees zeros outside the image
    N, C, H = 2, 2, 5
    x = synth.small_ints(N * C * H * H, 21).reshape(N, C, H, H)
    V = oracle.wino_input_transform(x, pad=1, m=2)
    assert V.shape == (16, C, N * 9)
    xp = np.pad(x, [(0, 0), (0, 0), (1, 2), (1, 2)])
    for n, c, ty, tx in itertools.product(range(N), range(C), range(3), range(3)):
        d = xp[n, c, 2 * ty:2 * ty + 4, 2 * tx:2 * tx + 4].copy().reshape(1, 1, 4, 4)
        one = oracle.wino_input_transform(d, pad=0, m=2).reshape(16)
        assert np.array_equal(V[:, c, (n * 3 + ty) * 3 + tx], one)
    for layout in LAYOUTS:
        assert np.array_equal(oracle.wino_input_transform(synth.act_to_layout(x, layout), 1, layout, m=2), V)


# F(4x4,3x3): the matrices of comparison/wrapedConv_NCHW.cuh:836-855 (B^T), :879-899 (G), :1084-1101 (A^T), written
# out here as data and used only as the expected values of one-hot probes
BT4 = np.array([[4, 0, -5, 0, 1, 0], [0, -4, -4, 1, 1, 0], [0, 4, -4, -1, 1, 0],
                [0, -2, -1, 2, 1, 0], [0, 2, -1, -2, 1, 0], [0, 4, 0, -5, 0, 1]], np.float64)
G4 = np.array([[1 / 4, 0, 0], [-1 / 6, -1 / 6, -1 / 6], [-1 / 6, 1 / 6, -1 / 6],
               [1 / 24, 1 / 12, 1 / 6], [1 / 24, -1 / 12, 1 / 6], [0, 0, 1]], np.float64)
AT4 = np.array([[1, 1, 1, 1, 1, 0], [0, 1, -1, 2, -2, 0], [0, 1, 1, 4, 4, 0], [0, 1, -1, 8, -8, 1]], np.float64)


def test_f4_filter_transform_one_hot_taps(oracle):
    # a single 1 at tap (r, s) gives outer(G[:, r], G[:, s]): nine probes pin every column of G on both sides
    for r, s in itertools.product(range(3), range(3)):
        w = np.zeros((1, 1, 3, 3), np.float32)
        w[0, 0, r, s] = 1.0
        U = oracle.wino_filter_transform(w, m=4).reshape(6, 6)
        assert np.allclose(U, np.outer(G4[:, r], G4[:, s]), rtol=0, atol=1e-7), (r, s)
    # multiples of 24 make every entry an integer: exact
    w = np.zeros((1, 1, 3, 3), np.float32)
    w[0, 0, 0, 2] = 576.0
    assert np.array_equal(oracle.wino_filter_transform(w, m=4).reshape(6, 6), np.outer(24 * G4[:, 0], 24 * G4[:, 2]).astype(np.float32))
    # index order U[xi][c][k] as for F(2x2)
    K, C = 3, 2
    w = synth.small_ints(K * C * 9, 8).reshape(K, C, 3, 3)
    base = oracle.wino_filter_transform(w, 0, m=4)
    assert base.shape == (36, C, K)
    for k, c in itertools.product(range(K), range(C)):
        assert np.array_equal(base[:, c, k], oracle.wino_filter_transform(w[k:k + 1, c:c + 1].copy(), 0, m=4)[:, 0, 0])


def test_f4_input_transform_one_hot_pixels_and_tiling(oracle):
    # B^T of F(4x4) is integral: a single 1 at d[r][s] of one 6x6 tile gives outer(B^T[:, r], B^T[:, s]) exactly
    for r, s in itertools.product(range(6), range(6)):
        x = np.zeros((1, 1, 6, 6), np.float32)
        x[0, 0, r, s] = 1
        V = oracle.wino_input_transform(x, pad=0, m=4).reshape(6, 6)
        assert np.array_equal(V, np.outer(BT4[:, r], BT4[:, s]).astype(np.float32)), (r, s)
    # a tile of ones: the row sums of B^T are (0, -6, 0, 0, 0, 0) -> only V[1][1] = 36
    V = oracle.wino_input_transform(np.ones((1, 1, 6, 6), np.float32), pad=0, m=4).reshape(6, 6)
    want = np.zeros((6, 6), np.float32)
    want[1, 1] = 36
    assert np.array_equal(V, want)
    # pad 1, H = W = 7 -> 2x2 tiles of 4x4 outputs with origin (4ty-1, 4tx-1), zeros outside the image;
    # tile (ty, tx) of image n is column p = (n*2 + ty)*2 + tx
    N, C, H = 2, 2, 7
    x = synth.small_ints(N * C * H * H, 23).reshape(N, C, H, H)
    V = oracle.wino_input_transform(x, pad=1, m=4)
    assert V.shape == (36, C, N * 4)
    xp = np.pad(x, [(0, 0), (0, 0), (1, 4), (1, 4)])
    for n, c, ty, tx in itertools.product(range(N), range(C), range(2), range(2)):
        d = xp[n, c, 4 * ty:4 * ty + 6, 4 * tx:4 * tx + 6].copy().reshape(1, 1, 6, 6)
        assert np.array_equal(V[:, c, (n * 2 + ty) * 2 + tx], oracle.wino_input_transform(d, pad=0, m=4).reshape(36))
    for layout in LAYOUTS:
        assert np.array_equal(oracle.wino_input_transform(synth.act_to_layout(x, layout), 1, layout, m=4), V)


def test_f4_output_transform_one_hot_products(oracle):
    # Mo = one-hot at (i, j) -> Y = outer(A^T[:, i], A^T[:, j]), exactly (A^T is integral)
    for i, j in itertools.product(range(6), range(6)):
        Mo = np.zeros((36, 1, 1), np.float32)
        Mo[i * 6 + j] = 1
        y = oracle.wino_output_transform(Mo, 1, 4, 4, m=4).reshape(4, 4)
        assert np.array_equal(y, np.outer(AT4[:, i], AT4[:, j]).astype(np.float32)), (i, j)
    # Ho = Wo = 6 -> 2x2 tiles, the last two rows and columns of the second tiles clipped
    Mo = synth.small_ints(36 * 2 * 4, 5).reshape(36, 2, 4)
    y = oracle.wino_output_transform(Mo, 1, 6, 6, m=4)
    assert y.shape == (1, 2, 6, 6)
    for k, ty, tx in itertools.product(range(2), range(2), range(2)):
        tile = AT4 @ Mo[:, k, ty * 2 + tx].reshape(6, 6).astype(np.float64) @ AT4.T
        hh, ww = min(4, 6 - 4 * ty), min(4, 6 - 4 * tx)
        assert np.array_equal(y[0, k, 4 * ty:4 * ty + hh, 4 * tx:4 * tx + ww], tile[:hh, :ww].astype(np.float32))


def test_f4_gemm_matches_einsum(oracle):
    U = synth.small_ints(36 * 5 * 7, 1).reshape(36, 5, 7)
    V = synth.small_ints(36 * 5 * 11, 2).reshape(36, 5, 11)
    assert np.array_equal(oracle.wino_gemm(U, V, m=4), np.einsum("xck,xcp->xkp", U, V))


def test_gemm_matches_einsum(oracle):
    U = synth.small_ints(16 * 5 * 7, 1).reshape(16, 5, 7)
    V = synth.small_ints(16 * 5 * 11, 2).reshape(16, 5, 11)
    assert np.array_equal(oracle.wino_gemm(U, V), np.einsum("xck,xcp->xkp", U, V))


def test_output_transform_closed_forms(oracle):
    # Mo = one-hot at (i, j) -> Y = outer(A^T[:, i], A^T[:, j]);  A^T = [1 1 1 0; 0 1 -1 -1]
    AT = np.array([[1, 1, 1, 0], [0, 1, -1, -1]], np.float32)
    for i, j in itertools.product(range(4), range(4)):
        Mo = np.zeros((16, 1, 1), np.float32)
        Mo[i * 4 + j] = 1
        y = oracle.wino_output_transform(Mo, 1, 2, 2, m=2).reshape(2, 2)
        assert np.array_equal(y, np.outer(AT[:, i], AT[:, j]))


def test_output_transform_clips_partial_tiles(oracle):
    # Ho = Wo = 3 -> 2x2 tiles, last row/col of outputs clipped; layouts agree
    N, K = 2, 3
    Mo = synth.small_ints(16 * K * N * 4, 5).reshape(16, K, N * 4)
    y = oracle.wino_output_transform(Mo, N, 3, 3, m=2)
    full = oracle.wino_output_transform(Mo, N, 4, 4, m=2)
    assert np.array_equal(y, full[:, :, :3, :3])
    for layout in LAYOUTS:
        yl = oracle.wino_output_transform(Mo, N, 3, 3, layout, m=2)
        assert np.array_equal(synth.act_from_layout(yl, layout), y)


def test_tile_geometry(oracle):
    assert oracle.wino_tiles(2, 56, 56, 1) == (28, 28)
    assert oracle.wino_tiles(2, 224, 224, 1) == (112, 112)      # 32 images -> 401,408 tiles
    assert oracle.wino_tiles(2, 5, 7, 1) == (3, 4)
    assert oracle.wino_tiles(2, 5, 5, 0) == (2, 2)
    # the reference's F(4x4) instance: inside=22, pad 1 -> blockn 6 (M = 64*36 = 2304)
    assert oracle.wino_tiles(4, 22, 22, 1) == (6, 6)
    assert oracle.wino_tiles(4, 224, 224, 1) == (56, 56)
    assert oracle.wino_tiles(4, 14, 14, 1) == (4, 4)


@pytest.mark.parametrize("m", [2, 4])
@pytest.mark.parametrize("pad", [2, 3, 5])
def test_wide_padding_is_a_padded_image(oracle, m, pad):
    """The reference takes `padding` arithmetically (comparison/wrapedConv_NCHW.cuh:346-362): a transform with padding
    p is the transform without padding of the image with p rings of zeros around it, and the whole Winograd
    convolution is the direct one."""
    N, C, K, H, W = 2, 3, 4, 6, 5
    x = synth.small_ints(N * C * H * W, 40 + pad).reshape(N, C, H, W)
    xp = np.pad(x, [(0, 0), (0, 0), (pad, pad), (pad, pad)])
    assert oracle.wino_tiles(m, H, W, pad) == oracle.wino_tiles(m, H + 2 * pad, W + 2 * pad, 0)
    for layout in LAYOUTS:
        got = oracle.wino_input_transform(synth.act_to_layout(x, layout), pad, layout, m=m)
        assert np.array_equal(got, oracle.wino_input_transform(synth.act_to_layout(xp, layout), 0, layout, m=m))
    w = synth.small_ints(K * C * 9, 41 + pad).reshape(K, C, 3, 3) * (576 if m == 4 else 1)
    assert np.array_equal(oracle.wino_conv(x, w, pad, m=m), oracle.direct_conv(x, w, pad))
    assert np.array_equal(oracle.direct_conv(x, w, pad), oracle.direct_conv(xp, w, 0))
