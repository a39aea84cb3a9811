"""F(4x4,3x3) mode -- the reference's own tile size (6x6 tiles, 36 coordinates,
comparison/wrapedConv_NCHW.cuh:836-855,879-899,1084-1101) -- against the oracle's
F(4x4) stage functions (oracle m=4, pinned in tests/test_oracle_winograd.py) and
against the direct convolution.  B^T and A^T are integer matrices, so the input
and output transforms are bit-exact on integers; G has 1/6, 1/12, 1/24, so the
filter transform and whole layers are compared with a tolerance (fp32: 1e-4
relative L2 as for the F(2x2) path)."""
import itertools

import numpy as np
import pytest
import torch

from cudnntest_amd import ops, synth
from gpu_util import TOL, batch_minor_perm, dev, host, pack_operand, unpack_operand

pytestmark = pytest.mark.gpu
LAYOUTS = [ops.NCHW, ops.NHWC, ops.CHWN]


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("K,C", [(4, 3), (64, 64), (130, 17)])
def test_f4_filter_transform(oracle, layout, K, C):
    w = synth.normal(K * C * 9, 5 + K, 0.1).reshape(K, C, 3, 3)
    wl = synth.flt_to_layout(w, layout)
    U = unpack_operand(ops.f4_filter_transform(dev(wl), layout))
    want = oracle.wino_filter_transform(wl, layout, m=4)
    np.testing.assert_allclose(U[:, :C, :K], want, rtol=2e-6, atol=1e-7)
    assert not U[:, C:, :].any() and not U[:, :, K:].any()
    assert oracle.rel_l2(np.ascontiguousarray(U[:, :C, :K]), want) < 1e-6


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("order", [ops.TILES_BATCH_MAJOR, ops.TILES_BATCH_MINOR])
@pytest.mark.parametrize("shape,pad", [((2, 3, 5, 5), 1), ((3, 17, 9, 6), 1), ((1, 64, 14, 14), 1), ((2, 5, 8, 7), 0),
                                       ((2, 16, 22, 22), 1),
                                       # the NCHW LDS-halo kernels: a whole 56x56 image per workgroup, row blocks with a
                                       # ragged last one (112 wide), two column blocks (tw = 68), odd sizes without padding,
                                       # small images with several channel vectors to a workgroup and a ragged last group
                                       ((2, 9, 56, 56), 1), ((1, 5, 112, 110), 1), ((1, 4, 10, 270), 1), ((2, 6, 47, 51), 0),
                                       ((3, 44, 14, 14), 1), ((2, 21, 28, 26), 1)])
def test_f4_input_transform(oracle, layout, order, shape, pad):
    N, C, H, W = shape
    x = synth.small_ints(N * C * H * W, 77 + sum(shape), -8, 8).reshape(N, C, H, W)
    xl = synth.act_to_layout(x, layout)
    V = unpack_operand(ops.f4_input_transform(dev(xl), pad, layout, order))
    want = oracle.wino_input_transform(xl, pad, layout, m=4)
    th, tw = oracle.wino_tiles(4, H, W, pad)
    P = N * th * tw
    got = V[:, :C, :P]
    if order == ops.TILES_BATCH_MINOR:
        got = got[:, :, np.argsort(batch_minor_perm(N, th, tw))]
    assert np.array_equal(got, want)
    assert not V[:, C:, :P].any()


@pytest.mark.parametrize("porder", [ops.PRODUCT_KP, ops.PRODUCT_PK])
def test_f4_batched_gemm(oracle, porder):
    C, K, P = 40, 130, 300
    g = ops.f4_geometry(ops.F32, 1, C, K, 6, 6, 1)
    Cp, Kp, Pp = g["Cp"], g["Kp"], 384
    U = np.zeros((36, Cp, Kp), np.float32)
    V = np.zeros((36, Cp, Pp), np.float32)
    U[:, :C, :K] = synth.small_ints(36 * C * K, 3, -3, 3).reshape(36, C, K)
    V[:, :C, :P] = synth.small_ints(36 * C * P, 4, -5, 5).reshape(36, C, P)
    Mo = host(ops.f4_batched_gemm(pack_operand(U), pack_operand(V), C, K, P, porder))
    if porder == ops.PRODUCT_PK:
        Mo = Mo.transpose(0, 2, 1)
    want = oracle.wino_gemm(np.ascontiguousarray(U[:, :C, :K]), np.ascontiguousarray(V[:, :C, :P]), m=4)
    assert np.array_equal(Mo[:, :K, :P], want)


@pytest.mark.parametrize("porder", [ops.PRODUCT_KP, ops.PRODUCT_PK])
@pytest.mark.parametrize("C,K,P", [(16, 70, 128 * 70), (80, 200, 128 * 22 - 5), (380, 600, 128 * 9)])
def test_f4_batched_gemm_walking_workgroups(oracle, porder, C, K, P):
    """Products with work for three and more rounds of the resident workgroups and a reduction of at most 24 stages run
    on the kernel whose workgroups walk the (coordinate, tile column) pairs in one pipeline: one, two and five filter
    tiles (groups of workgroups that do and do not divide an XCD's share), reductions of 1, 5 and 24 stages, a ragged
    last tile column; bit-exact on integers, twice (nothing may depend on what a previous launch left in LDS)."""
    g = ops.f4_geometry(ops.F32, 1, C, K, 6, 6, 1)
    Cp, Kp, Pp = g["Cp"], g["Kp"], (P + 127) // 128 * 128
    U = np.zeros((36, Cp, Kp), np.float32)
    V = np.zeros((36, Cp, Pp), np.float32)
    U[:, :C, :K] = synth.small_ints(36 * C * K, 13, -2, 2).reshape(36, C, K)
    V[:, :C, :P] = synth.small_ints(36 * C * P, 14, -3, 3).reshape(36, C, P)
    Ud, Vd = pack_operand(U), pack_operand(V)
    want = np.einsum("xck,xcp->xkp", U[:, :C, :K], V[:, :C, :P], optimize=True)
    pins = [(0, 0, 0), (35, K - 1, P - 1), (17, K // 2, P // 3)]
    ref = oracle.wino_gemm(np.ascontiguousarray(U[:, :C, :K]), np.ascontiguousarray(V[:, :C, :P]), m=4) if C * K * P < 2e8 else None
    for rep in range(2):
        Mo = host(ops.f4_batched_gemm(Ud, Vd, C, K, P, porder))
        if porder == ops.PRODUCT_PK:
            Mo = Mo.transpose(0, 2, 1)
        assert np.array_equal(Mo[:, :K, :P], want), rep
    if ref is not None:
        assert np.array_equal(ref, want)
    for xi, k, p_ in pins:                       # the einsum itself against a plain dot product
        assert want[xi, k, p_] == float(np.dot(U[xi, :C, k].astype(np.float64), V[xi, :C, p_].astype(np.float64)))


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("order", [ops.TILES_BATCH_MAJOR, ops.TILES_BATCH_MINOR])
@pytest.mark.parametrize("porder", [ops.PRODUCT_KP, ops.PRODUCT_PK])
@pytest.mark.parametrize("N,K,Ho,Wo", [(2, 4, 5, 5), (3, 7, 9, 6), (1, 130, 16, 16), (2, 3, 1, 1)])
def test_f4_output_transform(oracle, layout, order, porder, N, K, Ho, Wo):
    th, tw = (Ho + 3) // 4, (Wo + 3) // 4
    P = N * th * tw
    Kp, Pp = (K + 127) // 128 * 128, (P + 127) // 128 * 128
    M = synth.small_ints(36 * K * P, 13 + K, -6, 6).reshape(36, K, P)
    Mo = np.full((36, Kp, Pp), 1e30, np.float32)
    Mo[:, :K, :P] = M[:, :, batch_minor_perm(N, th, tw)] if order == ops.TILES_BATCH_MINOR else M
    Md = dev(np.ascontiguousarray(Mo.transpose(0, 2, 1))) if porder == ops.PRODUCT_PK else dev(Mo)
    for relu in (False, True):
        y = host(ops.f4_output_transform(Md, N, K, Ho, Wo, layout, order, relu, product_order=porder))
        want = oracle.wino_output_transform(M, N, Ho, Wo, layout, m=4)
        assert np.array_equal(y, np.maximum(want, 0) if relu else want)


F4_ALGOS = [ops.ALGO_STAGED_F4, ops.ALGO_EPILOGUE_F4]


@pytest.mark.parametrize("layout,order", [(ops.NCHW, ops.TILES_BATCH_MAJOR), (ops.NHWC, ops.TILES_BATCH_MAJOR),
                                          (ops.CHWN, ops.TILES_BATCH_MINOR), (ops.NCHW, ops.TILES_BATCH_MINOR)])
@pytest.mark.parametrize("C,K,N,Ho,Wo", [(16, 64, 1, 8, 8),        # one patch: a single workgroup or a few sharing it
                                         (40, 130, 3, 40, 40),      # 15 patches, filters and tiles ragged
                                         (80, 200, 2, 56, 60),      # 28 patches on 8 XCDs: uneven shares
                                         (256, 64, 8, 28, 28),      # one filter tile, 7 tile patches, 16 stages to a row
                                         (48, 256, 16, 30, 30)])    # 64 patches: most workgroups hold parts of two
def test_f4_gemm_with_the_output_transform_in_its_epilogue(oracle, layout, order, C, K, N, Ho, Wo):
    """y straight from U and V (gemm_rows_f4_kernel): the persistent workgroups cut the stage sequence of their XCD's
    patches into equal runs, so most patches are summed from the partial outputs of two or more workgroups.  Small
    integers: every product and partial sum is exact, so the result equals the oracle's GEMM followed by its output
    transform bit for bit -- twice in a row (the arrival counters return to zero), with ReLU the second time."""
    g = ops.f4_geometry(ops.F32, N, C, K, Ho, Wo, 1)
    Cp, Kp, Pp, P, th, tw = g["Cp"], g["Kp"], g["Pp"], g["P"], g["th"], g["tw"]
    U = np.zeros((36, Cp, Kp), np.float32)
    V = np.full((36, Cp, Pp), 3.0e38, np.float32)        # tile columns past P hold anything: they may not leak
    U[:, :C, :K] = synth.small_ints(36 * C * K, 13 + C, -2, 2).reshape(36, C, K)
    Vm = synth.small_ints(36 * C * P, 14 + K, -3, 3).reshape(36, C, P)
    V[:, :, :P] = 0
    V[:, :C, :P] = Vm[:, :, batch_minor_perm(N, th, tw)] if order == ops.TILES_BATCH_MINOR else Vm
    M = oracle.wino_gemm(np.ascontiguousarray(U[:, :C, :K]), np.ascontiguousarray(Vm), m=4)
    want = oracle.wino_output_transform(M, N, Ho, Wo, layout, m=4)
    Ud, Vd = pack_operand(U), pack_operand(V)
    for relu in (False, True):
        y = host(ops.f4_gemm_output(Ud, Vd, N, C, K, Ho, Wo, layout, order, relu))
        assert np.array_equal(y, np.maximum(want, 0) if relu else want), relu


@pytest.mark.parametrize("algo", F4_ALGOS)
@pytest.mark.parametrize("shape", [(2, 3, 4, 5, 5), (1, 8, 8, 6, 6), (3, 5, 7, 9, 9), (2, 16, 130, 7, 10), (1, 1, 1, 3, 3)])
def test_f4_layers_all_layout_pairs(oracle, shape, algo):
    N, C, K, H, W = shape
    x, w = synth.conv_inputs(N, C, K, H, W, seed=sum(shape))
    for src, dst in itertools.product(LAYOUTS, LAYOUTS):
        xs, ws = synth.act_to_layout(x, src), synth.flt_to_layout(w, src)
        want = oracle.direct_conv(xs, ws, 1, src, dst)
        got = host(ops.conv(dev(xs), dev(ws), 1, src, dst, algo))
        assert oracle.rel_l2(got, want) <= TOL[ops.F32], (src, dst)


@pytest.mark.parametrize("algo", F4_ALGOS)
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("shape", [(1, 64, 64, 56, 56), (64, 128, 128, 22, 22), (4, 128, 96, 14, 14), (2, 3, 64, 32, 32)])
def test_f4_floats_within_tolerance(oracle, layout, shape, algo):
    # second shape is the one the reference's notebooks use: N=64, C=K=128, H=22
    N, C, K, H, W = shape
    x, w = synth.conv_inputs(N, C, K, H, W, seed=2000 + sum(shape), layout=layout)
    want = oracle.direct_conv(x, w, 1, layout)
    got = host(ops.conv(dev(x), dev(w), 1, layout, algo=algo))
    err = oracle.rel_l2(got, want)
    print(f"F(4x4) algo {algo} layout {layout} shape {shape}: rel L2 {err:.2e}, sum|err| {np.abs(got - want).sum():.2f}")
    assert err <= TOL[ops.F32], err


def test_the_two_f4_pipelines_agree_on_the_headline_layer_bit_for_bit_from_call_to_call():
    """N=32, C=K=256, 56x56: 392 patches on 256 workgroups -- every workgroup holds parts of two or three patches.
    Against the staged F(4x4) pipeline (same products, another order of the sums: 1e-5), and twice the same bits."""
    N, C, K, H = 32, 256, 256, 56
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.rand((N, C, H, H), device="cuda", generator=g) * 2 - 1
    w = torch.randn((K, C, 3, 3), device="cuda", generator=g) * (2.0 / (9 * C)) ** 0.5
    for dst in LAYOUTS:
        a = ops.conv(x, w, 1, ops.NCHW, dst, algo=ops.ALGO_STAGED_F4)
        b = ops.conv(x, w, 1, ops.NCHW, dst, algo=ops.ALGO_EPILOGUE_F4)
        c = ops.conv(x, w, 1, ops.NCHW, dst, algo=ops.ALGO_EPILOGUE_F4)
        assert torch.equal(b, c)
        assert ((a - b).double().norm() / a.double().norm()).item() <= 1e-5
