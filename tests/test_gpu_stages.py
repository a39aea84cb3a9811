"""Stage-by-stage parity of the HIP kernels against the CPU oracle, through the
C ABI -- the reference's Module1/2/3.bin idea (layoutTest/NCHW/data/
ConvTest_V3_NCHW-Mar18.ipynb cells 10-11), seeded and asserted.

Integer-valued inputs make every F(2x2) intermediate exact in fp32, so the
transform stages must match the oracle bit-for-bit; the GEMM is checked
bit-for-bit on integers too (sums stay far below 2^24)."""
import itertools

import numpy as np
import pytest
import torch

from cudnntest_amd import ops, synth
from gpu_util import batch_minor_perm, dev, host, pack_operand, unpack_operand

pytestmark = pytest.mark.gpu
LAYOUTS = [ops.NCHW, ops.NHWC, ops.CHWN]


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("K,C", [(4, 3), (64, 64), (130, 17), (7, 40)])
def test_filter_transform(oracle, layout, K, C):
    w = synth.small_ints(K * C * 9, 31 + K + C, -4, 4).reshape(K, C, 3, 3)
    wl = synth.flt_to_layout(w, layout)
    U = unpack_operand(ops.filter_transform(dev(wl), layout))
    want = oracle.wino_filter_transform(wl, layout)
    assert np.array_equal(U[:, :C, :K], want)
    assert not U[:, C:, :].any() and not U[:, :, K:].any(), "padding must be zero"
    # float data: same arithmetic order is not promised, closeness is
    wf = synth.normal(K * C * 9, 5, 0.1).reshape(K, C, 3, 3)
    wfl = synth.flt_to_layout(wf, layout)
    Uf = unpack_operand(ops.filter_transform(dev(wfl), layout))[:, :C, :K]
    np.testing.assert_allclose(Uf, oracle.wino_filter_transform(wfl, layout), rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("order", [ops.TILES_BATCH_MAJOR, ops.TILES_BATCH_MINOR])
@pytest.mark.parametrize("shape,pad", [((2, 3, 5, 5), 1), ((3, 17, 9, 6), 1), ((1, 64, 14, 14), 1),
                                       ((2, 5, 8, 7), 0), ((4, 16, 28, 28), 1), ((1, 2, 3, 3), 1)])
def test_input_transform(oracle, layout, order, shape, pad):
    N, C, H, W = shape
    x = synth.small_ints(N * C * H * W, 77 + sum(shape), -8, 8).reshape(N, C, H, W)
    xl = synth.act_to_layout(x, layout)
    V = unpack_operand(ops.input_transform(dev(xl), pad, layout, order))
    want = oracle.wino_input_transform(xl, pad, layout)          # batch-major columns
    th, tw = oracle.wino_tiles(2, H, W, pad)
    P = N * th * tw
    got = V[:, :C, :P]
    if order == ops.TILES_BATCH_MINOR:
        got = got[:, :, np.argsort(batch_minor_perm(N, th, tw))]
    assert np.array_equal(got, want)
    assert not V[:, C:, :P].any(), "channel padding must be zero"


@pytest.mark.parametrize("layout", [ops.NCHW, ops.NHWC])
@pytest.mark.parametrize("dtype", [ops.F32, ops.F16, ops.BF16])
@pytest.mark.parametrize("shape,pad", [((2, 170, 14, 14), 1),     # several channel vectors per workgroup, ragged last group
                                       ((3, 136, 7, 7), 1),       # 16 tiles per image
                                       ((2, 20, 22, 20), 1),      # two channel vectors per workgroup
                                       ((1, 9, 28, 30), 1),       # one image per workgroup, channel padding
                                       ((2, 12, 15, 13), 0),      # odd width: 2-byte elements move one by one
                                       ((2, 12, 16, 12), 0),      # no padding, even width
                                       ((2, 512, 14, 14), 1),     # NHWC: 8-tile-wide blocks
                                       ((1, 256, 28, 28), 1),     # NHWC: 16-tile-wide blocks (2-byte)
                                       ((300, 4, 2, 2), 1)])      # one tile per image, many images
def test_input_transform_small_images(oracle, layout, dtype, shape, pad):
    """Images that fit one workgroup take their own NCHW kernel (a contiguous run of channel planes per workgroup)
    and narrow NHWC blocks: bit-exact on small integers for every element type."""
    N, C, H, W = shape
    x = synth.small_ints(N * C * H * W, 91 + sum(shape), -8, 8).reshape(N, C, H, W)
    xl = synth.act_to_layout(x, layout)
    V = unpack_operand(ops.input_transform(dev(xl, dtype), pad, layout, ops.TILES_BATCH_MAJOR), dtype)
    want = oracle.wino_input_transform(xl, pad, layout)
    th, tw = oracle.wino_tiles(2, H, W, pad)
    P = N * th * tw
    assert np.array_equal(V[:, :C, :P], want)
    assert not V[:, C:, :P].any(), "channel padding must be zero"


@pytest.mark.parametrize("dtype", [ops.F16, ops.BF16])
@pytest.mark.parametrize("shape,pad", [((2, 17, 9, 6), 1), ((4, 16, 28, 28), 1), ((6, 40, 8, 7), 0), ((32, 8, 12, 12), 1),
                                       ((3, 9, 6, 6), 1)])
def test_input_transform_chwn_two_byte(oracle, dtype, shape, pad):
    """2-byte CHWN sources, batch-minor tiles (eight channels per thread, lanes along n): bit-exact on small
    integers, channel padding zero."""
    N, C, H, W = shape
    x = synth.small_ints(N * C * H * W, 123 + sum(shape), -8, 8).reshape(N, C, H, W)
    xl = synth.act_to_layout(x, ops.CHWN)
    V = unpack_operand(ops.input_transform(dev(xl, dtype), pad, ops.CHWN, ops.TILES_BATCH_MINOR), dtype)
    want = oracle.wino_input_transform(xl, pad, ops.CHWN)
    th, tw = oracle.wino_tiles(2, H, W, pad)
    P = N * th * tw
    got = V[:, :C, :P][:, :, np.argsort(batch_minor_perm(N, th, tw))]
    assert np.array_equal(got, want)
    assert not V[:, C:, :P].any(), "channel padding must be zero"


def test_input_transform_small_images_unaligned_view(oracle):
    """A 2-byte NCHW tensor that starts on an odd element: same bits as the aligned one."""
    N, C, H, W = 2, 24, 14, 14
    x = synth.small_ints(N * C * H * W, 5, -8, 8).reshape(N, C, H, W)
    flat = torch.zeros(N * C * H * W + 1, dtype=torch.bfloat16, device="cuda")
    flat[1:] = dev(x, ops.BF16).reshape(-1)
    view = flat[1:].view(N, C, H, W)
    assert view.data_ptr() % 4 == 2
    got = ops.input_transform(view, 1, ops.NCHW, ops.TILES_BATCH_MAJOR)
    want = ops.input_transform(dev(x, ops.BF16), 1, ops.NCHW, ops.TILES_BATCH_MAJOR)
    assert torch.equal(got, want)
    ref = oracle.wino_input_transform(x, 1, ops.NCHW)
    assert np.array_equal(unpack_operand(got, ops.BF16)[:, :C, :N * 49], ref)


@pytest.mark.parametrize("porder", [ops.PRODUCT_KP, ops.PRODUCT_PK])
@pytest.mark.parametrize("C,K,P", [(16, 128, 128), (3, 5, 30), (64, 64, 784), (40, 130, 300), (256, 256, 512)])
def test_batched_gemm(oracle, C, K, P, porder):
    g = ops.geometry(ops.F32, 1, C, K, 4, 4, 1)
    Cp, Kp = g["Cp"], g["Kp"]
    Pp = (P + 127) // 128 * 128
    U = np.zeros((16, Cp, Kp), np.float32)
    V = np.zeros((16, Cp, Pp), np.float32)
    U[:, :C, :K] = synth.small_ints(16 * C * K, 3, -3, 3).reshape(16, C, K)
    V[:, :C, :P] = synth.small_ints(16 * C * P, 4, -5, 5).reshape(16, C, P)
    Mo = host(ops.batched_gemm(pack_operand(U), pack_operand(V), C, K, P, porder))
    if porder == ops.PRODUCT_PK:
        Mo = Mo.transpose(0, 2, 1)
    want = oracle.wino_gemm(np.ascontiguousarray(U[:, :C, :K]), np.ascontiguousarray(V[:, :C, :P]))
    assert np.array_equal(Mo[:, :K, :P], want)


@pytest.mark.parametrize("porder", [ops.PRODUCT_KP, ops.PRODUCT_PK])
@pytest.mark.parametrize("C,K,P", [(64, 256, 6272), (128, 256, 6272), (256, 128, 12544), (256, 256, 6300), (512, 256, 6272),
                                   (48, 256, 6272), (80, 256, 6272)])
def test_batched_gemm_over_the_resident_set(oracle, C, K, P, porder):
    """Shapes with several rounds of work for a resident set of workgroups: the GEMM then walks its (coordinate, tile
    column) pairs, with a finished pair's product stored during the next pair's first stages when the reduction is
    a multiple of four stages long (4, 8, 16, 32 here; 3 and 5: stored in one go).  Small integers: the product is
    exact, compared over all of it with a device-side fp32 matrix product (itself exact on these values) and, for the
    first and the last 70 tiles, with the oracle."""
    g = ops.geometry(ops.F32, 1, C, K, 4, 4, 1)
    Cp, Kp = g["Cp"], g["Kp"]
    Pp = (P + 127) // 128 * 128
    gen = torch.Generator(device="cuda").manual_seed(C * 7 + K)
    Ud = torch.zeros((16, Cp, Kp), device="cuda")
    Vd = torch.zeros((16, Cp, Pp), device="cuda")
    Ud[:, :C, :K] = torch.randint(-3, 4, (16, C, K), device="cuda", generator=gen).float()
    Vd[:, :C, :P] = torch.randint(-5, 6, (16, C, P), device="cuda", generator=gen).float()
    pack = lambda t: t.reshape(16, Cp // 4, 4, -1).permute(0, 1, 3, 2).contiguous()
    Mo = ops.batched_gemm(pack(Ud), pack(Vd), C, K, P, porder)
    if porder == ops.PRODUCT_PK:
        Mo = Mo.transpose(1, 2)
    want = torch.matmul(Ud.transpose(1, 2), Vd)               # [16][Kp][Pp]
    assert torch.equal(Mo[:, :K, :P], want[:, :K, :P])
    for p0 in (0, P - 70):
        ref = oracle.wino_gemm(np.ascontiguousarray(host(Ud[:, :C, :K])), np.ascontiguousarray(host(Vd[:, :C, p0:p0 + 70])))
        assert np.array_equal(host(Mo[:, :K, p0:p0 + 70]), ref)


def test_batched_gemm_floats(oracle):
    C, K, P = 64, 128, 256
    U = synth.normal(16 * C * K, 8, 0.2).reshape(16, C, K)
    V = synth.uniform_pm1(16 * C * P, 9).reshape(16, C, P)
    Mo = host(ops.batched_gemm(pack_operand(U), pack_operand(V), C, K, P))
    assert oracle.rel_l2(Mo, oracle.wino_gemm(U, V)) < 1e-6


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("order", [ops.TILES_BATCH_MAJOR, ops.TILES_BATCH_MINOR])
@pytest.mark.parametrize("N,K,Ho,Wo", [(2, 4, 5, 5), (3, 7, 9, 6), (1, 130, 14, 14), (4, 16, 28, 28), (2, 3, 1, 1)])
@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("porder", [ops.PRODUCT_KP, ops.PRODUCT_PK])
def test_output_transform(oracle, layout, order, N, K, Ho, Wo, relu, porder):
    th, tw = (Ho + 1) // 2, (Wo + 1) // 2
    P = N * th * tw
    g = ops.geometry(ops.F32, 1, 1, K, 4, 4, 1)
    Kp, Pp = g["Kp"], (P + 127) // 128 * 128
    M = synth.small_ints(16 * K * P, 13 + K, -6, 6).reshape(16, K, P)     # batch-major columns
    Mo = np.full((16, Kp, Pp), 1e30, np.float32)                         # poison the padding
    if order == ops.TILES_BATCH_MINOR:
        Mo[:, :K, :P] = M[:, :, batch_minor_perm(N, th, tw)]
    else:
        Mo[:, :K, :P] = M
    Md = dev(np.ascontiguousarray(Mo.transpose(0, 2, 1))) if porder == ops.PRODUCT_PK else dev(Mo)
    y = host(ops.output_transform(Md, N, K, Ho, Wo, layout, order, relu, product_order=porder))
    want = oracle.wino_output_transform(M, N, Ho, Wo, layout)
    if relu:
        want = np.maximum(want, 0)
    assert np.array_equal(y, want)


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("order", [ops.TILES_BATCH_MAJOR, ops.TILES_BATCH_MINOR])
@pytest.mark.parametrize("N,C,K,Ho,Wo", [(2, 3, 4, 5, 5), (3, 20, 70, 9, 6), (1, 64, 130, 14, 14), (4, 16, 64, 28, 28)])
@pytest.mark.parametrize("relu", [False, True])
def test_gemm_with_output_epilogue(oracle, layout, order, N, C, K, Ho, Wo, relu):
    """y straight from U and V: must equal oracle GEMM followed by oracle output transform."""
    th, tw = (Ho + 1) // 2, (Wo + 1) // 2
    P = N * th * tw
    g = ops.geometry(ops.F32, N, C, K, Ho, Wo, 1)
    Cp, Kp, Pp = g["Cp"], g["Kp"], g["Pp"]
    Uc = synth.small_ints(16 * C * K, 3 + K, -3, 3).reshape(16, C, K)
    Vc = synth.small_ints(16 * C * P, 4 + C, -5, 5).reshape(16, C, P)       # batch-major columns
    U = np.zeros((16, Cp, Kp), np.float32)
    V = np.zeros((16, Cp, Pp), np.float32)
    U[:, :C, :K] = Uc
    V[:, :C, :P] = Vc[:, :, batch_minor_perm(N, th, tw)] if order == ops.TILES_BATCH_MINOR else Vc
    y = host(ops.gemm_output(pack_operand(U), pack_operand(V), N, C, K, Ho, Wo, layout, order, relu))
    want = oracle.wino_output_transform(oracle.wino_gemm(Uc, Vc), N, Ho, Wo, layout)
    if relu:
        want = np.maximum(want, 0)
    assert np.array_equal(y, want)


@pytest.mark.parametrize("src,dst", list(itertools.permutations(LAYOUTS, 2)))
def test_layout_transform(oracle, src, dst):
    N, C, H, W = 3, 5, 7, 6
    x = synth.uniform_pm1(N * C * H * W, 2).reshape(N, C, H, W)
    xs = synth.act_to_layout(x, src)
    got = host(ops.layout_transform(dev(xs), src, dst))
    assert np.array_equal(got, synth.act_to_layout(x, dst))
    xh = dev(xs, ops.F16)
    assert torch.equal(ops.layout_transform(xh, src, dst).cpu(),
                       torch.from_numpy(synth.act_to_layout(x, dst)).half())


@pytest.mark.parametrize("shape", [(4, 6, 10, 8), (2, 64, 14, 14), (32, 66, 6, 6), (34, 130, 4, 2), (3, 8, 5, 6), (1, 2, 2, 2)])
@pytest.mark.parametrize("src,dst", list(itertools.permutations(LAYOUTS, 2)))
def test_layout_transform_two_byte_pairs(src, dst, shape):
    """2-byte tensors with even extents move as 4-byte pairs (tiles of 8192 elements in four shapes); odd extents
    and views that are only 2-byte aligned take the one-element kernel.  Bit-exact against torch's permute."""
    N, C, H, W = shape
    g = torch.Generator(device="cuda").manual_seed(N * 1000 + C)
    x = torch.randn((N, C, H, W), device="cuda", generator=g).to(torch.bfloat16)
    perm = {ops.NCHW: (0, 1, 2, 3), ops.NHWC: (0, 2, 3, 1), ops.CHWN: (1, 2, 3, 0)}
    xs = x.permute(perm[src]).contiguous()
    want = x.permute(perm[dst]).contiguous()
    assert torch.equal(ops.layout_transform(xs, src, dst), want)
    flat = torch.empty(xs.numel() + 1, dtype=xs.dtype, device="cuda")       # a view that starts on an odd element
    odd = flat[1:].view(xs.shape)
    odd.copy_(xs)
    assert torch.equal(ops.layout_transform(odd, src, dst), want)
