"""The benchmark configurations at their full sizes, every pipeline against the oracle and against each other:
the layer table of the reference's driver (comparison/layoutCompare.cu:38-148) at the batches the headline
numbers are quoted on.

  * N=64, C=K=512 at H=W=28 and H=W=14, fp32 (1,568 / 392 tile patches of 64: other round counts and another
    cut-up last round than the N=32 layers), three layouts, the automatic choice and every pipeline by name,
    and the filter bank transformed beforehand;
  * N=32, C=K=64, H=W=224, fp32 (401,408 tiles): the staged, epilogue and single-kernel pipelines agree
    over the whole tensor and each matches the oracle;
  * the thirteen VGG-16 convolutions chained with ReLU at N=32 in f16 and bf16: every layer against the oracle
    fed the device's own input of that layer, and the chain against the same chain in fp32 on the device
    (whose layers are checked against the oracle in the same way).

The CPU oracle cannot convolve whole layers of these sizes in test time: it convolves the last image with three
filters (first, middle, last) and those planes are compared; agreement between pipelines and layouts is checked
over the whole tensor on the device.  Tolerances: relative L2 1e-4 (fp32), 2e-2 (f16, bf16) against the oracle,
1e-6 between fp32 pipelines (same products, another summation order)."""
import numpy as np
import pytest
import torch

from cudnntest_amd import ops, synth
from gpu_util import TOL, TORCH_DT, host

pytestmark = pytest.mark.gpu
LAYOUTS = [ops.NCHW, ops.NHWC, ops.CHWN]


def to_layout(t_nchw, layout):
    """activations [N][C][H][W] or a filter bank [K][C][3][3] in `layout`'s convention"""
    if layout == ops.NCHW:
        return t_nchw.contiguous()
    if layout == ops.NHWC:
        return t_nchw.permute(0, 2, 3, 1).contiguous()
    return t_nchw.permute(1, 2, 3, 0).contiguous()


def from_layout(t, layout):
    if layout == ops.NCHW:
        return t
    if layout == ops.NHWC:
        return t.permute(0, 3, 1, 2)
    return t.permute(3, 0, 1, 2)


def rel(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm()).item()


def oracle_planes(oracle, x_nchw, w_kc33, relu=False):
    """the oracle's convolution of the last image with three filters, and their indices"""
    K = w_kc33.shape[0]
    ks = sorted({0, K // 2, K - 1})
    return ks, oracle.direct_conv_f32(host(x_nchw[-1:]), host(w_kc33[ks]), 1, relu=relu)


def seeded(N, C, K, H, seed, dtype=ops.F32):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = (torch.rand((N, C, H, H), device="cuda", generator=g) * 2 - 1).to(TORCH_DT[dtype])
    w = (torch.randn((K, C, 3, 3), device="cuda", generator=g) * (2.0 / (9 * C)) ** 0.5).to(TORCH_DT[dtype])
    return x, w


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("H", [28, 14])
def test_n64_c512_every_pipeline(oracle, H, layout):
    N, C, K = 64, 512, 512
    x, w = seeded(N, C, K, H, 0xC3 + H)
    ks, want = oracle_planes(oracle, x, w)
    xl, wl = to_layout(x, layout), to_layout(w, layout)
    base = None
    for algo in (ops.ALGO_STAGED, ops.ALGO_EPILOGUE, ops.ALGO_FUSED, ops.ALGO_STAGED_F4, ops.ALGO_EPILOGUE_F4, ops.ALGO_AUTO):
        y = from_layout(ops.conv(xl, wl, 1, layout, algo=algo), layout)
        assert tuple(y.shape) == (N, K, H, H)
        err = oracle.rel_l2(host(y[-1:][:, ks]), want)
        assert err <= TOL[ops.F32], (algo, err)
        if base is None:
            base = y.clone()
        else:
            # the F(2x2) pipelines differ by summation order; F(4x4) -- by name, or as the automatic choice for
            # these long reductions -- has other transforms and three to four times the rounding error
            assert rel(y, base) <= (1e-6 if algo in (ops.ALGO_EPILOGUE, ops.ALGO_FUSED) else 2e-5), algo
    # the filter bank transformed once (F(2x2)), then the automatic choice among the F(2x2) pipelines: the same bits
    # as that pipeline gives with the bank itself
    U = ops.filter_transform(wl, layout)
    yp = from_layout(ops.conv_prepared(xl, U, K, 1, layout), layout)
    assert rel(yp, base) <= 1e-6
    assert any(torch.equal(yp, from_layout(ops.conv(xl, wl, 1, layout, algo=a), layout))
               for a in (ops.ALGO_STAGED, ops.ALGO_EPILOGUE, ops.ALGO_FUSED))
    # and in the other two destination layouts (the cross-layout entry points)
    for dst in LAYOUTS:
        if dst != layout:
            yd = from_layout(ops.conv(xl, wl, 1, layout, dst), dst)
            assert rel(yd, base) <= 2e-5, dst


def test_n64_c512_h14_cut_rounds_repeat_bit_for_bit():
    """392 tile patches x 8 filter tiles: the workgroups that share a patch's reduction combine their partial sums
    in a fixed order, so every run gives the same bits."""
    x, w = seeded(64, 512, 512, 14, 0x514)
    for algo in (ops.ALGO_EPILOGUE, ops.ALGO_STAGED, ops.ALGO_AUTO):
        first = ops.conv(x, w, algo=algo).clone()
        for _ in range(3):
            assert torch.equal(ops.conv(x, w, algo=algo), first), algo


def test_headline_layer_cut_up_last_round(oracle):
    """N=32, C=K=256, H=W=56 (1,568 tile patches x 4 filter tiles on 512 resident workgroups: the last, small round
    is cut four ways): the same bits on every run, the oracle's planes, and the staged pipeline's tensor."""
    x, w = seeded(32, 256, 256, 56, 0x256)
    ks, want = oracle_planes(oracle, x, w)
    first = ops.conv(x, w, algo=ops.ALGO_EPILOGUE).clone()
    for _ in range(3):
        assert torch.equal(ops.conv(x, w, algo=ops.ALGO_EPILOGUE), first)
    assert oracle.rel_l2(host(first[-1:][:, ks]), want) <= TOL[ops.F32]
    # the last patches of the tensor are the ones the cut-up round computes
    tail = oracle.direct_conv_f32(host(x[-1:]), host(w[-2:]), 1)
    assert oracle.rel_l2(host(first[-1:, -2:]), tail) <= TOL[ops.F32]
    assert rel(ops.conv(x, w, algo=ops.ALGO_STAGED), first) <= 1e-6


@pytest.mark.parametrize("layout", LAYOUTS)
def test_n32_c64_h224_staged_epilogue_fused_agree(oracle, layout):
    N, C, K, H = 32, 64, 64, 224
    x, w = seeded(N, C, K, H, 0xC4)
    ks, want = oracle_planes(oracle, x, w)
    xl, wl = to_layout(x, layout), to_layout(w, layout)
    del x
    base = None
    for algo in (ops.ALGO_FUSED, ops.ALGO_EPILOGUE, ops.ALGO_STAGED, ops.ALGO_AUTO):
        y = from_layout(ops.conv(xl, wl, 1, layout, algo=algo), layout)
        err = oracle.rel_l2(host(y[-1:][:, ks]), want)
        assert err <= TOL[ops.F32], (algo, err)
        if base is None:
            base = y
        else:
            assert rel(y, base) <= 1e-6, algo
        del y
    # the first image as well: the oracle's first plane of image 0
    first = oracle.direct_conv_f32(np.ascontiguousarray(host(from_layout(xl, layout)[:1])), host(w[:1]), 1)
    assert oracle.rel_l2(host(base[:1, :1]), first) <= TOL[ops.F32]


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("dtype", [ops.F16, ops.BF16])
def test_vgg16_relu_chain_n32(oracle, dtype, layout):
    """13 layers, ReLU in every output stage, 2x sub-sampling between blocks (pooling is not part of the path),
    the 16-bit chain and the fp32 chain side by side on the device, both fed the same rounded input and filters."""
    N, H = 32, 224
    tdt = TORCH_DT[dtype]
    g = torch.Generator(device="cuda").manual_seed(0xC5)
    x16 = (torch.rand((N, 3, H, H), device="cuda", generator=g) * 2 - 1).to(tdt)
    x32 = x16.float()
    for li, (C, K, Hl) in enumerate(synth.VGG16_CONV):
        if Hl != x16.shape[2]:
            x16 = x16[:, :, ::2, ::2].contiguous()
            x32 = x32[:, :, ::2, ::2].contiguous()
        assert tuple(x16.shape) == (N, C, Hl, Hl)
        w16 = (torch.randn((K, C, 3, 3), device="cuda", generator=g) * (2.0 / (9 * C)) ** 0.5).to(tdt)
        w32 = w16.float()
        y16 = from_layout(ops.conv(to_layout(x16, layout), to_layout(w16, layout), 1, layout, relu=True), layout)
        y32 = from_layout(ops.conv(to_layout(x32, layout), to_layout(w32, layout), 1, layout, relu=True), layout)
        # each layer on its own: the oracle is fed the very activation the device consumed
        ks, want16 = oracle_planes(oracle, x16, w16, relu=True)
        err16 = oracle.rel_l2(host(y16[-1:][:, ks]), want16)
        assert err16 <= TOL[dtype], (li, err16)
        _, want32 = oracle_planes(oracle, x32, w32, relu=True)
        err32 = oracle.rel_l2(host(y32[-1:][:, ks]), want32)
        assert err32 <= TOL[ops.F32], (li, err32)
        x16, x32 = y16.contiguous(), y32.contiguous()
    chain = rel(x16, x32)
    print(f"dtype={dtype} layout={layout} 13-layer chain at N=32 against the fp32 chain: {chain:.3e}")
    assert chain <= TOL[dtype], chain


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("N", [1, 2, 4, 8, 16, 32, 64, 128])
def test_the_references_published_sweep(oracle, N, layout):
    """The one shape the reference commits latencies for (layoutTest/NHWC/test.sh:3-8: `a.out <N> 22 128 128` for
    N = 1 .. 128, the shape of its notebooks' accuracy checks at N = 64): the automatic choice -- F(2x2) up to
    N = 8, F(4x4) beyond -- against the oracle's convolution of the whole batch, and against the F(2x2) pipeline."""
    C = K = 128
    H = 22
    x, w = seeded(N, C, K, H, 0x2200 + N)
    want = oracle.direct_conv_f32(host(x), host(w), 1)
    xl, wl = to_layout(x, layout), to_layout(w, layout)
    y = from_layout(ops.conv(xl, wl, 1, layout), layout)
    assert oracle.rel_l2(host(y), want) <= TOL[ops.F32]
    y2 = from_layout(ops.conv(xl, wl, 1, layout, algo=ops.ALGO_STAGED), layout)
    assert rel(y, y2) <= 2e-5
