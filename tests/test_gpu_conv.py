"""Whole-layer parity of the HIP path against the CPU oracle's direct
convolution, through the C ABI: the reference notebooks' cells 4-6
(layoutTest/*/data/ConvTest_V3_*.ipynb), but seeded, asserted, over several
shapes, every layout pair, and with the tolerance the task states:
relative L2 <= 1e-4 for fp32 (bit-exact on small integers)."""
import itertools

import numpy as np
import pytest
import torch

import cudnntest_amd as wa
from cudnntest_amd import ops, synth
from gpu_util import TOL, dev, host

pytestmark = pytest.mark.gpu
LAYOUTS = [ops.NCHW, ops.NHWC, ops.CHWN]
ALGOS = [ops.ALGO_STAGED, ops.ALGO_EPILOGUE, ops.ALGO_FUSED]

SMALL = [(2, 3, 4, 5, 5), (1, 8, 8, 6, 6), (3, 5, 7, 9, 9), (2, 16, 130, 7, 10), (1, 1, 1, 3, 3), (5, 40, 24, 14, 14),
         # channel counts that take two k-groups per stage in the single-kernel path; odd and minimal widths
         (2, 32, 20, 11, 13), (1, 64, 70, 8, 4), (3, 36, 9, 6, 7)]


@pytest.mark.parametrize("algo", ALGOS)
@pytest.mark.parametrize("shape", SMALL)
def test_integers_bit_exact_all_layout_pairs(oracle, algo, shape):
    N, C, K, H, W = shape
    x, w = synth.conv_inputs(N, C, K, H, W, seed=sum(shape), integer=True)
    for src, dst in itertools.product(LAYOUTS, LAYOUTS):
        xs, ws = synth.act_to_layout(x, src), synth.flt_to_layout(w, src)
        want = oracle.direct_conv(xs, ws, 1, src, dst)
        got = host(ops.conv(dev(xs), dev(ws), 1, src, dst, algo))
        assert np.array_equal(got, want), (src, dst)


@pytest.mark.parametrize("algo", ALGOS)
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("shape", [(1, 64, 64, 56, 56), (2, 3, 64, 32, 32), (4, 128, 96, 14, 14), (2, 32, 32, 27, 27)])
def test_floats_within_tolerance(oracle, algo, layout, shape):
    # first shape is the reference-runnable configuration: N=1, C=K=64, H=W=56
    N, C, K, H, W = shape
    x, w = synth.conv_inputs(N, C, K, H, W, seed=1000 + sum(shape), layout=layout)
    want = oracle.direct_conv(x, w, 1, layout)
    got = host(ops.conv(dev(x), dev(w), 1, layout, algo=algo))
    err = oracle.rel_l2(got, want)
    assert err <= TOL[ops.F32], err


@pytest.mark.parametrize("algo", ALGOS)
def test_pad0_and_relu(oracle, algo):
    N, C, K, H, W = 2, 6, 5, 9, 8
    x, w = synth.conv_inputs(N, C, K, H, W, seed=3, integer=True)
    want = oracle.direct_conv(x, w, 0)
    assert np.array_equal(host(ops.conv(dev(x), dev(w), 0, algo=algo)), want)
    got = host(ops.conv(dev(x), dev(w), 1, algo=algo, relu=True))
    assert np.array_equal(got, np.maximum(oracle.direct_conv(x, w, 1), 0))


def test_prepared_filters_match(oracle):
    N, C, K, H, W = 2, 16, 24, 12, 12
    x, w = synth.conv_inputs(N, C, K, H, W, seed=8)
    xd, wd = dev(x), dev(w)
    U = ops.filter_transform(wd)
    # (with the filter bank itself AUTO may leave the Winograd kernels for so small a layer; with its transform it cannot)
    assert torch.equal(ops.conv_prepared(xd, U, K), ops.conv(xd, wd, algo=ops.ALGO_STAGED))
    assert oracle.rel_l2(host(ops.conv_prepared(xd, U, K)), host(ops.conv(xd, wd))) <= 1e-5


def test_reference_call_surface(oracle):
    """wrapedConv_* / layoutManager with the reference's argument list."""
    N, C, K, H = 2, 8, 12, 10
    x, w = synth.conv_inputs(N, C, K, H, H, seed=21, integer=True)
    for name, src in [("wrapedConv_NCHW", ops.NCHW), ("wrapedConv_NHWC", ops.NHWC), ("wrapedConv_CHWN", ops.CHWN)]:
        xs, ws = dev(synth.act_to_layout(x, src)), dev(synth.flt_to_layout(w, src))
        out = torch.zeros(ops.act_shape(src, N, K, H, H), device="cuda")
        chn = getattr(wa, name)(N, H, C, K, 1, xs, ws, None, None, None, out)
        assert chn == K      # the reference overwrites chn with numOfFilter (wrapedConv_NCHW.cuh:479)
        assert np.array_equal(host(out), oracle.direct_conv(host(xs), host(ws), 1, src))
    for src, dst in itertools.product(LAYOUTS, LAYOUTS):
        xs, ws = dev(synth.act_to_layout(x, src)), dev(synth.flt_to_layout(w, src))
        out = torch.zeros(ops.act_shape(dst, N, K, H, H), device="cuda")
        wa.layoutManager(wa.DataLayout(src), wa.DataLayout(dst), N, H, C, K, 1, xs, ws, None, None, None, out)
        assert np.array_equal(host(out), oracle.direct_conv(host(xs), host(ws), 1, src, dst))
    xs, ws = dev(synth.act_to_layout(x, ops.NHWC)), dev(synth.flt_to_layout(w, ops.NHWC))
    out = torch.zeros(ops.act_shape(ops.CHWN, N, K, H, H), device="cuda")
    wa.convLayoutTrans_NHWC_to_CHWN(N, H, C, K, 1, xs, ws, None, None, None, out)
    assert np.array_equal(host(out), oracle.direct_conv(host(xs), host(ws), 1, ops.NHWC, ops.CHWN))


def test_properties_at_full_size():
    """Size-independent checks on the headline layer (N=32, C=K=256, H=W=56):
    linearity in x, delta filter = identity, and agreement between layouts."""
    N, C, K, H = 32, 256, 256, 56
    g = torch.Generator(device="cuda").manual_seed(7)
    x1 = torch.rand((N, C, H, H), device="cuda", generator=g) * 2 - 1
    x2 = torch.rand((N, C, H, H), device="cuda", generator=g) * 2 - 1
    w = torch.randn((K, C, 3, 3), device="cuda", generator=g) * (2.0 / (9 * C)) ** 0.5
    y1, y2 = ops.conv(x1, w), ops.conv(x2, w)
    # the F(2x2) pipelines agree to summation order; the automatic choice may be the F(4x4) pipeline (other
    # transforms, three to four times the rounding error of F(2x2), still a twentieth of the 1e-4 layer tolerance)
    ys = ops.conv(x1, w, algo=ALGOS[1])
    for algo in ALGOS[2:]:
        ya = ops.conv(x1, w, algo=algo)
        assert ((ya - ys).norm() / ys.norm()).item() < 1e-6, algo
    assert ((y1 - ys).norm() / ys.norm()).item() < 1e-5
    y12 = ops.conv(x1 + x2, w)
    rel = ((y12 - (y1 + y2)).norm() / y12.norm()).item()
    assert rel < 1e-5, rel
    wd = torch.zeros((K, C, 3, 3), device="cuda")
    idx = torch.arange(K, device="cuda")
    wd[idx, idx, 1, 1] = 1.0
    yd = ops.conv(x1, wd)
    assert ((yd - x1).norm() / x1.norm()).item() < 1e-6
    y_nhwc = ops.conv(x1.permute(0, 2, 3, 1).contiguous(), w.permute(0, 2, 3, 1).contiguous(), src=ops.NHWC)
    y_chwn = ops.conv(x1.permute(1, 2, 3, 0).contiguous(), w.permute(1, 2, 3, 0).contiguous(), src=ops.CHWN)
    assert ((y_nhwc.permute(0, 3, 1, 2) - y1).norm() / y1.norm()).item() < 1e-5
    assert ((y_chwn.permute(3, 0, 1, 2) - y1).norm() / y1.norm()).item() < 1e-5


def test_caller_owned_workspace(oracle):
    """wino_set_workspace: too small a buffer is refused with WINO_ERR_WORKSPACE, a big enough one is used."""
    from cudnntest_amd import _lib
    L = _lib.load()
    N, C, K, H, W = 2, 16, 24, 12, 12
    x, w = synth.conv_inputs(N, C, K, H, W, seed=8, integer=True)
    xd, wd = dev(x), dev(w)
    want = oracle.direct_conv(x, w, 1)
    need = ops.workspace_bytes(ops.F32, N, C, K, H, W, 1)
    small = torch.empty(8192, dtype=torch.uint8, device="cuda")
    big = torch.empty(need, dtype=torch.uint8, device="cuda")
    try:
        assert L.wino_set_workspace(small.data_ptr(), 1024) == -4      # not even room for the arrival counters
        assert L.wino_set_workspace(small.data_ptr(), small.numel()) == 0
        with pytest.raises(_lib.WinoError) as e:
            ops.conv(xd, wd, algo=ops.ALGO_STAGED)
        assert e.value.code == -4
        assert L.wino_set_workspace(big.data_ptr(), big.numel()) == 0
        for algo in ALGOS:
            assert np.array_equal(host(ops.conv(xd, wd, algo=algo)), want)
    finally:
        assert L.wino_set_workspace(None, 0) == 0
    assert np.array_equal(host(ops.conv(xd, wd)), want)


@pytest.mark.parametrize("dtype,N", [(ops.F32, 65), (ops.F32, 66), (ops.F32, 96)])
@pytest.mark.parametrize("layout", LAYOUTS)
def test_epilogue_gemm_with_a_cut_up_last_round(oracle, layout, dtype, N):
    """Patch counts just above a whole number of rounds of resident workgroups (512 for fp32): the
    last patches (8, 16, and with N=96 a last round of 256) are computed by four workgroups each, one
    Winograd row per workgroup, combined by the last to arrive.  Exact on integers, and the same bits on
    every run."""
    from gpu_util import TORCH_DT
    C, K, H, W = 8, 64, 32, 64                      # 512 tiles per image, one filter tile: N*8 patches
    x, w = synth.conv_inputs(N, C, K, H, W, seed=5150 + N, layout=layout, integer=True)
    bias = synth.small_ints(K, seed=3, lo=-2, hi=2).astype(np.float32)
    want = oracle.direct_conv(x, w, 1, layout)
    want = np.maximum(synth.act_from_layout(want, layout) + bias[None, :, None, None], 0)
    want = synth.act_to_layout(np.ascontiguousarray(want.astype(np.float32)), layout)
    xd, wd, bd = dev(x, dtype), dev(w, dtype), dev(bias, dtype)
    got = ops.conv(xd, wd, 1, layout, algo=ops.ALGO_EPILOGUE, relu=True, bias=bd)
    assert np.array_equal(host(got), want)
    xf, wf = synth.conv_inputs(N, C, K, H, W, seed=77, layout=layout)
    xfd, wfd = dev(xf, dtype), dev(wf, dtype)
    first = ops.conv(xfd, wfd, 1, layout, algo=ops.ALGO_EPILOGUE)
    for _ in range(3):
        assert torch.equal(ops.conv(xfd, wfd, 1, layout, algo=ops.ALGO_EPILOGUE), first)
    assert torch.equal(ops.conv(xd, wd, 1, layout, algo=ops.ALGO_EPILOGUE, relu=True, bias=bd), got)


def _view_at(t, shift):
    """A contiguous copy of `t` that starts `shift` elements into its allocation (element-aligned only)."""
    flat = torch.empty(t.numel() + shift, dtype=t.dtype, device=t.device)
    v = flat[shift:].view(t.shape)
    v.copy_(t)
    return v


@pytest.mark.parametrize("algo", [ops.ALGO_STAGED, ops.ALGO_EPILOGUE, ops.ALGO_FUSED, ops.ALGO_AUTO])
@pytest.mark.parametrize("layout", [ops.NCHW, ops.NHWC, ops.CHWN])
@pytest.mark.parametrize("dtype", [ops.F32, ops.F16])
@pytest.mark.parametrize("C", [32, 3])
def test_tensors_that_are_only_element_aligned(C, dtype, layout, algo):
    """x, w, bias and y may be any view of an allocation: only the alignment of the element type is
    required.  The vector paths either test the address or use loads that need no alignment; the result
    must be bit-identical with that of 256-byte aligned tensors."""
    from gpu_util import TORCH_DT
    N, K, H = 2, 64, 16
    g = torch.Generator(device="cuda").manual_seed(5)
    x = (torch.rand(ops.act_shape(layout, N, C, H, H), device="cuda", generator=g) - 0.5).to(TORCH_DT[dtype])
    wshape = {ops.NCHW: (K, C, 3, 3), ops.NHWC: (K, 3, 3, C), ops.CHWN: (C, 3, 3, K)}[layout]
    w = (torch.randn(wshape, device="cuda", generator=g) * 0.1).to(TORCH_DT[dtype])
    b = torch.randn(K, device="cuda", generator=g).to(TORCH_DT[dtype])
    want = ops.conv(x, w, 1, layout, algo=algo, bias=b, relu=True)
    for shift in (1, 3):
        out = _view_at(torch.zeros_like(want), shift)
        got = ops.conv(_view_at(x, shift), _view_at(w, shift), 1, layout, algo=algo, bias=_view_at(b, shift),
                       relu=True, out=out)
        assert got.data_ptr() % 16 != 0
        assert torch.equal(got, want), (shift, (got.float() - want.float()).abs().max().item())


@pytest.mark.parametrize("shape", [(1, 512, 128, 14, 14), (1, 144, 130, 10, 12), (2, 208, 64, 7, 7), (1, 256, 512, 28, 28)])
def test_staged_gemm_with_its_reduction_cut_into_runs(oracle, shape):
    """Layers with few workgroups have the channel reduction of the staged GEMM cut into runs (several partial
    products, summed by the output transform): deep reductions on small images, with run lengths that
    do and do not divide the channel count, both product orientations.  Integers: bit-exact."""
    N, C, K, H, W = shape
    x, w = synth.conv_inputs(N, C, K, H, W, seed=sum(shape), integer=True)
    want = oracle.direct_conv(x, w, 1)
    for dst in LAYOUTS:
        got = host(ops.conv(dev(x), dev(w), 1, ops.NCHW, dst, ops.ALGO_STAGED, relu=True))
        assert np.array_equal(got, synth.act_to_layout(np.maximum(want, 0), dst)), dst
    for dtype in (ops.F16, ops.BF16):
        xf, wf = synth.conv_inputs(N, C, K, H, W, seed=7 + sum(shape))
        got = host(ops.conv(dev(xf, dtype), dev(wf, dtype), 1, ops.NCHW, ops.NCHW, ops.ALGO_STAGED))
        from gpu_util import rounded
        ref = oracle.direct_conv(rounded(xf, dtype, oracle), rounded(wf, dtype, oracle), 1)
        assert oracle.rel_l2(got, ref) <= TOL[dtype]


@pytest.mark.parametrize("algo", [ops.ALGO_STAGED, ops.ALGO_EPILOGUE, ops.ALGO_STAGED_F4])
@pytest.mark.parametrize("dtype", [ops.F32, ops.F16, ops.BF16])
def test_element_aligned_views_of_images_larger_than_a_workgroup(dtype, algo):
    """H=W=40 (400 tiles per image: the LDS-tiled NCHW input transform, whose 2-byte form loads 4-byte pairs
    only from 4-byte aligned tensors) and, for F(4x4,3x3), an output tensor whose 4-element row stores need a
    16- or 8-byte aligned base: odd element offsets give the bits of the aligned call."""
    from gpu_util import TORCH_DT
    N, C, K, H = 2, 16, 64, 40
    g = torch.Generator(device="cuda").manual_seed(11)
    x = (torch.rand((N, C, H, H), device="cuda", generator=g) - 0.5).to(TORCH_DT[dtype])
    w = (torch.randn((K, C, 3, 3), device="cuda", generator=g) * 0.1).to(TORCH_DT[dtype])
    want = ops.conv(x, w, 1, ops.NCHW, algo=algo, relu=True)
    for shift in (1, 3):
        out = _view_at(torch.zeros_like(want), shift)
        got = ops.conv(_view_at(x, shift), _view_at(w, shift), 1, ops.NCHW, algo=algo, relu=True, out=out)
        assert got.data_ptr() % 8 != 0
        assert torch.equal(got, want), (shift, (got.float() - want.float()).abs().max().item())


@pytest.mark.parametrize("layouts", [(ops.NHWC, ops.NHWC), (ops.NCHW, ops.NHWC), (ops.NHWC, ops.NCHW)])
def test_auto_with_an_nhwc_side_and_an_output_that_is_only_element_aligned(layouts):
    """A 2-byte layer large enough for the direct path, x aligned, y at an odd element offset: with an NHWC side only
    the 8-wave direct kernel could run, and it stores 4-byte pairs -- the automatic choice has to see y's alignment
    and take the Winograd pipelines instead of refusing.  Small integers: every pipeline gives the same bits."""
    src, dst = layouts
    N, C, K, H = 32, 64, 64, 56
    x, w = synth.conv_inputs(N, C, K, H, H, seed=31, layout=src, integer=True)
    xd, wd = dev(x, ops.BF16), dev(w, ops.BF16)
    want = ops.conv(xd, wd, 1, src, dst, algo=ops.ALGO_AUTO, relu=True)
    out = _view_at(torch.zeros_like(want), 1)
    assert out.data_ptr() % 4 != 0
    got = ops.conv(xd, wd, 1, src, dst, algo=ops.ALGO_AUTO, relu=True, out=out)
    assert torch.equal(got, want)
