"""Index arithmetic past 2^31: a layer whose transformed operands hold more than 2^31 elements (N=768, C=K=256,
H=W=56 in fp32: x and y 617 M elements = 2.5 GB each, the transformed input V 2.47 G elements = 9.9 GB, the product
tensor of the staged pipeline as much again, byte offsets past 2^33).  The oracle convolves the LAST image (the far
end of every index space) with three filters; the pipelines must agree with each other over the whole tensor."""
import pytest
import torch

from cudnntest_amd import ops
from gpu_util import TOL, host

pytestmark = pytest.mark.gpu
N, C, K, H = 768, 256, 256, 56


def _rel(a, b):
    # norms in chunks: a float64 copy of a 2.5 GB tensor is not needed
    num = sum(((a[i:i + 64].double() - b[i:i + 64].double()) ** 2).sum().item() for i in range(0, a.shape[0], 64))
    den = sum((b[i:i + 64].double() ** 2).sum().item() for i in range(0, b.shape[0], 64))
    return (num / den) ** 0.5


@pytest.mark.parametrize("layout", [ops.NCHW, ops.NHWC])
def test_more_than_2_31_elements_per_operand(oracle, layout):
    free, _ = torch.cuda.mem_get_info()
    if free < 40 * 2 ** 30:
        pytest.skip("needs 40 GB of free device memory")
    g = torch.Generator(device="cuda").manual_seed(31)
    x = torch.rand((N, C, H, H), device="cuda", generator=g) * 2 - 1
    w = torch.randn((K, C, 3, 3), device="cuda", generator=g) * (2.0 / (9 * C)) ** 0.5
    assert 16 * (N * 28 * 28) * C > 2 ** 31
    ks = [0, K // 2, K - 1]
    want = oracle.direct_conv_f32(host(x[N - 1:]), host(w[ks]), 1)
    if layout == ops.NHWC:
        xl, wl = x.permute(0, 2, 3, 1).contiguous(), w.permute(0, 2, 3, 1).contiguous()
        del x
    else:
        xl, wl = x, w
    ys = {}
    for algo in (ops.ALGO_EPILOGUE, ops.ALGO_STAGED, ops.ALGO_STAGED_F4):
        y = ops.conv(xl, wl, 1, layout, algo=algo)
        y_nchw = y.permute(0, 3, 1, 2) if layout == ops.NHWC else y
        assert tuple(y_nchw.shape) == (N, K, H, H)
        err = oracle.rel_l2(host(y_nchw[N - 1:][:, ks]), want)
        assert err <= TOL[ops.F32], (algo, err)
        ys[algo] = y
    assert _rel(ys[ops.ALGO_STAGED], ys[ops.ALGO_EPILOGUE]) <= 1e-5
    # the F(4x4) pipeline (what the automatic choice runs at this size): 5.5 GB of transformed input, as much product
    assert ops.pick_algo(layout, ops.F32, N, C, K, H, H, 1) == ops.ALGO_STAGED_F4
    assert _rel(ys[ops.ALGO_STAGED_F4], ys[ops.ALGO_STAGED]) <= 2e-5
    # leave the scratch arena at its usual size for the tests that follow
    del ys, y, xl
    torch.cuda.empty_cache()


@pytest.mark.parametrize("Nl", [208, 334])
def test_first_layer_with_byte_offsets_past_2_31(oracle, Nl):
    """The few-channel direct kernels address x and y with 32-bit byte offsets off a scalar base; the library offers
    them up to 2^30 elements a tensor.  208 and 334 images of 3 x 224 x 224 into 64 filters in fp32: y holds 668 M and
    1073 M elements (the last below 2^30 by a thousandth), byte offsets past 2^31 and up to 4.29 GB.  The tiled
    kernel against the oracle on the last image, and against the gathering kernel (an element-aligned view of x) over
    the whole tensor.  (2-byte tensors of 2^30 elements end below 2^31 bytes.)"""
    free, _ = torch.cuda.mem_get_info()
    if free < 16 * 2 ** 30:
        pytest.skip("needs 16 GB of free device memory")
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.rand((Nl, 3, 224, 224), device="cuda", generator=g) * 2 - 1
    w = torch.randn((64, 3, 3, 3), device="cuda", generator=g) * 0.2
    assert 2 ** 31 < Nl * 64 * 224 * 224 * 4 < 2 ** 32 and Nl * 64 * 224 * 224 < 2 ** 30
    y = ops.conv(x, w, 1, algo=ops.ALGO_DIRECT)
    want = oracle.direct_conv_f32(host(x[Nl - 1:]), host(w), 1)
    assert oracle.rel_l2(host(y[Nl - 1:]), want) <= 1e-6
    shifted = torch.empty(x.numel() + 1, dtype=x.dtype, device="cuda")[1:].view(x.shape)
    shifted.copy_(x)
    y2 = ops.conv(shifted, w, 1, algo=ops.ALGO_DIRECT)
    assert all(torch.equal(y[i:i + 16], y2[i:i + 16]) for i in range(0, Nl, 16))
    del x, y, y2, shifted
    torch.cuda.empty_cache()


def test_first_layer_from_nhwc_with_byte_offsets_past_2_31(oracle):
    """The same for the NHWC tiles: 334 images, y of 4.29 GB; the last image against the oracle, the whole tensor
    against the gathering kernel (an element-aligned view of x)."""
    free, _ = torch.cuda.mem_get_info()
    if free < 16 * 2 ** 30:
        pytest.skip("needs 16 GB of free device memory")
    Nl = 334
    g = torch.Generator(device="cuda").manual_seed(8)
    xn = torch.rand((Nl, 3, 224, 224), device="cuda", generator=g) * 2 - 1
    wn = torch.randn((64, 3, 3, 3), device="cuda", generator=g) * 0.2
    x, w = xn.permute(0, 2, 3, 1).contiguous(), wn.permute(0, 2, 3, 1).contiguous()
    y = ops.conv(x, w, 1, ops.NHWC, algo=ops.ALGO_DIRECT)
    want = oracle.direct_conv_f32(host(xn[Nl - 1:]), host(wn), 1)
    assert oracle.rel_l2(host(y[Nl - 1:].permute(0, 3, 1, 2).contiguous()), want) <= 1e-6
    del xn
    shifted = torch.empty(x.numel() + 1, dtype=x.dtype, device="cuda")[1:].view(x.shape)
    shifted.copy_(x)
    y2 = ops.conv(shifted, w, 1, ops.NHWC, algo=ops.ALGO_DIRECT)
    assert all(torch.equal(y[i:i + 16], y2[i:i + 16]) for i in range(0, Nl, 16))
    del x, y, y2, shifted
    torch.cuda.empty_cache()

