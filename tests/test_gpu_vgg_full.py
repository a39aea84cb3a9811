"""Every VGG-16 3x3 layer at its full size (N=32), in all three layouts, fp32, f16 and bf16, with the
algorithm AUTO picks: the configuration list of the reference's layer driver
(comparison/layoutCompare.cu:38-148, one case per (C, K, H) of the network) at the batch the
headline numbers are quoted on.

The CPU oracle cannot convolve whole layers of this size in test time, so the check is in two parts:
  * the planes (n, k) for n = N-1 and three filters k are compared with the oracle's direct convolution
    of that image with those filters (the oracle sees exactly the values the device was given);
  * the NHWC and CHWN results must agree with the NCHW result of the same values over the whole tensor
    (different input kernels, tile orders, store paths; the same arithmetic up to summation order).
Tolerances: relative L2 1e-4 (fp32), 2e-2 (f16, bf16)."""
import numpy as np
import pytest
import torch

from cudnntest_amd import ops, synth
from gpu_util import TOL, TORCH_DT, host

pytestmark = pytest.mark.gpu
N = 32


def to_layout(t_nchw, layout, flt=False):
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


@pytest.mark.parametrize("dtype", [ops.F32, ops.F16, ops.BF16])
@pytest.mark.parametrize("layer", range(len(synth.VGG16_CONV)))
def test_full_size_layer_all_layouts(oracle, layer, dtype):
    C, K, H = synth.VGG16_CONV[layer]
    g = torch.Generator(device="cuda").manual_seed(0xF00 + layer)
    tdt = TORCH_DT[dtype]
    x = (torch.rand((N, C, H, H), device="cuda", generator=g) * 2 - 1).to(tdt)
    w = (torch.randn((K, C, 3, 3), device="cuda", generator=g) * (2.0 / (9 * C)) ** 0.5).to(tdt)
    ks = sorted({0, K // 2, K - 1})
    want = oracle.direct_conv_f32(host(x[N - 1:N]), host(w[ks]), 1)          # [1][len(ks)][H][H]
    y_nchw = None
    for layout in (ops.NCHW, ops.NHWC, ops.CHWN):
        y = from_layout(ops.conv(to_layout(x, layout), to_layout(w, layout, flt=True), 1, layout), layout)
        assert tuple(y.shape) == (N, K, H, H)
        got = host(y[N - 1:N][:, ks])
        err = oracle.rel_l2(got, want)
        assert err <= TOL[dtype], (layout, err)
        if y_nchw is None:
            y_nchw = y.float()
        else:
            rel = ((y.float() - y_nchw).norm() / y_nchw.norm()).item()
            assert rel <= (1e-5 if dtype == ops.F32 else 1e-2), (layout, rel)
        del y
