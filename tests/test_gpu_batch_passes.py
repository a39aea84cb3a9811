"""Whole-layer calls that the library runs as several passes over the batch (2-byte epilogue pipeline with a
transformed input far larger than the last-level cache: each pass transforms and multiplies a slice of the
images, reusing the same scratch).  The result must not depend on the cut: on small integers it is bit-identical
with the staged pipeline, which always runs the batch in one pass, and image by image with the CPU oracle."""
import numpy as np
import pytest
import torch

from cudnntest_amd import ops, synth
from gpu_util import TORCH_DT, dev, host

pytestmark = pytest.mark.gpu


def _ints(shape, seed, lo, hi, dtype):
    return dev(synth.small_ints(int(np.prod(shape)), seed, lo, hi).reshape(shape), dtype)


@pytest.mark.parametrize("dtype", [ops.F16, ops.BF16])
@pytest.mark.parametrize("src,dst", [(ops.NCHW, ops.NCHW), (ops.NHWC, ops.NHWC), (ops.NCHW, ops.NHWC)])
@pytest.mark.parametrize("pool", [False, True])
def test_uneven_passes_match_single_pass(oracle, dtype, src, dst, pool):
    # 33 images of 64 channels at 112x112: 212 MB of transformed input in 2-byte elements -> two passes, 17 + 16 images
    N, C, K, H = 33, 64, 128, 112
    x = synth.act_to_layout(host(_ints((N, C, H, H), 11, -2, 2, dtype)), src)
    w_kcrs = host(_ints((K, C, 3, 3), 12, -1, 1, dtype))
    w = {ops.NCHW: w_kcrs, ops.NHWC: w_kcrs.transpose(0, 2, 3, 1)}[src]
    bias = _ints((K,), 13, -3, 3, dtype)
    xd, wd = dev(x, dtype), dev(w, dtype)
    got = ops.conv(xd, wd, 1, src, dst, algo=ops.ALGO_EPILOGUE, relu=True, bias=bias, pool=pool)
    ref = ops.conv(xd, wd, 1, src, dst, algo=ops.ALGO_STAGED, relu=True, bias=bias, pool=pool)
    assert torch.equal(got, ref)
    # the first and the last image (one in each pass) against the CPU oracle
    y = got if dst == ops.NCHW else got.permute(0, 3, 1, 2)
    x_nchw = x if src == ops.NCHW else x.transpose(0, 3, 1, 2)
    for n in (0, N - 1):
        want = oracle.direct_conv_f32(np.ascontiguousarray(x_nchw[n:n + 1]), w_kcrs[:3], 1) + host(bias)[:3, None, None]
        want = np.maximum(want, 0.0)
        if pool:
            want = want.reshape(1, 3, H // 2, 2, H // 2, 2).max(axis=(3, 5))
        assert np.array_equal(host(y[n:n + 1, :3]), host(dev(want, dtype)))


def test_prepared_filters_and_passes(oracle):
    """The same cut with the filter bank transformed beforehand (no filter work in any pass)."""
    N, C, K, H = 32, 64, 128, 112
    x = _ints((N, C, H, H), 21, -2, 2, ops.BF16)
    w = _ints((K, C, 3, 3), 22, -1, 1, ops.BF16)
    U = ops.filter_transform(w, ops.NCHW)
    got = ops.conv_prepared(x, U, K, 1, ops.NCHW, algo=ops.ALGO_EPILOGUE)
    ref = ops.conv(x, w, 1, ops.NCHW, algo=ops.ALGO_STAGED)
    assert torch.equal(got, ref)


@pytest.mark.parametrize("layout", [ops.NCHW, ops.NHWC])
def test_stack_with_multi_pass_layers_eager_and_graph(oracle, layout):
    """Two bf16 layers of the size that is cut into passes (and that AUTO runs on the 16-bit direct kernel, the second
    one with pooling in its stores), as a conv stack: the eager pass equals the layers run one by one through the
    one-pass staged pipeline, and graph replays equal the eager pass."""
    N, C, K, H = 32, 64, 128, 112
    layers = [dict(K=K, relu=True, pool=False, layout_in=layout), dict(K=K, relu=True, pool=True)]
    st = ops.ConvStack(torch.bfloat16, N, C, H, H, layers)
    perm = (lambda t: t.permute(0, 2, 3, 1).contiguous()) if layout == ops.NHWC else (lambda t: t)
    w1, w2 = perm(_ints((K, C, 3, 3), 31, -1, 1, ops.BF16)), perm(_ints((K, K, 3, 3), 32, -1, 1, ops.BF16))
    b1, b2 = _ints((K,), 33, -2, 2, ops.BF16), _ints((K,), 34, -2, 2, ops.BF16)
    st.set_layer(0, w1, b1)
    st.set_layer(1, w2, b2)
    x = perm(_ints((N, C, H, H), 35, -1, 1, ops.BF16))
    mid = ops.conv(x, w1, 1, layout, algo=ops.ALGO_STAGED, relu=True, bias=b1)
    ref = ops.conv(mid, w2, 1, layout, algo=ops.ALGO_STAGED, relu=True, bias=b2, pool=True)
    want = st.forward(x).clone()
    assert torch.equal(want, ref)
    out = torch.empty(st.out_shape, dtype=torch.bfloat16, device="cuda")
    for rep in range(3):
        out.zero_()
        st.forward(x, out=out, graph=True)
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep
    st.close()
