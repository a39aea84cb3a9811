"""The thirteen VGG-16 3x3 convolutions chained (C/K 64 -> 512, H/W 224 -> 14,
ReLU after every layer, no pooling fusion), f16 and bf16 storage with fp32
accumulation -- the call sequence of the reference's network driver
(netTest/cudnn_test_0124/VGG_Batched/Network.h:603-669: conv, ReLU, pool
between blocks).  The 2x2/2 pooling between blocks is not part of the
convolution path; here the activation is sub-sampled [::2, ::2] between blocks,
identically on both sides.

Oracle: fp32 direct convolution (+ReLU) of the same rounded input and weights.
Each layer is gated on its own (oracle fed the device's input of that layer),
and the error of the whole chain against an all-fp32 chain is gated as well:
relative L2 <= 2e-2."""
import numpy as np
import pytest
import torch

from cudnntest_amd import ops, synth
from gpu_util import TOL, dev, host, rounded

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [ops.F16, ops.BF16])
@pytest.mark.parametrize("algo", [ops.ALGO_AUTO, ops.ALGO_STAGED, ops.ALGO_EPILOGUE, ops.ALGO_FUSED])
def test_vgg16_conv_chain(oracle, dtype, algo):
    N = 2
    H = 224
    x_ref = rounded(synth.uniform_pm1(N * 3 * H * H, 0xC5).reshape(N, 3, H, H), dtype, oracle)   # fp32 chain
    x_dev = dev(x_ref, dtype)
    worst_layer, chain_err = 0.0, 0.0
    for li, (C, K, Hl) in enumerate(synth.VGG16_CONV):
        if Hl != x_ref.shape[2]:                      # block boundary: 2x sub-sampling on both sides
            x_ref = np.ascontiguousarray(x_ref[:, :, ::2, ::2])
            x_dev = x_dev[:, :, ::2, ::2].contiguous()
        assert x_ref.shape == (N, C, Hl, Hl)
        w = rounded(synth.normal(K * C * 9, 0x100 + li, float(np.sqrt(2.0 / (9.0 * C)))).reshape(K, C, 3, 3),
                    dtype, oracle)
        y_dev = ops.conv(x_dev, dev(w, dtype), 1, ops.NCHW, algo=algo, relu=True)
        # this layer on its own: oracle fed the very activation the device consumed
        want_layer = oracle.direct_conv_f32(host(x_dev), w, 1, relu=True)
        err = oracle.rel_l2(host(y_dev), want_layer)
        assert err <= TOL[dtype], (li, err)
        worst_layer = max(worst_layer, err)
        # the all-fp32 chain
        x_ref = oracle.direct_conv_f32(x_ref, w, 1, relu=True)
        chain_err = oracle.rel_l2(host(y_dev), x_ref)
        x_dev = y_dev
    print(f"dtype={dtype} algo={algo} worst single layer {worst_layer:.3e}, 13-layer chain {chain_err:.3e}")
    assert chain_err <= TOL[dtype], chain_err
