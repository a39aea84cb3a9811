"""The conv-stack driver (wino_stack_*): the convolution part of the reference's network driver
classify_example_modified (netTest/cudnn_test_0124/VGG_Batched/Network.h:603-669) -- per layer a
3x3 convolution in the layer's own layout pair, bias, ReLU, and 2x2 pooling after some layers --
with the filter transforms cached.  Oracle: the CPU direct convolution layer by layer, bias / ReLU /
pooling in NumPy."""
import numpy as np
import pytest
import torch

from cudnntest_amd import _lib, ops, synth
from gpu_util import TOL, TORCH_DT, dev, host, rounded

pytestmark = pytest.mark.gpu


def reference_chain(oracle, x_nchw, params, layers):
    """fp32 chain in NCHW: conv + bias -> relu -> pool, per layer."""
    a = x_nchw
    for (w, b), L in zip(params, layers):
        a = oracle.direct_conv_f32(a, w, 1)
        a = a + b[None, :, None, None]
        if L.get("relu"):
            a = np.maximum(a, 0)
        if L.get("pool"):
            N, K, H, W = a.shape
            a = a[:, :, :H // 2 * 2, :W // 2 * 2].reshape(N, K, H // 2, 2, W // 2, 2).max(axis=(3, 5))
        a = np.ascontiguousarray(a.astype(np.float32))
    return a


def make_params(oracle, C, layers, dtype):
    params = []
    for i, L in enumerate(layers):
        K = L["K"]
        w = rounded(synth.normal(K * C * 9, 0x300 + i, float(np.sqrt(2.0 / (9.0 * C)))).reshape(K, C, 3, 3), dtype, oracle)
        b = rounded(synth.normal(K, 0x400 + i, 0.1).astype(np.float32), dtype, oracle)
        params.append((w, b))
        C = K
    return params


VGG_LIKE = [dict(K=16, relu=True), dict(K=16, relu=True, pool=True), dict(K=32, relu=True),
            dict(K=32, relu=True, pool=True), dict(K=64, relu=True), dict(K=64, relu=True, pool=True)]


@pytest.mark.parametrize("dtype", [ops.F32, ops.F16, ops.BF16])
@pytest.mark.parametrize("layout", [ops.NCHW, ops.NHWC, ops.CHWN])
def test_stack_matches_the_layerwise_oracle(oracle, layout, dtype):
    N, C, H = 3, 3, 36
    layers = [dict(L, layout_in=layout, layout_out=layout) for L in VGG_LIKE]
    # the reference hands the activations over to NCHW at its last convolution (vggCUDNN.cu:173-176)
    layers[-1]["layout_out"] = ops.NCHW
    params = make_params(oracle, C, layers, dtype)
    x = rounded(synth.uniform_pm1(N * C * H * H, 0xA1).reshape(N, C, H, H), dtype, oracle)
    want = reference_chain(oracle, x, params, layers)

    st = ops.ConvStack(TORCH_DT[dtype], N, C, H, H, layers)
    assert tuple(st.out_shape) == want.shape and st.out_layout == ops.NCHW
    for i, (w, b) in enumerate(params):
        st.set_layer(i, dev(synth.flt_to_layout(w, layout), dtype), dev(b, dtype))
    xd = dev(synth.act_to_layout(x, layout), dtype)
    got = st.forward(xd)
    assert oracle.rel_l2(host(got), want) <= TOL[dtype]

    # the same layers one wino_conv_ex call at a time give the same bits
    a = xd
    for (w, b), L in zip(params, layers):
        a = ops.conv(a, dev(synth.flt_to_layout(w, layout), dtype), 1, L["layout_in"], L["layout_out"],
                     relu=L.get("relu", False), pool=L.get("pool", False), bias=dev(b, dtype))
    assert torch.equal(a, got)
    # a second pass over the cached transforms gives the same bits again
    assert torch.equal(st.forward(xd), got)
    st.close()


def test_stack_rejects_bad_requests():
    with pytest.raises(_lib.WinoError):          # layer 1 reads what layer 0 does not write
        ops.ConvStack(torch.float32, 1, 3, 8, 8, [dict(K=4, layout_in=ops.NCHW, layout_out=ops.NHWC),
                                                   dict(K=4, layout_in=ops.CHWN)])
    st = ops.ConvStack(torch.float32, 1, 3, 8, 8, [dict(K=4), dict(K=4, pool=True)])
    assert tuple(st.out_shape) == (1, 4, 4, 4)
    x = torch.zeros((1, 3, 8, 8), device="cuda")
    with pytest.raises(_lib.WinoError):          # no filters yet
        st.forward(x)
    st.set_layer(0, torch.zeros((4, 3, 3, 3), device="cuda"))
    with pytest.raises(_lib.WinoError):          # layer 1 still missing
        st.forward(x)
    with pytest.raises(_lib.WinoError):
        st.set_layer(2, torch.zeros((4, 4, 3, 3), device="cuda"))
    st.set_layer(1, torch.zeros((4, 4, 3, 3), device="cuda"), torch.ones(4, device="cuda"))
    assert torch.equal(st.forward(x), torch.ones((1, 4, 4, 4), device="cuda"))
    st.close()


def test_stack_replayed_from_a_graph_matches_eager_launches(oracle):
    """wino_stack_forward_graph: every replay -- with eager work of the library and synchronisations in
    between, after the input changed in place, after a change of tensors and after the scratch arena moved --
    gives the bits of the eager pass."""
    N, C, H = 2, 3, 20
    layers = [dict(L, layout_in=ops.NCHW, layout_out=ops.NCHW) for L in VGG_LIKE[:4]]
    params = make_params(oracle, C, layers, ops.F32)
    st = ops.ConvStack(torch.float32, N, C, H, H, layers)
    for i, (w, b) in enumerate(params):
        st.set_layer(i, dev(w), dev(b))
    x = dev(synth.uniform_pm1(N * C * H * H, 0xC1).reshape(N, C, H, H))
    other_x, other_w = synth.conv_inputs(2, 8, 8, 12, 12, seed=5)
    other_x, other_w = dev(other_x), dev(other_w)
    out = torch.empty(st.out_shape, device="cuda")
    want = st.forward(x).clone()
    for rep in range(4):
        out.zero_()
        st.forward(x, out=out, graph=True)
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep
        ops.conv(other_x, other_w)                    # eager work between the replays
        torch.cuda.synchronize()
    x.mul_(-0.5)                                      # new values behind the same pointer
    want2 = st.forward(x).clone()
    assert not torch.equal(want2, want)
    assert torch.equal(st.forward(x, out=out, graph=True), want2)
    x2, out2 = x.clone(), torch.empty_like(out)       # other tensors: recorded again
    assert torch.equal(st.forward(x2, out=out2, graph=True), want2)
    big_x, big_w = synth.conv_inputs(4, 64, 64, 40, 40, seed=6)
    ops.conv(dev(big_x), dev(big_w), algo=ops.ALGO_STAGED)   # grows the arena: its address may change
    torch.cuda.synchronize()
    for rep in range(2):
        out2.zero_()
        assert torch.equal(st.forward(x2, out=out2, graph=True), want2), rep
    st.close()


def test_stack_graph_follows_a_change_of_bias(oracle):
    """set_layer after a recorded pass -- a bias added, then removed again -- is seen by the next replay: the
    recorded launches hold the bias pointer (or its absence), so setting a layer drops the recording."""
    N, C, H = 2, 3, 12
    layers = [dict(K=8, relu=True), dict(K=8, relu=True)]
    params = make_params(oracle, C, layers, ops.F32)
    st = ops.ConvStack(torch.float32, N, C, H, H, layers)
    x = dev(synth.uniform_pm1(N * C * H * H, 0xB5).reshape(N, C, H, H))
    out = torch.empty(st.out_shape, device="cuda")
    for i, (w, b) in enumerate(params):
        st.set_layer(i, dev(w), None)
    no_bias = st.forward(x).clone()
    assert torch.equal(st.forward(x, out=out, graph=True), no_bias)
    for i, (w, b) in enumerate(params):
        st.set_layer(i, dev(w), dev(b + 0.5))
    with_bias = st.forward(x).clone()
    assert not torch.equal(with_bias, no_bias)
    assert torch.equal(st.forward(x, out=out, graph=True), with_bias)
    assert torch.equal(st.forward(x, out=out, graph=True), with_bias)
    st.set_layer(1, dev(params[1][0]), None)
    want = st.forward(x).clone()
    assert torch.equal(st.forward(x, out=out, graph=True), want)
    with pytest.raises(ValueError):          # a bank of the wrong size is refused before it reaches the device
        st.set_layer(0, torch.zeros((8, 4, 3, 3), device="cuda"))
    with pytest.raises(ValueError):
        st.set_layer(0, dev(params[0][0]), torch.zeros(7, device="cuda"))
    st.close()


@pytest.mark.parametrize("layout", [ops.NCHW, ops.NHWC, ops.CHWN])
def test_stack_layers_on_the_f4_pipeline(oracle, layout):
    """fp32 layers that the automatic choice runs through F(4x4,3x3) (C, K >= 128, one of them 256, 512 tiles and
    more): the stack transforms their filters for that pipeline when they are set; the pass gives the bits of the
    layers run one by one with the algorithm named, and the oracle's planes within the fp32 tolerance."""
    N, C, H = 32, 128, 32
    layers = [dict(K=256, relu=True, pool=True, layout_in=layout, layout_out=layout),
              dict(K=128, relu=True, pool=False, layout_in=layout, layout_out=layout)]
    assert ops.pick_algo(layout, ops.F32, N, C, 256, H, H, 1) == ops.ALGO_STAGED_F4
    assert ops.pick_algo(layout, ops.F32, N, 256, 128, H // 2, H // 2, 1) == ops.ALGO_STAGED_F4
    st = ops.ConvStack(torch.float32, N, C, H, H, layers)
    g = torch.Generator(device="cuda").manual_seed(0xF4)
    x = torch.rand((N, C, H, H), device="cuda", generator=g) * 2 - 1
    ws, bs = [], []
    c = C
    for i, L in enumerate(layers):
        ws.append(torch.randn((L["K"], c, 3, 3), device="cuda", generator=g) * (2.0 / (9 * c)) ** 0.5)
        bs.append(torch.randn((L["K"],), device="cuda", generator=g) * 0.1)
        c = L["K"]

    def lay(t, flt=False):
        if layout == ops.NCHW:
            return t.contiguous()
        return (t.permute(0, 2, 3, 1) if layout == ops.NHWC else t.permute(1, 2, 3, 0)).contiguous()

    for i in range(2):
        st.set_layer(i, lay(ws[i]), bs[i])
    got = st.forward(lay(x)).clone()
    a = lay(x)
    for i, L in enumerate(layers):
        a = ops.conv(a, lay(ws[i]), 1, layout, algo=ops.ALGO_STAGED_F4, relu=True, pool=L["pool"], bias=bs[i])
    assert torch.equal(got, a)
    got_nchw = got if layout == ops.NCHW else (got.permute(0, 3, 1, 2) if layout == ops.NHWC else got.permute(3, 0, 1, 2))
    want = reference_chain(oracle, host(x[-1:]), [(host(w), host(b)) for w, b in zip(ws, bs)], layers)
    assert oracle.rel_l2(host(got_nchw[-1:]), want) <= TOL[ops.F32]
    out = torch.empty_like(got)
    for rep in range(2):
        out.zero_()
        st.forward(lay(x), out=out, graph=True)
        torch.cuda.synchronize()
        assert torch.equal(out, got), rep
