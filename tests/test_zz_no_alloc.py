"""wino_conv_noalloc -- the whole-layer call whose scratch is a fixed buffer inside the library's device image --
against wino_conv_ex, the entry point it is a variant of: the same kernels, so the same bits.  Two calls in a
row, the second on a smaller input (the buffer keeps the first call's contents; what must start at zero is the
arrival counters, which the kernels leave at zero), for every pipeline that uses scratch; a problem beyond the
buffer is refused with the workspace status and nothing is launched."""
import numpy as np
import pytest
import torch

from cudnntest_amd import _lib, ops, synth
from gpu_util import TORCH_DT, dev, host

pytestmark = pytest.mark.gpu
LIMIT = 64 << 20          # WINO_NOALLOC_SCRATCH_BYTES


def both(x, w, b, layout, algo, **kw):
    want = ops.conv(x, w, 1, layout, algo=algo, bias=b, **kw)
    got = torch.full_like(want, float("nan"))
    ops.conv_noalloc(x, w, got, 1, layout, algo=algo, bias=b, **kw)
    return got, want


ALGOS = [ops.ALGO_AUTO, ops.ALGO_STAGED, ops.ALGO_EPILOGUE, ops.ALGO_FUSED, ops.ALGO_STAGED_F4]
# (the F(4x4) GEMM with the output transform in its epilogue is fp32 only)
CASES = [(ops.F32, a) for a in ALGOS + [ops.ALGO_EPILOGUE_F4]] + [(ops.BF16, a) for a in ALGOS]


@pytest.mark.parametrize("layout", [ops.NCHW, ops.NHWC, ops.CHWN])
@pytest.mark.parametrize("dtype,algo", CASES)
def test_two_calls_in_a_row_match_the_allocating_entry_point(oracle, dtype, algo, layout):
    # first a layer that fills a good part of the buffer, then a smaller one with other channel and filter counts
    for (N, C, K, H) in [(4, 64, 96, 56), (1, 24, 40, 13)]:
        resolved = ops.pick_algo(layout, dtype, N, C, K, H, H) if algo == ops.ALGO_AUTO else algo
        f4 = resolved in (ops.ALGO_STAGED_F4, ops.ALGO_EPILOGUE_F4)      # (F(4x4) rounds where F(2x2) is exact)
        x, w = synth.conv_inputs(N, C, K, H, H, seed=900 + C, layout=layout, integer=True)
        bias = dev(synth.small_ints(K, seed=4, lo=-2, hi=2).astype(np.float32), dtype)
        got, want = both(dev(x, dtype), dev(w, dtype), bias, layout, algo, relu=True)
        assert torch.equal(got, want), (N, C, K, H)
        if not f4 and dtype == ops.F32:     # and the oracle itself: small integers are exact in every fp32 pipeline
            ref = oracle.direct_conv(x, w, 1, layout)
            ref = synth.act_from_layout(ref, layout) + host(bias)[None, :, None, None]
            ref = synth.act_to_layout(np.ascontiguousarray(np.maximum(ref, 0).astype(np.float32)), layout)
            assert np.array_equal(host(got), ref)


def test_the_call_leaves_the_free_device_memory_unchanged():
    """No hipMalloc on the call path: the device's free memory is the same before and after calls on shapes the
    library has not seen (the arena would have to grow for them), for every pipeline that keeps scratch."""
    ops.warmup()
    N, C, K, H = 3, 40, 72, 30
    x, w = synth.conv_inputs(N, C, K, H, H, seed=77)
    xd, wd = dev(x), dev(w)
    out = torch.empty((N, K, H, H), device="cuda")
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for algo in (ops.ALGO_STAGED, ops.ALGO_EPILOGUE, ops.ALGO_FUSED, ops.ALGO_STAGED_F4, ops.ALGO_EPILOGUE_F4, ops.ALGO_AUTO):
        ops.conv_noalloc(xd, wd, out, 1, ops.NCHW, algo=algo)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0


def test_cut_up_rounds_share_the_counters_from_call_to_call():
    """fp32 epilogue GEMM with a small last round (N=65: 520 patches on 512 places): the cut-up patches use the
    arrival counters and the partial-sum region of the buffer; three calls in a row, then a smaller problem."""
    C, K, H, W = 8, 64, 32, 64
    for N in (65, 65, 65, 3):
        x, w = synth.conv_inputs(N, C, K, H, W, seed=70 + N)
        got, want = both(dev(x), dev(w), None, ops.NCHW, ops.ALGO_EPILOGUE)
        assert torch.equal(got, want), N


def test_a_problem_beyond_the_buffer_is_refused():
    N, C, K, H = 8, 64, 64, 112          # V alone: 16 * 25088 * 64 * 4 bytes = 103 MB
    x = torch.zeros((N, C, H, H), device="cuda")
    w = torch.zeros((K, C, 3, 3), device="cuda")
    out = torch.full((N, K, H, H), 7.0, device="cuda")
    with pytest.raises(_lib.WinoError) as e:
        ops.conv_noalloc(x, w, out, algo=ops.ALGO_EPILOGUE)
    assert e.value.code == -4 and str(LIMIT) in str(e.value)
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())      # nothing ran
    # the single-kernel pipeline keeps only the transformed filters and fits
    x.uniform_(-1, 1)
    w.normal_(0, 0.05)
    ops.conv_noalloc(x, w, out, algo=ops.ALGO_FUSED)
    assert torch.equal(out, ops.conv(x, w, algo=ops.ALGO_FUSED))


def test_pooled_chwn_layers_with_and_without_room_for_the_unpooled_tensor(oracle):
    """A pooled 2-byte CHWN layer on the direct path keeps the unpooled tensor in scratch.  N = 32, C = K = 64: at 56 x 56
    it fits the buffer (12.8 MB) and the call runs the same two kernels as wino_conv_ex; at 160 x 160 it does not
    (105 MB), and the automatic choice falls back to a Winograd pipeline that fits -- small integers, so both are exact
    and agree bit for bit."""
    for H in (56, 160):
        N, C, K = 32, 64, 64
        x, w = synth.conv_inputs(N, C, K, H, H, seed=H, layout=ops.CHWN, integer=True)
        bias = dev(synth.small_ints(K, seed=4, lo=-2, hi=2).astype(np.float32), ops.BF16)
        got, want = both(dev(x, ops.BF16), dev(w, ops.BF16), bias, ops.CHWN, ops.ALGO_AUTO, relu=True, pool=True)
        assert (N * K * H * H * 2 > LIMIT) == (H == 160)
        assert torch.equal(got, want), H


@pytest.mark.parametrize("layout", [ops.NCHW, ops.NHWC, ops.CHWN])
def test_pooled_first_layers_with_and_without_room_for_the_unpooled_tensor(oracle, layout):
    """The same for a pooled layer of three channels (direct into scratch, then the pooling kernel): N = 32, K = 64 in
    bf16 at 56 x 56 (12.8 MB unpooled) and at 160 x 160 (105 MB: NCHW and NHWC layers run in two passes of 16 images,
    a CHWN layer, whose images cannot be cut, goes to the single Winograd kernel, which keeps only its filters in
    scratch)."""
    for H in (56, 160):
        N, C, K = 32, 3, 64
        x, w = synth.conv_inputs(N, C, K, H, H, seed=H, layout=layout, integer=True)
        bias = dev(synth.small_ints(K, seed=4, lo=-2, hi=2).astype(np.float32), ops.BF16)
        got, want = both(dev(x, ops.BF16), dev(w, ops.BF16), bias, layout, ops.ALGO_AUTO, relu=True, pool=True)
        assert (N * K * H * H * 2 > LIMIT) == (H == 160)
        assert torch.equal(got, want), H



def test_the_automatic_choice_stays_inside_the_buffer(oracle):
    """fp32, N = 8, C = 512, K = 64, 56 x 56: the automatic choice is F(4x4), whose transformed input and product take 130 MB;
    inside the 64 MB buffer the call runs the single Winograd kernel instead (2 MB of transformed filters) -- the same bits
    as that kernel by name."""
    N, C, K, H = 8, 512, 64, 56
    x, w = synth.conv_inputs(N, C, K, H, H, seed=5)
    xd, wd = dev(x), dev(w)
    assert ops.pick_algo(ops.NCHW, ops.F32, N, C, K, H, H) == ops.ALGO_STAGED_F4
    out = torch.empty((N, K, H, H), device="cuda")
    ops.conv_noalloc(xd, wd, out, 1, ops.NCHW, algo=ops.ALGO_AUTO)
    assert torch.equal(out, ops.conv(xd, wd, 1, ops.NCHW, algo=ops.ALGO_FUSED))
