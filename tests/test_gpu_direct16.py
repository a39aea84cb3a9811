"""The direct (implicit-GEMM) path for 2-byte NCHW tensors (WINO_ALGO_DIRECT with more than four channels): the
convolution itself on the 16-bit matrix instruction with fp32 accumulation, no Winograd transform.  Oracle: the CPU
direct convolution (layoutTest/NCHW/data/WinoTran_NCHW.py:200-228 restated).  On small integers every product and
sum is exact in fp32, so the result must be the oracle's value rounded once to the tensor's type, bit for bit; on
floats the layer tolerance applies (relative L2 2e-2)."""
import numpy as np
import pytest
import torch

from cudnntest_amd import _lib, ops, synth
from gpu_util import TOL, TORCH_DT, dev, host, rounded

pytestmark = pytest.mark.gpu
# (N, C, K, H, W): blocks that span several images (14x14, 6x8), widths that do and do not fill a block's columns,
# channel counts with half a stage left over (8, 24, 40), filter counts off the 64-filter tile, a single row
SHAPES = [(2, 16, 64, 14, 14), (5, 8, 40, 6, 8), (1, 24, 130, 37, 20), (3, 40, 70, 9, 66), (2, 64, 64, 40, 34),
          (1, 16, 8, 1, 2), (4, 32, 96, 28, 28), (2, 16, 64, 224, 224),
          # the bank is padded to 32 channels: with C = 8, 40, 72 the last stage of 16 channels lies wholly past C
          # (its loads must stay inside the tensor: the first stage's channels again, masked)
          (3, 72, 64, 30, 34), (2, 8, 128, 100, 130), (1, 40, 64, 64, 62)]


@pytest.mark.parametrize("dtype", [ops.F16, ops.BF16])
@pytest.mark.parametrize("shape", SHAPES)
def test_integers_round_once(oracle, shape, dtype):
    N, C, K, H, W = shape
    x = synth.small_ints(N * C * H * W, sum(shape), -2, 2).reshape(N, C, H, W)
    w = synth.small_ints(K * C * 9, 7 + sum(shape), -1, 1).reshape(K, C, 3, 3)
    bias = synth.small_ints(K, 3, -2, 2).astype(np.float32)
    for pad in (1, 0):
        if H + 2 * pad - 2 <= 0 or W + 2 * pad - 2 <= 0:
            continue
        want = np.maximum(oracle.direct_conv(x, w, pad) + bias[None, :, None, None], 0).astype(np.float32)
        got = ops.conv(dev(x, dtype), dev(w, dtype), pad, algo=ops.ALGO_DIRECT, relu=True, bias=dev(bias, dtype))
        assert np.array_equal(host(got), rounded(want, dtype, oracle)), pad


# Layers with at least one tile per CU, output heights that are multiples of 4, even widths and filter counts that
# are multiples of 64 run on the 8-wave kernel (one workgroup per CU, tiles of 64 or 128 filters x 4-row strips):
# (N, C, K, H, W, pad)
#   * 128-filter tiles, a block as wide as the image, 4 stages per tile;
#   * 64-filter tiles (K = 64), 200 columns in a block of 256, a last stage whose second channel vector lies past C;
#   * K = 192 (64-filter tiles, three of them), no padding, blocks of 8 rows x 128 columns;
#   * 12-row images under blocks of 16 rows: a block spans three images;
#   * two column blocks, the second one half empty (this one stays on the 4-wave kernel: its block does not fit the
#     8-wave kernel's LDS plane).
BIG_SHAPES = [(32, 64, 128, 112, 112, 1), (16, 24, 64, 64, 200, 1), (12, 16, 192, 66, 130, 0), (192, 16, 256, 12, 24, 1),
              (16, 32, 128, 32, 160, 1)]


@pytest.mark.parametrize("dtype", [ops.F16, ops.BF16])
@pytest.mark.parametrize("shape", BIG_SHAPES)
def test_integers_round_once_one_tile_per_cu_and_more(oracle, shape, dtype):
    """Whole tensors against the staged Winograd pipeline (exact on these integers as well: every transformed value
    is a multiple of 1/4 far inside the 16-bit formats' exact range), the first and the last image's planes of
    three filters against the oracle, twice (the kernel's workgroups are persistent: the second run must not depend
    on what the first left in LDS)."""
    N, C, K, H, W, pad = shape
    x = synth.small_ints(N * C * H * W, sum(shape), -1, 1).reshape(N, C, H, W)
    w = synth.small_ints(K * C * 9, 7 + sum(shape), -1, 1).reshape(K, C, 3, 3)
    bias = synth.small_ints(K, 3, -2, 2).astype(np.float32)
    xd, wd, bd = dev(x, dtype), dev(w, dtype), dev(bias, dtype)
    ref = ops.conv(xd, wd, pad, algo=ops.ALGO_STAGED, relu=True, bias=bd)
    ks = sorted({0, K // 2, K - 1})
    for rep in range(2):
        got = ops.conv(xd, wd, pad, algo=ops.ALGO_DIRECT, relu=True, bias=bd)
        assert torch.equal(got, ref), rep
        for n in (0, N - 1):
            want = np.maximum(oracle.direct_conv(x[n:n + 1], w[ks], pad) + bias[ks][None, :, None, None], 0)
            assert np.array_equal(host(got[n:n + 1][:, ks]), rounded(want.astype(np.float32), dtype, oracle)), (rep, n)
    # 2x2 max pooling in the kernel's stores: the maximum of values that are rounded afterwards is the maximum of the
    # rounded values (rounding is monotonic), so the pooled tensor is the pooling of the unpooled one, bit for bit
    Ho, Wo = got.shape[2], got.shape[3]
    if shape == BIG_SHAPES[4]:
        # (130 columns of a 128-filter block x 6 rows do not fit the 8-wave kernel's LDS plane: this layer runs on the
        # 4-wave kernel, which has no pooling)
        with pytest.raises(_lib.WinoError):
            ops.conv(xd, wd, pad, algo=ops.ALGO_DIRECT, relu=True, bias=bd, pool=True)
        return
    pooled = ops.conv(xd, wd, pad, algo=ops.ALGO_DIRECT, relu=True, bias=bd, pool=True)
    assert tuple(pooled.shape) == (N, K, Ho // 2, Wo // 2)
    assert torch.equal(pooled, torch.nn.functional.max_pool2d(got.float(), 2).to(got.dtype))
    assert torch.equal(pooled, ops.conv(xd, wd, pad, algo=ops.ALGO_STAGED, relu=True, bias=bd, pool=True))


@pytest.mark.parametrize("dtype", [ops.F16, ops.BF16])
@pytest.mark.parametrize("shape", BIG_SHAPES[:4] + [(64, 256, 256, 28, 28, 1), (8, 72, 320, 56, 60, 1)])
def test_nhwc_tensors_on_the_8_wave_kernel(oracle, shape, dtype):
    """[N][H][W][C] tensors and [K][3][3][C] filters: the pixel's channel vectors are loaded as they lie, the
    multiplies run with the operands exchanged and the stores are along the filters.  Whole tensors against the staged
    Winograd pipeline from the same layout and against the NCHW direct kernel (same products, same order of
    summation: the same bits), planes of the first and last image against the oracle; twice."""
    N, C, K, H, W, pad = shape
    x = synth.small_ints(N * C * H * W, sum(shape), -1, 1).reshape(N, C, H, W)
    w = synth.small_ints(K * C * 9, 7 + sum(shape), -1, 1).reshape(K, C, 3, 3)
    bias = synth.small_ints(K, 3, -2, 2).astype(np.float32)
    xl, wl = synth.act_to_layout(x, ops.NHWC), synth.flt_to_layout(w, ops.NHWC)
    xd, wd, bd = dev(xl, dtype), dev(wl, dtype), dev(bias, dtype)
    if shape[:5] in ((64, 256, 256, 28, 28), (32, 64, 128, 112, 112)):                  # what AUTO takes for such layers
        assert ops.pick_algo(ops.NHWC, dtype, N, C, K, H, W, pad) == ops.ALGO_DIRECT
    ref = ops.conv(xd, wd, pad, ops.NHWC, algo=ops.ALGO_STAGED, relu=True, bias=bd)
    nchw = ops.conv(dev(x, dtype), dev(w, dtype), pad, algo=ops.ALGO_DIRECT, relu=True, bias=bd)
    ks = sorted({0, K // 2, K - 1})
    for rep in range(2):
        got = ops.conv(xd, wd, pad, ops.NHWC, algo=ops.ALGO_DIRECT, relu=True, bias=bd)
        assert torch.equal(got, ref), rep
        assert torch.equal(got.permute(0, 3, 1, 2), nchw), rep
        for n in (0, N - 1):
            want = np.maximum(oracle.direct_conv(x[n:n + 1], w[ks], pad) + bias[ks][None, :, None, None], 0)
            assert np.array_equal(host(got[n:n + 1].permute(0, 3, 1, 2)[:, ks]), rounded(want.astype(np.float32), dtype, oracle)), (rep, n)
    # the two sides are independent: NCHW in and NHWC out, NHWC in and NCHW out (the filters in the source's layout)
    cross = ops.conv(dev(x, dtype), dev(w, dtype), pad, ops.NCHW, ops.NHWC, algo=ops.ALGO_DIRECT, relu=True, bias=bd)
    assert torch.equal(cross, got)
    cross = ops.conv(xd, wd, pad, ops.NHWC, ops.NCHW, algo=ops.ALGO_DIRECT, relu=True, bias=bd)
    assert torch.equal(cross, nchw)
    cross = ops.conv(xd, wd, pad, ops.NHWC, ops.NCHW, algo=ops.ALGO_DIRECT, relu=True, bias=bd, pool=True)
    assert torch.equal(cross, torch.nn.functional.max_pool2d(nchw.float(), 2).to(nchw.dtype))
    # 2x2 pooling in the stores (rounding is monotonic: the pooled tensor is the pooling of the unpooled one)
    pooled = ops.conv(xd, wd, pad, ops.NHWC, algo=ops.ALGO_DIRECT, relu=True, bias=bd, pool=True)
    assert tuple(pooled.shape) == (N, got.shape[1] // 2, got.shape[2] // 2, K)
    assert torch.equal(pooled.permute(0, 3, 1, 2), torch.nn.functional.max_pool2d(got.permute(0, 3, 1, 2).float(), 2).to(got.dtype))
    assert torch.equal(pooled, ops.conv(xd, wd, pad, ops.NHWC, algo=ops.ALGO_STAGED, relu=True, bias=bd, pool=True))
    # floats: only the final rounding separates it from the oracle
    xf, wf = synth.conv_inputs(min(N, 2), C, K, H, W, seed=5 + sum(shape))
    xr, wr = rounded(xf, dtype, oracle), rounded(wf, dtype, oracle)
    if ops.pick_algo(ops.NHWC, dtype, min(N, 2), C, K, H, W, pad) == ops.ALGO_DIRECT:
        gotf = ops.conv(dev(synth.act_to_layout(xr, ops.NHWC), dtype), dev(synth.flt_to_layout(wr, ops.NHWC), dtype), pad, ops.NHWC)
        err = oracle.rel_l2(host(gotf.permute(0, 3, 1, 2)), oracle.direct_conv(xr, wr, pad))
        assert err <= (1e-3 if dtype == ops.F16 else 5e-3), err


# (N, C, K, H, W, pad) for [C][H][W][N] tensors, which the 8-wave kernel takes as ONE image of width W * N with its tap
# columns N elements apart:
#   * N = 32, 128-filter tiles: a block is 4 rows x 4 columns x 32 images, 14 x 14 blocks per filter tile;
#   * N = 32, K = 64 (64-filter tiles, 8 waves side by side: 8 columns x 32 images), a last stage half past C;
#   * N = 8: four columns to a wave, a row of 60 x 8 elements that ends inside a block; K = 192, no padding;
#   * N = 6: pairs of images, a block's 128 elements are 21 1/3 columns;
#   * 28 x 28 images, 512 filters: 7 x 7 blocks per filter tile, 16 stages.
CHWN_SHAPES = [(32, 64, 128, 56, 56, 1), (32, 24, 64, 64, 80, 1), (8, 16, 192, 130, 62, 0), (6, 32, 256, 96, 100, 1),
               (32, 256, 512, 28, 28, 1)]


@pytest.mark.parametrize("dtype", [ops.F16, ops.BF16])
@pytest.mark.parametrize("shape", CHWN_SHAPES)
def test_chwn_tensors_on_the_8_wave_kernel(oracle, shape, dtype):
    """[C][H][W][N] tensors and [C][3][3][K] filters.  Whole tensors against the staged Winograd pipeline from the same
    layout and against the NCHW direct kernel (same products, same order of summation: the same bits), planes of
    the first and last image against the oracle; twice; floats within the direct path's rounding."""
    N, C, K, H, W, pad = shape
    x = synth.small_ints(N * C * H * W, sum(shape), -1, 1).reshape(N, C, H, W)
    w = synth.small_ints(K * C * 9, 7 + sum(shape), -1, 1).reshape(K, C, 3, 3)
    bias = synth.small_ints(K, 3, -2, 2).astype(np.float32)
    xl, wl = synth.act_to_layout(x, ops.CHWN), synth.flt_to_layout(w, ops.CHWN)
    xd, wd, bd = dev(xl, dtype), dev(wl, dtype), dev(bias, dtype)
    if shape[:5] == (32, 64, 128, 56, 56):                  # what AUTO takes for such layers (at 28 x 28: Winograd)
        assert ops.pick_algo(ops.CHWN, dtype, N, C, K, H, W, pad) == ops.ALGO_DIRECT
    if shape[:5] == (32, 256, 512, 28, 28):
        assert ops.pick_algo(ops.CHWN, dtype, N, C, K, H, W, pad) != ops.ALGO_DIRECT
    ref = ops.conv(xd, wd, pad, ops.CHWN, algo=ops.ALGO_STAGED, relu=True, bias=bd)
    nchw = ops.conv(dev(x, dtype), dev(w, dtype), pad, algo=ops.ALGO_DIRECT, relu=True, bias=bd)
    ks = sorted({0, K // 2, K - 1})
    for rep in range(2):
        got = ops.conv(xd, wd, pad, ops.CHWN, algo=ops.ALGO_DIRECT, relu=True, bias=bd)
        assert torch.equal(got, ref), rep
        assert torch.equal(got.permute(3, 0, 1, 2), nchw), rep
        for n in (0, N - 1):
            want = np.maximum(oracle.direct_conv(x[n:n + 1], w[ks], pad) + bias[ks][None, :, None, None], 0)
            assert np.array_equal(host(got.permute(3, 0, 1, 2)[n:n + 1][:, ks]), rounded(want.astype(np.float32), dtype, oracle)), (rep, n)
    # pooling windows span columns N elements apart, in different waves: the layer runs unpooled into scratch and a
    # pooling kernel follows (rounding is monotonic: the same bits as pooling before the rounding)
    pooled = ops.conv(xd, wd, pad, ops.CHWN, algo=ops.ALGO_DIRECT, relu=True, bias=bd, pool=True)
    assert tuple(pooled.shape) == (K, got.shape[1] // 2, got.shape[2] // 2, N)
    assert torch.equal(pooled.permute(3, 0, 1, 2), torch.nn.functional.max_pool2d(nchw.float(), 2).to(nchw.dtype))
    assert torch.equal(pooled, ops.conv(xd, wd, pad, ops.CHWN, algo=ops.ALGO_STAGED, relu=True, bias=bd, pool=True))
    # other layouts on one side: not built
    with pytest.raises(_lib.WinoError) as e:
        ops.conv(xd, wd, pad, ops.CHWN, ops.NCHW, algo=ops.ALGO_DIRECT)
    assert e.value.code == -2
    assert torch.equal(ops.conv(xd, wd, pad, ops.CHWN, relu=True, bias=bd, pool=True),
                       ops.conv(xd, wd, pad, ops.CHWN, algo=ops.ALGO_STAGED, relu=True, bias=bd, pool=True))
    # floats: only the final rounding separates it from the oracle
    xf, wf = synth.conv_inputs(N, C, K, H, W, seed=5 + sum(shape))
    xr, wr = rounded(xf, dtype, oracle), rounded(wf, dtype, oracle)
    gotf = ops.conv(dev(synth.act_to_layout(xr, ops.CHWN), dtype), dev(synth.flt_to_layout(wr, ops.CHWN), dtype), pad, ops.CHWN,
                    algo=ops.ALGO_DIRECT)
    for n in (0, N - 1):
        err = oracle.rel_l2(host(gotf.permute(3, 0, 1, 2)[n:n + 1]), oracle.direct_conv(xr[n:n + 1], wr, pad))
        assert err <= (1e-3 if dtype == ops.F16 else 5e-3), err


@pytest.mark.parametrize("shape,layout", [((32, 64, 256, 56, 56), ops.NCHW), ((32, 64, 256, 56, 56), ops.NHWC),
                                          ((32, 32, 128, 112, 112), ops.NCHW), ((32, 64, 256, 56, 56), ops.CHWN),
                                          ((20, 48, 128, 60, 56), ops.NCHW)])
def test_layers_whose_images_are_cut_into_4_row_and_3_row_blocks(oracle, shape, layout):
    """Layers whose tiles would leave a good part of the chip idle in their last round: the 8-wave kernel's host side
    cuts every image into blocks whose waves own 4 rows and blocks whose waves own 3 (the VGG geometries at N = 32 with
    fewer channels: 56 x 56 with two filter tiles, 448 tiles -> 256 + 256; 112 x 112, 896 -> 512 + 512; the CHWN layer as
    one wide image; an image height that is a multiple of 4 but not of 8).  Small integers: the staged Winograd
    pipeline's bits, and the oracle's on the first and last image."""
    N, C, K, H, W = shape
    dtype = ops.BF16
    x = synth.small_ints(N * C * H * W, sum(shape), -1, 1).reshape(N, C, H, W)
    w = synth.small_ints(K * C * 9, 7 + sum(shape), -1, 1).reshape(K, C, 3, 3)
    bias = synth.small_ints(K, 3, -2, 2).astype(np.float32)
    xd, wd, bd = dev(synth.act_to_layout(x, layout), dtype), dev(synth.flt_to_layout(w, layout), dtype), dev(bias, dtype)
    ref = ops.conv(xd, wd, 1, layout, algo=ops.ALGO_STAGED, relu=True, bias=bd)
    got = ops.conv(xd, wd, 1, layout, algo=ops.ALGO_DIRECT, relu=True, bias=bd)
    assert torch.equal(got, ref)
    ks = sorted({0, K // 2, K - 1})
    g = synth.act_from_layout(host(got), layout)
    for n in (0, N - 1):
        want = np.maximum(oracle.direct_conv(x[n:n + 1], w[ks], 1) + bias[ks][None, :, None, None], 0)
        assert np.array_equal(g[n:n + 1][:, ks], rounded(want.astype(np.float32), dtype, oracle)), n
    # pooled: whole row pairs in a wave, so no cut (CHWN: the cut layer unpooled, then a pooling kernel) -- the same values, pooled
    pooled = ops.conv(xd, wd, 1, layout, algo=ops.ALGO_DIRECT, relu=True, bias=bd, pool=True)
    want = ops.conv(xd, wd, 1, layout, algo=ops.ALGO_STAGED, relu=True, bias=bd, pool=True)
    assert torch.equal(pooled, want)


def test_chwn_layers_the_8_wave_kernel_does_not_take():
    """An odd batch, a batch whose halo does not fit the LDS plane (N = 64), an output height off the 4-row strips: refused
    by name, and the automatic choice runs them through the Winograd pipelines."""
    for (N, C, K, H) in [(5, 16, 64, 32), (64, 16, 128, 32), (16, 16, 64, 30)]:
        x = torch.zeros((C, H, H, N), device="cuda", dtype=torch.bfloat16)
        w = torch.zeros((C, 3, 3, K), device="cuda", dtype=torch.bfloat16)
        with pytest.raises(_lib.WinoError) as e:
            ops.conv(x, w, 1, ops.CHWN, algo=ops.ALGO_DIRECT)
        assert e.value.code == -2
        assert ops.pick_algo(ops.CHWN, ops.BF16, N, C, K, H, H, 1) != ops.ALGO_DIRECT
        ops.conv(x, w, 1, ops.CHWN)


@pytest.mark.parametrize("dtype", [ops.F16, ops.BF16])
@pytest.mark.parametrize("shape", [(2, 64, 64, 56, 56), (1, 128, 256, 28, 28), (3, 256, 64, 14, 14)])
def test_floats_within_tolerance(oracle, shape, dtype):
    N, C, K, H, W = shape
    x, w = synth.conv_inputs(N, C, K, H, W, seed=61 + sum(shape))
    xr, wr = rounded(x, dtype, oracle), rounded(w, dtype, oracle)
    want = oracle.direct_conv(xr, wr, 1)
    got = ops.conv(dev(xr, dtype), dev(wr, dtype), 1, algo=ops.ALGO_DIRECT)
    err = oracle.rel_l2(host(got), want)
    assert err <= TOL[dtype], err
    # only the final rounding separates it from the oracle: far inside the layer tolerance
    assert err <= (1e-3 if dtype == ops.F16 else 5e-3), err
    # and the Winograd pipelines agree with it within their own rounding
    other = ops.conv(dev(xr, dtype), dev(wr, dtype), 1, algo=ops.ALGO_EPILOGUE)
    assert oracle.rel_l2(host(other), host(got)) <= TOL[dtype]


def test_element_aligned_views_and_what_is_refused():
    g = torch.Generator(device="cuda").manual_seed(3)
    x = (torch.rand((2, 16, 12, 12), device="cuda", generator=g) - 0.5).to(torch.bfloat16)
    w = (torch.randn((64, 16, 3, 3), device="cuda", generator=g) * 0.1).to(torch.bfloat16)
    want = ops.conv(x, w, algo=ops.ALGO_DIRECT)
    # w, bias and y may sit at any element offset; x must be 4-byte aligned (column pairs) and is refused otherwise
    flat = torch.empty(w.numel() + 1, dtype=w.dtype, device="cuda")
    w1 = flat[1:].view(w.shape)
    w1.copy_(w)
    out = torch.empty(want.numel() + 1, dtype=want.dtype, device="cuda")[1:].view(want.shape)
    assert torch.equal(ops.conv(x, w1, algo=ops.ALGO_DIRECT, out=out), want)
    xf = torch.empty(x.numel() + 1, dtype=x.dtype, device="cuda")
    x1 = xf[1:].view(x.shape)
    x1.copy_(x)
    with pytest.raises(_lib.WinoError) as e:
        ops.conv(x1, w, algo=ops.ALGO_DIRECT)
    assert e.value.code == -2
    assert torch.equal(ops.conv(x1, w, algo=ops.ALGO_EPILOGUE), ops.conv(x, w, algo=ops.ALGO_EPILOGUE))
    with pytest.raises(_lib.WinoError) as e:                   # pooling stays with the Winograd pipelines
        ops.conv(x, w, algo=ops.ALGO_DIRECT, pool=True)
    assert e.value.code == -2
    with pytest.raises(_lib.WinoError) as e:                   # and so do the other layouts
        ops.conv(x.permute(0, 2, 3, 1).contiguous(), w.permute(0, 2, 3, 1).contiguous(), src=ops.NHWC, algo=ops.ALGO_DIRECT)
    assert e.value.code == -2
    with pytest.raises(_lib.WinoError):                        # an odd width
        ops.conv(x[:, :, :, :11].contiguous(), w, algo=ops.ALGO_DIRECT)
    with pytest.raises(_lib.WinoError):                        # fp32 with more than four channels: small layers only
        ops.conv(x.float().repeat(64, 1, 4, 4), w.float(), algo=ops.ALGO_DIRECT)
