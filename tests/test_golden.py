"""The committed golden fixtures (tests/golden/conv3x3_fixtures.npz, written by tests/golden/make_fixtures.py
from the float64 definition of the convolution and the closed-form F(2x2,3x3) matrices, cross-checked there
against torch's float64 conv2d): the CPU oracle must reproduce them (no GPU needed), and the HIP path must
match them through the C ABI -- bit-exact on the integer problems, relative L2 <= 1e-4 on the float ones."""
import itertools
import os

import numpy as np
import pytest

from cudnntest_amd import ops, synth

FIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "conv3x3_fixtures.npz"))
PROBLEMS = sorted({k[:-2] for k in FIX.files if k.endswith("_x")})      # "s0_int", "s0_flt", ...
LAYOUTS = [ops.NCHW, ops.NHWC, ops.CHWN]


def test_fixture_file_is_complete():
    assert len(PROBLEMS) == 8
    for p in PROBLEMS:
        for part in ("x", "w", "y_pad0", "y_pad1"):
            assert f"{p}_{part}" in FIX.files
    assert all(FIX[k].dtype == np.float32 for k in FIX.files)
    for part in "UVM":
        assert "s0_int_" + part in FIX.files


@pytest.mark.parametrize("problem", PROBLEMS)
def test_oracle_reproduces_the_fixtures(oracle, problem):
    x, w = FIX[problem + "_x"], FIX[problem + "_w"]
    for pad in (0, 1):
        want = FIX[f"{problem}_y_pad{pad}"]
        for src, dst in itertools.product(LAYOUTS, LAYOUTS):
            got = oracle.direct_conv(synth.act_to_layout(x, src), synth.flt_to_layout(w, src), pad, src, dst)
            got = synth.act_from_layout(got, dst)
            if problem.endswith("_int"):
                assert np.array_equal(got, want), (pad, src, dst)
            else:
                assert oracle.rel_l2(got, want) <= 1e-6, (pad, src, dst)


def test_oracle_winograd_stages_reproduce_the_fixtures(oracle):
    x, w = FIX["s0_int_x"], FIX["s0_int_w"]
    U, V = oracle.wino_filter_transform(w), oracle.wino_input_transform(x, 1)
    assert np.array_equal(U, FIX["s0_int_U"]) and np.array_equal(V, FIX["s0_int_V"])
    M = oracle.wino_gemm(U, V)
    assert np.array_equal(M, FIX["s0_int_M"])
    assert np.array_equal(oracle.wino_output_transform(M, 2, 5, 5), FIX["s0_int_y_pad1"])


@pytest.mark.gpu
@pytest.mark.parametrize("algo", [ops.ALGO_AUTO, ops.ALGO_STAGED, ops.ALGO_EPILOGUE, ops.ALGO_FUSED, ops.ALGO_STAGED_F4,
                                  ops.ALGO_EPILOGUE_F4])
@pytest.mark.parametrize("problem", PROBLEMS)
def test_hip_path_matches_the_fixtures(oracle, problem, algo):
    from gpu_util import TOL, dev, host
    x, w = FIX[problem + "_x"], FIX[problem + "_w"]
    exact = problem.endswith("_int") and algo not in (ops.ALGO_STAGED_F4, ops.ALGO_EPILOGUE_F4)     # F(4x4)'s 1/6, 1/24 are not dyadic
    for pad in (0, 1):
        want = FIX[f"{problem}_y_pad{pad}"]
        for src, dst in itertools.product(LAYOUTS, LAYOUTS):
            got = host(ops.conv(dev(synth.act_to_layout(x, src)), dev(synth.flt_to_layout(w, src)), pad, src, dst, algo))
            got = synth.act_from_layout(got, dst)
            if exact:
                assert np.array_equal(got, want), (pad, src, dst)
            else:
                assert oracle.rel_l2(got, want) <= TOL[ops.F32], (pad, src, dst)


@pytest.mark.gpu
def test_hip_stages_match_the_fixtures():
    from gpu_util import dev, host, pack_operand, unpack_operand
    x, w = FIX["s0_int_x"], FIX["s0_int_w"]
    U, V, M = FIX["s0_int_U"], FIX["s0_int_V"], FIX["s0_int_M"]
    _, C, K = U.shape
    P = V.shape[2]
    Ud, Vd = ops.filter_transform(dev(w)), ops.input_transform(dev(x), 1)
    Uh, Vh = unpack_operand(Ud), unpack_operand(Vd)
    assert np.array_equal(Uh[:, :C, :K], U) and not Uh[:, C:, :].any() and not Uh[:, :C, K:].any()
    assert np.array_equal(Vh[:, :C, :P], V) and not Vh[:, C:, :P].any()
    Mh = host(ops.batched_gemm(Ud, Vd, C, K, P))
    assert np.array_equal(Mh[:, :K, :P], M)
    y = host(ops.output_transform(ops.batched_gemm(Ud, Vd, C, K, P), 2, K, 5, 5))
    assert np.array_equal(y, FIX["s0_int_y_pad1"])
    assert np.array_equal(host(ops.gemm_output(Ud, Vd, 2, C, K, 5, 5)), FIX["s0_int_y_pad1"])
