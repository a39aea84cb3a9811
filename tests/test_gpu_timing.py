"""The library's per-stage timing: the event pairs that the reference's wrapper keeps commented out around
its four stages (comparison/wrapedConv_NCHW.cuh:88-138) and the average / minimum / maximum report of its
per-stage harness (delayTest/testbench/src/M1/M1Test.h:100-151).  Checked here: which stages each algorithm
records, how many spans, that min <= mean <= max, that reading the statistics forgets them, and that
nothing is recorded (and results are the same) while timing is off."""
import pytest
import torch

from cudnntest_amd import ops

pytestmark = pytest.mark.gpu
RUNS = 5


def _inputs():
    g = torch.Generator(device="cuda").manual_seed(77)
    x = torch.rand((4, 32, 28, 28), device="cuda", generator=g) - 0.5
    w = torch.randn((64, 32, 3, 3), device="cuda", generator=g) * 0.1
    return x, w


@pytest.mark.parametrize("algo,expect", [
    (ops.ALGO_STAGED, {"filter": RUNS, "input": RUNS, "gemm": RUNS, "output": RUNS}),
    (ops.ALGO_EPILOGUE, {"filter": RUNS, "input": RUNS, "gemm": RUNS, "output": 0}),
    (ops.ALGO_FUSED, {"filter": RUNS, "input": 0, "gemm": RUNS, "output": 0}),
])
def test_stage_statistics(algo, expect):
    x, w = _inputs()
    ref = ops.conv(x, w, 1, ops.NCHW, algo=algo).clone()
    torch.cuda.synchronize()
    ops.stage_stats()                                   # forget whatever earlier tests left
    ops.stage_timing(True)
    try:
        for _ in range(RUNS):
            y = ops.conv(x, w, 1, ops.NCHW, algo=algo)
        st = ops.stage_stats()
    finally:
        ops.stage_timing(False)
    assert torch.equal(y, ref)
    for name, n in expect.items():
        total, lo, hi, calls = st[name]
        assert calls == n, (name, st)
        if n == 0:
            assert total == 0.0 and lo == 0.0 and hi == 0.0
            continue
        assert 0.0 < lo <= hi < 50.0, (name, st)
        assert lo * n <= total * 1.0001 and total <= hi * n * 1.0001, (name, st)
    again = ops.stage_stats()                           # reading forgets
    assert all(v == (0.0, 0.0, 0.0, 0) for v in again.values())


def test_nothing_recorded_while_timing_is_off():
    x, w = _inputs()
    ops.stage_stats()
    ops.conv(x, w, 1, ops.NCHW, algo=ops.ALGO_STAGED)
    torch.cuda.synchronize()
    assert all(v[1] == 0 for v in ops.stage_times().values())


def test_totals_only_call_agrees_with_statistics():
    x, w = _inputs()
    ops.stage_stats()
    ops.stage_timing(True)
    try:
        ops.conv(x, w, 1, ops.NCHW, algo=ops.ALGO_STAGED)
        st = ops.stage_times()
    finally:
        ops.stage_timing(False)
    assert [st[s][1] for s in ops.STAGES] == [1, 1, 1, 1]
    assert all(st[s][0] > 0 for s in ops.STAGES)
