"""CPU-side checks of the C-ABI library: it loads, exports every function that
include/wino_amd.h declares, validates arguments before touching a GPU, and its
geometry matches the oracle's tile arithmetic."""
import ctypes
import os
import re

import pytest

from cudnntest_amd import _lib, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    text = open(os.path.join(ROOT, "include", "wino_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(wino_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = ctypes.CDLL(_lib.LIB_PATH)
    names = header_functions()
    assert len(names) >= 14
    for n in names:
        assert hasattr(L, n), f"{n} declared in wino_amd.h but not exported"
    assert sorted(_lib.SYMBOLS) == names, "ctypes table and header disagree"


def test_version_string():
    assert b"gfx950" in _lib.load().wino_version()


@pytest.mark.parametrize("shape,want", [
    ((32, 256, 256, 56, 56, 1), dict(th=28, tw=28, P=25088, Cp=256, Kp=256, Pp=25088)),
    ((1, 64, 64, 56, 56, 1), dict(th=28, tw=28, P=784, Cp=64, Kp=128, Pp=896)),
    ((32, 3, 64, 224, 224, 1), dict(th=112, tw=112, P=401408, Cp=16, Kp=128, Pp=401408)),
    ((2, 5, 7, 9, 6, 1), dict(th=5, tw=3, P=30, Cp=16, Kp=128, Pp=128)),
    ((1, 1, 1, 5, 5, 0), dict(th=2, tw=2, P=4, Cp=16, Kp=128, Pp=128)),
])
def test_geometry(oracle, shape, want):
    N, C, K, H, W, pad = shape
    g = ops.geometry(ops.F32, N, C, K, H, W, pad)
    assert g == want
    assert (g["th"], g["tw"]) == oracle.wino_tiles(2, H, W, pad)


def test_workspace_bytes_covers_operands():
    N, C, K, H, W = 32, 256, 256, 56, 56
    g = ops.geometry(ops.F32, N, C, K, H, W, 1)
    need = 4 * 16 * (g["Cp"] * g["Kp"] + g["Cp"] * g["Pp"] + g["Kp"] * g["Pp"])
    assert ops.workspace_bytes(ops.F32, N, C, K, H, W, 1) >= need
    assert ops.workspace_bytes(ops.F16, N, C, K, H, W, 1) < ops.workspace_bytes(ops.F32, N, C, K, H, W, 1)


def test_invalid_arguments_are_rejected_without_a_gpu():
    L = _lib.load()
    one = ctypes.c_void_p(16)   # never dereferenced: validation fails first
    # null tensors
    assert L.wino_conv(0, 0, 0, 0, 0, 1, 1, 1, 4, 4, 1, None, one, one, None) == -1
    assert L.wino_conv(0, 0, 0, 0, 0, 1, 1, 1, 4, 4, 1, one, None, one, None) == -1
    assert b"null" in L.wino_last_error()
    # bad enums
    assert L.wino_conv(7, 0, 0, 0, 0, 1, 1, 1, 4, 4, 1, one, one, one, None) == -1
    assert L.wino_conv(0, 0, 9, 0, 0, 1, 1, 1, 4, 4, 1, one, one, one, None) == -1
    assert L.wino_conv(0, 0, 0, 12, 0, 1, 1, 1, 4, 4, 1, one, one, one, None) == -1
    # bad shapes: zero batch, image too small for pad 0, negative and absurd pad
    assert L.wino_conv(0, 0, 0, 0, 0, 0, 1, 1, 4, 4, 1, one, one, one, None) == -1
    assert L.wino_conv(0, 0, 0, 0, 0, 1, 1, 1, 2, 2, 0, one, one, one, None) == -1
    assert L.wino_conv(0, 0, 0, 0, 0, 1, 1, 1, 4, 4, -1, one, one, one, None) == -1
    assert L.wino_conv(0, 0, 0, 0, 0, 1, 1, 1, 4, 4, 1025, one, one, one, None) == -1
    assert b"bad shape" in L.wino_last_error()
    assert L.wino_filter_transform(0, 0, 0, 4, one, one, None) == -1
    assert L.wino_input_transform(0, 0, 5, 1, 1, 4, 4, 1, one, one, None) == -1
    assert L.wino_batched_gemm(0, 0, 0, 1, 1, one, one, one, None) == -1
    assert L.wino_batched_gemm(0, 5, 1, 1, 1, one, one, one, None) == -1
    assert L.wino_output_transform(3, 0, 0, 0, 0, 1, 1, 4, 4, one, one, None) == -1
    assert L.wino_layout_transform(0, 1, 0, 1, 1, 0, 4, one, one, None) == -1
    assert L.wino_workspace_bytes(0, 0, 1, 1, 4, 4, 1) == 0
    # alignment: tensors to their element size, Winograd-domain operands to 16 bytes
    odd, off8 = ctypes.c_void_p(18), ctypes.c_void_p(24)
    assert L.wino_conv(0, 0, 0, 0, 0, 1, 1, 1, 4, 4, 1, odd, one, one, None) == -1
    assert b"aligned" in L.wino_last_error()
    assert L.wino_conv(0, 0, 1, 0, 0, 1, 1, 1, 4, 4, 1, one, one, ctypes.c_void_p(17), None) == -1
    assert L.wino_conv_prepared(0, 0, 0, 0, 0, 1, 1, 1, 4, 4, 1, one, off8, one, None) == -1
    assert b"16-byte" in L.wino_last_error()
    assert L.wino_filter_transform(0, 0, 4, 4, one, off8, None) == -1
    assert L.wino_input_transform(0, 0, 0, 1, 1, 4, 4, 1, one, off8, None) == -1
    assert L.wino_batched_gemm(0, 0, 4, 4, 4, one, off8, one, None) == -1
    assert L.wino_output_transform(0, 0, 0, 0, 0, 1, 1, 4, 4, off8, one, None) == -1
    assert L.wino_gemm_output(0, 0, 0, 0, 1, 4, 4, 4, 4, off8, one, one, None) == -1


def test_operator_layer_refuses_cpu_tensors():
    import torch
    x = torch.zeros(1, 1, 4, 4)
    w = torch.zeros(1, 1, 3, 3)
    with pytest.raises(ValueError):
        ops.conv(x, w)


def test_datalayout_enum_order_matches_reference():
    # enum class DataLayout { NCHW, NHWC, CHWN }  comparison/DataLayoutTrans.cuh:587-591
    assert [int(v) for v in ops.DataLayout] == [0, 1, 2]
    assert [v.name for v in ops.DataLayout] == ["NCHW", "NHWC", "CHWN"]


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    """There is no fallback path: without the built library, loading raises."""
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libwino_amd.so"))
    monkeypatch.setattr(_lib, "_lib", None)
    with pytest.raises(RuntimeError, match="missing"):
        _lib.load()


def test_product_never_imports_the_oracle():
    import glob
    for f in glob.glob(os.path.join(ROOT, "cudnntest_amd", "*.py")):
        text = open(f).read()
        assert "import oracle" not in text and "from oracle" not in text, f


def test_bench_refuses_more_than_one_gpu_and_runs_nothing_without_one():
    """bench.py measures one GPU: --gpus N > 1 exits with a message before touching a device; without a GPU the
    default run exits with a message as well (no CPU path stands in for the kernels)."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "ONE GPU" in r.stderr
    import torch
    if not torch.cuda.is_available():
        r = subprocess.run([sys.executable, os.path.join(root, "bench.py")], capture_output=True, text=True)
        assert r.returncode != 0 and "no GPU" in r.stderr


def test_the_algorithm_sweep_tool_imports_without_a_gpu():
    """python3 -m cudnntest_amd.algo_sweep needs a GPU to run; its grids and the algorithm table load without one."""
    from cudnntest_amd import algo_sweep, ops
    assert set(algo_sweep.GRIDS) == {"f32", "f16", "bf16"}
    assert algo_sweep.ALGOS["f4"] == ops.ALGO_STAGED_F4 and algo_sweep.ALGOS["direct"] == ops.ALGO_DIRECT
