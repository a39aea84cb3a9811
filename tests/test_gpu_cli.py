"""The command-line driver cudnntest_amd/cli/layout_compare: the reference's `batch= opt= layer=`
interface (comparison/layoutCompare.cu:32-148) and its raw float32 files (get_parameter /
save_parameter, comparison/util.h:99-127).  The program is given files written here, run for each
layout, and its saved output compared with the CPU oracle."""
import os
import re
import subprocess

import numpy as np
import pytest

from cudnntest_amd import ops, synth

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "..", "cudnntest_amd", "cli", "layout_compare")


@pytest.mark.parametrize("opt,layout", [(0, ops.NCHW), (1, ops.NHWC), (2, ops.CHWN)])
def test_cli_reads_bin_files_and_matches_the_oracle(oracle, tmp_path, opt, layout):
    assert os.path.exists(EXE), "build it with `make -C cudnntest_amd/cli` (done by __graft_entry__.build())"
    N, C, K, H = 2, 512, 512, 14                    # layer=9 of the reference's table
    x, w = synth.conv_inputs(N, C, K, H, H, seed=909, layout=layout)
    (tmp_path / "vggData").mkdir()
    (tmp_path / "binImage").mkdir()
    w.astype("<f4").tofile(tmp_path / "vggData" / "conv13.bin")
    for i in range(2):
        x.astype("<f4").tofile(tmp_path / "binImage" / f"file_{i}.bin")
    out = tmp_path / "y.bin"
    r = subprocess.run([EXE, f"batch={N}", f"opt={opt}", "layer=9", f"data={tmp_path}", "runs=2", f"save={out}"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "synthetic" not in r.stdout              # both files were found and read
    assert r.stdout.count(["Conv_NCHW", "Conv_NHWC", "Conv_CHWN"][opt]) == 2
    times = re.findall(r"time:([0-9.]+) ms", r.stdout)
    assert len(times) == 2 and all(float(t) > 0 for t in times)
    want = oracle.direct_conv(x, w, 1, layout)
    got = np.fromfile(out, dtype="<f4").reshape(want.shape)
    assert oracle.rel_l2(got, want) <= 1e-4
    first = float(re.findall(r"convOutput_cpu\[0\]:(-?[0-9.]+)", r.stdout)[-1])
    assert abs(first - want.ravel()[0]) <= 1e-3 * max(1.0, abs(want.ravel()[0]))


def test_cli_falls_back_to_synthetic_data_and_rejects_bad_options(tmp_path):
    r = subprocess.run([EXE, "batch=1", "opt=0", "layer=9", f"data={tmp_path}", "runs=1"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "synthetic filters" in r.stdout and "time:" in r.stdout
    assert subprocess.run([EXE, "batch=1", "opt=3", "layer=9"], capture_output=True, text=True).returncode == 2
    assert subprocess.run([EXE, "batch=1", "opt=0", "layer=12"], capture_output=True, text=True).returncode == 2


MODULE = os.path.join(HERE, "..", "cudnntest_amd", "cli", "conv_module")


@pytest.mark.parametrize("layout,name", [(ops.NCHW, "NCHW"), (ops.NHWC, "NHWC"), (ops.CHWN, "CHWN")])
@pytest.mark.parametrize("algo", ["auto", "f4"])
def test_conv_module_reads_its_two_files_and_matches_the_oracle(oracle, tmp_path, layout, name, algo):
    """cudnntest_amd/cli/conv_module: the reference's per-layout stand-alone driver
    (layoutTest/NHWC/convModule_NHWC_padding.cu:8-121; `a.out <N> <inside> <chn> <numOfFilter>`,
    data/input.bin + data/filter.bin -> data/ConvModule_<LAYOUT>.bin), at the shape its notebooks use
    (inside 22, 128 channels and filters) with a small batch."""
    assert os.path.exists(MODULE), "build it with `make -C cudnntest_amd/cli` (done by __graft_entry__.build())"
    N, C, K, H = 3, 128, 128, 22
    x, w = synth.conv_inputs(N, C, K, H, H, seed=2222, layout=layout)
    (tmp_path / "data").mkdir()
    x.astype("<f4").tofile(tmp_path / "data" / "input.bin")
    w.astype("<f4").tofile(tmp_path / "data" / "filter.bin")
    r = subprocess.run([MODULE, str(N), str(H), str(C), str(K), f"layout={name}", f"data={tmp_path}", f"algo={algo}"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "synthetic" not in r.stdout
    assert f"inside: {H}, oside:{H}" in r.stdout
    us = re.findall(r"([0-9]+\.[0-9]+) us", r.stdout)          # what layoutTest/NHWC/test.sh greps for
    assert len(us) == 1 and float(us[0]) > 0
    want = oracle.direct_conv(x, w, 1, layout)
    got = np.fromfile(tmp_path / "data" / f"ConvModule_{name}.bin", dtype="<f4").reshape(want.shape)
    assert oracle.rel_l2(got, want) <= 1e-4
    first = float(re.findall(r"convOutput_cpu\[0\]:(-?[0-9.]+)", r.stdout)[-1])
    assert abs(first - want.ravel()[0]) <= 1e-3 * max(1.0, abs(want.ravel()[0]))


def test_conv_module_without_files_and_with_bad_arguments(tmp_path):
    r = subprocess.run([MODULE, "2", "22", "128", "128", f"data={tmp_path}", "padding=0", "runs=2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "synthetic input" in r.stdout and "inside: 22, oside:20" in r.stdout
    assert "Bad file path" in r.stdout              # no data directory: the output is not saved, the run still counts
    assert subprocess.run([MODULE, "2", "22", "128"], capture_output=True, text=True).returncode == 2
    assert subprocess.run([MODULE, "2", "22", "128", "128", "layout=HWCN"], capture_output=True, text=True).returncode == 2
    assert subprocess.run([MODULE, "0", "22", "128", "128"], capture_output=True, text=True).returncode == 2
