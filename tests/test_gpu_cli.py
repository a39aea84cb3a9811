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
