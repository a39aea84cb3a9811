"""Runs the C++ host program built from tests/host/dropin_test.cpp: a caller
written against the reference's own names (wrapedConv_*, layoutManager,
DataLayout) through include/wino_dropin.hpp, for all nine layout pairs."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def test_cpp_dropin_program():
    exe = os.path.join(HERE, "host", "dropin_test")
    assert os.path.exists(exe), "build it with `make -C tests/host` (done by __graft_entry__.build())"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "DROPIN OK" in r.stdout
