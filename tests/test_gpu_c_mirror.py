"""Runs the C test program of the reference-shaped wrappers (include/qlinear_tf.h): a plain C caller,
qtensor structs over host memory, every linear call checked against decoded rows in double."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "c", "test_tf_mirror")


def test_c_caller_through_reference_shaped_wrappers():
    assert os.path.exists(EXE), "run `python -m gemm_amd.build` first"
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all C-mirror checks passed" in r.stdout
    assert "qmatvec failed" in r.stderr  # the unsupported-type case reports on stderr, as the reference does
