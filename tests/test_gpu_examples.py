"""The example programs (examples/101_gemm) run on the GPU and check themselves against a CPU
fp32 loop; a non-zero exit status is a mismatch."""

import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DIR = os.path.join(ROOT, "examples", "101_gemm")


@pytest.mark.parametrize("binary", ["01_gemm_global_reg/gemm_global_reg", "02_gemm_all_mem/gemm_all_mem"])
def test_example_runs_and_checks_itself(binary):
    path = os.path.join(DIR, binary)
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", DIR])
    out = subprocess.run([path], capture_output=True, text=True, timeout=100)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "(ok)" in out.stdout and "TFLOP/s" in out.stdout
