"""The micro-benchmarks under benchmarks/ run on the GPU and check their own results."""

import io
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_g2s_copy_benchmark_checks_itself():
    d = os.path.join(ROOT, "benchmarks", "cpp", "g2s_copy")
    path = os.path.join(d, "g2s_copy")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", d])
    out = subprocess.run([path], capture_output=True, text=True, timeout=100)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.count("|ok|") == 22 and "all configurations ok" in out.stdout


def test_fused_two_gemms_sweep_is_correct_on_a_few_shapes():
    import importlib.util

    spec = importlib.util.spec_from_file_location("fused_bench", os.path.join(ROOT, "benchmarks", "fused_two_gemms", "bench.py"))
    fused_bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(fused_bench)

    buf = io.StringIO()
    assert fused_bench.run(shapes=[(512, 512), (2048, 2048), (4096, 1024)], out=buf), buf.getvalue()
    assert "MISMATCH" not in buf.getvalue()


def test_fused_launch_floor_table():
    import importlib.util

    spec = importlib.util.spec_from_file_location("fused_bench2", os.path.join(ROOT, "benchmarks", "fused_two_gemms", "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    # the table has its three rows and every time is a positive finite number; how long a launch
    # takes is the box's business and is reported, not asserted
    rows = mod.launch_floor(out=io.StringIO())
    assert len(rows) == 3 and all(t > 0 and t == t and t != float("inf") for _, t in rows), rows


def test_gemm_sweep_is_correct_on_the_small_shapes():
    sys.path.insert(0, os.path.join(ROOT, "benchmarks", "gemm"))
    import importlib.util

    spec = importlib.util.spec_from_file_location("gemm_bench", os.path.join(ROOT, "benchmarks", "gemm", "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    buf = io.StringIO()
    assert mod.run(shapes=mod.SHAPES[:5], out=buf), buf.getvalue()
    assert "MISMATCH" not in buf.getvalue()


def test_header_kernel_gemm_table_is_correct():
    import importlib.util

    spec = importlib.util.spec_from_file_location("header_kernels", os.path.join(ROOT, "benchmarks", "gemm", "header_kernels.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    buf = io.StringIO()
    assert mod.run(out=buf), buf.getvalue()
    assert "MISMATCH" not in buf.getvalue()


def test_attention_head_dim_table_is_correct_on_a_small_problem():
    import importlib.util

    import torch

    spec = importlib.util.spec_from_file_location("attn_bench", os.path.join(ROOT, "benchmarks", "attention", "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    buf = io.StringIO()
    cases = [(128, torch.float16, True, "tuned"), (64, torch.bfloat16, False, "tuned"), (96, torch.float16, True, "tuned"),
             (160, torch.float16, True, "header kernel"), (32, torch.bfloat16, False, "header kernel"),
             (80, torch.float16, False, "torch op: padded to 96, tuned")]
    assert mod.run(cases=cases, bh=2, s=512, out=buf), buf.getvalue()
    assert "MISMATCH" not in buf.getvalue()
