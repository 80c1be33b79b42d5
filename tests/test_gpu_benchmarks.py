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


def test_mfma_ceiling_probe_runs_and_stays_under_the_peak():
    d = os.path.join(ROOT, "benchmarks", "cpp", "mfma_ceiling")
    path = os.path.join(d, "mfma_ceiling")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", d])
    out = subprocess.run([path], capture_output=True, text=True, timeout=100)
    assert out.returncode == 0, out.stdout + out.stderr
    rows = [line.split("|") for line in out.stdout.splitlines() if line.startswith("|v_mfma")]
    assert len(rows) == 2
    for r in rows:
        tflops, cycles = float(r[3]), float(r[5])
        assert 500 < tflops < 2500 and 250 <= cycles < 400, out.stdout


def test_simd_issue_probe_shows_what_the_attention_schedule_relies_on():
    d = os.path.join(ROOT, "benchmarks", "cpp", "simd_issue")
    path = os.path.join(d, "simd_issue")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", d])
    out = subprocess.run([path], capture_output=True, text=True, timeout=100)
    assert out.returncode == 0 and out.stdout.rstrip().endswith("done"), out.stdout + out.stderr
    rows = {line.split("|")[1]: [float(x) for x in line.split("|")[2:5]]
            for line in out.stdout.splitlines() if line.startswith("|v_")}
    # ordinary VALU instructions run at about half rate next to an MFMA stream; v_dot2 is far worse,
    # which is why the attention kernel adds up its row sums on the matrix pipe
    assert 4.0 < rows["v_fma_f32"][0] < 7.0 and 6.5 < rows["v_fma_f32"][1] < 11.0, out.stdout
    assert rows["v_dot2c_f32_f16"][1] > 1.5 * rows["v_fma_f32"][1], out.stdout
    blocks = [line.split("|") for line in out.stdout.splitlines() if line.startswith("|alone|") and line.count("|") == 4]
    assert blocks and 1088 <= float(blocks[0][2]) < 2000 and 1088 <= float(blocks[0][3]) < 2000, out.stdout


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
    rows = mod.launch_floor(out=io.StringIO())
    (_, empty), (_, cached), (_, hbm) = rows
    assert 0.5 < empty < cached * 1.05 and cached < 20 and hbm < 20, rows


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
    cases = [(128, torch.float16, True, "tuned"), (64, torch.bfloat16, False, "tuned"),
             (96, torch.float16, True, "header kernel"), (32, torch.bfloat16, False, "header kernel")]
    assert mod.run(cases=cases, bh=2, s=512, out=buf), buf.getvalue()
    assert "MISMATCH" not in buf.getvalue()
