"""Throughput of the header macro kernels (kernels/gemm_device.hpp) instantiated at run time,
beside the tuned ahead-of-time GEMM and hipBLASLt, at the 4096^3 fp16 shape.

ke_gemm is the synchronous composition of the tile movers (include/kernels/gemm_device.cuh:134-208
in the reference), ke_gemm_level1_pipeline keeps num_stages - 1 asynchronous global -> LDS chunks in
flight (gemm_device.cuh:210-250), ke_gemm_level2_pipeline adds the one-step-ahead LDS -> register
prefetch (gemm_device.cuh:252-419).  Every row is checked against an fp32 product of 256 rows.

    python benchmarks/gemm/header_kernels.py     # prints a markdown table
"""

import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from tilefusion_amd.jit import gemm_jit  # noqa: E402
from tilefusion_amd.ops import gemm  # noqa: E402

M = N = K = 4096
# (label, tile_m, tile_n, tile_k, num_stages, pipeline_level, wavefront layout)
CASES = [
    ("ke_gemm, 1 buffer", 128, 128, 64, 1, 0, (2, 2)),
    ("ke_gemm, 2 buffers", 128, 128, 64, 2, 0, (2, 2)),
    ("ke_gemm_level1_pipeline, 2 stages", 128, 128, 64, 2, 1, (2, 2)),
    ("ke_gemm_level1_pipeline, 3 stages", 128, 128, 64, 3, 1, (2, 2)),
    ("ke_gemm_level2_pipeline, 3 stages", 128, 128, 64, 3, 2, (2, 2)),
    ("ke_gemm_level2_pipeline, 3 stages, 256x128 tile", 256, 128, 64, 3, 2, (4, 2)),
]


def _time_ms(fn, warm=5, reps=20):
    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def run(out=sys.stdout):
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(7)
    a = (torch.randn(M, K, device=dev, generator=g) / K ** 0.5).half()
    b = torch.randn(N, K, device=dev, generator=g).half()
    ref = a[:256].float() @ b.float().T
    ok_all = True
    print("|kernel|tiles (M, N, K)|ms|TFLOP/s|rel-L2 error|", file=out)
    print("|:---|:---:|:---:|:---:|:---:|", file=out)

    def row(label, tiles, fn, c):
        nonlocal ok_all
        t = _time_ms(fn)
        err = float((c[:256].float() - ref).norm() / ref.norm())
        ok = err <= 1e-3
        ok_all &= ok
        print(f"|{label}|{tiles}|{t:.4f}|{2.0 * M * N * K / t / 1e9:.0f}|{err:.2e}{'' if ok else ' MISMATCH'}|",
              file=out, flush=True)

    for label, tm, tn, tk, stages, level, wl in CASES:
        c = torch.zeros(M, N, device=dev, dtype=torch.float32)
        row(label, f"{tm}, {tn}, {tk}", lambda: gemm_jit(a, b, c, tm, tn, tk, stages, level, wl), c)
    c16 = torch.zeros(M, N, device=dev, dtype=torch.float16)
    row("tuned ring kernel (the op)", "256, 256, 64", lambda: gemm(a, b, c16, 64, 128, 128, 2, 1), c16)
    c16b = torch.zeros(M, N, device=dev, dtype=torch.float16)
    row("hipBLASLt (torch.matmul)", "-", lambda: torch.matmul(a, b.T, out=c16b), c16b)
    return ok_all


if __name__ == "__main__":
    sys.exit(0 if run() else 1)
