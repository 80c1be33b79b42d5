"""GEMM shape sweep (the shapes of the table in benchmarks/cpp/gemm/README.md:8-18 of the
reference; method of benchmarks/cpp/gemm/bench.cu:155-176: 10 warm-up + 50 timed launches in
one event pair, inputs U[1e-4, 5e-3]) against hipBLASLt (torch.matmul) on the same inputs.
The A100 column repeats the reference's published TileFusion times for orientation only.

    python benchmarks/gemm/bench.py            # prints a markdown table
"""

import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from tilefusion_amd.ops import gemm  # noqa: E402

# [M, N, K] -> the reference's published time on an A100 in ms (benchmarks/cpp/gemm/README.md:10-18)
SHAPES = [((1024, 1024, 512), 0.016548), ((1024, 1024, 1024), 0.027156), ((2048, 2048, 1024), 0.070431),
          ((2048, 2048, 2048), 0.128143), ((4096, 4096, 4096), 0.969605), ((8192, 8192, 1024), 0.971059),
          ((8192, 8192, 2048), 1.931223), ((8192, 8192, 4096), 3.956757), ((8192, 8192, 8192), 8.080589)]
TILE = (64, 128, 128)


def _time_ms(fn, warm=10, reps=50):
    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def run(shapes=SHAPES, out=sys.stdout):
    dev = "cuda"
    ok_all = True
    print("|[M, N, K]|this library (ms)|TFLOP/s|hipBLASLt (ms)|ratio|rel-L2 error|reference on A100 (ms)|", file=out)
    print("|:---|:---:|:---:|:---:|:---:|:---:|:---:|", file=out)
    for (m, n, k), a100 in shapes:
        g = torch.Generator(device=dev).manual_seed(m + n + k)
        a = (torch.rand(m, k, device=dev, generator=g) * (5e-3 - 1e-4) + 1e-4).half()
        b = (torch.rand(n, k, device=dev, generator=g) * (5e-3 - 1e-4) + 1e-4).half()   # B as its [N, K] buffer
        c = torch.empty(m, n, device=dev, dtype=torch.float16)
        c2 = torch.empty(m, n, device=dev, dtype=torch.float16)
        t_ours = _time_ms(lambda: gemm(a, b, c, *TILE, 2, 1))
        t_lib = _time_ms(lambda: torch.matmul(a, b.T, out=c2))
        rows = slice(0, min(m, 512))
        ref = a[rows].float() @ b.float().T
        err = float((c[rows].float() - ref).norm() / ref.norm())
        ok = err <= 1e-3
        ok_all &= ok
        print(f"|[{m}, {n}, {k}]|{t_ours:.4f}|{2.0 * m * n * k / t_ours / 1e9:.0f}|{t_lib:.4f}|{t_ours / t_lib:.3f}|"
              f"{err:.2e}{'' if ok else ' MISMATCH'}|{a100:.4f}|", file=out, flush=True)
    return ok_all


if __name__ == "__main__":
    sys.exit(0 if run() else 1)
