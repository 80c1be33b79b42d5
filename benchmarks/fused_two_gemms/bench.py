"""Shape sweep of the fused back-to-back GEMM (the shapes of benchmarks/cpp/fused_two_gemms/
bench.cu:197-245 in the reference: D = (A[M,K] B[K,N]) C[N,P] with K = P = 128 and tile
[64, 128, 128, 128]) against two library GEMMs (torch.matmul, i.e. hipBLASLt) on the same
inputs.  Every shape is checked against an fp32 computation of the same expression with the
intermediate rounded to fp16, as the kernel does.

    python benchmarks/fused_two_gemms/bench.py            # prints a markdown table
"""

import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from tilefusion_amd.ops import fused_two_gemms  # noqa: E402

SHAPES = [(4096, 1024), (4096, 2048), (8192, 1024), (8192, 2048), (4096, 4096), (8192, 8192), (8192, 4096),
          (2048, 2048), (1024, 1024), (512, 512)]
K = P = 128
TILE = (64, 128, 128, 128)


def _time_us(fn, reps=50):
    for _ in range(10):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps * 1e3


def run(shapes=SHAPES, out=sys.stdout):
    dev = "cuda"
    ok_all = True
    print("|[M, N, K, P]|tile|two library GEMMs (us)|fused (us)|ratio|rel-L2 error|", file=out)
    print("|:---|:---:|:---:|:---:|:---:|:---:|", file=out)
    for m, n in shapes:
        g = torch.Generator(device=dev).manual_seed(m + n)
        a = (torch.randn(m, K, device=dev, generator=g) / K**0.5).half()
        b = (torch.randn(n, K, device=dev, generator=g) / K**0.5).half()   # B as its [N, K] buffer
        c = (torch.randn(P, n, device=dev, generator=g) / n**0.5).half()   # C as its [P, N] buffer
        d = torch.empty(m, P, device=dev, dtype=torch.float16)
        tmp = torch.empty(m, n, device=dev, dtype=torch.float16)

        def ours():
            fused_two_gemms(a, b, c, d, *TILE)

        def library():
            torch.matmul(a, b.T, out=tmp)
            torch.matmul(tmp, c.T, out=d)

        t_lib = _time_us(library)
        t_ours = _time_us(ours)
        ours()
        ref = ((a.float() @ b.float().T).half().float() @ c.float().T)
        err = float((d.float() - ref).norm() / ref.norm())
        ok = err <= 1e-3
        ok_all &= ok
        print(f"|[{m}, {n}, {K}, {P}]|{list(TILE)}|{t_lib:.1f}|{t_ours:.1f}|{t_ours / t_lib:.3f}|{err:.2e}{'' if ok else ' MISMATCH'}|",
              file=out, flush=True)
    return ok_all


if __name__ == "__main__":
    sys.exit(0 if run() else 1)
