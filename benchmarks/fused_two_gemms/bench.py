"""Shape sweep of the fused back-to-back GEMM (the shapes of benchmarks/cpp/fused_two_gemms/
bench.cu:197-245 in the reference: D = (A[M,K] B[K,N]) C[N,P] with K = P = 128 and tile
[64, 128, 128, 128]) against two library GEMMs (torch.matmul, i.e. hipBLASLt) on the same
inputs.  Every shape is checked against an fp32 computation of the same expression with the
intermediate rounded to fp16, as the kernel does.

    python benchmarks/fused_two_gemms/bench.py            # prints a markdown table
    python benchmarks/fused_two_gemms/bench.py --floor    # launch-to-launch floor at the 16384-row shape
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


def _graph_us(launch, n=200):
    """Microseconds per launch of n launches recorded once into a HIP graph and replayed: the
    host side of a launch is out of the figure, what is left is kernel time plus the GPU's
    own hand-over from one kernel to the next."""
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        for i in range(10):
            launch(i, s.cuda_stream)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            for i in range(n):
                launch(i, s.cuda_stream)
        best = float("inf")
        for _ in range(5):
            g.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(s)
            g.replay()
            e1.record(s)
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) * 1e3 / n)
    return best


def launch_floor(out=sys.stdout):
    """The 16384 x 128 x 128 x 128 shape (256 workgroups, 8.45 MB) next to a kernel of the same
    launch geometry that does nothing: how much of a step is the launch itself."""
    from tilefusion_amd import _capi
    from tilefusion_amd.jit import JitCompiler

    lib = _capi.load()
    dev = "cuda"
    m, n = 16384, 128
    g = torch.Generator(device=dev).manual_seed(3)
    b = (torch.randn(n, K, device=dev, generator=g) / K**0.5).half()
    c = (torch.randn(P, n, device=dev, generator=g) / n**0.5).half()
    sets = [((torch.randn(m, K, device=dev, generator=g) / K**0.5).half(), torch.empty(m, P, device=dev, dtype=torch.float16))
            for _ in range(40)]   # 40 x 8 MiB: more than the 256 MB last-level cache
    empty = JitCompiler.get_or_compile_kernel(
        "empty_kernel_256", 'extern "C" __global__ __launch_bounds__(256) void empty_kernel_256(const void* p) {}')

    def fused(nsets):
        def launch(i, st):
            a, d = sets[i % nsets]
            rc = lib.tf_fused_two_gemms_f16(a.data_ptr(), b.data_ptr(), c.data_ptr(), d.data_ptr(), 1, m, n, K, P, *TILE, st)
            assert rc == 0, lib.tf_last_error()
        return launch

    rows = [("empty kernel, 256 workgroups x 256 threads, 64 KiB of LDS",
             _graph_us(lambda i, st: empty.launch((256,), (256,), (b,), 64 * 1024, stream=st))),
            ("fused kernel, one operand set (inputs stay in the caches)", _graph_us(fused(1))),
            ("fused kernel, 40 rotating A/D sets (inputs from HBM)", _graph_us(fused(40)))]
    print("|200 launches in one HIP graph|us per launch|", file=out)
    print("|:---|:---:|", file=out)
    for label, us in rows:
        print(f"|{label}|{us:.2f}|", file=out, flush=True)
    return rows


if __name__ == "__main__":
    if "--floor" in sys.argv:
        launch_floor()
        sys.exit(0)
    sys.exit(0 if run() else 1)
