"""Flash-attention forward over head dimensions: the tuned kernels (D = 64, 96, 128; fp16 and bf16)
next to the header macro kernel ke_flash_attention compiled at run time (what any other head
dimension runs, here D = 160 and D = 32), all through the same entry point
tf_flash_attention_fwd; and the torch op, which zero-pads a head dimension below 128 without a
tuned kernel to the next tuned size instead (TFLOP/s count the unpadded problem).  Counterpart of the reference's benchmarks/cpp/flashattention
program; every row is checked against an fp32 softmax(QK^T)V of one (batch, head) slice.

    python benchmarks/attention/bench.py      # prints a markdown table
"""

import math
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from tilefusion_amd import _capi  # noqa: E402

BH, S = 32, 4096
# (head dim, dtype, causal, what runs)
CASES = [(128, torch.float16, False, "tuned"), (128, torch.float16, True, "tuned"), (128, torch.bfloat16, False, "tuned"),
         (96, torch.float16, False, "tuned"), (96, torch.float16, True, "tuned"), (96, torch.bfloat16, False, "tuned"),
         (64, torch.float16, False, "tuned"),
         (160, torch.float16, False, "header kernel"), (160, torch.float16, True, "header kernel"),
         (32, torch.float16, False, "header kernel"),
         (80, torch.float16, False, "torch op: padded to 96, tuned"), (80, torch.float16, True, "torch op: padded to 96, tuned"),
         (32, torch.float16, False, "torch op: padded to 64, tuned")]


def _time_ms(fn, warm=60, reps=40):
    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def run(cases=CASES, bh=BH, s=S, out=sys.stdout):
    lib = _capi.load()
    dev = "cuda"
    ok_all = True
    print("|head dim|type|causal|kernel|ms|TFLOP/s|rel-L2 error|", file=out)
    print("|:---:|:---:|:---:|:---|:---:|:---:|:---:|", file=out)
    for d, dtype, causal, what in cases:
        g = torch.Generator(device=dev).manual_seed(d + causal)
        q, k, v = (torch.randn(bh, s, d, device=dev, generator=g).to(dtype) for _ in range(3))
        vt = v.transpose(1, 2).contiguous()   # the reference hands V over transposed
        o = torch.empty(bh, s, d, device=dev, dtype=dtype)
        scale = 1.0 / math.sqrt(d)
        code = _capi.TF_DTYPE_BF16 if dtype == torch.bfloat16 else _capi.TF_DTYPE_F16
        st = torch.cuda.current_stream().cuda_stream

        def call_op():
            torch.ops.tilefusion.flash_attention(q, k, vt, o, 64, 64, d, d, scale, causal)

        def call():
            if what.startswith("torch op"):
                return call_op()
            rc = lib.tf_flash_attention_fwd(q.data_ptr(), k.data_ptr(), vt.data_ptr(), o.data_ptr(), code, bh, s, s, d, d,
                                            1, 64, 64, d, d, scale, int(causal), st)
            assert rc == 0, lib.tf_last_error()

        t = _time_ms(call)
        logits = (q[0].float() @ k[0].float().T) * scale
        if causal:
            logits = logits.masked_fill(torch.ones(s, s, device=dev, dtype=torch.bool).triu(1), float("-inf"))
        ref = torch.softmax(logits, -1) @ v[0].float()
        err = float((o[0].float() - ref).norm() / ref.norm())
        ok = err <= (4e-3 if dtype == torch.bfloat16 else 1e-3)
        ok_all &= ok
        flops = 4.0 * bh * s * s * d * (0.5 if causal else 1.0)
        print(f"|{d}|{'bf16' if dtype == torch.bfloat16 else 'fp16'}|{'yes' if causal else 'no'}|{what}|{t:.4f}|"
              f"{flops / t / 1e9:.0f}|{err:.2e}{'' if ok else ' MISMATCH'}|", file=out, flush=True)
    return ok_all


if __name__ == "__main__":
    sys.exit(0 if run() else 1)
