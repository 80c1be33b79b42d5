#!/usr/bin/env python3
"""Benchmark of the MI355X TileFusion hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

One "step" is one pass of a hot-path kernel over one batch of synthetic input that is
already resident in HBM.  The default workload is the configuration the headline metric is
quoted on - the 4096^3 fp16 GEMM (fp32 accumulate, fp16 out); the other benchmark
configurations (fused back-to-back GEMM, flash-attention forward +/- causal, split-KV
flash-decoding) are measured in the same run and reported under "workloads".  Prints ONE
JSON line.

Timing: W untimed warm-up steps, then exactly K steps between two HIP events recorded on the
stream the kernels are launched on, bracketed by torch.cuda.synchronize().  Input sets rotate
so that consecutive launches do not hit the 256 MB last-level cache with the same operands.
The roofline entry is algorithmic flops (or bytes) per launch divided by the measured average
launch duration; its "traffic" is read from the rocprofv3 summary of the workload under profiles/
(counter runs are separate processes).  A second, separate pass times every step with its own
event pair and reports the fastest and the median step next to the mean.  The CPU baseline is the
fp32 torch oracle timed on this host.
"""

import argparse
import json
import math
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2516.6   # 256 CU x 2.4 GHz x 4096 flop/clk/CU (dense fp16 MFMA, "2.5 PFLOP/s")
PEAK_HBM_GBS = 8000.0       # HBM3E, 8 TB/s


PRE_WARM_MS = 300.0


def _time_steps(fn, steps, warmup, pre_warm_ms=PRE_WARM_MS):
    import torch
    # Untimed pre-warm with the kernel under test so that the W warm-up steps start from the
    # clocks this kernel settles at: the power management needs a few hundred ms of sustained
    # load to converge (launch durations first swing by 10-20%), and a different pre-warm load
    # would leave the clocks where THAT load settles.
    t_end = time.perf_counter() + pre_warm_ms / 1e3
    i = 0
    while time.perf_counter() < t_end:
        fn(i)
        i += 1
        if i % 16 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        fn(warmup + i)
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_time(e1) / steps, wall / steps


def _time_each_step(fn, steps, first):
    """Fastest and median of `steps` individually timed steps (one event pair each; the pairs add
    a few microseconds of launch gap, so these figures are reported next to the mean of the
    back-to-back region, they do not replace it)."""
    import torch
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for i, (e0, e1) in enumerate(pairs):
        e0.record()
        fn(first + i)
        e1.record()
    torch.cuda.synchronize()
    t = [e0.elapsed_time(e1) for e0, e1 in pairs]
    return min(t), statistics.median(t)


def _profile_traffic(name):
    """Bytes per step between the L2 caches and the fabric, as the rocprofv3 summary of the workload
    states them (FETCH_SIZE + WRITE_SIZE per launch, each scaled by what the counter reads for a
    1 GiB copy); None when the summary is missing or does not carry the figure."""
    try:
        text = open(os.path.join(ROOT, "profiles", name + ".txt")).read()
    except OSError:
        return None
    m = re.search(r"scaled traffic per step:.*\((\d+) bytes\)", text)
    return int(m.group(1)) if m else None


def _bound_calls(fn, arg_lists, err):
    """One closure per operand set with every argument already converted: a step is then a
    single C call, so that the host side of a step stays well under a few-microsecond kernel."""
    import functools

    def make(args):
        call = functools.partial(fn, *args)

        def run():
            if call() != 0:
                raise RuntimeError(err())
        return run
    return [make(a) for a in arg_lists]


def _cpu_times(fn, reps=3, warm=True):
    """(best, median) wall time of `reps` calls, after one untimed call when `warm`."""
    if warm:
        fn()
    t = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        t.append(time.perf_counter() - t0)
    return min(t), statistics.median(t)


class Gemm4096:
    name = "gemm_fp16_4096x4096x4096"
    profile = "gemm_fp16_4096"   # profiles/<this>.txt
    metric, unit, bound = "gemm_fp16_tflops", "TFLOP/s", "mfma"
    M = N = K = 4096
    flops = 2.0 * 4096 ** 3
    bytes = 3 * 4096 * 4096 * 2

    def setup(self, dev):
        import torch
        import oracle
        self.lib = _capi().load()
        a, b = oracle.make_c2_gemm_inputs()
        self.host = (a, b)
        g = torch.Generator(device=dev).manual_seed(2)
        s = 1.0 / 64.0
        self.sets = [(a.to(dev), b.to(dev), torch.empty(4096, 4096, device=dev, dtype=torch.float16))]
        for _ in range(3):  # 4 sets x 96 MiB > 256 MB of last-level cache
            self.sets.append(((torch.randn(4096, 4096, device=dev, generator=g) * s).half(),
                              (torch.randn(4096, 4096, device=dev, generator=g) * s).half(),
                              torch.empty(4096, 4096, device=dev, dtype=torch.float16)))
        st = torch.cuda.current_stream().cuda_stream
        self.calls = _bound_calls(self.lib.tf_gemm_f16,
                                  [(a.data_ptr(), b.data_ptr(), c.data_ptr(), 1, 4096, 4096, 4096, 64, 128, 128, 2, 1, st)
                                   for a, b, c in self.sets], self.lib.tf_last_error)

    def step(self, i):
        self.calls[i % len(self.calls)]()

    def check(self):
        import oracle
        self.step(0)
        return oracle.check_close(self.sets[0][2], oracle.gemm_ref(*self.host))

    def cpu_baseline(self):
        import torch
        a32, b32 = self.host[0].float(), self.host[1].float()
        best, med = _cpu_times(lambda: torch.matmul(a32, b32.T))
        return {"value": self.flops / best / 1e12, "median": self.flops / med / 1e12, "unit": "TFLOP/s",
                "sample": "full 4096^3 fp32 torch.matmul, 1 warm-up + 3 repetitions (value = best, median beside it)"}

    config = {"workload": "fp16 GEMM M=N=K=4096, A row-major, B col-major, fp32 accumulate, fp16 out",
              "inputs": "N(0,1)/sqrt(K), seed 1002; 4 rotating operand sets"}


class Fused:
    name = "fused_two_gemms_16384x128x128x128"
    metric, unit, bound = "fused_two_gemms_gbs", "GB/s", "hbm"
    M, N, K, P = 16384, 128, 128, 128
    flops = 2.0 * 2 * 16384 * 128 * 128
    bytes = (16384 * 128 * 2 + 2 * 128 * 128) * 2

    def setup(self, dev):
        import torch
        import oracle
        self.lib = _capi().load()
        a, b, c = oracle.make_c3_fused_inputs()
        self.host = (a, b, c)
        self.sets = []
        for i in range(40):  # 40 x 8.4 MB > 256 MB
            self.sets.append((a.to(dev) if i == 0 else torch.roll(a.to(dev), i, 0), b.to(dev), c.to(dev),
                              torch.empty(16384, 128, device=dev, dtype=torch.float16)))
        st = torch.cuda.current_stream().cuda_stream
        self.calls = _bound_calls(self.lib.tf_fused_two_gemms_f16,
                                  [(a.data_ptr(), b.data_ptr(), c.data_ptr(), d.data_ptr(), 1, self.M, self.N, self.K,
                                    self.P, 64, 128, 128, 128, st) for a, b, c, d in self.sets], self.lib.tf_last_error)

    def step(self, i):
        self.calls[i % len(self.calls)]()

    def check(self):
        import oracle
        self.step(0)
        return oracle.check_close(self.sets[0][3], oracle.fused_two_gemms_ref(*self.host))

    def cpu_baseline(self):
        a, b, c = (t.float() for t in self.host)
        best, med = _cpu_times(lambda: (a @ b.T) @ c.T)
        return {"value": self.bytes / best / 1e9, "median": self.bytes / med / 1e9, "unit": "GB/s",
                "sample": "full problem, two fp32 torch.matmul, 1 warm-up + 3 repetitions (value = best, median beside it)"}

    config = {"workload": "fused (A[16384x128] @ B[128x128]) @ C[128x128], fp16 in/out, fp32 accumulate",
              "inputs": "N(0,1)/sqrt(128), seed 1003; 40 rotating A/D sets"}


class Attention:
    unit, bound = "TFLOP/s", "mfma"
    B, H, S, D = 2, 32, 4096, 128

    def __init__(self, causal):
        self.causal = causal
        self.name = "flash_attention_fwd_b2_h32_s4096_d128" + ("_causal" if causal else "")
        self.metric = "flash_attention_fwd_tflops" + ("_causal" if causal else "")
        self.flops = 4.0 * 64 * 4096 * 4096 * 128 * (0.5 if causal else 1.0)
        self.bytes = 4 * 64 * 4096 * 128 * 2
        self.config = {"workload": "flash-attention fwd fp16 B=2 H=32 S=4096 D=128 %s, scale 1/sqrt(128), fp32 softmax stats"
                       % ("causal" if causal else "non-causal"),
                       "inputs": "N(0,1), seed 1004; V in natural [S, D] layout; 2 rotating Q/K/V/O sets"}

    def setup(self, dev):
        import torch
        import oracle
        self.lib = _capi().load()
        q, k, v = oracle.make_c4_attention_inputs()
        self.host = (q, k, v)
        mk = lambda t: t.reshape(64, 4096, 128).to(dev)
        self.sets = [(mk(q), mk(k), mk(v), torch.empty(64, 4096, 128, device=dev, dtype=torch.float16))]
        self.sets.append((mk(k), mk(v), mk(q), torch.empty(64, 4096, 128, device=dev, dtype=torch.float16)))
        st = torch.cuda.current_stream().cuda_stream
        self.calls = _bound_calls(self.lib.tf_flash_attention_fwd_f16,
                                  [(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), 64, 4096, 4096, 128, 128, 0, 128,
                                    64, 128, 128, 1.0 / math.sqrt(128), int(self.causal), st) for q, k, v, o in self.sets],
                                  self.lib.tf_last_error)

    def step(self, i):
        self.calls[i % len(self.calls)]()

    _sample = [(0, 0), (1, 31)]

    def check(self):
        import oracle
        self.step(0)
        q, k, v = self.host
        o = self.sets[0][3].cpu().reshape(2, 32, 4096, 128)
        worst = (True, 0.0, 0.0)
        for b, h in self._sample:
            ok, r, m = oracle.check_close(o[b, h], oracle.attention_ref(q[b, h], k[b, h], v[b, h], causal=self.causal))
            worst = (worst[0] and ok, max(worst[1], r), max(worst[2], m))
        return worst

    def cpu_baseline(self):
        import oracle
        q, k, v = self.host
        oracle.attention_ref(q[0, 0], k[0, 0], v[0, 0], causal=self.causal)   # untimed warm-up slice
        per_slice = []
        for b in range(self.B):
            for h in range(self.H):
                t0 = time.perf_counter()
                oracle.attention_ref(q[b, h], k[b, h], v[b, h], causal=self.causal)
                per_slice.append(time.perf_counter() - t0)
        total = sum(per_slice)
        per = self.flops / 64
        return {"value": self.flops / total / 1e12, "unit": "TFLOP/s",
                "best_slice": per / min(per_slice) / 1e12, "median_slice": per / statistics.median(per_slice) / 1e12,
                "sample": "all 64 (batch, head) slices, one repetition after one warm-up slice: fp32 softmax(QK^T)V per "
                          "slice (value = whole-workload flops / total time; rate of the best and of the median slice beside it)"}


class Decode:
    name = "flash_decode_b16_h32_kv32768_d128_splits64"
    metric, unit, bound = "flash_decode_hbm_gbs", "GB/s", "hbm"
    BH, LKV, D, SPLITS = 512, 32768, 128, 64
    bytes = 2 * 512 * 32768 * 128 * 2 + 2 * 512 * 128 * 2
    flops = 4.0 * 512 * 32768 * 128

    def setup(self, dev):
        import torch
        import oracle
        self.lib = _capi().load()
        g = torch.Generator(device=dev).manual_seed(oracle.SEEDS["c5"])
        self.q = torch.randn(self.BH, self.D, device=dev, dtype=torch.float16, generator=g)
        self.k = torch.randn(self.BH, self.LKV, self.D, device=dev, dtype=torch.float16, generator=g)
        self.v = torch.randn(self.BH, self.LKV, self.D, device=dev, dtype=torch.float16, generator=g)
        self.o = torch.empty(self.BH, self.D, device=dev, dtype=torch.float16)
        self.ws_bytes = self.lib.tf_flash_decode_workspace_bytes(self.BH, self.D, self.SPLITS)
        self.ws = torch.empty(self.ws_bytes, device=dev, dtype=torch.uint8)

        st = torch.cuda.current_stream().cuda_stream
        self.calls = _bound_calls(self.lib.tf_flash_decode_f16,
                                  [(self.q.data_ptr(), self.k.data_ptr(), self.v.data_ptr(), self.o.data_ptr(),
                                    self.ws.data_ptr(), self.ws_bytes, self.BH, self.LKV, self.D, self.SPLITS,
                                    1.0 / math.sqrt(self.D), st)], self.lib.tf_last_error)

    def step(self, i):
        self.calls[0]()

    _sample = [0, 100, 255, 511]
    _cpu_slices = 64

    def check(self):
        import oracle
        self.step(0)
        worst = (True, 0.0, 0.0)
        for i in self._sample:
            ok, r, m = oracle.check_close(self.o[i], oracle.flash_decode_ref(self.q[i].cpu(), self.k[i].cpu(), self.v[i].cpu()))
            worst = (worst[0] and ok, max(worst[1], r), max(worst[2], m))
        return worst

    def cpu_baseline(self):
        import oracle
        idx = list(range(0, self.BH, self.BH // self._cpu_slices))
        per_slice = []
        for n, i in enumerate([idx[0]] + idx):   # the first one twice: warm-up
            q, k, v = self.q[i].cpu(), self.k[i].cpu(), self.v[i].cpu()
            t0 = time.perf_counter()
            oracle.flash_decode_ref(q, k, v)
            if n:
                per_slice.append(time.perf_counter() - t0)
        per = self.bytes / self.BH
        return {"value": per * len(idx) / sum(per_slice) / 1e9, "unit": "GB/s",
                "best_slice": per / min(per_slice) / 1e9, "median_slice": per / statistics.median(per_slice) / 1e9,
                "sample": "%d of 512 (batch, head) slices (every 8th), one repetition after one warm-up slice: fp32 "
                          "softmax(qK^T)V per slice with K, V upcast per slice (value = sampled bytes / sampled time; "
                          "rate of the best and of the median slice beside it)" % len(idx)}

    config = {"workload": "flash-decoding fp16 B=16 H=32 q_len=1 KV=32768 D=128, 64 splits + LSE combine (2 kernels per step)",
              "inputs": "N(0,1) drawn on the device, seed 1005; 8 GiB of K,V (exceeds the last-level cache)"}


def _capi():
    from tilefusion_amd import _capi as m
    return m


class Copy:
    """Calibration only: a plain device-to-device copy of known size, the yardstick the
    FETCH_SIZE / WRITE_SIZE counters of the other workloads are scaled by."""
    name = "copy_1gib"
    metric, unit, bound = "copy_gbs", "GB/s", "hbm"
    nbytes = 1 << 30
    bytes = 2 * nbytes
    flops = 0.0
    traffic = None
    config = {"workload": "torch copy_ of 1 GiB (reads 1 GiB, writes 1 GiB)", "inputs": "uint8 zeros"}

    def setup(self, dev):
        import torch
        self.src = torch.zeros(self.nbytes, device=dev, dtype=torch.uint8)
        self.dst = torch.empty_like(self.src)

    def step(self, i):
        self.dst.copy_(self.src)

    def check(self):
        return True, 0.0, 0.0

    def cpu_baseline(self):
        return {"value": 0.0, "unit": "GB/s", "sample": "none"}


def run_workload(w, steps, warmup, with_cpu, pre_warm_ms=PRE_WARM_MS):
    import torch
    dev = "cuda:0"
    w.setup(dev)
    ok, rel, mabs = w.check()
    ms, wall_ms = _time_steps(w.step, steps, warmup, pre_warm_ms)
    step_min, step_median = _time_each_step(w.step, steps, warmup + steps)
    if w.bound == "mfma":
        achieved, peak, runit = w.flops / ms / 1e9, PEAK_FP16_TFLOPS, "TFLOP/s"
    else:
        achieved, peak, runit = w.bytes / ms / 1e6, PEAK_HBM_GBS, "GB/s"
    out = {
        "metric": w.metric, "value": round(achieved, 2), "unit": w.unit, "ms_per_step": round(ms, 5),
        "wall_ms_per_step": round(wall_ms, 5),
        "step_ms_individually_timed": {"min": round(step_min, 5), "median": round(step_median, 5)},
        "roofline": {"bound": w.bound, "achieved": round(achieved, 2), "peak": peak, "unit": runit,
                     "frac": round(achieved / peak, 4),
                     "traffic": None if isinstance(w, Copy) else _profile_traffic(getattr(w, "profile", w.name))},
        "tflops": round(w.flops / ms / 1e9, 2), "algorithmic_gbs": round(w.bytes / ms / 1e6, 1),
        "parity": {"ok": bool(ok), "rel_l2": float("%.3e" % rel), "max_abs": float("%.3e" % mabs),
                   "tolerance": "rel_l2<=1e-3, max_abs<=2e-2 vs fp32 CPU oracle"},
        "config": w.config,
    }
    if with_cpu:
        cb = w.cpu_baseline()
        for key in ("value", "median", "best_slice", "median_slice"):
            if key in cb:
                cb[key] = round(cb[key], 4)
        cb["cores"] = torch.get_num_threads()
        cb["kind"] = "port"
        out["cpu_baseline"] = cb
    del w
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all",
                    choices=["all", "gemm", "fused", "attention", "attention_causal", "decode", "copy"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--prewarm-ms", type=float, default=PRE_WARM_MS,
                    help="untimed run of the kernel under test before each workload (0 for counter runs)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the hot path on ONE GPU; --gpus N with N > 1 is not supported "
              "(every kernel shards over independent rows / heads without exchange).", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.set_num_threads(max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))))
    table = {"gemm": Gemm4096(), "fused": Fused(), "attention": Attention(False),
             "attention_causal": Attention(True), "decode": Decode(), "copy": Copy()}
    head_key = "gemm" if args.workload == "all" else args.workload
    head = run_workload(table[head_key], args.steps, args.warmup, not args.no_cpu and head_key != "copy", args.prewarm_ms)
    prop = torch.cuda.get_device_properties(0)
    line = {
        "metric": head["metric"], "value": head["value"], "unit": head["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic", "config": head["config"], "roofline": head["roofline"],
        "parity": head["parity"],
        "step_ms_individually_timed": head["step_ms_individually_timed"],
        "device": {"name": prop.name, "cus": prop.multi_processor_count, "host_cores": os.cpu_count()},
    }
    if "cpu_baseline" in head:
        line["cpu_baseline"] = head["cpu_baseline"]
    if args.workload == "all":
        others = {}
        for key in ("fused", "attention", "attention_causal", "decode"):
            steps = args.steps if key != "decode" else max(5, min(args.steps, 20))
            others[key] = run_workload(table[key], steps, min(args.warmup, 5), not args.no_cpu, args.prewarm_ms)
        line["workloads"] = others
    print(json.dumps(line))


if __name__ == "__main__":
    main()
