"""Run-time compilation of kernels written against the tile headers.

Python face of tilefusion::jit::JitCompiler (include/jit/compiler.hpp:21-81 in the reference):
source text + the name of an `extern "C" __global__` function -> a launchable kernel, cached
in the process and, as a code object, on disk.  The three `*_jit` functions below generate
the same kind of wrapper source as the reference's host launchers (src/kernels/gemm.cu:21-59,
fused_two_gemms.cu:35-63, flash_attn.cu:16-55): the whole problem shape and the tile sizes
become template arguments of the macro kernels in `kernels/*_device.hpp`, so - unlike the
ahead-of-time entry points, which treat tile sizes as hints - the launch uses exactly the
tiling that was asked for.
"""

import ctypes
import math
import os
import struct
from typing import Sequence

import torch

from . import _capi

INCLUDE_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "include")

_PRELUDE = """#include "kernels/gemm_device.hpp"
#include "kernels/fused_two_gemms_device.hpp"
#include "kernels/flash_attention_device.hpp"
using namespace tilefusion;
using namespace tilefusion::kernels;
namespace tl = tile_layout;
"""


class Kernel:
    """A compiled kernel.  `launch` takes device pointers / ints / floats as arguments."""

    def __init__(self, handle: int, name: str):
        self._handle, self.name = handle, name
        self._generation = JitCompiler._generation

    def launch(self, grid: Sequence[int], block: Sequence[int], args: Sequence, shared_mem: int = 0,
               stream=None) -> None:
        if self._generation != JitCompiler._generation:
            raise RuntimeError(f"kernel {self.name} was unloaded by JitCompiler.clear_cache(); compile it again")
        lib = _capi.load()
        boxed = []
        for a in args:
            if isinstance(a, torch.Tensor):
                boxed.append(ctypes.c_void_p(a.data_ptr()))
            elif isinstance(a, float):
                boxed.append(ctypes.c_float(a))
            elif isinstance(a, int):
                boxed.append(ctypes.c_int(a))
            else:
                boxed.append(a)  # already a ctypes value
        argv = (ctypes.c_void_p * len(boxed))(*[ctypes.cast(ctypes.pointer(b), ctypes.c_void_p) for b in boxed])
        g = tuple(grid) + (1,) * (3 - len(grid))
        b = tuple(block) + (1,) * (3 - len(block))
        st = torch.cuda.current_stream().cuda_stream if stream is None else stream
        _capi.check(lib.tf_jit_launch(self._handle, g[0], g[1], g[2], b[0], b[1], b[2], shared_mem, st, argv),
                    f"launch of {self.name}")


class JitCompiler:
    """Mirror of tilefusion::jit::JitCompiler (a process-wide singleton in the library)."""

    # clear_cache() unloads the modules, which kills every function handle handed out so far:
    # Kernel objects remember the generation they were made in and refuse to launch afterwards.
    _generation = 0

    @staticmethod
    def get_or_compile_kernel(kernel_name: str, source: str, include_paths: Sequence[str] = (),
                              compile_args: Sequence[str] = ()) -> Kernel:
        lib = _capi.load()
        inc = (ctypes.c_char_p * max(1, len(include_paths)))(*[p.encode() for p in include_paths])
        arg = (ctypes.c_char_p * max(1, len(compile_args)))(*[a.encode() for a in compile_args])
        out = ctypes.c_void_p()
        status = lib.tf_jit_compile(kernel_name.encode(), source.encode(), inc, len(include_paths), arg,
                                    len(compile_args), ctypes.byref(out))
        if status != _capi.TF_OK:
            # same wording as the reference's launchers (src/kernels/gemm.cu:104-106)
            raise RuntimeError("Failed to compile or retrieve kernel: " +
                               lib.tf_last_error().decode("utf-8", "replace"))
        return Kernel(out.value, kernel_name)

    compile_kernel = get_or_compile_kernel

    @staticmethod
    def clear_cache() -> None:
        JitCompiler._generation += 1
        _capi.load().tf_jit_clear_cache()

    @staticmethod
    def cache_dir() -> str:
        return _capi.load().tf_jit_cache_dir().decode()


def _check(t: torch.Tensor, name: str, dtype) -> None:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise ValueError(f"{name} must be a cuda tensor")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def gemm_jit(a, b, c, tile_m, tile_n, tile_k, num_stages=1, pipeline_level=0, warp_layout=(2, 2)) -> None:
    """C[M,N] (fp32) = A[M,K] @ B with B given as its [N,K] buffer, by a run-time instantiation
    of ke_gemm with exactly these tile sizes (src/kernels/gemm.cu:21-59,63-142)."""
    _check(a, "a", torch.float16), _check(b, "b", torch.float16), _check(c, "c", torch.float32)
    m, k = a.shape
    n = b.shape[0]
    if b.shape[1] != k or tuple(c.shape) != (m, n):
        raise ValueError("shapes must be a [M,K], b [N,K], c [M,N]")
    if m % tile_m or n % tile_n or k % tile_k:
        raise ValueError("tile sizes must divide the problem")
    if pipeline_level > 0 and num_stages < 2:
        raise ValueError("the pipelined kernels (pipeline_level 1 and 2) need num_stages >= 2")
    wr, wc = warp_layout
    rk = 32
    entry = {0: "ke_gemm", 1: "ke_gemm_level1_pipeline", 2: "ke_gemm_level2_pipeline"}[pipeline_level]
    name = f"gemm_kernel_{m}_{n}_{k}_{tile_m}_{tile_n}_{tile_k}_{num_stages}_{pipeline_level}_{wr}x{wc}"
    src = _PRELUDE + f"""
using Config = KeGemmTraits<__half, float, tl::RowMajor<{wr}, {wc}>, {m}, {n}, {k}, {tile_m}, {tile_n}, {tile_k}, {rk}, {num_stages}, 64>;
extern "C" __global__ __launch_bounds__({wr * wc * 64}) void {name}(const __half* A, const __half* B, float* C) {{
  {entry}<__half, float, Config>(A, B, C);
}}
"""
    # ke_gemm keeps at most two LDS buffers; the pipelined kernels keep num_stages ring slots
    slots = num_stages if pipeline_level > 0 else (2 if num_stages >= 2 else 1)
    lds = (tile_m * tile_k + tile_k * tile_n) * slots * 2
    kern = JitCompiler.get_or_compile_kernel(name, src)
    kern.launch((m // tile_m, n // tile_n), (wr * wc * 64,), (a, b, c), lds)


def fused_two_gemms_jit(a, b, c, d, tm=64, tn=64, tk=64, tp=64, warp_layout=(2, 1)) -> None:
    """D = (A @ B) @ C with B as its [N,K] and C as its [P,N] buffer, by a run-time instantiation
    of ke_fused_two_gemms (src/kernels/fused_two_gemms.cu:35-63,66-144)."""
    for t, nm in ((a, "a"), (b, "b"), (c, "c"), (d, "d")):
        _check(t, nm, torch.float16)
    m, k = a.shape[-2:]
    n, p = b.shape[-2], c.shape[-2]
    batch = a.numel() // (m * k)
    if m % tm or n % tn or k % tk or p % tp:
        raise ValueError("tile sizes must divide the problem")
    wr, wc = warp_layout
    name = f"fused_two_gemms_kernel_{m}_{n}_{k}_{p}_{tm}_{tn}_{tk}_{tp}_{wr}"
    src = _PRELUDE + f"""
using Config = FusedTwoGemmsTraits<__half, float, tl::RowMajor<{wr}, {wc}>, {m}, {n}, {k}, {p}, {tm}, {tn}, {tk}, {tp}>;
extern "C" __global__ __launch_bounds__({wr * wc * 64}) void {name}(const __half* A, const __half* B, const __half* C, __half* D) {{
  ke_fused_two_gemms<__half, float, Config>(A, B, C, D);
}}
"""
    lds = (tm * tk + tk * tn + tn * tp + tm * tn) * 2
    kern = JitCompiler.get_or_compile_kernel(name, src)
    kern.launch((m // tm, p // tp, batch), (wr * wc * 64,), (a, b, c, d), lds)


def flash_attention_jit(q, k, v_t, o, tile_length_q=64, tile_length_kv=64, tile_hidden_qk=None, tile_hidden_v=None,
                        softmax_scale=None, causal=False, warp_layout=(4, 1)) -> None:
    """O = softmax(scale Q K^T (+ causal mask)) V with V given transposed ([.., Dv, Lkv], the
    reference's convention), by a run-time instantiation of ke_flash_attention
    (src/kernels/flash_attn.cu:16-55,58-152)."""
    for t, nm in ((q, "q"), (k, "k"), (v_t, "v_t"), (o, "o")):
        _check(t, nm, torch.float16)
    lq, d = q.shape[-2:]
    lkv = k.shape[-2]
    dv = v_t.shape[-2]
    batch = q.numel() // (lq * d)
    tk_ = d if tile_hidden_qk is None else tile_hidden_qk
    tp_ = dv if tile_hidden_v is None else tile_hidden_v
    if lq % tile_length_q or lkv % tile_length_kv or d % tk_ or dv % tp_:
        raise ValueError("tile sizes must divide the problem")
    scale = 1.0 / math.sqrt(d) if softmax_scale is None else float(softmax_scale)
    wr, wc = warp_layout
    tag = f"{lq}_{lkv}_{d}_{dv}_{tile_length_q}_{tile_length_kv}_{tk_}_{tp_}_{int(causal)}_{wr}_{struct.pack('<d', float(scale)).hex()}"
    name = f"flash_attention_kernel_{tag}"
    src = _PRELUDE + f"""
using Config = FlashAttentionTraits<__half, float, __half, TileShape<{lq}, {lkv}, {d}, {dv}>,
                                    TileShape<{tile_length_q}, {tile_length_kv}, {tk_}, {tp_}>, tl::RowMajor<{wr}, {wc}>,
                                    {scale!r}, {str(bool(causal)).lower()}>;
extern "C" __global__ __launch_bounds__({wr * wc * 64}) void {name}(const __half* Q, const __half* K, const __half* V, __half* O) {{
  ke_flash_attention<__half, float, __half, Config>(Q, K, V, O);
}}
"""
    lds = (tile_length_q * tk_ + tk_ * tile_length_kv + tile_length_kv * tp_ + tile_length_q * tile_length_kv) * 2
    kern = JitCompiler.get_or_compile_kernel(name, src)
    kern.launch((lq // tile_length_q, dv // tp_, batch), (wr * wc * 64,), (q, k, v_t, o), lds)
