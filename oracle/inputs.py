"""Seeded synthetic inputs for the five benchmark configurations (test infrastructure).

Inputs are drawn in fp32 from torch.Generator("cpu").manual_seed(seed) and rounded to fp16;
both the GPU kernels and the fp32 oracles consume the rounded values.
"""

import math

import torch

SEEDS = {"c1": 1001, "c2": 1002, "c3": 1003, "c4": 1004, "c5": 1005}


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def _uniform(shape, g, lo=-1.0, hi=1.0):
    return (torch.rand(shape, generator=g, dtype=torch.float32) * (hi - lo) + lo).half()


def _normal(shape, g, std=1.0):
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).half()


def make_c1_gemm_inputs(m=128, n=64, k=256, seed=SEEDS["c1"]):
    """README single-tile GEMM: A [m,k] row-major, B as an [n,k] buffer (col-major k x n)."""
    g = _gen(seed)
    return _uniform((m, k), g), _uniform((n, k), g)


def make_c2_gemm_inputs(m=4096, n=4096, k=4096, seed=SEEDS["c2"]):
    """Large GEMM: N(0,1)/sqrt(k)."""
    g = _gen(seed)
    s = 1.0 / math.sqrt(k)
    return _normal((m, k), g, s), _normal((n, k), g, s)


def make_c3_fused_inputs(m=16384, n=128, k=128, p=128, seed=SEEDS["c3"]):
    """Fused back-to-back GEMM: A [m,k], B buffer [n,k], C buffer [p,n]; N(0,1)/sqrt(128)."""
    g = _gen(seed)
    s = 1.0 / math.sqrt(128.0)
    return _normal((m, k), g, s), _normal((n, k), g, s), _normal((p, n), g, s)


def make_c4_attention_inputs(batch=2, heads=32, seq=4096, dim=128, seed=SEEDS["c4"], seq_kv=None):
    """Flash-attention forward: Q,K,V [batch, heads, seq, dim] ~ N(0,1)."""
    g = _gen(seed)
    seq_kv = seq if seq_kv is None else seq_kv
    q = _normal((batch, heads, seq, dim), g)
    k = _normal((batch, heads, seq_kv, dim), g)
    v = _normal((batch, heads, seq_kv, dim), g)
    return q, k, v


def make_c5_decode_slice(b, h, kv_len=32768, dim=128, heads=32, seed=SEEDS["c5"]):
    """One (batch, head) slice of the flash-decoding workload: q [dim], K,V [kv_len, dim]."""
    g = _gen(seed * 1_000_000 + b * heads + h)
    q = _normal((dim,), g)
    k = _normal((kv_len, dim), g)
    v = _normal((kv_len, dim), g)
    return q, k, v
