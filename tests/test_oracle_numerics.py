"""Pins the fp32 oracles by closed forms, invariants and an independent C loop."""

import ctypes
import math
import os

import numpy as np
import pytest
import torch

import oracle
from oracle import numerics as N

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _naive_lib():
    path = os.path.join(ROOT, "oracle", "liboracle_naive.so")
    if not os.path.exists(path):
        import subprocess
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    lib = ctypes.CDLL(path)
    lib.oracle_naive_gemm.argtypes = [ctypes.c_int] * 3 + [ctypes.c_void_p] * 3
    lib.oracle_naive_decode.argtypes = [ctypes.c_int] * 3 + [ctypes.c_void_p] * 3 + [ctypes.c_double, ctypes.c_void_p]
    return lib


def test_inputs_are_seeded_and_fp16():
    a1, b1 = oracle.make_c1_gemm_inputs()
    a2, b2 = oracle.make_c1_gemm_inputs()
    assert a1.dtype == torch.float16 and a1.shape == (128, 256) and b1.shape == (64, 256)
    assert torch.equal(a1, a2) and torch.equal(b1, b2)
    assert a1.abs().max() <= 1.0
    q, k, v = oracle.make_c5_decode_slice(3, 7, kv_len=64)
    q2, _, _ = oracle.make_c5_decode_slice(3, 8, kv_len=64)
    assert q.shape == (128,) and k.shape == (64, 128) and not torch.equal(q, q2)


def test_gemm_ref_hand_case_catches_transposed_operand():
    # A 2x3, B given as [n=2, k=3]; C = A @ B^T by hand
    a = torch.tensor([[1., 2., 3.], [4., 5., 6.]]).half()
    b = torch.tensor([[1., 0., -1.], [2., 1., 0.]]).half()
    assert N.gemm_ref(a, b).tolist() == [[-2., 4.], [-2., 13.]]


def test_gemm_ref_vs_naive_c_loop():
    lib = _naive_lib()
    a, b = oracle.make_c1_gemm_inputs()
    ref = N.gemm_ref(a, b)
    a32, b32 = a.float().contiguous(), b.float().contiguous()
    out = torch.empty(128, 64)
    lib.oracle_naive_gemm(128, 64, 256, a32.data_ptr(), b32.data_ptr(), out.data_ptr())
    assert N.rel_l2(ref, out) < 1e-6 and N.max_abs(ref, out) < 1e-4


def test_fused_ref_hand_case_and_rounding_bound():
    a = torch.tensor([[1., 2.]]).half()
    b = torch.tensor([[1., 1.], [0., 2.]]).half()      # B[k,n] = b[n,k] -> A@B = [3, 4]
    c = torch.tensor([[1., -1.], [2., 0.], [0., 1.]]).half()   # C[n,p] = c[p,n] -> [-1, 6, 4]
    assert N.fused_two_gemms_ref(a, b, c).tolist() == [[-1., 6., 4.]]
    a, b, c = oracle.make_c3_fused_inputs(m=256)
    d, dr = N.fused_two_gemms_ref(a, b, c), N.fused_two_gemms_ref_rounded(a, b, c)
    assert N.rel_l2(dr, d) < 5e-4  # the fp16 intermediate costs < half the tolerance


def test_fused_ref_rounded_rounds_the_intermediate_to_fp16():
    # A@B = [2049, 4099]: 2049 is a tie between the fp16 neighbours 2048 and 2050 (-> even, 2048),
    # 4099 lies between 4096 and 4100 (-> 4100).  Without the rounding D would be 2049 / 4099.
    a = torch.tensor([[2048., 1.], [4096., 3.]]).half()
    b = torch.tensor([[1., 1.]]).half()                 # N = 1, K = 2
    c = torch.tensor([[1.], [0.5]]).half()              # P = 2, N = 1
    assert N.fused_two_gemms_ref(a, b, c).tolist() == [[2049., 1024.5], [4099., 2049.5]]
    assert N.fused_two_gemms_ref_rounded(a, b, c).tolist() == [[2048., 1024.], [4100., 2050.]]


def test_attention_ref_invariants():
    g = torch.Generator().manual_seed(7)
    q = torch.randn(3, 16, 8, generator=g).half()
    k = torch.randn(3, 24, 8, generator=g).half()
    v = torch.randn(3, 24, 5, generator=g).half()
    # causal row 0 attends only to key 0
    o = N.attention_ref(q, k, v, causal=True)
    assert torch.allclose(o[:, 0], v[:, 0].float(), atol=1e-6)
    # all-equal keys -> uniform weights -> mean of V
    k_eq = k[:, :1].expand(-1, 24, -1)
    o = N.attention_ref(q, k_eq, v)
    assert torch.allclose(o, v.float().mean(dim=1, keepdim=True).expand_as(o), atol=1e-5)
    # V = ones -> rows of P sum to one
    o = N.attention_ref(q, k, torch.ones_like(v))
    assert torch.allclose(o, torch.ones_like(o), atol=1e-6)
    # scale is applied to the logits (a dropped scale changes the answer)
    assert not torch.allclose(N.attention_ref(q, k, v, scale=1.0), N.attention_ref(q, k, v, scale=0.1), atol=1e-3)
    # brute force on one row
    s = [sum(float(q[0, 2, i]) * float(k[0, n, i]) for i in range(8)) / math.sqrt(8) for n in range(24)]
    mx = max(s); e = [math.exp(x - mx) for x in s]; den = sum(e)
    want = [sum(e[n] * float(v[0, n, j]) for n in range(24)) / den for j in range(5)]
    assert np.allclose(N.attention_ref(q, k, v)[0, 2].numpy(), want, atol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("tile_kv", [16, 32, 128])
def test_blockwise_online_softmax_equals_direct(causal, tile_kv):
    g = torch.Generator().manual_seed(11)
    q = torch.randn(128, 64, generator=g).half()
    k = torch.randn(128, 64, generator=g).half()
    v = torch.randn(128, 32, generator=g).half()
    d = N.attention_ref(q, k, v, causal=causal)
    b = N.attention_blockwise_ref(q, k, v, tile_kv, causal=causal)
    assert N.max_abs(b, d) < 1e-5


@pytest.mark.parametrize("splits", [1, 3, 8, 64])
def test_split_combine_identity(splits):
    q, k, v = oracle.make_c5_decode_slice(0, 1, kv_len=640)
    direct = N.flash_decode_ref(q, k, v)
    o, m, l = N.split_kv_partials(q, k, v, splits)
    assert N.max_abs(N.combine_partials(o, m, l), direct) < 1e-5


def test_decode_ref_vs_naive_c_loop_and_attention_ref():
    lib = _naive_lib()
    q, k, v = oracle.make_c5_decode_slice(1, 2, kv_len=512)
    ref = N.flash_decode_ref(q, k, v)
    out = torch.empty(128)
    q32, k32, v32 = q.float().contiguous(), k.float().contiguous(), v.float().contiguous()
    lib.oracle_naive_decode(512, 128, 128, q32.data_ptr(), k32.data_ptr(), v32.data_ptr(), 1.0 / math.sqrt(128), out.data_ptr())
    assert N.max_abs(ref, out) < 1e-5
    assert N.max_abs(ref, N.attention_ref(q[None], k, v)[0]) < 1e-6


def test_check_close_uses_contract_tolerances():
    ref = torch.ones(100)
    assert N.check_close(ref + 5e-4, ref)[0]
    assert not N.check_close(ref + 5e-3, ref)[0]
    assert N.REL_L2_TOL == 1e-3 and N.MAX_ABS_TOL == 2e-2


def test_scatter_nd_ref_matches_a_plain_loop():
    # pins the index_put_ restatement: a dropped "accumulate", a transposed index or a wrong
    # slice shape each fail this hand-written loop
    g = torch.Generator().manual_seed(5)
    data = torch.randn(3, 4, 5, generator=g)
    idx = torch.tensor([[0, 1], [2, 3], [0, 1], [1, 0]])           # row 0 repeats
    upd = torch.randn(4, 5, generator=g)
    want = data.clone()
    for i in range(idx.shape[0]):
        for e in range(5):
            want[idx[i, 0], idx[i, 1], e] += upd[i, e]
    assert torch.allclose(N.scatter_nd_ref(data, idx, upd), want, atol=1e-6)
    # index depth == rank: single elements
    idx3 = torch.tensor([[0, 0, 0], [2, 3, 4], [0, 0, 0]])
    upd3 = torch.tensor([1.0, 2.0, 4.0])
    want = data.clone()
    want[0, 0, 0] += 5.0
    want[2, 3, 4] += 2.0
    assert torch.allclose(N.scatter_nd_ref(data, idx3, upd3), want, atol=1e-6)
