"""The torch.ops.tilefusion.* / tilefusion_amd.ops path (binding -> C ABI -> HIP kernels),
restating the reference's op-level tests (tests/python/test_{gemm,fused_two_gemms,flash_attn}.py)
with fp32 CPU oracles.  Tolerance: rel-L2 <= 1e-3, max-abs <= 2e-2."""

import math

import pytest
import torch

import oracle
from oracle import numerics as N

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_gemm_op_reference_signature():
    from tilefusion_amd.ops import gemm
    a, b = oracle.make_c1_gemm_inputs(256, 256, 256)
    for dt in (torch.float32, torch.float16):
        c = torch.zeros(256, 256, device=DEV, dtype=dt)
        gemm(a.to(DEV), b.to(DEV), c, 64, 64, 64, 2, 1)
        ok, r, m = N.check_close(c, N.gemm_ref(a, b))
        assert ok, (r, m)
    with pytest.raises(RuntimeError, match="does not divide"):
        gemm(a.to(DEV), b.to(DEV), torch.zeros(256, 256, device=DEV), 96, 64, 64, 1, 0)
    with pytest.raises(RuntimeError, match="contiguous"):
        gemm(a.to(DEV).t(), b.to(DEV), torch.zeros(256, 256, device=DEV), 64, 64, 64, 1, 0)
    with pytest.raises(RuntimeError, match="float16"):
        gemm(a.to(DEV).float(), b.to(DEV), torch.zeros(256, 256, device=DEV), 64, 64, 64, 1, 0)


def test_fused_two_gemms_op():
    from tilefusion_amd.ops import fused_two_gemms
    a, b, c = oracle.make_c3_fused_inputs(256, 128, 64, 64)
    d = torch.zeros(256, 64, device=DEV, dtype=torch.float16)
    fused_two_gemms(a.to(DEV), b.to(DEV), c.to(DEV), d)  # default tiles 64
    ok, r, m = N.check_close(d, N.fused_two_gemms_ref(a, b, c))
    assert ok, (r, m)
    with pytest.raises(TypeError):
        fused_two_gemms(a.to(DEV).float(), b.to(DEV), c.to(DEV), d)


@pytest.mark.parametrize("lq,lkv,causal", [(64, 128, False), (128, 128, True)])
def test_flash_attention_op(lq, lkv, causal):
    # tests/python/test_flash_attn.py:173-199: query [Lq, D], key [D, Lkv], value [Lkv, Dv]
    from tilefusion_amd.ops import flash_attention
    torch.manual_seed(1234)
    q = torch.randn(lq, 128, dtype=torch.float16)
    k = torch.randn(128, lkv, dtype=torch.float16)
    v = torch.randn(lkv, 128, dtype=torch.float16)
    scale = 1.0 / math.sqrt(128)
    o = flash_attention(q.to(DEV), k.to(DEV), v.to(DEV), 64, 128, 128, 128, scale, causal)
    assert o.shape == (lq, 128)
    ok, r, m = N.check_close(o, N.attention_ref(q, k.t(), v, scale, causal))
    assert ok, (r, m)
    # the raw op keeps the reference contract: K [Lkv, D], V transposed [Dv, Lkv]
    o2 = torch.zeros_like(o)
    torch.ops.tilefusion.flash_attention(q.to(DEV), k.t().contiguous().to(DEV), v.t().contiguous().to(DEV), o2,
                                         64, 128, 128, 128, scale, causal)
    ok, r, m = N.check_close(o2, N.attention_ref(q, k.t(), v, scale, causal))
    assert ok, (r, m)


def test_flash_attention_batched_and_decode_ops():
    from tilefusion_amd.ops import flash_attention, flash_decode
    q, k, v = oracle.make_c4_attention_inputs(2, 3, 256, 128)
    o = flash_attention(q.to(DEV), k.transpose(-1, -2).contiguous().to(DEV), v.to(DEV), 64, 64, 128, 128,
                        1.0 / math.sqrt(128), True)
    ok, r, m = N.check_close(o, N.attention_ref(q, k, v, causal=True))
    assert ok, (r, m)
    qs, ks, vs = zip(*[oracle.make_c5_decode_slice(0, h, kv_len=3000) for h in range(6)])
    q, k, v = torch.stack(qs).view(2, 3, 1, 128), torch.stack(ks).view(2, 3, 3000, 128), torch.stack(vs).view(2, 3, 3000, 128)
    o = flash_decode(q.to(DEV), k.to(DEV), v.to(DEV), num_splits=8)
    assert o.shape == q.shape
    ok, r, m = N.check_close(o.view(6, 128), N.flash_decode_ref(q.view(6, 128), k.view(6, 3000, 128), v.view(6, 3000, 128)))
    assert ok, (r, m)


def test_ops_run_on_the_current_stream():
    from tilefusion_amd.ops import gemm
    a, b = oracle.make_c1_gemm_inputs(512, 512, 512)
    ad, bd = a.to(DEV), b.to(DEV)
    s = torch.cuda.Stream()
    c = torch.zeros(512, 512, device=DEV)
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(3):
            gemm(ad, bd, c, 64, 64, 64, 1, 0)
    s.synchronize()
    ok, r, m = N.check_close(c, N.gemm_ref(a, b))
    assert ok, (r, m)


def test_smoke_entry():
    import __graft_entry__
    __graft_entry__.smoke()
