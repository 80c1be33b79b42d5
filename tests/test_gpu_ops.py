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


def test_flash_decode_op_takes_bf16_and_head_dimension_64():
    from tilefusion_amd.ops import flash_decode
    g = torch.Generator().manual_seed(31)
    q = torch.randn(2, 4, 1, 64, generator=g).bfloat16()
    k = torch.randn(2, 4, 1500, 64, generator=g).bfloat16()
    v = torch.randn(2, 4, 1500, 64, generator=g).bfloat16()
    o = flash_decode(q.to(DEV), k.to(DEV), v.to(DEV), num_splits=5)
    assert o.shape == q.shape and o.dtype == torch.bfloat16
    ref = N.flash_decode_ref(q.view(8, 64), k.view(8, 1500, 64), v.view(8, 1500, 64))
    # bf16 output: 8 mantissa bits
    assert N.rel_l2(o.view(8, 64), ref) <= 4e-3 and N.max_abs(o.view(8, 64), ref) <= 4e-2
    with pytest.raises(RuntimeError, match="same dtype"):
        flash_decode(q.to(DEV), k.half().to(DEV), v.to(DEV), num_splits=5)


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


# ---- shapes and element types without a tuned kernel: never an error for a legal call ---------------
# bf16 tolerance: the oracle consumes the bf16-rounded inputs in fp32; products are accumulated in
# fp32; what remains is the bf16 rounding (8 mantissa bits, 2^-9 relative) of the intermediate
# (fused: A*B, attention: the softmax weights) and of the output: rel-L2 <= 4e-3, max-abs <= 4e-2.

def _close_bf16(out, ref):
    return N.rel_l2(out, ref) <= 4e-3 and N.max_abs(out, ref) <= 4e-2 * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("d,dv,lq,lkv,causal", [(64, 128, 128, 256, False), (96, 96, 128, 128, True),
                                                (48, 80, 64, 128, False), (128, 64, 40, 64, True),
                                                (48, 48, 200, 160, True), (32, 16, 64, 96, False)])
def test_flash_attention_ops_for_head_dims_without_a_tuned_kernel(d, dv, lq, lkv, causal):
    # Head dimensions up to 128 without a tuned kernel are zero-padded by the op to the next tuned
    # size ((48, 48) and (32, 16) -> 64, (48, 80) -> 96, mixed ones above that -> 128) and run the
    # tuned kernel, any Lq and Lkv; (96, 96) has a tuned kernel of its own.  Both op forms (natural
    # and transposed V).
    from tilefusion_amd.ops import flash_attention
    g = torch.Generator().manual_seed(d * 1000 + dv)
    q = torch.randn(2, lq, d, generator=g).half()
    k = torch.randn(2, lkv, d, generator=g).half()
    v = torch.randn(2, lkv, dv, generator=g).half()
    scale = 1.0 / math.sqrt(d)
    ref = N.attention_ref(q, k, v, scale, causal)
    o = flash_attention(q.to(DEV), k.transpose(1, 2).contiguous().to(DEV), v.to(DEV), 8, 32, d, dv, scale, causal)
    assert o.shape == (2, lq, dv)
    ok, r, m = N.check_close(o, ref)
    assert ok, (r, m)
    o2 = torch.full((2, lq, dv), float("nan"), dtype=torch.float16, device=DEV)
    torch.ops.tilefusion.flash_attention(q.to(DEV), k.to(DEV), v.transpose(1, 2).contiguous().to(DEV), o2,
                                         8, 32, d, dv, scale, causal)
    ok, r, m = N.check_close(o2, ref)
    assert ok, (r, m)


@pytest.mark.parametrize("d,dv,lq,lkv", [(160, 160, 48, 64), (192, 128, 40, 96)])
def test_flash_attention_ops_for_head_dims_above_128_run_the_header_kernel(d, dv, lq, lkv):
    # no tuned kernel and nothing to pad to: compiled at run time from the header kernel (query rows
    # padded to whole MFMA tiles by the op)
    g = torch.Generator().manual_seed(d + dv)
    q = torch.randn(1, lq, d, generator=g).half()
    k = torch.randn(1, lkv, d, generator=g).half()
    v = torch.randn(1, lkv, dv, generator=g).half()
    scale = 1.0 / math.sqrt(d)
    o = torch.full((1, lq, dv), float("nan"), dtype=torch.float16, device=DEV)
    torch.ops.tilefusion.flash_attention_fwd(q.to(DEV), k.to(DEV), v.to(DEV), o, scale, False)
    ok, r, m = N.check_close(o, N.attention_ref(q, k, v, scale, False))
    assert ok, (r, m)


@pytest.mark.parametrize("d,dv,lq,lkv,tq,tkv,causal", [(256, 256, 64, 128, 64, 64, False),
                                                         (512, 512, 64, 128, 64, 64, False),
                                                         (384, 384, 128, 256, 128, 128, True),
                                                         (512, 256, 48, 96, 48, 32, True)])
def test_flash_attention_ops_shrink_tiles_that_do_not_fit_the_lds(d, dv, lq, lkv, tq, tkv, causal):
    # Whole-head-dimension tiles of these shapes need more than a CU's 160 KiB of LDS (512 x 512
    # with 64 x 64 sequence tiles: 192 KiB; 384 x 384 with 128 x 128: 288 KiB).  The launcher cuts
    # the head dimension into chunks, then the sequence tiles, until they fit.
    from tilefusion_amd.ops import flash_attention
    g = torch.Generator().manual_seed(d * 7 + dv)
    q = torch.randn(2, lq, d, generator=g).half()
    k = torch.randn(2, lkv, d, generator=g).half()
    v = torch.randn(2, lkv, dv, generator=g).half()
    scale = 1.0 / math.sqrt(d)
    ref = N.attention_ref(q, k, v, scale, causal)
    o = flash_attention(q.to(DEV), k.transpose(1, 2).contiguous().to(DEV), v.to(DEV), tq, tkv, d, dv, scale, causal)
    assert o.shape == (2, lq, dv)
    ok, r, m = N.check_close(o, ref)
    assert ok, (r, m)


def test_flash_attention_key_length_that_cannot_be_padded_is_a_clear_error():
    # above 128 the header kernel is what runs, and its key tiles are 32 wide
    q = torch.randn(16, 160, dtype=torch.float16, device=DEV)
    k = torch.randn(48, 160, dtype=torch.float16, device=DEV)
    v = torch.randn(48, 160, dtype=torch.float16, device=DEV)
    o = torch.zeros(16, 160, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="multiple of 32"):
        torch.ops.tilefusion.flash_attention_fwd(q, k, v, o, 0.1, False)


@pytest.mark.parametrize("m,n,k,p", [(128, 64, 48, 64), (64, 48, 64, 32), (96, 80, 112, 48), (256, 128, 64, 72)])
def test_fused_two_gemms_op_pads_what_the_kernels_cannot_tile(m, n, k, p):
    # K = 48, N = 48 ...: legal for the reference's 16-wide base tiles, not whole 32-deep MFMAs
    from tilefusion_amd.ops import fused_two_gemms
    a, b, c = oracle.make_c3_fused_inputs(m, n, k, p)
    d = torch.full((m, p), float("nan"), device=DEV, dtype=torch.float16)
    fused_two_gemms(a.to(DEV), b.to(DEV), c.to(DEV), d, 16, 16, 16, 8)
    ok, r, mx = N.check_close(d, N.fused_two_gemms_ref(a, b, c))
    assert ok, (r, mx)


@pytest.mark.parametrize("m,n,k", [(256, 256, 128), (4096, 512, 256), (96, 160, 64), (128, 128, 96),
                                   (4096, 2048, 96), (32, 32, 32)])
def test_gemm_op_bf16(m, n, k):
    # every kernel of the GEMM is a template of the operand type: the ring kernel (first two shapes),
    # the bounds-checked kernel (96 x 160), the 32-deep direct-to-LDS kernels with 128- and 256-wide
    # tiles (K = 96)
    from tilefusion_amd.ops import gemm
    a, b = oracle.make_c1_gemm_inputs(m, n, k, seed=77)
    a, b = a.bfloat16(), b.bfloat16()
    ref = N.gemm_ref(a, b)
    c32 = torch.full((m, n), float("nan"), device=DEV)
    gemm(a.to(DEV), b.to(DEV), c32, 32, 32, 32, 2, 1)
    assert N.rel_l2(c32, ref) <= 1e-5, N.rel_l2(c32, ref)
    c16 = torch.full((m, n), float("nan"), device=DEV, dtype=torch.bfloat16)
    gemm(a.to(DEV), b.to(DEV), c16, 32, 32, 32, 3, 2)
    assert _close_bf16(c16, ref), (N.rel_l2(c16, ref), N.max_abs(c16, ref))
    # integer operands: exact
    g = torch.Generator().manual_seed(3)
    ai = torch.randint(-3, 4, (m, k), generator=g).bfloat16()
    bi = torch.randint(-3, 4, (n, k), generator=g).bfloat16()
    gemm(ai.to(DEV), bi.to(DEV), c32, 32, 32, 32, 1, 0)
    assert torch.equal(c32.cpu(), N.gemm_ref(ai, bi))
    with pytest.raises(RuntimeError, match="same dtype"):
        gemm(a.to(DEV), b.half().to(DEV), c32, 32, 32, 32, 1, 0)


def test_fused_two_gemms_and_flash_attention_ops_bf16():
    from tilefusion_amd.ops import flash_attention, fused_two_gemms
    a, b, c = [t.bfloat16() for t in oracle.make_c3_fused_inputs(256, 128, 64, 64)]
    d = torch.full((256, 64), float("nan"), device=DEV, dtype=torch.bfloat16)
    fused_two_gemms(a.to(DEV), b.to(DEV), c.to(DEV), d)
    ref = N.fused_two_gemms_ref(a, b, c)
    assert _close_bf16(d, ref), (N.rel_l2(d, ref), N.max_abs(d, ref))
    with pytest.raises(TypeError):
        fused_two_gemms(a.to(DEV), b.half().to(DEV), c.to(DEV), d)
    g = torch.Generator().manual_seed(9)
    q = torch.randn(128, 128, generator=g).bfloat16()
    k = torch.randn(256, 128, generator=g).bfloat16()
    v = torch.randn(256, 128, generator=g).bfloat16()
    for causal in (False, True):
        o = flash_attention(q.to(DEV), k.t().contiguous().to(DEV), v.to(DEV), 64, 64, 128, 128, 1 / math.sqrt(128), causal)
        assert o.dtype == torch.bfloat16
        ref = N.attention_ref(q, k, v, 1 / math.sqrt(128), causal)
        assert _close_bf16(o, ref), (causal, N.rel_l2(o, ref), N.max_abs(o, ref))
