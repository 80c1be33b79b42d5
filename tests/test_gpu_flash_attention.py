"""GPU parity of flash-attention forward through the C ABI against the fp32 CPU oracle.
Tolerance: rel-L2 <= 1e-3, max-abs <= 2e-2 (fp16 in/out, fp32 scores and statistics)."""

import math

import pytest
import torch

import oracle
from oracle import numerics as N
from tests.gpu_util import DEV, c_attention

pytestmark = pytest.mark.gpu


def _inputs(b, lq, lkv, d, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(b, lq, d, generator=g).half(), torch.randn(b, lkv, d, generator=g).half(),
            torch.randn(b, lkv, d, generator=g).half())


# tests/python/test_flash_attn.py:202-233: (Lq, Lkv, D, Dv) = (64,128,128,128) non-causal and
# (128,128,128,128) causal, tiles (64,128,128,128), seed 1234; V handed over transposed as the
# reference op receives it
@pytest.mark.parametrize("lq,lkv,causal", [(64, 128, False), (128, 128, True)])
@pytest.mark.parametrize("v_transposed", [True, False])
def test_reference_cases(lq, lkv, causal, v_transposed):
    q, k, v = _inputs(1, lq, lkv, 128, 1234)
    vd = v.transpose(1, 2).contiguous() if v_transposed else v
    o = c_attention(q.to(DEV), k.to(DEV), vd.to(DEV), causal, 1.0 / math.sqrt(128), v_transposed, (64, 128, 128, 128))
    ok, r, m = N.check_close(o, N.attention_ref(q, k, v, causal=causal))
    assert ok, f"rel_l2={r:.3e} max_abs={m:.3e}"


@pytest.mark.parametrize("b,lq,lkv,d", [(3, 200, 136, 128), (2, 1, 16, 128), (2, 128, 1000, 128), (1, 513, 513, 128),
                                        (2, 256, 512, 64), (4, 96, 72, 64), (1, 1024, 2048, 128),
                                        (2, 256, 512, 96), (3, 200, 136, 96), (1, 1024, 1100, 96), (2, 100, 40, 96)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("v_transposed", [False, True])
def test_shapes(b, lq, lkv, d, causal, v_transposed):
    q, k, v = _inputs(b, lq, lkv, d, b * 7 + lq + lkv)
    vd = v.transpose(1, 2).contiguous() if v_transposed else v
    if v_transposed and lkv % 8:
        # rows of a transposed V must stay 16-byte aligned: rejected, not mis-computed
        with pytest.raises(RuntimeError, match="Lkv % 8"):
            c_attention(q.to(DEV), k.to(DEV), vd.to(DEV), causal, None, v_transposed)
        return
    o = c_attention(q.to(DEV), k.to(DEV), vd.to(DEV), causal, None, v_transposed)
    assert not torch.isnan(o).any()
    ok, r, m = N.check_close(o, N.attention_ref(q, k, v, causal=causal))
    assert ok, f"rel_l2={r:.3e} max_abs={m:.3e}"


# The 256-query workgroup keeps a five-tile ring with two tiles live and requests three tiles
# ahead: key ranges of one to seven tiles, with and without a ragged last tile, exercise its fill,
# the clamped requests past the end and the hand-over between the two wavefront sets; 768 queries
# (an odd number of query tiles) take the one-pass causal order, 512 and 1024 the paired one.
@pytest.mark.parametrize("lkv", [8, 64, 72, 128, 192, 200, 256, 320, 384, 448])
@pytest.mark.parametrize("causal", [False, True])
def test_short_key_ranges_through_the_eight_wavefront_ring(lkv, causal):
    q, k, v = _inputs(2, 256, lkv, 128, 900 + lkv)
    o = c_attention(q.to(DEV), k.to(DEV), v.to(DEV), causal, None, False)
    ok, r, m = N.check_close(o, N.attention_ref(q, k, v, causal=causal))
    assert ok, f"rel_l2={r:.3e} max_abs={m:.3e}"


@pytest.mark.parametrize("lq,d", [(512, 128), (768, 128), (1024, 64), (300, 128), (512, 96), (768, 96)])
def test_causal_pass_orders(lq, d):
    q, k, v = _inputs(3, lq, lq, d, 77 + lq)
    o = c_attention(q.to(DEV), k.to(DEV), v.to(DEV), True, None, False)
    ok, r, m = N.check_close(o, N.attention_ref(q, k, v, causal=True))
    assert ok, f"rel_l2={r:.3e} max_abs={m:.3e}"


def test_scale_and_large_logits():
    # scale enters the logits; big logits need the running max (exp would overflow otherwise)
    q, k, v = _inputs(2, 128, 256, 128, 77)
    for scale in (1.0, 0.02, -0.1):
        o = c_attention(q.to(DEV), k.to(DEV), v.to(DEV), False, scale)
        ok, r, m = N.check_close(o, N.attention_ref(q, k, v, scale=scale))
        assert ok, f"scale={scale}: rel_l2={r:.3e} max_abs={m:.3e}"


@pytest.mark.parametrize("causal", [False, True])
def test_reference_maximum_moves_both_ways(causal):
    # The kernel starts every score at minus a lazily updated reference maximum.  Keys whose
    # scores are far below zero first, far above later (and the reverse) force the reference
    # down on the first tile and up by hundreds of log2 units afterwards; a stale reference
    # would underflow every weight to 0 (division by zero) or overflow fp16.
    g = torch.Generator().manual_seed(99)
    d, lq, lkv = 128, 256, 512
    q = torch.randn(1, lq, d, generator=g).half()
    k = torch.randn(1, lkv, d, generator=g).half()
    v = torch.randn(1, lkv, d, generator=g).half()
    q[..., 0] = 8.0                       # a strong common component ...
    ramp = torch.linspace(-6.0, 6.0, lkv)  # ... that the keys weight from very negative to very positive
    for direction in (1.0, -1.0):
        k2 = k.clone()
        k2[0, :, 0] = (direction * ramp).half()
        o = c_attention(q.to(DEV), k2.to(DEV), v.to(DEV), causal, 1.0)   # scale 1: logits span +-48
        assert not torch.isnan(o).any() and not torch.isinf(o).any()
        ok, r, m = N.check_close(o, N.attention_ref(q, k2, v, scale=1.0, causal=causal))
        assert ok, f"direction={direction}: rel_l2={r:.3e} max_abs={m:.3e}"


def test_invariants():
    q, k, v = _inputs(2, 256, 256, 128, 5)
    # causal row 0 sees only key 0
    o = c_attention(q.to(DEV), k.to(DEV), v.to(DEV), True)
    assert torch.equal(o[:, 0].cpu(), v[:, 0])
    # V = 1 -> every output is exactly 1 (weights sum to one)
    o = c_attention(q.to(DEV), k.to(DEV), torch.ones_like(v).to(DEV), False)
    assert (o.float() - 1).abs().max() < 2e-3
    # all keys equal -> mean of V
    keq = k[:, :1].expand(-1, 256, -1).contiguous()
    o = c_attention(q.to(DEV), keq.to(DEV), v.to(DEV), False)
    assert N.max_abs(o, v.float().mean(dim=1, keepdim=True).expand(-1, 256, -1)) < 2e-3


@pytest.mark.parametrize("causal", [False, True])
def test_c4_full_size(causal):
    # B2 H32 S4096 D128: all 64 slices on the GPU; the oracle runs on a sample of slices (a
    # 4096x4096 fp32 softmax each), every other slice is covered by the V = 1 property below
    q, k, v = oracle.make_c4_attention_inputs()
    qd, kd, vd = (t.reshape(64, 4096, 128).to(DEV) for t in (q, k, v))
    o = c_attention(qd, kd, vd, causal).cpu().reshape(2, 32, 4096, 128)
    assert not torch.isnan(o).any()
    for b, h in [(0, 0), (0, 17), (1, 5), (1, 31)]:
        ok, r, m = N.check_close(o[b, h], N.attention_ref(q[b, h], k[b, h], v[b, h], causal=causal))
        assert ok, f"slice ({b},{h}) causal={causal}: rel_l2={r:.3e} max_abs={m:.3e}"
    ones = c_attention(qd, kd, torch.ones_like(vd), causal)
    assert (ones.float() - 1).abs().max() < 2e-3


def test_large_scale_and_large_q_stay_finite():
    # The tuned kernels fold scale * log2(e) into an fp16 copy of Q.  |Q * scale * 1.4427| beyond
    # 65504 saturates instead of turning into inf / NaN scores; well inside the range (here up to
    # ~600) the result still matches the oracle, whose softmax is then nearly one-hot.
    g = torch.Generator().manual_seed(5)
    q = (torch.randn(2, 128, 128, generator=g) * 30).half()
    k = torch.randn(2, 256, 128, generator=g).half()
    v = torch.randn(2, 256, 128, generator=g).half()
    o = c_attention(q.to(DEV), k.to(DEV), v.to(DEV), scale=4.0)
    assert torch.isfinite(o).all()
    ref = N.attention_ref(q, k, v, 4.0)
    # rows whose winning key leads by a clear margin are that key's value row
    logits = (q.float() @ k.float().transpose(1, 2)) * 4.0
    top2 = logits.topk(2, dim=-1).values
    clear = (top2[..., 0] - top2[..., 1]) > 50
    assert clear.float().mean() > 0.5
    assert (o.float().cpu() - ref)[clear].abs().max() < 2e-2
    q_huge = (torch.randn(1, 64, 128, generator=g) * 3e4).half()
    o = c_attention(q_huge.to(DEV), k[:1].to(DEV), v[:1].to(DEV), scale=8.0)
    assert torch.isfinite(o).all()


# bf16 runs the same tuned kernels with the bf16 MFMA, bf16 softmax weights and bf16 output.  The
# oracle consumes the bf16-rounded inputs in fp32; what is left is the rounding of the weights and
# of the output to 8 mantissa bits: rel-L2 <= 4e-3, max-abs <= 4e-2.
@pytest.mark.parametrize("bh,lq,lkv,d,causal,vt", [
    (3, 256, 512, 128, False, False), (2, 384, 384, 128, True, False), (2, 200, 333, 128, False, False),
    (2, 100, 100, 128, True, False), (2, 256, 256, 64, True, False), (3, 130, 517, 64, False, False),
    (2, 256, 512, 128, False, True), (2, 320, 320, 64, True, True),
    (2, 256, 512, 96, False, False), (2, 384, 384, 96, True, False), (2, 130, 520, 96, False, True),
])
def test_bf16_tuned_kernels_match_the_oracle(bh, lq, lkv, d, causal, vt):
    g = torch.Generator().manual_seed(bh * 1000 + lq + lkv + d)
    q = torch.randn(bh, lq, d, generator=g).bfloat16()
    k = torch.randn(bh, lkv, d, generator=g).bfloat16()
    v = torch.randn(bh, lkv, d, generator=g).bfloat16()
    v_dev = v.transpose(1, 2).contiguous().to(DEV) if vt else v.to(DEV)
    o = c_attention(q.to(DEV), k.to(DEV), v_dev, causal=causal, v_transposed=vt)
    assert o.dtype == torch.bfloat16
    ref = N.attention_ref(q, k, v, 1.0 / math.sqrt(d), causal)
    assert N.rel_l2(o, ref) <= 4e-3 and N.max_abs(o, ref) <= 4e-2, (N.rel_l2(o, ref), N.max_abs(o, ref))


def test_bf16_and_fp16_kernels_agree_on_inputs_both_can_hold():
    # inputs with 3 significant bits are exact in both types: the two kernels then differ only in
    # how they round the softmax weights and the output
    g = torch.Generator().manual_seed(77)
    mk = lambda *shape: (torch.randint(-7, 8, shape, generator=g).float() / 4)
    q, k, v = mk(2, 256, 128), mk(2, 384, 128), mk(2, 384, 128)
    o16 = c_attention(q.half().to(DEV), k.half().to(DEV), v.half().to(DEV), causal=True, scale=0.05)
    ob = c_attention(q.bfloat16().to(DEV), k.bfloat16().to(DEV), v.bfloat16().to(DEV), causal=True, scale=0.05)
    ref = N.attention_ref(q, k, v, 0.05, True)
    assert N.rel_l2(o16, ref) <= 1e-3
    assert N.rel_l2(ob, ref) <= 4e-3
    assert N.rel_l2(ob.float(), o16.float().cpu()) <= 4e-3


def test_head_dimension_96_never_reads_the_padding_of_its_lds_rows():
    # Head dimension 96 is kept in 128-element LDS rows; the 32 elements of padding hold copies of
    # the row's last 8 columns (the requests re-fetch the last 16-byte chunk).  Those columns are
    # made to dominate the scores and the values: a fragment read that strayed into the padding
    # would count them more than once.
    g = torch.Generator().manual_seed(96)
    q = torch.randn(2, 256, 96, generator=g)
    k = torch.randn(2, 192, 96, generator=g)
    v = torch.randn(2, 192, 96, generator=g)
    q[..., 88:] *= 3.0
    k[..., 88:] *= 3.0
    v[..., 88:] += 4.0
    q, k, v = q.half(), k.half(), v.half()
    for causal in (False, True):
        for vt in (False, True):
            vd = v.transpose(1, 2).contiguous() if vt else v
            o = c_attention(q.to(DEV), k.to(DEV), vd.to(DEV), causal, None, vt)
            ok, r, m = N.check_close(o, N.attention_ref(q, k, v, causal=causal))
            assert ok, f"causal={causal} vt={vt}: rel_l2={r:.3e} max_abs={m:.3e}"
