"""GPU parity of split-KV flash-decoding (split kernel + combine kernel) through the C ABI
against the fp32 CPU oracle.  Tolerance: rel-L2 <= 1e-3, max-abs <= 2e-2.
The reference has no decoding kernel: the oracle is the closed form, itself pinned by the
split/combine identity and an independent C loop (tests/test_oracle_numerics.py)."""

import math

import pytest
import torch

import oracle
from oracle import numerics as N
from tests.gpu_util import DEV, c_decode

pytestmark = pytest.mark.gpu


def _slices(bh, lkv):
    qs, ks, vs = zip(*[oracle.make_c5_decode_slice(i // 32, i % 32, kv_len=lkv) for i in range(bh)])
    return torch.stack(qs), torch.stack(ks), torch.stack(vs)


@pytest.mark.parametrize("bh,lkv,splits", [(4, 1000, 3), (2, 777, 64), (3, 1, 1), (3, 5, 8), (8, 4096, 1),
                                           (8, 4096, 64), (2, 32768, 64), (1, 20000, 7), (5, 128, 128),
                                           (2, 128, 1), (2, 256, 1), (2, 384, 1), (3, 129, 1), (3, 257, 2)])
def test_shapes_and_ragged_splits(bh, lkv, splits):
    q, k, v = _slices(bh, lkv)
    o = c_decode(q.to(DEV), k.to(DEV), v.to(DEV), splits)
    assert not torch.isnan(o).any()
    ok, r, m = N.check_close(o, N.flash_decode_ref(q, k, v))
    assert ok, f"rel_l2={r:.3e} max_abs={m:.3e}"


# The kernels are templates of the element type and the head dimension (the reference's 16-bit
# types, include/kernels/dispatch_macros.hpp:6-23).  bf16: the oracle consumes the bf16-rounded
# inputs in fp32, what is left is the rounding of the output to 8 mantissa bits (rel-L2 <= 4e-3,
# max-abs <= 4e-2); head dimension 64 puts two key rows in a 16-lane group (8-lane reductions).
@pytest.mark.parametrize("dtype,tol", [(torch.float16, (1e-3, 2e-2)), (torch.bfloat16, (4e-3, 4e-2))])
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("bh,lkv,splits", [(4, 1000, 3), (3, 5, 8), (2, 32768, 64), (5, 128, 128), (3, 257, 2),
                                           (16, 4096, 16), (2, 2048, 1)])
def test_element_types_and_head_dimensions(dtype, tol, d, bh, lkv, splits):
    g = torch.Generator().manual_seed(bh * 100 + lkv + d)
    q = torch.randn(bh, d, generator=g).to(dtype)
    k = torch.randn(bh, lkv, d, generator=g).to(dtype)
    v = torch.randn(bh, lkv, d, generator=g).to(dtype)
    o = c_decode(q.to(DEV), k.to(DEV), v.to(DEV), splits)
    assert o.dtype == dtype and not torch.isnan(o).any()
    ref = N.flash_decode_ref(q, k, v, 1.0 / math.sqrt(d))
    assert N.rel_l2(o, ref) <= tol[0] and N.max_abs(o, ref) <= tol[1], (N.rel_l2(o, ref), N.max_abs(o, ref))


def test_one_hot_keys_pick_single_value_rows_exactly():
    # a key that dominates by a wide margin makes the output that key's value row, bit for bit,
    # in every type and head dimension (a wrong lane-group reduction or row mapping cannot hide)
    for dtype in (torch.float16, torch.bfloat16):
        for d in (64, 128):
            g = torch.Generator().manual_seed(d)
            bh, lkv = 6, 3000
            q = torch.zeros(bh, d); q[:, 0] = 8.0
            k = torch.zeros(bh, lkv, d)
            hot = torch.randint(0, lkv, (bh,), generator=g)
            k[torch.arange(bh), hot, 0] = 16.0          # logit 128 * scale against 0 everywhere else
            v = torch.randint(-8, 9, (bh, lkv, d), generator=g).float()
            o = c_decode(q.to(dtype).to(DEV), k.to(dtype).to(DEV), v.to(dtype).to(DEV), 7, 1.0)
            assert torch.equal(o.float().cpu(), v[torch.arange(bh), hot]), (dtype, d)


def test_scale_and_extreme_logits():
    q, k, v = _slices(4, 2048)
    for scale in (1.0, 1e-3, -0.2):
        o = c_decode(q.to(DEV), k.to(DEV), v.to(DEV), 16, scale)
        ok, r, m = N.check_close(o, N.flash_decode_ref(q, k, v, scale))
        assert ok, f"scale={scale}: rel_l2={r:.3e} max_abs={m:.3e}"


def test_split_count_invariance_and_invariants():
    q, k, v = _slices(4, 4096)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    base = c_decode(qd, kd, vd, 1).float()
    for splits in (2, 16, 64, 257):
        assert (c_decode(qd, kd, vd, splits).float() - base).abs().max() < 2e-3
    assert (c_decode(qd, kd, torch.ones_like(vd), 64).float() - 1).abs().max() < 2e-3
    # one dominant key: the output is that key's value row
    k2 = k.clone(); k2[:, 1234] = q * 8
    o = c_decode(qd, k2.to(DEV), vd, 64)
    assert N.max_abs(o, v[:, 1234]) < 2e-3


def test_c5_full_size():
    # B16 H32 q1 KV32768 D128, 64 splits: 8 GiB of K,V are drawn on the device; a sample of
    # (batch, head) slices is copied back so the oracle consumes identical values, and the
    # split-count invariance covers every slice.
    bh, lkv, d = 512, 32768, 128
    g = torch.Generator(device=DEV).manual_seed(oracle.SEEDS["c5"])
    q = torch.randn(bh, d, device=DEV, dtype=torch.float16, generator=g)
    k = torch.randn(bh, lkv, d, device=DEV, dtype=torch.float16, generator=g)
    v = torch.randn(bh, lkv, d, device=DEV, dtype=torch.float16, generator=g)
    o = c_decode(q, k, v, 64)
    assert not torch.isnan(o).any()
    for i in (0, 100, 255, 511):
        ok, r, m = N.check_close(o[i], N.flash_decode_ref(q[i].cpu(), k[i].cpu(), v[i].cpu()))
        assert ok, f"slice {i}: rel_l2={r:.3e} max_abs={m:.3e}"
    o16 = c_decode(q, k, v, 16)
    assert (o.float() - o16.float()).abs().max() < 1e-3
