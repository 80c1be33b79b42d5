"""GPU parity of the fused back-to-back GEMM through the C ABI against the fp32 CPU oracle.
Tolerance: rel-L2 <= 1e-3, max-abs <= 2e-2."""

import pytest
import torch

import oracle
from oracle import numerics as N
from tests.gpu_util import DEV, c_fused

pytestmark = pytest.mark.gpu


def test_reference_case():
    # tests/python/test_fused_two_gemms.py:55-60: M,N,K,P = 256,128,64,64, tiles 64,
    # inputs normal(5e-3, 1e-2)
    g = torch.Generator().manual_seed(0)
    mk = lambda *s: (torch.randn(*s, generator=g) * 1e-2 + 5e-3).half()
    a, b, c = mk(256, 64), mk(128, 64), mk(64, 128)
    d = c_fused(a.to(DEV), b.to(DEV), c.to(DEV), (64, 64, 64, 64))
    ref = N.fused_two_gemms_ref(a, b, c)
    assert torch.allclose(d.float().cpu(), ref, rtol=1e-3, atol=1e-3)  # the reference's own bar
    assert N.rel_l2(d, ref) <= 2e-3  # tiny magnitudes: fp16 output rounding dominates


def test_c3_full_size():
    a, b, c = oracle.make_c3_fused_inputs()
    d = c_fused(a.to(DEV), b.to(DEV), c.to(DEV), (64, 128, 128, 128))
    ok, r, m = N.check_close(d, N.fused_two_gemms_ref(a, b, c))
    assert ok, f"C3: rel_l2={r:.3e} max_abs={m:.3e}"
    # and it must sit closer to the oracle that rounds the intermediate like the kernel
    assert N.rel_l2(d, N.fused_two_gemms_ref_rounded(a, b, c)) <= r + 1e-5


@pytest.mark.parametrize("m,n,k,p", [(64, 32, 32, 16), (100, 32, 32, 16), (1, 128, 128, 128), (512, 512, 128, 128),
                                     (300, 256, 64, 64), (256, 160, 96, 48), (1024, 1024, 256, 128),
                                     (128, 128, 512, 256), (2048, 96, 32, 80)])
def test_shapes(m, n, k, p):
    a, b, c = oracle.make_c3_fused_inputs(m, n, k, p, seed=m + n + k + p)
    d = c_fused(a.to(DEV), b.to(DEV), c.to(DEV))
    assert not torch.isnan(d).any()
    ref = N.fused_two_gemms_ref(a, b, c)
    assert N.rel_l2(d, ref) <= 1e-3 and N.max_abs(d, ref) <= 2e-2 * max(1.0, float(ref.abs().max()))


# The streaming kernel (K = P = 128, N a multiple of 64 from 256 on): two wavefront sets take
# alternate n-tiles and their partial sums are added at the end.  Tile counts that are even, odd
# and not a multiple of the ring length; a ragged last row block; one row; a batch.  Operands are
# small integers times a power of two, so both products, the fp16 rounding of the intermediate
# and the final sums are exact and the comparison with the oracle is bit-exact.
@pytest.mark.parametrize("batch,m,n", [(1, 64, 256), (1, 70, 320), (1, 1, 448), (1, 200, 1088), (3, 96, 384)])
def test_streaming_kernel_exact(batch, m, n):
    g = torch.Generator().manual_seed(17 * m + n + batch)
    a = torch.randint(-2, 3, (batch, m, 128), generator=g).half()
    b = (torch.randint(-2, 3, (batch, n, 128), generator=g) / 4).half()
    c = (torch.randint(-2, 3, (batch, 128, n), generator=g) / 8).half()
    d = c_fused(a.to(DEV), b.to(DEV), c.to(DEV)).cpu()
    for i in range(batch):
        ref = N.fused_two_gemms_ref_rounded(a[i], b[i], c[i])
        assert torch.equal(d[i].float(), ref.half().float()), f"batch {i}"


def test_batched():
    g = torch.Generator().manual_seed(4)
    a = (torch.randn(3, 192, 64, generator=g) / 8).half()
    b = (torch.randn(3, 128, 64, generator=g) / 8).half()
    c = (torch.randn(3, 64, 128, generator=g) / 8).half()
    d = c_fused(a.to(DEV), b.to(DEV), c.to(DEV))
    for i in range(3):
        ok, r, m = N.check_close(d[i], N.fused_two_gemms_ref(a[i], b[i], c[i]))
        assert ok, f"batch {i}: rel_l2={r:.3e} max_abs={m:.3e}"


def test_integer_inputs_are_exact():
    g = torch.Generator().manual_seed(8)
    a = torch.randint(-2, 3, (256, 64), generator=g).half()
    b = torch.randint(-2, 3, (128, 64), generator=g).half()
    c = torch.randint(-1, 2, (64, 128), generator=g).half()
    d = c_fused(a.to(DEV), b.to(DEV), c.to(DEV))
    ref = N.fused_two_gemms_ref(a, b, c)
    assert ref.abs().max() < 2048  # exactly representable in fp16
    assert torch.equal(d.float().cpu(), ref)
