"""GPU parity of the fused back-to-back GEMM through the C ABI against the fp32 CPU oracle.
Tolerance: rel-L2 <= 1e-3, max-abs <= 2e-2."""

import pytest
import torch

import oracle
from oracle import numerics as N
from tests.gpu_util import DEV, c_fused, c_fused_dtype, c_fused_ws

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


# With a workspace the long-N problems are cut along N (fp32 partial sums per part, added up by a
# second kernel).  The same exact-integer construction: the cut result must equal the oracle and the
# uncut kernel bit for bit.  Shapes: parts of equal and of unequal length, a ragged last row block,
# a batch, one row (all with 64-row blocks, four wavefronts x two sets); 4096 and 4000 rows x 4096
# take 128-row blocks (eight wavefronts, every one on every tile), the second with a ragged block.
@pytest.mark.parametrize("batch,m,n", [(1, 64, 2048), (1, 70, 1856), (1, 1, 2048), (1, 200, 2112), (3, 96, 1600),
                                       (1, 4096, 2048), (1, 4096, 4096), (1, 4000, 4096)])
def test_split_along_n_is_exact(batch, m, n):
    g = torch.Generator().manual_seed(19 * m + n + batch)
    a = torch.randint(-2, 3, (batch, m, 128), generator=g).half()
    b = (torch.randint(-2, 3, (batch, n, 128), generator=g) / 4).half()
    c = (torch.randint(-2, 3, (batch, 128, n), generator=g) / 8).half()
    ad, bd, cd = a.to(DEV), b.to(DEV), c.to(DEV)
    d, want = c_fused_ws(ad, bd, cd)
    assert want > 0 and want % (batch * m * 128 * 4) == 0
    assert torch.equal(d, c_fused(ad, bd, cd))
    d = d.cpu()
    for i in range(batch if m <= 200 else 0):
        ref = N.fused_two_gemms_ref_rounded(a[i], b[i], c[i])
        assert torch.equal(d[i].float(), ref.half().float()), f"batch {i}"


def test_many_rows_take_128_row_blocks_exactly():
    # 256 blocks of 128 rows and more run eight wavefronts on every tile; the last block is ragged
    g = torch.Generator().manual_seed(23)
    m, n = 256 * 128 + 40, 576
    a = torch.randint(-2, 3, (m, 128), generator=g).half()
    b = (torch.randint(-2, 3, (n, 128), generator=g) / 4).half()
    c = (torch.randint(-2, 3, (128, n), generator=g) / 8).half()
    d = c_fused(a.to(DEV), b.to(DEV), c.to(DEV)).cpu()
    for rows in (slice(0, 300), slice(m - 300, m)):
        ref = N.fused_two_gemms_ref_rounded(a[rows], b, c)
        assert torch.equal(d[rows].float(), ref.half().float())
    # every row block agrees with the 64-row kernel, which a shorter problem runs
    d_small = c_fused(a[:8192].to(DEV), b.to(DEV), c.to(DEV)).cpu()
    assert torch.equal(d[:8192], d_small)


def test_workspace_form_without_a_cut_is_the_plain_op():
    g = torch.Generator().manual_seed(5)
    a = (torch.randn(300 * 64, 128, generator=g) / 8).half().to(DEV)
    b = (torch.randn(2048, 128, generator=g) / 8).half().to(DEV)
    c = (torch.randn(128, 2048, generator=g) / 8).half().to(DEV)
    d, want = c_fused_ws(a, b, c)
    assert want == 0 and torch.equal(d, c_fused(a, b, c))          # enough row blocks: not cut
    d, want = c_fused_ws(a[:64], b[:512].contiguous(), c[:, :512].contiguous())
    assert want == 0                                               # eight n-tiles: a cut would not pay
    a = a[:4096].contiguous()
    d, want = c_fused_ws(a, b, c, workspace_bytes=0)               # no workspace handed over: not cut
    assert want > 0 and torch.equal(d, c_fused(a, b, c))
    d2, _ = c_fused_ws(a, b, c)                                    # cut: same sums in another order
    ok, r, m = N.check_close(d2, d.float().cpu())
    assert ok and r < 1e-3


# bf16 runs the same kernels with the bf16 MFMA.  Small integers are exact in bf16 too, so the plain
# kernel (one n-tile, several n-tiles, ragged rows), the streaming kernel and the cut along N are
# compared bit for bit with the oracle evaluated on the same values; a random case bounds the error
# of the bf16 rounding of the intermediate (8 mantissa bits): rel-L2 <= 4e-3.
@pytest.mark.parametrize("m,n,k,p,workspace", [(256, 128, 128, 128, False), (70, 96, 64, 48, False), (130, 384, 128, 128, False),
                                               (64, 2048, 128, 128, True), (4096, 4096, 128, 128, True)])
def test_bf16_kernels_exact(m, n, k, p, workspace):
    g = torch.Generator().manual_seed(m + n + k + p)
    a = torch.randint(-2, 3, (m, k), generator=g).bfloat16()
    b = (torch.randint(-2, 3, (n, k), generator=g) / 4).bfloat16()
    c = (torch.randint(-2, 3, (p, n), generator=g) / 8).bfloat16()
    d = c_fused_dtype(a.to(DEV), b.to(DEV), c.to(DEV), workspace=workspace).cpu()
    rows = slice(0, min(m, 256))
    inter = (a[rows].float() @ b.float().T)
    assert torch.equal(inter.bfloat16().float(), inter)            # the intermediate is exact in bf16
    ref = inter @ c.float().T
    assert torch.equal(d[rows].float(), ref.bfloat16().float())
    if workspace:
        assert torch.equal(d, c_fused_dtype(a.to(DEV), b.to(DEV), c.to(DEV)).cpu())


# Every instance of the plain kernel - n-tiles of 128 / 32, p-tiles of 128 / 64 / 16, k-chunks of
# 128 / 32, fp16 and bf16 - on problems with several k-chunks (K > KC) and several n-tiles (N > TN)
# and a ragged row count.  The kernel requests its A fragments from assembly and waits for them by
# counting requests; a fragment register read before its data has arrived, in any instance, shows as
# a wrong integer here.  B and C are sparse (+-1 in a few places of every row), so that both products
# stay small integers, exact even in bf16, while every k-chunk and n-tile contributes to them.
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k", [256, 96])      # k-chunks of 128 (two of them) and of 32 (three)
@pytest.mark.parametrize("p", [256, 192, 48])  # p-tiles of 128, 64, 16
@pytest.mark.parametrize("n", [256, 192, 96])  # n-tiles of 128 (two), 32 (six), 32 (three)
def test_every_plain_kernel_instance_is_exact(dtype, k, p, n):
    g = torch.Generator().manual_seed(n + p + k)
    m = 100

    def sparse_rows(rows, cols, per_row):
        t = torch.zeros(rows, cols)
        for r in range(rows):
            idx = torch.randperm(cols, generator=g)[:per_row]
            t[r, idx] = (torch.randint(0, 2, (per_row,), generator=g) * 2 - 1).float()
        return t
    a = torch.randint(-2, 3, (m, k), generator=g).float()
    b = sparse_rows(n, k, 6)     # every row of B picks six entries of a row of A
    c = sparse_rows(p, n, 4)     # every row of C picks four entries of the intermediate
    inter = a @ b.T
    ref = inter @ c.T
    assert float(inter.abs().max()) <= 12 and float(ref.abs().max()) <= 48   # integers, exact in bf16 too
    assert (b.abs().sum(0).reshape(-1, 32).sum(1) > 0).all() and (c.abs().sum(0).reshape(-1, 32).sum(1) > 0).all()
    for _ in range(2):
        d = c_fused_dtype(a.to(dtype).to(DEV), b.to(dtype).to(DEV), c.to(dtype).to(DEV)).cpu()
        assert torch.equal(d.float(), ref)


def test_bf16_random_inputs_within_tolerance():
    g = torch.Generator().manual_seed(77)
    a = (torch.randn(512, 128, generator=g) / 11).bfloat16()
    b = (torch.randn(128, 128, generator=g) / 11).bfloat16()
    c = (torch.randn(128, 128, generator=g) / 11).bfloat16()
    d = c_fused_dtype(a.to(DEV), b.to(DEV), c.to(DEV))
    ref = N.fused_two_gemms_ref(a, b, c)
    assert N.rel_l2(d, ref) <= 4e-3 and N.max_abs(d, ref) <= 4e-2 * max(1.0, float(ref.abs().max()))


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
