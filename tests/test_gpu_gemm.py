"""GPU parity of the GEMM macro kernel through the C ABI against the fp32 CPU oracle.
Tolerance (benchmark contract): rel-L2 <= 1e-3 and max-abs <= 2e-2, fp16 in / fp32 accumulate."""

import pytest
import torch

import oracle
from oracle import numerics as N
from tests.gpu_util import DEV, c_gemm

pytestmark = pytest.mark.gpu


def _check(c, ref, what):
    ok, r, m = N.check_close(c, ref)
    assert ok, f"{what}: rel_l2={r:.3e} max_abs={m:.3e}"


def test_readme_single_tile_gemm_c1():
    # README example: A 128x256 row-major, B 256x64 col-major, C 128x64 fp32
    a, b = oracle.make_c1_gemm_inputs()
    c = c_gemm(a.to(DEV), b.to(DEV), torch.float32, (128, 64, 32))
    _check(c, N.gemm_ref(a, b), "C1")
    assert N.max_abs(c, N.gemm_ref(a, b)) < 1e-4  # fp32 output: only summation order differs


# tests/python/test_gemm.py:75-135: (128^3, 256^3, 512^3) x tile 64^3 x (stages, level)
@pytest.mark.parametrize("size,stages,level", [(128, 1, 0), (256, 1, 0), (256, 2, 1), (512, 2, 1), (512, 3, 2)])
def test_reference_op_cases(size, stages, level):
    g = torch.Generator().manual_seed(size + level)
    a = torch.randn(size, size, generator=g).half()
    b = torch.randn(size, size, generator=g).half()
    c = c_gemm(a.to(DEV), b.to(DEV), torch.float32, (64, 64, 64), stages, level)
    _check(c, N.gemm_ref(a, b), f"gemm {size}^3")


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_large_gemm_c2(out_dtype):
    a, b = oracle.make_c2_gemm_inputs()
    c = c_gemm(a.to(DEV), b.to(DEV), out_dtype, (64, 128, 128), 2, 1)
    _check(c, N.gemm_ref(a, b), "C2 4096^3")


# shapes of tests/cpp/cell/test_gemm.cu:316-375 (M,N in 16..128, K in 32..256) plus ragged
# ones that exercise the bounds-checked path, non-square and mid-size direct-LDS tiles
@pytest.mark.parametrize("m,n,k", [(16, 16, 32), (32, 32, 64), (64, 64, 128), (128, 128, 256), (64, 128, 64),
                                   (100, 72, 40), (1, 1, 8), (33, 257, 136), (384, 128, 192), (256, 512, 64),
                                   (1024, 768, 320), (2048, 256, 64)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_shapes(m, n, k, out_dtype):
    g = torch.Generator().manual_seed(m * 131 + n * 17 + k)
    a = torch.rand(m, k, generator=g).half()
    b = torch.rand(n, k, generator=g).half()
    c = c_gemm(a.to(DEV), b.to(DEV), out_dtype)
    assert not torch.isnan(c).any()
    ref = N.gemm_ref(a, b)
    # U[0,1) inputs give outputs of size ~k/4: compare relative to that scale
    assert N.rel_l2(c, ref) <= 1e-3
    assert N.max_abs(c, ref) <= 2e-2 * max(1.0, float(ref.abs().max()))


def test_integer_inputs_are_exact():
    # products and sums of small integers are exact in fp32: bit-exact against the oracle
    g = torch.Generator().manual_seed(3)
    a = torch.randint(-3, 4, (512, 256), generator=g).half()
    b = torch.randint(-3, 4, (384, 256), generator=g).half()
    for dt in (torch.float32, torch.float16):
        c = c_gemm(a.to(DEV), b.to(DEV), dt)
        assert torch.equal(c.float().cpu(), N.gemm_ref(a, b))


# The 256x256x64 ring kernel (grids of more than 128 tiles of 256x256, K % 64 == 0): one k-tile,
# fewer k-tiles than ring units, counts that are not multiples of the ring length, non-square
# tile grids.
# Small integers make every product and partial sum exact, so the comparison is bit-exact and
# a single misplaced fragment, a stale ring unit or a missed wait cannot hide in a tolerance.
@pytest.mark.parametrize("m,n,k", [(4096, 3072, 64), (3072, 4096, 128), (4096, 4096, 192), (2304, 4096, 320),
                                   (6144, 2048, 448), (4096, 4096, 1088)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_ring_kernel_exact(m, n, k, out_dtype):
    g = torch.Generator(device=DEV).manual_seed(m + 3 * n + 7 * k)
    a = torch.randint(-2, 3, (m, k), generator=g, device=DEV).half()
    b = torch.randint(-2, 3, (n, k), generator=g, device=DEV).half()
    c = c_gemm(a, b, out_dtype)
    ref = torch.matmul(a.float(), b.float().T)  # exact in fp32 (|sum| < 2^24), any summation order
    if out_dtype == torch.float16:
        ref = ref.half()                        # |values| <= 4k <= 4352: exact or one correctly rounded step
    assert torch.equal(c, ref)
    # and against the CPU oracle on a sampled block (the oracle is the reference, torch only scales it up)
    blk = N.gemm_ref(a[256:384].cpu(), b[512:576].cpu())
    assert torch.equal(c[256:384, 512:576].float().cpu(), blk if out_dtype == torch.float32 else blk.half().float())


# The same ring kernel with 128x128 tiles (grids with fewer than 128 tiles of 256x256; a ring of
# 9 units, requests 4 tiles ahead): fewer k-tiles than the look-ahead, counts around the ring
# length, one tile, non-square grids.
@pytest.mark.parametrize("m,n,k", [(128, 128, 64), (128, 256, 128), (256, 128, 256), (384, 640, 320), (640, 384, 576),
                                   (1024, 1024, 1216), (2048, 2048, 2048),
                                   # more tiles than CUs: the 5-unit variant with two workgroups per CU
                                   (2048, 2176, 64), (2176, 2048, 192), (2048, 2304, 448), (3072, 2560, 704)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_ring_kernel_mid_tiles_exact(m, n, k, out_dtype):
    g = torch.Generator(device=DEV).manual_seed(m + 3 * n + 7 * k)
    a = torch.randint(-2, 3, (m, k), generator=g, device=DEV).half()
    b = torch.randint(-2, 3, (n, k), generator=g, device=DEV).half()
    c = c_gemm(a, b, out_dtype)
    ref = torch.matmul(a.float(), b.float().T)
    if out_dtype == torch.float16:
        ref = ref.half()   # |values| <= 4k = 8192 at most; sums of a few thousand terms of size <= 4 stay far below it
    assert torch.equal(c, ref)
    blk = N.gemm_ref(a[:128].cpu(), b[64:128].cpu())
    assert torch.equal(c[:128, 64:128].float().cpu(), blk if out_dtype == torch.float32 else blk.half().float())


def test_linearity_at_full_size():
    # size-independent property: (A1 + A2) B = A1 B + A2 B for integer-valued operands
    g = torch.Generator(device=DEV).manual_seed(5)
    a1 = torch.randint(-2, 3, (4096, 4096), generator=g, device=DEV).half()
    a2 = torch.randint(-2, 3, (4096, 4096), generator=g, device=DEV).half()
    b = torch.randint(-2, 3, (4096, 4096), generator=g, device=DEV).half()
    assert torch.equal(c_gemm(a1 + a2, b), c_gemm(a1, b) + c_gemm(a2, b))


def test_identity_operand():
    g = torch.Generator().manual_seed(9)
    a = torch.randn(256, 256, generator=g).half()
    eye = torch.eye(256).half()
    assert torch.equal(c_gemm(a.to(DEV), eye.to(DEV), torch.float16).cpu(), a)
    # B buffer is [N, K]: C = A @ B^T, so a non-symmetric B catches a transposed operand
    b = torch.randn(256, 256, generator=g).half()
    c = c_gemm(eye.to(DEV), b.to(DEV), torch.float16).cpu()
    assert torch.equal(c, b.T)
