"""GPU tests of the tile-programming headers (GlobalTile / SharedTile / RegTile, iterators,
loaders / storers, gemm(), reduce / broadcast / map / mask, ke_gemm, ke_fused_two_gemms,
ke_flash_attention).  The kernels live in
tests/cpp/tile_api_kernels.hip and are driven through ctypes.

Data-movement tests are bit-exact (integer-valued data `i % 2048` as in the reference's
tests/cpp/cell/test_g2s_load.cu:55); GEMM tests use the fp32 oracle with rel-L2 <= 1e-3,
max-abs <= 2e-2; softmax pieces are compared with numpy in fp32 (abs 1e-5)."""

import ctypes
import os
import subprocess

import numpy as np
import pytest
import torch

import oracle
from oracle import layout as L
from oracle import numerics as N

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
_vp, _i = ctypes.c_void_p, ctypes.c_int


@pytest.fixture(scope="module")
def lib():
    path = os.path.join(ROOT, "tests", "cpp", "libtile_api_tests.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", os.path.dirname(path), "libtile_api_tests.so"])
    lib = ctypes.CDLL(path)
    lib.tt_g2s_roundtrip.argtypes = [_i, _vp, _vp]
    lib.tt_g2s_shape.argtypes = [_i] + [ctypes.POINTER(_i)] * 4
    lib.tt_swizzled_fragments.argtypes = [_i, _vp, _vp, _vp]
    lib.tt_acc_roundtrip.argtypes = [_i, _vp, _vp, _vp, _vp]
    lib.tt_readme_gemm.argtypes = [_vp, _vp, _vp]
    lib.tt_atom_gemm.argtypes = [_i, _vp, _vp, _vp]
    lib.tt_ke_gemm.argtypes = [_i, _vp, _vp, _vp]
    lib.tt_ke_gemm_shape.argtypes = [_i] + [ctypes.POINTER(_i)] * 4
    lib.tt_softmax_pieces.argtypes = [_i, _vp, _vp, _vp, _vp, _i, _i]
    lib.tt_ke_fused.argtypes = [_i, _vp, _vp, _vp, _vp]
    lib.tt_ke_fused_shape.argtypes = [_i] + [ctypes.POINTER(_i)] * 5
    lib.tt_ke_flash.argtypes = [_i, _vp, _vp, _vp, _vp]
    lib.tt_ke_flash_shape.argtypes = [_i] + [ctypes.POINTER(_i)] * 6
    return lib


@pytest.mark.parametrize("variant", range(10))
def test_global_shared_roundtrip_is_exact(lib, variant):
    r, c, eb, cm = (_i(), _i(), _i(), _i())
    lib.tt_g2s_shape(variant, r, c, eb, cm)
    n = r.value * c.value
    dt = torch.float16 if eb.value == 2 else torch.float32
    src = (torch.arange(n) % 2048).to(dt).to(DEV)
    dst = torch.full((n,), -1, dtype=dt, device=DEV)
    assert lib.tt_g2s_roundtrip(variant, src.data_ptr(), dst.data_ptr()) == 0
    assert torch.equal(src, dst)


@pytest.mark.parametrize("variant,rows,cols", [(0, 64, 64), (1, 128, 128), (2, 64, 128), (3, 64, 64)])
def test_swizzled_and_plain_lds_give_identical_fragments(lib, variant, rows, cols):
    a = (torch.arange(rows * cols) % 2048).half().to(DEV)
    b = ((torch.arange(rows * cols) * 7) % 2048).half().to(DEV)
    bad = torch.zeros(1, dtype=torch.int32, device=DEV)
    assert lib.tt_swizzled_fragments(variant, a.data_ptr(), b.data_ptr(), bad.data_ptr()) == 0
    assert int(bad.item()) == 0


@pytest.mark.parametrize("variant,rows,cols", [(0, 32, 64), (1, 128, 64)])
def test_accumulator_tile_roundtrips(lib, variant, rows, cols):
    src = (torch.arange(rows * cols) % 2048).float().to(DEV)
    direct, via_lds = torch.full_like(src, -1), torch.full_like(src, -1)
    half = torch.full((rows * cols,), -1, dtype=torch.float16, device=DEV)
    assert lib.tt_acc_roundtrip(variant, src.data_ptr(), direct.data_ptr(), via_lds.data_ptr(), half.data_ptr()) == 0
    assert torch.equal(src, direct)      # global -> register -> global
    assert torch.equal(src, via_lds)     # global -> register -> LDS (swizzled) -> global
    assert torch.equal(src.half(), half)  # ... and through RegTileConvert to fp16


def test_readme_example_gemm(lib):
    # README.md:56-112: A 128x256 row-major, B 256x64 col-major, C 128x64 fp32, 2x2 wavefronts
    a, b = oracle.make_c1_gemm_inputs()
    c = torch.full((128, 64), float("nan"), device=DEV)
    assert lib.tt_readme_gemm(a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.data_ptr()) == 0
    ok, r, m = N.check_close(c, N.gemm_ref(a, b))
    assert ok and m < 1e-4, (r, m)
    # integer operands: exact
    g = torch.Generator().manual_seed(1)
    a = torch.randint(-3, 4, (128, 256), generator=g).half()
    b = torch.randint(-3, 4, (64, 256), generator=g).half()
    assert lib.tt_readme_gemm(a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.data_ptr()) == 0
    assert torch.equal(c.cpu(), N.gemm_ref(a, b))


def test_other_mma_atoms(lib):
    # bf16 x bf16 -> fp32, and fp16 x fp16 with an fp16 accumulator tile (rounded once per atom)
    a, b = oracle.make_c1_gemm_inputs()
    ref = N.gemm_ref(a.bfloat16(), b.bfloat16())
    c = torch.full((128, 64), float("nan"), device=DEV)
    assert lib.tt_atom_gemm(0, a.bfloat16().to(DEV).data_ptr(), b.bfloat16().to(DEV).data_ptr(), c.data_ptr()) == 0
    ok, r, m = N.check_close(c, ref)
    assert ok and m < 1e-4, (r, m)
    ch = torch.full((128, 64), float("nan"), device=DEV, dtype=torch.float16)
    assert lib.tt_atom_gemm(1, a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), ch.data_ptr()) == 0
    ref = N.gemm_ref(a, b)
    # 8 roundings to fp16 along K = 256 (one per 32-deep atom): a few fp16 ulps of |C| ~ 10
    assert N.rel_l2(ch, ref) <= 2e-3 and N.max_abs(ch, ref) <= 5e-2, (N.rel_l2(ch, ref), N.max_abs(ch, ref))


@pytest.mark.parametrize("variant", range(6))
def test_ke_gemm_composed_from_primitives(lib, variant):
    m, n, k, h = (_i(), _i(), _i(), _i())
    lib.tt_ke_gemm_shape(variant, m, n, k, h)
    a, b = oracle.make_c1_gemm_inputs(m.value, n.value, k.value, seed=100 + variant)
    c = torch.full((m.value, n.value), float("nan"), device=DEV, dtype=torch.float16 if h.value else torch.float32)
    assert lib.tt_ke_gemm(variant, a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.data_ptr()) == 0
    ref = N.gemm_ref(a, b)
    assert N.rel_l2(c, ref) <= 1e-3 and N.max_abs(c, ref) <= 2e-2 * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("variant,rows,cols", [(0, 16, 16), (1, 32, 64), (2, 128, 128)])
@pytest.mark.parametrize("row_off,col_off", [(0, 0), (64, 0), (0, 64), (5, 9)])
def test_reduce_broadcast_exp_mask(lib, variant, rows, cols, row_off, col_off):
    rng = np.random.default_rng(variant * 10 + row_off)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    src = torch.from_numpy(x).to(DEV)
    rmax = torch.zeros(rows, device=DEV)
    rsum = torch.zeros(rows, device=DEV)
    out = torch.zeros(rows, cols, device=DEV)
    assert lib.tt_softmax_pieces(variant, src.data_ptr(), rmax.data_ptr(), rsum.data_ptr(), out.data_ptr(), row_off, col_off) == 0
    # numpy restatement: causal mask in global coordinates (include/cell/mask.hpp:75-82), row max,
    # subtract, exp, row sum, divide, times 2
    rr = np.arange(rows)[:, None] + row_off
    cc = np.arange(cols)[None, :] + col_off
    xm = np.where(cc > rr, -np.inf, x)
    keep = np.isfinite(xm).any(axis=1)   # rows that are not fully masked
    mx = xm.max(axis=1)
    e = np.exp(xm - np.where(keep, mx, 0)[:, None])
    sm = e.sum(axis=1)
    assert np.array_equal(rmax.cpu().numpy()[keep], mx[keep])
    assert np.allclose(rsum.cpu().numpy()[keep], sm[keep], rtol=1e-5)
    want = 2 * e / np.where(keep, sm, 1)[:, None]
    assert np.allclose(out.cpu().numpy()[keep], want[keep], atol=1e-5)


@pytest.mark.parametrize("variant", range(4))
def test_ke_fused_two_gemms_composed_from_primitives(lib, variant):
    # variant 0 is the reference's own case (tests/python/test_fused_two_gemms.py: 256,128,64,64)
    bt, m, n, k, p = (_i(), _i(), _i(), _i(), _i())
    lib.tt_ke_fused_shape(variant, bt, m, n, k, p)
    g = torch.Generator().manual_seed(300 + variant)
    a = (torch.randn(bt.value, m.value, k.value, generator=g) / 8).half()
    b = (torch.randn(bt.value, n.value, k.value, generator=g) / 8).half()   # [n,k] buffer = col-major k x n
    c = (torch.randn(bt.value, p.value, n.value, generator=g) / 8).half()   # [p,n] buffer = col-major n x p
    d = torch.full((bt.value, m.value, p.value), float("nan"), dtype=torch.float16, device=DEV)
    assert lib.tt_ke_fused(variant, a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.to(DEV).data_ptr(), d.data_ptr()) == 0
    for i in range(bt.value):
        ref = N.fused_two_gemms_ref(a[i], b[i], c[i])
        ok, r, ab = N.check_close(d[i], ref)
        assert ok, (variant, i, r, ab)


@pytest.mark.parametrize("variant", range(6))
def test_ke_flash_attention_composed_from_primitives(lib, variant):
    # variants 0 and 1 are the reference's own cases (tests/python/test_flash_attn.py:
    # (64,128,128,128) plain, (128,128,128,128) causal; tiles (64,128,128,128))
    bt, m, n, k, p, causal = (_i(), _i(), _i(), _i(), _i(), _i())
    lib.tt_ke_flash_shape(variant, bt, m, n, k, p, causal)
    g = torch.Generator().manual_seed(400 + variant)
    q = torch.randn(bt.value, m.value, k.value, generator=g).half()
    kk = torch.randn(bt.value, n.value, k.value, generator=g).half()
    v = torch.randn(bt.value, n.value, p.value, generator=g).half()
    vt = v.transpose(1, 2).contiguous()   # the kernel takes V column-major: a [p, n] buffer
    o = torch.full((bt.value, m.value, p.value), float("nan"), dtype=torch.float16, device=DEV)
    assert lib.tt_ke_flash(variant, q.to(DEV).data_ptr(), kk.to(DEV).data_ptr(), vt.to(DEV).data_ptr(), o.data_ptr()) == 0
    ref = N.attention_ref(q, kk, v, causal=bool(causal.value))
    ok, r, ab = N.check_close(o, ref)
    assert ok, (variant, r, ab)
