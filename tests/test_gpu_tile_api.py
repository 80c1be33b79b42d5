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
    lib.tt_single_atom.argtypes = [_i, _vp, _vp, _vp]
    lib.tt_ke_gemm.argtypes = [_i, _vp, _vp, _vp]
    lib.tt_ke_gemm_shape.argtypes = [_i] + [ctypes.POINTER(_i)] * 4
    lib.tt_softmax_pieces.argtypes = [_i, _vp, _vp, _vp, _vp, _i, _i]
    lib.tt_ke_fused.argtypes = [_i, _vp, _vp, _vp, _vp]
    lib.tt_ke_fused_shape.argtypes = [_i] + [ctypes.POINTER(_i)] * 5
    lib.tt_ke_flash.argtypes = [_i, _vp, _vp, _vp, _vp]
    lib.tt_ke_flash_shape.argtypes = [_i] + [ctypes.POINTER(_i)] * 6
    lib.tt_ke_gemm_pipe.argtypes = [_i, _vp, _vp, _vp]
    lib.tt_ke_gemm_pipe_shape.argtypes = [_i] + [ctypes.POINTER(_i)] * 4
    lib.tt_pipeline_roundtrip.argtypes = [_i, _vp, _vp, _vp]
    lib.tt_pipeline_shape.argtypes = [_i] + [ctypes.POINTER(_i)] * 2
    lib.tt_g2s_subtile.argtypes = [_vp, _vp]
    lib.tt_warp_helpers.argtypes = [_i, _i, _vp]
    lib.tt_stile_iterator2.argtypes = [_i, _vp, _vp, _vp, _vp]
    lib.tt_reg_copy.argtypes = [_vp, _vp, _vp]
    lib.tt_vectorize.argtypes = [_vp, _vp, _vp, _vp]
    lib.tt_functors.argtypes = [_vp] * 9
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


@pytest.mark.parametrize("wide", [True, False])
@pytest.mark.parametrize("shape,rows,cols", [(0, 64, 64), (1, 128, 128), (2, 64, 128), (3, 64, 64)])
def test_swizzled_and_plain_lds_give_identical_fragments(lib, wide, shape, rows, cols):
    # wide 16 x 32 operand base tiles (variants 0-3) and the square 16 x 16 ones (4-7)
    variant = shape if wide else shape + 4
    a = (torch.arange(rows * cols) % 2048).half().to(DEV)
    b = ((torch.arange(rows * cols) * 7) % 2048).half().to(DEV)
    bad = torch.zeros(1, dtype=torch.int32, device=DEV)
    assert lib.tt_swizzled_fragments(variant, a.data_ptr(), b.data_ptr(), bad.data_ptr()) == 0
    assert int(bad.item()) == 0


@pytest.mark.parametrize("variant,rows,cols", [(0, 32, 64), (1, 128, 64), (2, 32, 64), (3, 128, 64)])
def test_accumulator_tile_roundtrips(lib, variant, rows, cols):
    # variants 0-1 hold the tile as row-major base tiles, 2-3 as column-major ones
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


def test_readme_example_gemm_is_exact_for_each_k_chunk(lib):
    # a wrong k assignment between the A and B fragments shows when only one 16-wide k block of
    # the 256 is non-zero: every such block must give the exact partial product
    g = torch.Generator().manual_seed(2)
    c = torch.full((128, 64), float("nan"), device=DEV)
    for blk in (0, 1, 6, 15):
        a = torch.zeros(128, 256)
        b = torch.randint(-3, 4, (64, 256), generator=g).float()
        a[:, 16 * blk:16 * blk + 16] = torch.randint(-3, 4, (128, 16), generator=g).float()
        a, b = a.half(), b.half()
        assert lib.tt_readme_gemm(a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.data_ptr()) == 0
        assert torch.equal(c.cpu(), N.gemm_ref(a, b)), blk


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 8, 9, 10])
def test_other_mma_atoms(lib, variant):
    # A [128, 192], B [192, 64]: bf16 / fp16 operands, fp32 / fp16 accumulators, row- and
    # column-major accumulator tiles, even and odd base-tile counts per chunk (16x16x32 pairs and a
    # 16x16x16 tail), square (0-4) and wide (8-10) operand tiles; integer data, so exact
    bf16 = variant in (0, 4, 8)
    half_acc = variant in (1, 9)
    g = torch.Generator().manual_seed(30 + variant)
    dt = torch.bfloat16 if bf16 else torch.float16
    a = torch.randint(-3, 4, (128, 192), generator=g).to(dt)
    b = torch.randint(-3, 4, (64, 192), generator=g).to(dt)
    c = torch.full((128, 64), float("nan"), device=DEV, dtype=torch.float16 if half_acc else torch.float32)
    assert lib.tt_atom_gemm(variant, a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.data_ptr()) == 0
    assert torch.equal(c.float().cpu(), N.gemm_ref(a, b))   # |C| <= 9 * 192 < 2048: exact in fp16 too
    # random data against the fp32 oracle
    a, b = oracle.make_c1_gemm_inputs(128, 64, 192, seed=40 + variant)
    a, b = a.to(dt), b.to(dt)
    assert lib.tt_atom_gemm(variant, a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.data_ptr()) == 0
    ref = N.gemm_ref(a, b)
    if half_acc:
        # the accumulator tile is rounded to fp16 once per gemm() call: a few fp16 ulps of |C| ~ 10
        assert N.rel_l2(c, ref) <= 2e-3 and N.max_abs(c, ref) <= 5e-2, (N.rel_l2(c, ref), N.max_abs(c, ref))
    else:
        ok, r, m = N.check_close(c, ref)
        assert ok and m < 1e-4, (r, m)


@pytest.mark.parametrize("variant", [0, 1])
def test_single_mma_atom_on_one_base_tile(lib, variant):
    # tests/cpp/cell/test_single_wmma.cu:222-231: one 16 x 16 x 16 atom against the naive loop
    dt = torch.float16 if variant == 0 else torch.bfloat16
    g = torch.Generator().manual_seed(50 + variant)
    a = torch.randint(-4, 5, (16, 16), generator=g).to(dt)
    b = torch.randint(-4, 5, (16, 16), generator=g).to(dt)   # [n, k] buffer = column-major k x n
    c = torch.full((16, 16), float("nan"), device=DEV)
    assert lib.tt_single_atom(variant, a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.data_ptr()) == 0
    assert torch.equal(c.cpu(), N.gemm_ref(a, b))


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


@pytest.mark.parametrize("variant", range(7))
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


# ---- asynchronous copies, Pipeline and the pipelined GEMMs ----------------------------------------

@pytest.mark.parametrize("variant", range(9))
def test_ke_gemm_level1_and_level2_pipelines(lib, variant):
    # variants 0-3 are the reference's cases 1-4 (tests/python/test_gemm.py:75-135): 64 x 64 x 64
    # tiles, level 1 with 2 ring slots, level 2 with 3; the others vary slots (2, 3, 4), register
    # steps per chunk (1, 2, 3), wavefront layouts and the output type
    m, n, k, h = (_i(), _i(), _i(), _i())
    lib.tt_ke_gemm_pipe_shape(variant, m, n, k, h)
    a, b = oracle.make_c1_gemm_inputs(m.value, n.value, k.value, seed=500 + variant)
    c = torch.full((m.value, n.value), float("nan"), device=DEV, dtype=torch.float16 if h.value else torch.float32)
    assert lib.tt_ke_gemm_pipe(variant, a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.data_ptr()) == 0
    ref = N.gemm_ref(a, b)
    assert N.rel_l2(c, ref) <= 1e-3 and N.max_abs(c, ref) <= 2e-2 * max(1.0, float(ref.abs().max()))
    # integer operands: the products and sums are exact in fp32, so any chunk read too early or
    # from the wrong ring slot shows as a wrong integer
    g = torch.Generator().manual_seed(variant)
    a = torch.randint(-2, 3, (m.value, k.value), generator=g).half()
    b = torch.randint(-2, 3, (n.value, k.value), generator=g).half()
    for _ in range(3):
        c.fill_(float("nan"))
        assert lib.tt_ke_gemm_pipe(variant, a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), c.data_ptr()) == 0
        assert torch.equal(c.float().cpu(), N.gemm_ref(a, b))


@pytest.mark.parametrize("variant", range(4))
def test_pipeline_ring_with_asynchronous_copies_is_exact(lib, variant):
    # 2, 3, 3 and 4 ring slots; stages - 1 chunks in flight, wait_group<stages - 2> per chunk
    r, c = _i(), _i()
    lib.tt_pipeline_shape(variant, r, c)
    n = r.value * c.value
    src = ((torch.arange(n) * 3 + variant) % 2048).half().to(DEV)
    for _ in range(3):
        dst = torch.full((n,), -1, dtype=torch.float16, device=DEV)
        err = torch.zeros(1, dtype=torch.int32, device=DEV)
        assert lib.tt_pipeline_roundtrip(variant, src.data_ptr(), dst.data_ptr(), err.data_ptr()) == 0
        assert int(err.item()) == 0          # get_dst_ptr_by_index / get_cur_dst / get_prev_dst
        assert torch.equal(src, dst)


def test_loader_fills_a_strided_subtile_through_registers(lib):
    src = (torch.arange(64 * 128) % 2048).half().reshape(64, 128)
    dst = torch.zeros(64, 128, dtype=torch.float16, device=DEV)
    assert lib.tt_g2s_subtile(src.to(DEV).data_ptr(), dst.data_ptr()) == 0
    want = torch.full((64, 128), -1.0, dtype=torch.float16)
    want[:, 64:] = src[:, 64:]
    assert torch.equal(dst.cpu(), want)


# ---- warp helpers ------------------------------------------------------------------------------------

@pytest.mark.parametrize("layout", range(4))
@pytest.mark.parametrize("mode", range(3))
def test_warp_offset_helpers_and_exec_counter(lib, layout, mode):
    # (wavefront grid, its order, tile layout, base tile) of tt_warp_helpers' four layouts
    wr, wc, wkind, tile, base = [
        (2, 2, L.ROW_MAJOR, L.row_major(128, 256, 512), (16, 32)),
        (4, 1, L.ROW_MAJOR, L.row_major(128, 64), (16, 32)),
        (2, 2, L.COL_MAJOR, L.col_major(128, 64, 256), (32, 16)),
        (2, 2, L.ROW_MAJOR, L.row_major(128, 256, 512), (16, 16)),
    ][layout]
    name = ["kCont", "kRowReuseCont", "kColReuseCont"][mode]
    out = torch.full((wr * wc, 6), -1, dtype=torch.int64, device=DEV)
    assert lib.tt_warp_helpers(layout, mode, out.data_ptr()) == 0
    got = out.cpu().tolist()
    rows, cols = L.warp_tile_shape(tile.rows, tile.cols, wr, wc, name)
    for wid in range(wr * wc):
        i, j = L.warp_coords(wid, wr, wc, wkind)
        off = L.warp_global_offset(tile, wr, wc, i, j, name)
        assert got[wid] == [i, j, off, off, rows // base[0], cols // base[1]], (wid, got[wid])


# ---- STileIterator2 -----------------------------------------------------------------------------------

def _stile2_case(variant):
    rm, cm = L.row_major, L.col_major
    B, S = L.BlockMatrixLayout, L.SwizzledLayout
    return [
        (rm(4, 24), 4, 8), (cm(24, 4), 8, 4),
        (B(rm(4, 16), rm(2, 4)), 4, 8), (B(cm(16, 4), cm(4, 2)), 8, 4),
        (B(rm(8, 16), S(rm(2, 4), 1, 0, 2)), 8, 4), (B(cm(32, 8), S(cm(4, 4), 2, 0, 2)), 8, 8),
        (B(rm(8, 16), rm(2, 4)), 4, 8), (rm(8, 16), 2, 4),
    ][variant]


@pytest.mark.parametrize("variant", range(8))
def test_stile_iterator2_subtiles_are_the_parents_elements(lib, variant):
    # the buffer holds its own index, so element (r, c) of sub-tile (x, y) must read
    # parent_layout(x * chunk_rows + r, y * chunk_cols + c); variants 0-5 are the layouts of
    # tests/cpp/types/test_stile_iterator.cu:48-236, 6-7 chunk in both dimensions
    layout, cr, cc = _stile2_case(variant)
    sc0, sc1 = layout.rows // cr, layout.cols // cc
    n = layout.rows * layout.cols
    outs = [torch.full((n,), -7.0, device=DEV) for _ in range(4)]
    assert lib.tt_stile_iterator2(variant, *[o.data_ptr() for o in outs]) == 0
    want = torch.tensor([layout(x * cr + r, y * cc + c) for x in range(sc0) for y in range(sc1)
                         for r in range(cr) for c in range(cc)], dtype=torch.float32)
    assert sorted(want.tolist()) == list(range(n))        # the layout is a bijection
    for o in outs[:3]:                                     # (x, y), (x, _)(y), (_, y)(x)
        assert torch.equal(o.cpu(), want)
    if sc0 == 1 or sc1 == 1:                               # single-index form
        assert torch.equal(outs[3].cpu(), want)


# ---- register copies, vector moves, remaining functors ----------------------------------------------

def test_reg_tile_copy_and_base_tile_copy(lib):
    src = torch.arange(32 * 64, dtype=torch.float32).reshape(32, 64)
    whole = torch.full((32, 64), -1.0, device=DEV)
    one = torch.full((32, 64), -1.0, device=DEV)
    assert lib.tt_reg_copy(src.to(DEV).data_ptr(), whole.data_ptr(), one.data_ptr()) == 0
    assert torch.equal(whole.cpu(), src)
    want = torch.zeros(32, 64)
    want[16:32, 32:48] = src[16:32, 32:48]                # base tile (1, 2) of the 2 x 4 grid
    assert torch.equal(one.cpu(), want)


def test_vectorize_moves_32_64_128_bits(lib):
    h = (torch.arange(896) % 2048).half().to(DEV)
    f = torch.arange(384, dtype=torch.float32, device=DEV)
    ho, fo = torch.full_like(h, -1), torch.full_like(f, -1)
    assert lib.tt_vectorize(h.data_ptr(), ho.data_ptr(), f.data_ptr(), fo.data_ptr()) == 0
    assert torch.equal(h, ho) and torch.equal(f, fo)


def test_remaining_broadcast_and_map_functors(lib):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((64, 32)).astype(np.float32)
    y = rng.standard_normal((64, 32)).astype(np.float32)
    outs = [torch.zeros(64, 32, device=DEV) for _ in range(7)]
    xd, yd = torch.from_numpy(x).to(DEV), torch.from_numpy(y).to(DEV)
    assert lib.tt_functors(xd.data_ptr(), yd.data_ptr(), *[o.data_ptr() for o in outs]) == 0
    o_add, o_log, o_min, o_div, o_max, o_mul, o_sub = [o.cpu().numpy() for o in outs]
    rs = x.sum(axis=1, keepdims=True)
    assert np.allclose(o_add, x + rs, atol=1e-5)                        # BroadcastAdd
    assert np.allclose(o_mul, x * rs, atol=1e-4)                        # BroadcastMul
    assert np.allclose(o_log, np.log(np.maximum(x, 0) + 1), atol=1e-5)  # Relu, scalar Add, Log
    assert np.array_equal(o_min, np.minimum(x, y)) and np.array_equal(o_max, np.maximum(x, y))
    assert np.array_equal(o_sub, x - y)
    assert np.allclose(o_div, x / (y * y + 1), rtol=1e-6, atol=1e-7)    # Mul, scalar Add, Div
