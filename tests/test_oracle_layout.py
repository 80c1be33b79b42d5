"""Pins oracle/layout.py against the reference's own integer known answers."""

import pytest

from oracle import layout as L


def test_matrix_layout_known_answers():
    # tests/cpp/types/test_layout.cu:12-38
    l1 = L.row_major(4, 7)
    assert (l1.rows, l1.cols, l1.numel, l1.row_stride, l1.col_stride, l1.kind) == (4, 7, 28, 7, 1, "RowMajor")
    l2 = L.col_major(4, 7)
    assert (l2.rows, l2.cols, l2.numel, l2.row_stride, l2.col_stride, l2.kind) == (4, 7, 28, 1, 4, "ColMajor")


def test_block_row_major_known_answers():
    # tests/cpp/types/test_layout.cu:40-60
    b = L.BlockMatrixLayout(L.row_major(14, 9), L.row_major(2, 3))
    assert (b.tile_rows, b.tile_cols, b.row_stride, b.col_stride, b.kind) == (7, 3, 18, 6, "RowMajor")
    assert [b(2, 0), b(2, 1), b(4, 3), b(4, 4)] == [18, 19, 42, 43]


def test_block_col_major_known_answers():
    # tests/cpp/types/test_layout.cu:62-82
    b = L.BlockMatrixLayout(L.col_major(14, 9), L.col_major(2, 3))
    assert (b.tile_rows, b.tile_cols, b.row_stride, b.col_stride, b.kind) == (7, 3, 6, 42, "ColMajor")
    assert [b(6, 0), b(7, 0), b(0, 3), b(1, 3)] == [18, 19, 42, 43]


def test_block_mixed_known_answers():
    # tests/cpp/types/test_layout.cu:84-120
    b = L.BlockMatrixLayout(L.row_major(14, 9), L.col_major(2, 3))
    assert (b.tile_rows, b.tile_cols, b.row_stride, b.col_stride, b.kind) == (7, 3, 18, 6, "RowMajor")
    assert [b(2, 0), b(3, 0), b(4, 3), b(5, 3)] == [18, 19, 42, 43]
    b = L.BlockMatrixLayout(L.col_major(14, 9), L.row_major(2, 3))
    assert (b.tile_rows, b.tile_cols, b.row_stride, b.col_stride, b.kind) == (7, 3, 6, 42, "ColMajor")
    assert [b(6, 0), b(6, 1), b(0, 3), b(0, 4)] == [18, 19, 42, 43]


def _swizzle_ref(x, y, b, m, s):
    # closed form of tests/cpp/types/test_swizzle.cu:19-29
    sw = x ^ (y >> m)
    return (x << (m + s)) | (sw << m) | (y & ((1 << m) - 1))


@pytest.mark.parametrize("bms", [(3, 3, 3), (2, 3, 2), (3, 2, 3), (2, 2, 2)])
def test_swizzle_function(bms):
    b, m, s = bms
    # the five points of tests/cpp/types/test_swizzle.cu:48-64 plus the whole domain
    for x, y in [(0, 0), (1, 0), (1, 4), (2, 0), (2, 4)]:
        assert L.swizzle(x * (1 << (m + s)) + y, b, m, s) == _swizzle_ref(x, y, b, m, s)
    seen = set()
    for x in range(1 << b):
        for y in range(1 << (m + s)):
            v = L.swizzle((x << (m + s)) | y, b, m, s)
            assert v == _swizzle_ref(x, y, b, m, s)
            seen.add(v)
    assert len(seen) == 1 << (b + m + s)  # a permutation


def test_swizzled_row_major_matches_cute_closed_form():
    # tests/cpp/types/test_swizzle.cu:66-86; the CuTe side composition(Swizzle<3,3,3>,
    # (8,64):(64,1)) tiled to (16,64) has the closed form idx ^ (((idx >> 6) & 7) << 3).
    lay = L.BlockMatrixLayout(L.row_major(16, 64), L.SwizzledLayout(L.row_major(8, 64), 3, 3, 3))
    for i in range(16):
        for j in range(64):
            idx = i * 64 + j
            assert lay(i, j) == idx ^ (((idx >> 6) & 7) << 3)


def test_swizzled_col_major_matches_cute_closed_form():
    # tests/cpp/types/test_swizzle.cu:88-105 (col-major 64 x 16, atom (64,8):(1,64))
    lay = L.BlockMatrixLayout(L.col_major(64, 16), L.SwizzledLayout(L.col_major(64, 8), 3, 3, 3))
    for i in range(64):
        for j in range(16):
            idx = j * 64 + i
            assert lay(i, j) == idx ^ (((idx >> 6) & 7) << 3)


@pytest.mark.parametrize("kind", ["RowMajor", "ColMajor"])
def test_gtile_iterator_known_answers(kind):
    # tests/cpp/types/test_gtile_iterator.cu:146-158: 4x9 tile in 2x3 chunks; every element
    # of chunk (i,j) equals start + m*rowstride + n (row-major) / start + m + n*colstride.
    lay = L.row_major(4, 9) if kind == "RowMajor" else L.col_major(4, 9)
    sc0, sc1 = L.gtile_strip_counts(lay, (2, 3))
    assert (sc0, sc1) == (2, 3)
    for i in range(sc0):
        for j in range(sc1):
            off, sub = L.gtile_chunk_offset(lay, (2, 3), i, j)
            if kind == "RowMajor":
                start = i * 2 * lay.row_stride + j * 3
            else:
                start = i * 2 + j * 3 * lay.col_stride
            assert off == start
            for m in range(2):
                for n in range(3):
                    assert off + sub(m, n) == lay(i * 2 + m, j * 3 + n)


# (elem_bytes, kind, tile, expected (rows, cols, row_threads, col_threads)) at 32 lanes:
# tests/cpp/types/test_warp_base_tile_shape.cu:10-188
_WBT_32 = [
    (2, "RowMajor", (128, 8), (32, 8, 32, 1)),
    (2, "RowMajor", (64, 16), (16, 16, 16, 2)),
    (2, "RowMajor", (16, 32), (8, 32, 8, 4)),
    (2, "RowMajor", (128, 128), (4, 64, 4, 8)),
    (2, "ColMajor", (8, 128), (8, 32, 1, 32)),
    (2, "ColMajor", (16, 64), (16, 16, 2, 16)),
    (2, "ColMajor", (32, 16), (32, 8, 4, 8)),
    (2, "ColMajor", (128, 128), (64, 4, 8, 4)),
    (4, "RowMajor", (128, 4), (32, 4, 32, 1)),
    (4, "RowMajor", (64, 8), (16, 8, 16, 2)),
    (4, "RowMajor", (16, 16), (8, 16, 8, 4)),
    (4, "RowMajor", (128, 128), (4, 32, 4, 8)),
    (4, "ColMajor", (4, 128), (4, 32, 1, 32)),
    (4, "ColMajor", (8, 64), (8, 16, 2, 16)),
    (4, "ColMajor", (16, 32), (16, 8, 4, 8)),
    (4, "ColMajor", (128, 128), (32, 4, 8, 4)),
]


@pytest.mark.parametrize("eb,kind,tile,want", _WBT_32)
def test_warp_base_tile_shape_reference_answers(eb, kind, tile, want):
    assert L.warp_base_tile_shape(eb, tile[0], tile[1], kind, 32) == want


def test_warp_base_tile_shape_wave64():
    # Same inference with 64 lanes: the strided dimension doubles.
    assert L.warp_base_tile_shape(2, 128, 128, "RowMajor", 64) == (8, 64, 8, 8)
    assert L.warp_base_tile_shape(2, 128, 128, "ColMajor", 64) == (64, 8, 8, 8)
    assert L.warp_base_tile_shape(4, 128, 128, "RowMajor", 64) == (8, 32, 8, 8)
    assert L.warp_base_tile_shape(2, 64, 16, "RowMajor", 64) == (32, 16, 32, 2)


def test_shared_physical_offset_is_bank_permutation():
    # include/types/shared.hpp:118-149: within each 8-row band the 16-byte chunk index inside a
    # 64-half column block is XORed with row % 8 (128-byte swizzle, fp16).
    lay = L.row_major(16, 128)
    seen = set()
    for r in range(16):
        for c in range(128):
            p = L.shared_physical_offset(lay(r, c), lay, 2, True, 128)
            chunk, blk = (c % 64) // 8, c // 64
            assert p == r * 128 + blk * 64 + ((chunk ^ (r % 8)) * 8) + c % 8
            seen.add(p)
            assert L.shared_physical_offset(lay(r, c), lay, 2, False, 128) == lay(r, c)
    assert seen == set(range(16 * 128))
    lay = L.row_major(8, 64)
    for r in range(8):
        for c in range(64):
            p = L.shared_physical_offset(lay(r, c), lay, 2, True, 64)
            chunk, blk = (c % 32) // 8, c // 32
            assert p == r * 64 + blk * 32 + ((chunk ^ (r % 4)) * 8) + c % 8


def test_warp_coords_and_reuse_offsets():
    # include/cell/copy/warp.hpp:65-130 (threadIdx 67 examples use 32 lanes: wid 2)
    assert L.warp_coords(2, 2, 2, "RowMajor") == (1, 0)
    assert L.warp_coords(2, 2, 2, "ColMajor") == (0, 1)
    lay = L.row_major(128, 32, 256)
    # 2x2 wavefronts: kCont -> own block; row reuse -> all columns of row block; col reuse
    assert L.warp_global_offset(lay, 2, 2, 1, 1, "kCont") == 64 * 256 + 16
    assert L.warp_global_offset(lay, 2, 2, 1, 1, "kRowReuseCont") == 64 * 256
    assert L.warp_global_offset(lay, 2, 2, 1, 1, "kColReuseCont") == 16
    assert L.warp_tile_shape(128, 32, 2, 2, "kRowReuseCont") == (64, 32)
    assert L.warp_tile_shape(128, 32, 2, 2, "kColReuseCont") == (128, 16)
    assert L.warp_tile_shape(128, 32, 2, 2, "kCont") == (64, 16)


def test_mfma_fragment_maps_cover_tiles():
    for ab, c, m, k, nreg in [(L.mfma_32x32x16_ab, L.mfma_32x32x16_c, 32, 16, 16),
                              (L.mfma_16x16x32_ab, L.mfma_16x16x32_c, 16, 32, 4)]:
        assert {ab(l, t) for l in range(64) for t in range(8)} == {(i, kk) for i in range(m) for kk in range(k)}
        assert {c(l, r) for l in range(64) for r in range(nreg)} == {(i, j) for i in range(m) for j in range(m)}


def test_golden_fixture():
    # tests/golden/layout_known_answers.json: the reference's asserted integers, as data
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "layout_known_answers.json")) as f:
        g = json.load(f)
    mk = {"RowMajor": L.row_major, "ColMajor": L.col_major}
    for m in g["matrix_layouts"]:
        lay = mk[m["kind"]](m["rows"], m["cols"])
        assert (lay.numel, lay.row_stride, lay.col_stride, lay.kind) == (m["numel"], m["row_stride"], m["col_stride"], m["kind"])
    for b in g["block_layouts"]:
        lay = L.BlockMatrixLayout(mk[b["outer"][0]](*b["outer"][1:]), mk[b["inner"][0]](*b["inner"][1:]))
        assert (lay.tile_rows, lay.tile_cols, lay.row_stride, lay.col_stride, lay.kind) == (
            b["tile_rows"], b["tile_cols"], b["row_stride"], b["col_stride"], b["kind"])
        for i, j, off in b["samples"]:
            assert lay(i, j) == off
    for x, y, want in g["swizzle_3_3_3_points"]:
        assert L.swizzle(x * 64 + y, 3, 3, 3) == want


def test_base_tile_lane_maps_cover_their_blocks():
    # every element of the 16 x 16 (wide: 16 x 32 / 32 x 16) block is held by exactly one
    # (lane, element) pair, for both orientations
    for row_major in (True, False):
        for per_lane in (4, 8):
            rows, cols = L.base_tile_shape(row_major, per_lane)
            seen = {L.base_tile_coord(lane, e, row_major, per_lane) for lane in range(64) for e in range(per_lane)}
            assert seen == {(r, c) for r in range(rows) for c in range(cols)}
    # the square row-major tile is the transpose of the square column-major one, lane for lane
    for lane in range(64):
        for e in range(4):
            r, c = L.base_tile_coord(lane, e, True)
            assert L.base_tile_coord(lane, e, False) == (c, r)


def test_paired_square_tiles_feed_one_32_deep_instruction_consistently():
    # two square base tiles adjacent in k, concatenated per lane, must give every k of the 32 to
    # exactly one (lane group, element) slot, and A and B (same map) meet on equal k
    for row in range(16):
        ks = sorted(L.paired_k_assignment(row + 16 * g, e) for g in range(4) for e in range(8))
        assert ks == list(range(32))
