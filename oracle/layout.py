"""Integer restatements of the reference's tile-layout arithmetic (TEST INFRASTRUCTURE).

Pure-Python / numpy closed forms of the compile-time index maps on the hot path.  Each
function cites the reference lines it follows; tests/test_oracle_layout.py pins them against
the reference's own integer known answers, and tests/test_types_host.py then checks the C++
headers under tilefusion_amd/include against these functions.
"""

from dataclasses import dataclass

ROW_MAJOR = "RowMajor"
COL_MAJOR = "ColMajor"


@dataclass(frozen=True)
class MatrixLayout:
    """(i, j) -> i*row_stride + j*col_stride; include/types/layout.hpp:49-66.
    The layout type is deduced from col_stride == 1 (layout.hpp:52-53), so ColMajor<1,1>
    reads as row-major."""

    rows: int
    cols: int
    row_stride: int
    col_stride: int

    @property
    def kind(self):
        return ROW_MAJOR if self.col_stride == 1 else COL_MAJOR

    @property
    def numel(self):
        return self.rows * self.cols

    def __call__(self, i, j):
        return i * self.row_stride + j * self.col_stride

    @property
    def contiguous(self):
        # include/types/layout.hpp:121-127
        if self.kind == ROW_MAJOR:
            return self.row_stride == self.cols and self.col_stride == 1
        return self.col_stride == self.rows and self.row_stride == 1


def row_major(rows, cols, stride=None):
    """include/types/layout.hpp:81-82"""
    return MatrixLayout(rows, cols, cols if stride is None else stride, 1)


def col_major(rows, cols, stride=None):
    """include/types/layout.hpp:86-87"""
    return MatrixLayout(rows, cols, 1, rows if stride is None else stride)


class BlockMatrixLayout:
    """Two-level layout: a grid of inner tiles; include/types/layout.hpp:129-194."""

    def __init__(self, outer: MatrixLayout, inner):
        assert outer.rows % inner.rows == 0 and outer.cols % inner.cols == 0
        self.outer, self.inner = outer, inner
        self.rows, self.cols = outer.rows, outer.cols
        self.tile_rows = outer.rows // inner.rows
        self.tile_cols = outer.cols // inner.cols
        inner_numel = inner.rows * inner.cols
        self.kind = outer.kind
        is_row = outer.kind == ROW_MAJOR
        if outer.contiguous:  # layout.hpp:156-161
            self.row_stride = self.tile_cols * inner_numel if is_row else inner_numel
            self.col_stride = inner_numel if is_row else self.tile_rows * inner_numel
        else:
            self.row_stride, self.col_stride = outer.row_stride, outer.col_stride

    def __call__(self, i, j):
        oi, ii = divmod(i, self.inner.rows)
        oj, ij = divmod(j, self.inner.cols)
        return oi * self.row_stride + oj * self.col_stride + self.inner(ii, ij)


def swizzle(idx, b, m, s):
    """Swizzle<B,M,S>: XOR the S 'chunk' bits with the B row bits above the M low bits;
    include/types/swizzle.hpp:28-42."""
    bs = idx >> m
    y = bs & ((1 << s) - 1)
    x = bs >> s
    return (x << (m + s)) | ((x ^ y) << m) | (idx & ((1 << m) - 1))


class SwizzledLayout:
    """Layout composed with a swizzle; include/types/swizzle.hpp:63-143."""

    def __init__(self, layout: MatrixLayout, b, m, s):
        self.layout, self.b, self.m, self.s = layout, b, m, s
        self.rows, self.cols = layout.rows, layout.cols
        self.kind = layout.kind
        if self.kind == ROW_MAJOR:
            assert layout.rows == 1 << b and layout.cols == 1 << (m + s)
        else:
            assert layout.cols == 1 << b and layout.rows == 1 << (m + s)

    def __call__(self, x, y):
        ms = self.m + self.s
        if self.kind == ROW_MAJOR:  # swizzle.hpp:90-97
            sw = swizzle((x << ms) | y, self.b, self.m, self.s)
            return self.layout(sw >> ms, sw & ((1 << ms) - 1))
        # swizzle.hpp:131-138 (note: shifts by B+M there; identical when B == S)
        sw = swizzle((y << (self.b + self.m)) | x, self.b, self.m, self.s)
        return self.layout(sw & ((1 << ms) - 1), sw >> ms)


def swizzle_base_tile_shape(elem_bytes, swizzle_bytes):
    """(rows, cols, B, M, S); include/types/swizzle.hpp:158-214."""
    table = {
        (2, 128): (8, 64, 3, 3, 3),
        (4, 128): (8, 32, 3, 2, 3),
        (2, 64): (4, 32, 2, 3, 2),
        (4, 64): (4, 16, 2, 2, 2),
    }
    return table[(elem_bytes, swizzle_bytes)]


def shared_physical_offset(offset, layout: MatrixLayout, elem_bytes, swizzled, swizzle_bytes=128):
    """SharedTile::fetch_physical_offset; include/types/shared.hpp:107-149."""
    sr, sc, b, m, s = swizzle_base_tile_shape(elem_bytes, swizzle_bytes)
    is_row = layout.kind == ROW_MAJOR
    if not is_row:
        sr, sc = sc, sr
    if is_row:
        row, col = offset // layout.row_stride, offset % layout.row_stride
        in_tile = MatrixLayout(sr, sc, layout.row_stride, 1)
        tiles = MatrixLayout(layout.rows // sr, layout.cols // sc, layout.row_stride * sr, sc)
    else:
        row, col = offset % layout.col_stride, offset // layout.col_stride
        in_tile = MatrixLayout(sr, sc, 1, layout.col_stride)
        tiles = MatrixLayout(layout.rows // sr, layout.cols // sc, sr, layout.col_stride * sc)
    tile_off = tiles(row // sr, col // sc)
    ir, ic = row % sr, col % sc
    if swizzled:
        return tile_off + SwizzledLayout(in_tile, b, m, s)(ir, ic)
    return tile_off + in_tile(ir, ic)


def gtile_chunk_offset(layout: MatrixLayout, chunk, x, y):
    """Offset of chunk (x, y) of a GTileIterator and the chunk's layout;
    include/types/global_tile_iterator.hpp:63-102."""
    c0, c1 = chunk
    if layout.kind == ROW_MAJOR:
        off = x * (c0 * layout.row_stride) + y * c1
    else:
        off = x * c0 + y * (layout.col_stride * c1)
    return off, MatrixLayout(c0, c1, layout.row_stride, layout.col_stride)


def gtile_strip_counts(layout: MatrixLayout, chunk):
    """(sc0, sc1); include/types/global_tile_iterator.hpp:49-50."""
    return layout.rows // chunk[0], layout.cols // chunk[1]


def warp_base_tile_shape(elem_bytes, tile_rows, tile_cols, kind, warp_size):
    """WarpBaseTileShape: per-wavefront copy atom (rows, cols, row_threads, col_threads);
    include/types/base_tile.hpp:28-115 with AccessBase (include/types/base.hpp:42-59):
    128-bit accesses, a 1024-bit contiguous run per group of lanes."""
    per_access = 16 // elem_bytes
    expected = 128 // elem_bytes
    if kind == ROW_MAJOR:
        assert tile_cols >= per_access
        assert tile_cols < expected or tile_cols % expected == 0
        cols = expected if tile_cols >= expected else tile_cols
        col_threads = cols // per_access
        assert warp_size % col_threads == 0
        row_threads = warp_size // col_threads
        assert tile_rows % row_threads == 0
        return row_threads, cols, row_threads, col_threads
    assert tile_rows >= per_access
    assert tile_rows < expected or tile_rows % expected == 0
    rows = expected if tile_rows >= expected else tile_rows
    row_threads = rows // per_access
    assert warp_size % row_threads == 0
    col_threads = warp_size // row_threads
    assert tile_cols % col_threads == 0
    return rows, col_threads, row_threads, col_threads


def warp_coords(wid, warp_rows, warp_cols, kind=ROW_MAJOR):
    """(warp_row, warp_col) of wavefront `wid`; include/cell/copy/warp.hpp:82-92,119-129."""
    if kind == ROW_MAJOR:
        return wid // warp_cols, wid % warp_cols
    return wid % warp_rows, wid // warp_rows


def warp_global_offset(layout: MatrixLayout, warp_rows, warp_cols, wr, wc, mode):
    """Start offset of a wavefront's share of a global tile for the three WarpReuse modes
    (include/cell/copy/constants.hpp:7-14; include/cell/copy/warp.hpp:20-47,206-231)."""
    shape_r, shape_c = layout.rows // warp_rows, layout.cols // warp_cols
    if layout.kind == ROW_MAJOR:
        rs, cs = layout.row_stride * shape_r, shape_c
    else:
        rs, cs = shape_r, layout.col_stride * shape_c
    if mode == "kCont":
        return wr * rs + wc * cs
    if mode == "kRowReuseCont":
        return wr * rs
    if mode == "kColReuseCont":
        return wc * cs
    raise ValueError(mode)


def warp_tile_shape(rows, cols, warp_rows, warp_cols, mode):
    """(rows, cols) of the share one wavefront owns; include/cell/copy/warp.hpp:132-156."""
    if mode == "kCont":
        return rows // warp_rows, cols // warp_cols
    if mode == "kRowReuseCont":
        return rows // warp_rows, cols
    if mode == "kColReuseCont":
        return rows, cols // warp_cols
    raise ValueError(mode)


# --- CDNA4 MFMA fragment maps (no reference counterpart: the reference's are for
# mma.m16n8k16, include/cell/copy/global_to_register.hpp:40-55).  Verified on hardware by
# the one-tile known-answer GPU test. -------------------------------------------------------

def mfma_32x32x16_ab(lane, t):
    """A/B operand element t (0..7) of lane: (row-or-col, k)."""
    return lane % 32, 8 * (lane // 32) + t


def mfma_32x32x16_c(lane, r):
    """Accumulator register r (0..15) of lane: (row, col)."""
    return 8 * (r // 4) + 4 * (lane // 32) + r % 4, lane % 32


def mfma_16x16x32_ab(lane, t):
    return lane % 16, 8 * (lane // 16) + t


def mfma_16x16x32_c(lane, r):
    return 4 * (lane // 16) + r, lane % 16


# --- base-tile lane maps of the tile API on a 64-lane wavefront (the reference's are for the
# 32-thread mma.m16n8k16 fragments, include/cell/copy/global_to_register.hpp:40-55).  A base tile
# covers the reference's 16 x 16 block (include/types/base.hpp:62-68); `per_lane` is 4 for it and
# 8 for the wide 16 x 32 / 32 x 16 operand block. ---------------------------------------------

def base_tile_coord(lane, e, row_major, per_lane=4):
    """(row, col) inside the block of per-lane element e: a row-major base tile gives lane l the
    columns per_lane*(l//16).. of row l%16, a column-major one the rows per_lane*(l//16).. of
    column l%16."""
    if row_major:
        return lane % 16, per_lane * (lane // 16) + e
    return per_lane * (lane // 16) + e, lane % 16


def base_tile_shape(row_major, per_lane=4):
    """(rows, cols) of the block one base tile covers."""
    return (16, 4 * per_lane) if row_major else (4 * per_lane, 16)


def paired_k_assignment(lane, e):
    """k index (0..31) that element e (0..7) of the 8-element operand fragment built from two
    square base tiles adjacent in k carries: elements 0-3 come from the first tile."""
    return 16 * (e // 4) + 4 * (lane // 16) + e % 4
