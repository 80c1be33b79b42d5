// Where a wavefront sits in the workgroup's WarpLayout and which part of a tile it owns
// (counterpart of include/cell/copy/warp.hpp:65-300).
#pragma once

#include <cstddef>

#include "cell/copy/constants.hpp"
#include "types/layout.hpp"
#include "types/tile_shape.hpp"

namespace tilefusion::cell::copy::warp {
namespace tl = tile_layout;

DEVICE int warp_id() { return threadIdx.x / WARP_SIZE; }
DEVICE int lane_id() { return threadIdx.x % WARP_SIZE; }

// wavefront ids run along rows of a row-major WarpLayout and along columns of a column-major one
template <typename WarpLayout>
DEVICE int warp_row_id() {
  return tl::layout_type<WarpLayout> == tl::Layout::kRowMajor ? warp_id() / (int)tl::num_cols<WarpLayout>
                                                              : warp_id() % (int)tl::num_rows<WarpLayout>;
}
template <typename WarpLayout>
DEVICE int warp_col_id() {
  return tl::layout_type<WarpLayout> == tl::Layout::kRowMajor ? warp_id() % (int)tl::num_cols<WarpLayout>
                                                              : warp_id() / (int)tl::num_rows<WarpLayout>;
}

template <int kTileRows, int kWarpRows, WarpReuse kMode = WarpReuse::kCont>
HOST_DEVICE constexpr int warp_tile_rows() {
  return kMode == WarpReuse::kColReuseCont ? kTileRows : kTileRows / kWarpRows;
}
template <int kTileCols, int kWarpCols, WarpReuse kMode = WarpReuse::kCont>
HOST_DEVICE constexpr int warp_tile_cols() {
  return kMode == WarpReuse::kRowReuseCont ? kTileCols : kTileCols / kWarpCols;
}

// How many base tiles a wavefront walks over in each dimension.
template <typename BaseShape_, typename Tile_, typename WarpLayout_, WarpReuse kMode_>
struct ExecCounter {
  using BaseShape = BaseShape_;
  using Tile = Tile_;
  static constexpr WarpReuse kMode = kMode_;
  static_assert(Tile::kRows % BaseShape::kRows == 0 && Tile::kCols % BaseShape::kCols == 0,
                "the tile must be a whole number of base tiles");
  static constexpr int kRowExec =
      warp_tile_rows<Tile::kRows, tl::num_rows<WarpLayout_>, kMode>() / BaseShape::kRows;
  static constexpr int kColExec =
      warp_tile_cols<Tile::kCols, tl::num_cols<WarpLayout_>, kMode>() / BaseShape::kCols;
  DEVICE static constexpr int row_exec_count() { return kRowExec; }
  DEVICE static constexpr int col_exec_count() { return kColExec; }
};

// (row, col) of the first element of this wavefront's share of `Tile`, in elements: with kCont
// wavefront (i, j) owns block (i, j); with kRowReuseCont the wavefronts of row i share row block
// i and start at column 0; with kColReuseCont those of column j share column block j and start
// at row 0 (include/cell/copy/warp.hpp:20-47,206-231).
template <typename WarpLayout, WarpReuse kMode, typename Tile>
DEVICE void warp_origin(int& row, int& col) {
  constexpr int kRowsPerWarp = Tile::kRows / (int)tl::num_rows<WarpLayout>;
  constexpr int kColsPerWarp = Tile::kCols / (int)tl::num_cols<WarpLayout>;
  row = kMode == WarpReuse::kColReuseCont ? 0 : warp_row_id<WarpLayout>() * kRowsPerWarp;
  col = kMode == WarpReuse::kRowReuseCont ? 0 : warp_col_id<WarpLayout>() * kColsPerWarp;
}

// Element offset of this wavefront's share inside a global tile (64-bit: a global tile may span
// more than 2^31 elements).  Used by the global <-> register movers.
template <typename WarpLayout_, WarpReuse kMode_>
struct GlobalOffsetHelper {
  using WarpLayout = WarpLayout_;
  static constexpr WarpReuse kMode = kMode_;
  template <typename Tile>
  DEVICE ptrdiff_t get_warp_offset() const {
    int r, c;
    warp_origin<WarpLayout, kMode, Tile>(r, c);
    return ptrdiff_t(r) * Tile::kRowStride + ptrdiff_t(c) * Tile::kColStride;
  }
};

// Logical element offset of this wavefront's share inside an LDS tile, to be passed through
// SharedTile::fetch_physical_offset together with the in-share offset.  Used by the LDS <->
// register movers.
template <typename WarpLayout_, typename BaseShape_, typename Shared_, WarpReuse kMode_>
struct SharedOffsetHelper {
  using WarpLayout = WarpLayout_;
  using BaseShape = BaseShape_;
  using Shared = Shared_;
  static constexpr WarpReuse kMode = kMode_;
  DEVICE int get_warp_offset() const {
    int r, c;
    warp_origin<WarpLayout, kMode, Shared>(r, c);
    return r * Shared::kRowStride + c * Shared::kColStride;
  }
};

}  // namespace tilefusion::cell::copy::warp
