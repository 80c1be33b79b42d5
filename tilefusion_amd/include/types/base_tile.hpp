// Per-wavefront copy atom inference (counterpart of include/types/base_tile.hpp:28-115) for
// 64 lanes: every lane moves one 128-bit vector, lanes first fill the contiguous dimension
// (at most one 128-byte line), the remaining lanes stack along the strided dimension.
#pragma once

#include "types/layout.hpp"
#include "types/tile_shape.hpp"

namespace tilefusion {
namespace tl = tile_layout;

template <typename DType, typename TileShape, tl::Layout kType, int kWarpSize_ = WARP_SIZE>
struct WarpBaseTileShape;

template <typename DType, typename TileShape, int kWarpSize_>
struct WarpBaseTileShape<DType, TileShape, tl::Layout::kRowMajor, kWarpSize_> {
  using AccessInfo = AccessBase<DType>;
  static constexpr int kTileRows = dim_size<0, TileShape>;
  static constexpr int kTileCols = dim_size<1, TileShape>;
  static_assert(kTileCols >= AccessInfo::kNumPerAccess, "the tile is narrower than one 128-bit access");
  static_assert(kTileCols < AccessInfo::kExpectedSize || kTileCols % AccessInfo::kExpectedSize == 0,
                "wide tiles must be a whole number of 128-byte lines");
  static constexpr int kCols = kTileCols >= AccessInfo::kExpectedSize ? AccessInfo::kExpectedSize : kTileCols;
  static constexpr int kColThreads = kCols / AccessInfo::kNumPerAccess;
  static_assert(kWarpSize_ % kColThreads == 0, "cannot arrange the lanes over this tile");
  static constexpr int kRowThreads = kWarpSize_ / kColThreads;
  static constexpr int kRows = kRowThreads;
  static_assert(kTileRows % kRowThreads == 0, "tile rows must be a multiple of the lane rows");
  static constexpr tl::Layout kType = tl::Layout::kRowMajor;
  static constexpr int kNumel = kRows * kCols;
  using WarpThreadLayout = tl::RowMajor<kRowThreads, kColThreads>;
};

template <typename DType, typename TileShape, int kWarpSize_>
struct WarpBaseTileShape<DType, TileShape, tl::Layout::kColMajor, kWarpSize_> {
  using AccessInfo = AccessBase<DType>;
  static constexpr int kTileRows = dim_size<0, TileShape>;
  static constexpr int kTileCols = dim_size<1, TileShape>;
  static_assert(kTileRows >= AccessInfo::kNumPerAccess, "the tile is shorter than one 128-bit access");
  static_assert(kTileRows < AccessInfo::kExpectedSize || kTileRows % AccessInfo::kExpectedSize == 0,
                "tall tiles must be a whole number of 128-byte lines");
  static constexpr int kRows = kTileRows >= AccessInfo::kExpectedSize ? AccessInfo::kExpectedSize : kTileRows;
  static constexpr int kRowThreads = kRows / AccessInfo::kNumPerAccess;
  static_assert(kWarpSize_ % kRowThreads == 0, "cannot arrange the lanes over this tile");
  static constexpr int kColThreads = kWarpSize_ / kRowThreads;
  static constexpr int kCols = kColThreads;
  static_assert(kTileCols % kColThreads == 0, "tile columns must be a multiple of the lane columns");
  static constexpr tl::Layout kType = tl::Layout::kColMajor;
  static constexpr int kNumel = kRows * kCols;
  using WarpThreadLayout = tl::ColMajor<kRowThreads, kColThreads>;
};

template <typename DType, typename TileShape, tl::Layout kType, int kW>
HOST std::ostream& operator<<(std::ostream& out, const WarpBaseTileShape<DType, TileShape, kType, kW>&) {
  using W = WarpBaseTileShape<DType, TileShape, kType, kW>;
  return out << "BaseShape = (" << W::kRows << ", " << W::kCols << "), Numel = " << W::kNumel
             << ", ThreadLayout = (" << W::kRowThreads << ", " << W::kColThreads << ")";
}

}  // namespace tilefusion
