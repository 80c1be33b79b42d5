// Masks on an accumulator register tile (counterpart of include/cell/mask.hpp:9-113).
// kCausal writes `mask_value` wherever the GLOBAL column index exceeds the global row index.
// For the row-major MFMA accumulator layout, element r of base tile (m, n) of lane l is
//   row = row_offset + warp_row * (tile rows) + 16*m + 4*(l/16) + r
//   col = col_offset + warp_col * (tile cols) + 16*n + l%16.
#pragma once

#include "cell/copy/warp.hpp"
#include "types/register.hpp"

namespace tilefusion::cell {
namespace tl = tile_layout;

enum class MaskMode { kNone = 0, kCausal = 1, kCustom = 2 };

template <typename RegTile, typename WarpLayout, typename BaseShape, MaskMode kMode>
struct ApplyMask {
  template <typename Element>
  DEVICE void operator()(RegTile&, int, int, Element) {}
};

template <typename RegTile, typename WarpLayout, typename BaseShape>
struct ApplyMask<RegTile, WarpLayout, BaseShape, MaskMode::kCausal> {
  using BaseTile = typename RegTile::DType;
  static_assert(BaseTile::kNumel == 4 && BaseTile::kType == tl::Layout::kRowMajor,
                "the causal mask works on row-major accumulator base tiles");

  template <typename Element>
  DEVICE void operator()(RegTile& tile, const int row_offset, const int col_offset, Element mask_value) {
    const int lane = copy::warp::lane_id();
    const int row0 = row_offset + copy::warp::warp_row_id<WarpLayout>() * RegTile::kRows * 16 + 4 * (lane / 16);
    const int col0 = col_offset + copy::warp::warp_col_id<WarpLayout>() * RegTile::kCols * 16 + lane % 16;
#pragma unroll
    for (int m = 0; m < RegTile::kRows; ++m)
#pragma unroll
      for (int n = 0; n < RegTile::kCols; ++n)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (col0 + 16 * n > row0 + 16 * m + r) tile(m, n)(r, 0) = mask_value;
  }
};

}  // namespace tilefusion::cell
