// Masks on a register tile (counterpart of include/cell/mask.hpp:9-113).
// kCausal writes `mask_value` wherever the GLOBAL column index exceeds the global row index.
// Per-lane element e of base tile (m, n) sits at
//   row = row_offset + warp_row * (tile rows) + 16*m + r,   col = col_offset + warp_col * (tile cols) + 16*n + c
// with (r, c) the base tile's lane map (types/register.hpp).
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
  using Traits = BaseTileTraits<BaseTile>;
  static_assert(!Traits::kIsWide, "the causal mask works on 16 x 16 base tiles");

  template <typename Element>
  DEVICE void operator()(RegTile& tile, const int row_offset, const int col_offset, Element mask_value) {
    const int lane = copy::warp::lane_id();
    int r0, c0;
    Traits::coord(lane, 0, r0, c0);
    const int row0 = row_offset + copy::warp::warp_row_id<WarpLayout>() * RegTile::kRows * 16 + r0;
    const int col0 = col_offset + copy::warp::warp_col_id<WarpLayout>() * RegTile::kCols * 16 + c0;
#pragma unroll
    for (int m = 0; m < RegTile::kRows; ++m)
#pragma unroll
      for (int n = 0; n < RegTile::kCols; ++n)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int dr = Traits::kIsRowMajor ? 0 : e, dc = Traits::kIsRowMajor ? e : 0;
          if (col0 + 16 * n + dc > row0 + 16 * m + dr) tile(m, n).mutable_data()[e] = mask_value;
        }
  }
};

}  // namespace tilefusion::cell
