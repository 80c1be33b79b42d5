// Register-to-register tile copies (counterpart of include/cell/copy/register.hpp:10-41).
// RegTileCopy walks the base tiles of a register tile and BaseTileCopy the elements of a base
// tile; both are the same element-wise walk over (rows, cols) applied at different depths.
#pragma once

#include "types/register.hpp"

namespace tilefusion::cell::copy {

namespace detail {
template <typename Element>
struct DataCopy {
  DEVICE void operator()(const Element& src, Element& dst) const { dst = src; }
};

template <typename RegTile, typename Copy>
struct RegCopy {
  static constexpr int kRows = RegTile::kRows;
  static constexpr int kCols = RegTile::kCols;
  DEVICE void operator()(const RegTile& src, RegTile& dst) const {
    Copy c;
#pragma unroll
    for (int i = 0; i < kRows; ++i)
#pragma unroll
      for (int j = 0; j < kCols; ++j) c(src(i, j), dst(i, j));
  }
};
}  // namespace detail

template <typename BaseTile>
using BaseTileCopy = detail::RegCopy<BaseTile, detail::DataCopy<typename BaseTile::DType>>;
template <typename RegTile>
using RegTileCopy = detail::RegCopy<RegTile, BaseTileCopy<typename RegTile::DType>>;

// Copies a tile of any nesting depth (a base tile or a tile of base tiles).
template <typename Tile>
DEVICE void copy_tile(const Tile& src, Tile& dst) {
  if constexpr (requires(const typename Tile::DType& d) { d.data(); }) {
    RegTileCopy<Tile>{}(src, dst);
  } else {
    BaseTileCopy<Tile>{}(src, dst);
  }
}

}  // namespace tilefusion::cell::copy
