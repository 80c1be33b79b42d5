// Register-to-register tile copies (counterpart of include/cell/copy/register.hpp:10-41).
#pragma once

#include "types/register.hpp"

namespace tilefusion::cell::copy {

template <typename Tile>
DEVICE void copy_tile(const Tile& src, Tile& dst) {
#pragma unroll
  for (int i = 0; i < Tile::kNumel; ++i) {
    if constexpr (requires(const typename Tile::DType& d) { d.data(); }) {
      copy_tile(src.data()[i], dst.mutable_data()[i]);
    } else {
      dst.mutable_data()[i] = src.data()[i];
    }
  }
}

template <typename BaseTile>
struct BaseTileCopy {
  DEVICE void operator()(const BaseTile& src, BaseTile& dst) const { copy_tile(src, dst); }
};
template <typename RegTile>
struct RegTileCopy {
  DEVICE void operator()(const RegTile& src, RegTile& dst) const { copy_tile(src, dst); }
};

}  // namespace tilefusion::cell::copy
