// Chunked iteration over a GlobalTile (counterpart of
// include/types/global_tile_iterator.hpp:33-151; the README calls it TileIterator).
//
// A tile of R x C is cut into sc0 x sc1 chunks of ChunkShape; chunk (x, y) is a GlobalTile of
// the chunk's shape that keeps the parent's strides.  Offsets are computed in ptrdiff_t:
// a 32-bit int overflows once a key/value tensor passes 2^31 elements.
#pragma once

#include <cstddef>

#include "types/global.hpp"
#include "types/tile_shape.hpp"

namespace tilefusion {
namespace tl = tile_layout;

template <class Tile_, class ChunkShape_>
class GTileIterator {
 public:
  using Tile = Tile_;
  using DType = typename Tile::DType;
  using ChunkShape = ChunkShape_;
  static constexpr int kStride0 = dim_size<0, ChunkShape>;
  static constexpr int kStride1 = dim_size<1, ChunkShape>;
  static_assert(Tile::kRows >= kStride0 && Tile::kCols >= kStride1, "the chunk is larger than the tile");
  static constexpr int sc0 = Tile::kRows / kStride0;
  static constexpr int sc1 = Tile::kCols / kStride1;

  using ChunkLayout = tl::MatrixLayout<kStride0, kStride1, Tile::kRowStride, Tile::kColStride>;
  using ChunkTile = GlobalTile<DType, ChunkLayout>;

  HOST_DEVICE GTileIterator() : data_(nullptr) {}
  HOST_DEVICE GTileIterator(DType* data) : data_(data) {}
  HOST_DEVICE GTileIterator(const DType* data) : data_(const_cast<DType*>(data)) {}

  HOST_DEVICE static constexpr ptrdiff_t chunk_offset(int x, int y) {
    return Tile::kType == tl::Layout::kRowMajor
               ? ptrdiff_t(x) * kStride0 * Tile::kRowStride + ptrdiff_t(y) * kStride1
               : ptrdiff_t(x) * kStride0 + ptrdiff_t(y) * kStride1 * Tile::kColStride;
  }

  // single index: allowed when the tile is only chunked along one dimension
  HOST_DEVICE ChunkTile operator()(int i) const {
    static_assert(sc0 == 1 || sc1 == 1, "a single index needs a 1-D chunking");
    return sc0 == 1 ? ChunkTile(data_ + chunk_offset(0, i)) : ChunkTile(data_ + chunk_offset(i, 0));
  }
  HOST_DEVICE ChunkTile operator()(int x, int y) const { return ChunkTile(data_ + chunk_offset(x, y)); }

  // (x, _): row strip x as an iterator over its sc1 chunks
  HOST_DEVICE auto operator()(int x, const Underscore&) const {
    using Strip = GlobalTile<DType, tl::MatrixLayout<kStride0, Tile::kCols, Tile::kRowStride, Tile::kColStride>>;
    return GTileIterator<Strip, ChunkShape>(data_ + chunk_offset(x, 0));
  }
  // (_, y): column strip y as an iterator over its sc0 chunks
  HOST_DEVICE auto operator()(const Underscore&, int y) const {
    using Strip = GlobalTile<DType, tl::MatrixLayout<Tile::kRows, kStride1, Tile::kRowStride, Tile::kColStride>>;
    return GTileIterator<Strip, ChunkShape>(data_ + chunk_offset(0, y));
  }

  HOST_DEVICE Tile to_tile() const { return Tile(data_); }

 private:
  DType* data_;
};

template <class Tile, class ChunkShape>
using TileIterator = GTileIterator<Tile, ChunkShape>;

}  // namespace tilefusion
