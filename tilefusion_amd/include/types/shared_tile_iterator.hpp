// Chunked iteration over a SharedTile (counterpart of
// include/types/shared_tile_iterator.hpp:84-177; the 2-D form is STileIterator2, :190-290).
// Sub-tiles keep the parent's base pointer, strides and swizzle parameters and carry their
// logical origin, so their elements are found at the same physical place as in the parent.
#pragma once

#include "types/shared.hpp"
#include "types/tile_shape.hpp"

namespace tilefusion {
namespace tl = tile_layout;

template <class Tile_, class ChunkShape_>
class STileIterator {
 public:
  using Tile = Tile_;
  using DType = typename Tile::DType;
  using ChunkShape = ChunkShape_;
  static constexpr int kChunkRows = dim_size<0, ChunkShape>;
  static constexpr int kChunkCols = dim_size<1, ChunkShape>;
  static_assert(Tile::kRows >= kChunkRows && Tile::kCols >= kChunkCols, "the chunk is larger than the tile");
  static constexpr int sc0 = Tile::kRows / kChunkRows;
  static constexpr int sc1 = Tile::kCols / kChunkCols;

  using ChunkLayout = tl::MatrixLayout<kChunkRows, kChunkCols, Tile::kRowStride, Tile::kColStride>;
  using NewTile = SharedTile<DType, ChunkLayout, Tile::kSwizzled, Tile::SwizzleBytes>;

  DEVICE STileIterator() : data_(nullptr), offset_(0) {}
  DEVICE STileIterator(DType* data) : data_(data), offset_(0) {}
  DEVICE STileIterator(const DType* data) : data_(const_cast<DType*>(data)), offset_(0) {}
  DEVICE STileIterator(DType* data, int offset) : data_(data), offset_(offset) {}

  DEVICE static constexpr int chunk_offset(int x, int y) {
    return Tile::kType == tl::Layout::kRowMajor ? x * kChunkRows * Tile::kRowStride + y * kChunkCols
                                                : x * kChunkRows + y * kChunkCols * Tile::kColStride;
  }

  DEVICE NewTile operator()(int i) const {
    static_assert(sc0 == 1 || sc1 == 1, "a single index needs a 1-D chunking");
    return NewTile(data_, offset_ + (sc0 == 1 ? chunk_offset(0, i) : chunk_offset(i, 0)));
  }
  DEVICE NewTile operator()(int x, int y) const { return NewTile(data_, offset_ + chunk_offset(x, y)); }

  DEVICE auto operator()(int x, const Underscore&) const {
    using Strip = SharedTile<DType, tl::MatrixLayout<kChunkRows, Tile::kCols, Tile::kRowStride, Tile::kColStride>,
                             Tile::kSwizzled, Tile::SwizzleBytes>;
    return STileIterator<Strip, ChunkShape>(data_, offset_ + chunk_offset(x, 0));
  }
  DEVICE auto operator()(const Underscore&, int y) const {
    using Strip = SharedTile<DType, tl::MatrixLayout<Tile::kRows, kChunkCols, Tile::kRowStride, Tile::kColStride>,
                             Tile::kSwizzled, Tile::SwizzleBytes>;
    return STileIterator<Strip, ChunkShape>(data_, offset_ + chunk_offset(0, y));
  }

  DEVICE Tile to_tile() const { return Tile(data_, offset_); }

 private:
  DType* data_;
  int offset_;
};

template <class Tile, class ChunkShape>
using STileIterator2 = STileIterator<Tile, ChunkShape>;

}  // namespace tilefusion
