// Chunked iteration over a SharedTile (counterpart of
// include/types/shared_tile_iterator.hpp:84-177 for STileIterator and :190-290 for
// STileIterator2).
//
// STileIterator: sub-tiles keep the parent's base pointer, strides and swizzle parameters and
// carry their logical origin, so their elements are found at the same physical place as in the
// parent.
// STileIterator2: for tiles whose LAYOUT does the placing - plain matrix layouts and
// BlockMatrxLayout (a grid of inner tiles, each possibly swizzled inside).  A chunk is a whole
// number of inner tiles; its sub-tile gets its own base pointer (the chunk's first inner tile)
// and a block layout of the chunk's extent that keeps the parent's tile strides and inner
// layout.  All four access forms work (the reference implements the single-index form only).
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

namespace detail {
template <typename Layout>
struct is_block_layout : std::false_type {};
template <typename Outer, typename Inner>
struct is_block_layout<tl::BlockMatrxLayout<Outer, Inner>> : std::true_type {};
template <typename Layout>
inline constexpr bool is_block_layout_v = is_block_layout<Layout>::value;

// layout of a kChunkRows x kChunkCols piece of a tile laid out by TileLayout
template <typename TileLayout, int kChunkRows, int kChunkCols, bool kIsBlock = is_block_layout_v<TileLayout>>
struct SubTileLayoutCreator {
  using type = tl::MatrixLayout<kChunkRows, kChunkCols, TileLayout::kRowStride, TileLayout::kColStride>;
};
template <typename TileLayout, int kChunkRows, int kChunkCols>
struct SubTileLayoutCreator<TileLayout, kChunkRows, kChunkCols, true> {
  static_assert(kChunkRows % TileLayout::kInnerRows == 0 && kChunkCols % TileLayout::kInnerCols == 0,
                "a chunk of a block layout is a whole number of inner tiles");
  // the outer strides are the parent's TILE strides (not contiguous for the chunk), which
  // BlockMatrxLayout then keeps as they are
  using Outer = tl::MatrixLayout<kChunkRows, kChunkCols, TileLayout::kRowStride, TileLayout::kColStride,
                                 TileLayout::kType>;
  using type = tl::BlockMatrxLayout<Outer, typename TileLayout::InnerLayout>;
};
template <typename TileLayout, int kChunkRows, int kChunkCols>
using SubTileLayout_t = typename SubTileLayoutCreator<TileLayout, kChunkRows, kChunkCols>::type;
}  // namespace detail
using detail::SubTileLayoutCreator;

template <class Tile_, class ChunkShape_>
class STileIterator2 {
 public:
  using Tile = Tile_;
  using DType = typename Tile::DType;
  using ChunkShape = ChunkShape_;
  using Layout = typename Tile::Layout;
  static constexpr int kChunkRows = dim_size<0, ChunkShape>;
  static constexpr int kChunkCols = dim_size<1, ChunkShape>;
  static_assert(Tile::kRows >= kChunkRows && Tile::kRows % kChunkRows == 0,
                "Tile::kRows must be a multiple of the chunk's rows");
  static_assert(Tile::kCols >= kChunkCols && Tile::kCols % kChunkCols == 0,
                "Tile::kCols must be a multiple of the chunk's columns");
  static_assert(!Tile::kSwizzled, "STileIterator2 is for layout-placed tiles; swizzle inside the inner layout");
  static constexpr int sc0 = Tile::kRows / kChunkRows;
  static constexpr int sc1 = Tile::kCols / kChunkCols;
  static constexpr int kNumel = sc0 * sc1;
  static constexpr bool kIsBlockLayout = detail::is_block_layout_v<Layout>;

  using NewTile = SharedTile<DType, detail::SubTileLayout_t<Layout, kChunkRows, kChunkCols>>;

  HOST_DEVICE STileIterator2() : tile_(nullptr), data_(nullptr) {}
  DEVICE explicit STileIterator2(Tile* tile) : tile_(tile), data_(tile->mutable_data() + tile->get_offset()) {}

  // element offset of chunk (x, y) from the parent's first element
  HOST_DEVICE static constexpr int chunk_offset(int x, int y) { return x * kChunkRowStride + y * kChunkColStride; }

  DEVICE NewTile operator()(int i) const {
    static_assert(sc0 == 1 || sc1 == 1, "a single index needs a 1-D chunking");
    return sc0 == 1 ? (*this)(0, i) : (*this)(i, 0);
  }
  DEVICE NewTile operator()(int x, int y) const { return NewTile(data_ + chunk_offset(x, y)); }

  // (x, _): row strip x as an iterator over its sc1 chunks; (_, y): column strip y
  DEVICE auto operator()(int x, const Underscore&) const {
    using Strip = SharedTile<DType, detail::SubTileLayout_t<Layout, kChunkRows, Tile::kCols>>;
    return StripIterator<Strip>(data_ + chunk_offset(x, 0));
  }
  DEVICE auto operator()(const Underscore&, int y) const {
    using Strip = SharedTile<DType, detail::SubTileLayout_t<Layout, Tile::kRows, kChunkCols>>;
    return StripIterator<Strip>(data_ + chunk_offset(0, y));
  }

  DEVICE Tile to_tile() const { return *tile_; }

 private:
  // a strip owns its tile object, so that it can hand out the same kind of iterator
  template <typename Strip>
  struct StripIterator {
    Strip strip;
    DEVICE explicit StripIterator(DType* data) : strip(data) {}
    DEVICE auto operator()(int i) { return STileIterator2<Strip, ChunkShape>(&strip)(i); }
    DEVICE Strip to_tile() const { return strip; }
    static constexpr int sc0 = Strip::kRows / kChunkRows, sc1 = Strip::kCols / kChunkCols;
  };

  // a step of one chunk: whole inner tiles for a block layout, elements otherwise
  template <typename L, bool kBlock>
  struct InnerExtent {
    static constexpr int kRows = 1, kCols = 1;
  };
  template <typename L>
  struct InnerExtent<L, true> {
    static constexpr int kRows = L::kInnerRows, kCols = L::kInnerCols;
  };
  using Inner = InnerExtent<Layout, kIsBlockLayout>;
  static constexpr int kChunkRowStride = Layout::kRowStride * (kChunkRows / Inner::kRows);
  static constexpr int kChunkColStride = Layout::kColStride * (kChunkCols / Inner::kCols);

  Tile* tile_;
  DType* data_;
};

}  // namespace tilefusion
