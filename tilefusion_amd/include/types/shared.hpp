// A view of a tile in LDS with an optional XOR swizzle (counterpart of
// include/types/shared.hpp:32-150).
//
// A SharedTile is (base pointer of the PARENT tile, logical origin inside it, static layout
// with the parent's strides).  fetch_physical_offset() maps a logical element offset - counted
// from the parent's base with the parent's strides - to where the element really sits: the
// tile is cut into swizzle blocks (8 rows x 128 bytes or 4 rows x 64 bytes) and inside a block
// the 16-byte vector index is XORed with the row index.  Because sub-tiles produced by
// STileIterator keep the parent's base and strides, they swizzle in parent coordinates.
#pragma once

#include <type_traits>

#include "types/layout.hpp"
#include "types/swizzle.hpp"
#include "util/print.hpp"

namespace tilefusion {
namespace tl = tile_layout;

template <typename Element_, typename Layout_, bool kSwizzled_ = false, int SwizzleBytes_ = 128>
class SharedTile {
 public:
  using DType = Element_;
  using Layout = Layout_;
  static constexpr int kRows = Layout::kRows;
  static constexpr int kCols = Layout::kCols;
  static constexpr int kRowStride = Layout::kRowStride;
  static constexpr int kColStride = Layout::kColStride;
  static constexpr tl::Layout kType = Layout::kType;
  static constexpr int kNumel = Layout::kNumel;
  static constexpr bool isRowMajor = tl::is_row_major<Layout>::value;
  static constexpr int SwizzleBytes = SwizzleBytes_;
  static constexpr bool kSwizzled = kSwizzled_;

  using SwizzleBaseShape = SwizzleBaseTileShape<DType, SwizzleBytes>;
  // block extent along (strided, contiguous) dimensions, in elements
  static constexpr int kSwizzleRows = isRowMajor ? SwizzleBaseShape::kRows : SwizzleBaseShape::kCols;
  static constexpr int kSwizzleCols = isRowMajor ? SwizzleBaseShape::kCols : SwizzleBaseShape::kRows;

  // the swizzle permutes 16-byte vectors inside kSwizzleCols-wide blocks of a row (column):
  // the contiguous extent of the (parent) tile must be whole blocks
  static_assert(!kSwizzled || (isRowMajor ? kRowStride : kColStride) % kSwizzleCols == 0,
                "a swizzled tile's contiguous dimension must be a multiple of the swizzle width "
                "(SwizzleBytes / sizeof(element))");

  DEVICE SharedTile() : data_(nullptr), offset_(0) {}
  DEVICE SharedTile(DType* data) : data_(data), offset_(0) {}
  DEVICE SharedTile(const DType* data) : data_(const_cast<DType*>(data)), offset_(0) {}
  DEVICE SharedTile(DType* data, int offset) : data_(data), offset_(offset) {}

  DEVICE DType* mutable_data() { return data_; }
  DEVICE const DType* data() const { return data_; }
  DEVICE int get_offset() const { return offset_; }
  HOST_DEVICE constexpr Layout layout() const { return Layout{}; }

  // logical element access (goes through the swizzle when there is one)
  DEVICE DType& operator()(int x, int y) { return data_[fetch_physical_offset(Layout{}(x, y))]; }
  DEVICE const DType& operator()(int x, int y) const { return data_[fetch_physical_offset(Layout{}(x, y))]; }

  // `offset` is relative to this tile's origin; the result is relative to data().
  DEVICE int fetch_physical_offset(int offset) const {
    const int logical = offset_ + offset;
    if constexpr (!kSwizzled) {
      return logical;
    } else {
      constexpr int kStrided = isRowMajor ? kRowStride : kColStride;
      const int line = logical / kStrided;  // row (row-major) or column (column-major)
      const int pos = logical % kStrided;   // position along the contiguous dimension
      constexpr int M = SwizzleBaseShape::M, S = SwizzleBaseShape::S, B = SwizzleBaseShape::B;
      const int vec = (pos >> M) & ((1 << S) - 1);
      const int swz = vec ^ (line & ((1 << B) - 1));
      return line * kStrided + ((pos >> (M + S)) << (M + S)) + (swz << M) + (pos & ((1 << M) - 1));
    }
  }

  DEVICE void dump_value() const {
    for (int i = 0; i < kRows; ++i) {
      for (int j = 0; j < kCols; ++j) printf("%.3f, ", to_float((*this)(i, j)));
      printf("\n");
    }
  }

 private:
  DType* data_;
  int offset_;
};

template <typename Element, typename Layout, bool kSwizzled, int kBytes>
HOST std::ostream& operator<<(std::ostream& out, const SharedTile<Element, Layout, kSwizzled, kBytes>&) {
  return out << "SharedTile { " << Layout{} << ", swizzled = " << kSwizzled << ", bytes = " << kBytes << " }";
}

}  // namespace tilefusion
