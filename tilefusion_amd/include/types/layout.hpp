// Static matrix layouts (counterpart of include/types/layout.hpp:20-231).
#pragma once

#include <cstdio>
#include <ostream>

#include "types/base.hpp"
#include "util/math_utils.hpp"

namespace tilefusion::tile_layout {

enum class Layout { kRowMajor = 0, kColMajor = 1 };

HOST_DEVICE constexpr const char* layout_type_to_str(Layout type) {
  return type == Layout::kRowMajor ? "RowMajor" : type == Layout::kColMajor ? "ColMajor" : "UnsupportedLayout";
}

// (i, j) -> i * row_stride + j * col_stride.  The kind is deduced from the unit stride, so a
// degenerate ColMajor<1, 1> reads as row-major (like the reference).
template <int kRows_, int kCols_, int kRowStride_, int kColStride_,
          Layout kType_ = (kColStride_ == 1 ? Layout::kRowMajor : Layout::kColMajor)>
struct MatrixLayout {
  static constexpr int kRows = kRows_;
  static constexpr int kCols = kCols_;
  static constexpr int kRowStride = kRowStride_;
  static constexpr int kColStride = kColStride_;
  static constexpr int kNumel = kRows * kCols;
  static constexpr Layout kType = kType_;

  HOST_DEVICE constexpr int operator()(int i, int j) const { return i * kRowStride + j * kColStride; }
};

template <int kRows, int kCols, int kRowStride, int kColStride, Layout kType>
HOST std::ostream& operator<<(std::ostream& out, const MatrixLayout<kRows, kCols, kRowStride, kColStride, kType>&) {
  return out << layout_type_to_str(kType) << "<" << kRows << ", " << kCols << ">, Strides<" << kRowStride
             << ", " << kColStride << ">, Numel = " << kRows * kCols;
}

template <int kRow, int kCol, int kStride = kCol>
using RowMajor = MatrixLayout<kRow, kCol, kStride, 1>;

template <int kRow, int kCol, int kStride = kRow>
using ColMajor = MatrixLayout<kRow, kCol, 1, kStride>;

template <typename L>
inline constexpr size_t num_rows = L::kRows;
template <typename L>
inline constexpr size_t num_cols = L::kCols;
template <typename L>
inline constexpr size_t row_stride = L::kRowStride;
template <typename L>
inline constexpr size_t col_stride = L::kColStride;
template <typename L>
inline constexpr size_t get_numel = L::kNumel;
template <typename L>
inline constexpr Layout layout_type = L::kType;

template <typename L>
struct is_row_major {
  static constexpr bool value = L::kType == Layout::kRowMajor;
};
template <typename L>
struct is_col_major {
  static constexpr bool value = L::kType == Layout::kColMajor;
};
template <typename L>
struct is_contiguous {
  static constexpr bool value = is_row_major<L>::value ? (L::kRowStride == L::kCols && L::kColStride == 1)
                                                       : (L::kColStride == L::kRows && L::kRowStride == 1);
};

// A grid of inner tiles: element (i, j) lives in tile (i / inner_rows, j / inner_cols).  When
// the outer layout is contiguous the tiles themselves are stored back to back (tile strides
// are multiples of the inner tile's numel); otherwise the outer strides are kept.
// (The reference spells the name without the second 'i'; both spellings are provided.)
template <typename OuterLayout_, typename InnerLayout_>
struct BlockMatrxLayout {
  using OuterLayout = OuterLayout_;
  using InnerLayout = InnerLayout_;
  static constexpr int kRows = OuterLayout::kRows;
  static constexpr int kCols = OuterLayout::kCols;
  static constexpr int kNumel = OuterLayout::kNumel;
  static constexpr int kInnerRows = InnerLayout::kRows;
  static constexpr int kInnerCols = InnerLayout::kCols;
  static constexpr int kInnerNumel = InnerLayout::kNumel;
  static_assert(kRows % kInnerRows == 0 && kCols % kInnerCols == 0,
                "the inner tile must divide the outer layout");
  static constexpr Layout kType = OuterLayout::kType;
  static constexpr int kTileRows = kRows / kInnerRows;
  static constexpr int kTileCols = kCols / kInnerCols;
  static constexpr bool kIsRowMajor = is_row_major<OuterLayout>::value;
  static constexpr bool kIsContiguous = is_contiguous<OuterLayout>::value;
  static constexpr int kRowStride =
      kIsContiguous ? (kIsRowMajor ? kTileCols * kInnerNumel : kInnerNumel) : OuterLayout::kRowStride;
  static constexpr int kColStride =
      kIsContiguous ? (kIsRowMajor ? kInnerNumel : kTileRows * kInnerNumel) : OuterLayout::kColStride;

  HOST_DEVICE constexpr int operator()(int i, int j) const {
    using RowDM = DivModSelector<is_power_of_2<kInnerRows>(), kInnerRows>;
    using ColDM = DivModSelector<is_power_of_2<kInnerCols>(), kInnerCols>;
    return RowDM::div(i) * kRowStride + ColDM::div(j) * kColStride + InnerLayout{}(RowDM::mod(i), ColDM::mod(j));
  }

  HOST_DEVICE void dump() const {
    for (int i = 0; i < kRows; ++i) {
      for (int j = 0; j < kCols; ++j) printf("%d, ", operator()(i, j));
      printf("\n");
    }
  }
};
template <typename O, typename I>
using BlockMatrixLayout = BlockMatrxLayout<O, I>;

template <typename O, typename I>
concept BlockRowMajorLayout = is_row_major<O>::value && is_row_major<I>::value;
template <typename O, typename I>
concept BlockColMajorLayout = is_col_major<O>::value && is_col_major<I>::value;
template <typename O, typename I>
concept BlockMixedLayout = (is_row_major<O>::value && is_col_major<I>::value) ||
                           (is_col_major<O>::value && is_row_major<I>::value);

template <typename O, typename I>
  requires BlockRowMajorLayout<O, I>
using BlockRowMajor = BlockMatrxLayout<O, I>;
template <typename O, typename I>
  requires BlockColMajorLayout<O, I>
using BlockColMajor = BlockMatrxLayout<O, I>;
template <typename O, typename I>
  requires BlockMixedLayout<O, I>
using BlockMixed = BlockMatrxLayout<O, I>;

}  // namespace tilefusion::tile_layout
