// Row / column reductions of register tiles (counterpart of include/cell/compute/reduce.hpp:16-152).
//
// A row-major base tile gives lane l the columns 4*(l/16) .. +3 of row l%16, so reducing
// along rows is
//   1. fold the lane's 4 elements of every base tile of a tile row,
//   2. combine over the four lanes l%16 + {0, 16, 32, 48} that share the row (two register
//      half-swaps, no LDS traffic), after which each of them holds the result.
// A lane therefore owns ONE row per base-tile row: the natural result vector of a tile with
// kRows base-tile rows is RegTile<T, RowMajor<kRows, 1>>, element (i, 0) belonging to tile row
// 16*i + l%16.  Kernels written for the reference declare the vector as RowMajor<kRows, 2>
// (its lanes own a top and a bottom row, include/cell/compute/reduce.hpp:52-68); any number of
// columns is accepted and every column receives the same value, which the element-wise vector
// ops and the Broadcast functors (they read column 0) are indifferent to.
// Column-major base tiles reduce along columns symmetrically into ColMajor<n, kCols>.
#pragma once

#include "cell/compute/math_functor.hpp"
#include "cell/warp.hpp"
#include "types/register.hpp"

namespace tilefusion::cell::compute {
namespace tl = tile_layout;

namespace detail {

template <typename RegTile, tl::Layout kLayout>
struct Reduce;

template <typename RegTile>
struct Reduce<RegTile, tl::Layout::kRowMajor> {
  using BaseTile = typename RegTile::DType;
  using DType = typename BaseTile::DType;
  static_assert(BaseTileTraits<BaseTile>::kIsRowMajor, "row reduction works on row-major base tiles");
  static constexpr int kRows = RegTile::kRows, kCols = RegTile::kCols;

  template <typename DstTile, typename Op>
  DEVICE void operator()(const RegTile& src, DstTile& dst, Op op) {
    static_assert(DstTile::kRows == kRows && DstTile::kCols >= 1, "the result vector has one row per base-tile row");
#pragma unroll
    for (int i = 0; i < kRows; ++i) {
      float v = to_float(src(i, 0).data()[0]);
#pragma unroll
      for (int j = 0; j < kCols; ++j)
#pragma unroll
        for (int e = (j == 0 ? 1 : 0); e < BaseTile::kNumel; ++e) v = op(v, to_float(src(i, j).data()[e]));
      const auto out = from_float<typename DstTile::DType>(quad16_allreduce(v, op));
#pragma unroll
      for (int c = 0; c < DstTile::kCols; ++c) dst(i, c) = out;
    }
  }
};

template <typename RegTile>
struct Reduce<RegTile, tl::Layout::kColMajor> {
  using BaseTile = typename RegTile::DType;
  using DType = typename BaseTile::DType;
  static_assert(!BaseTileTraits<BaseTile>::kIsRowMajor, "column reduction works on column-major base tiles");
  static constexpr int kRows = RegTile::kRows, kCols = RegTile::kCols;

  template <typename DstTile, typename Op>
  DEVICE void operator()(const RegTile& src, DstTile& dst, Op op) {
    static_assert(DstTile::kCols == kCols && DstTile::kRows >= 1, "the result vector has one column per base-tile column");
#pragma unroll
    for (int j = 0; j < kCols; ++j) {
      float v = to_float(src(0, j).data()[0]);
#pragma unroll
      for (int i = 0; i < kRows; ++i)
#pragma unroll
        for (int e = (i == 0 ? 1 : 0); e < BaseTile::kNumel; ++e) v = op(v, to_float(src(i, j).data()[e]));
      const auto out = from_float<typename DstTile::DType>(quad16_allreduce(v, op));
#pragma unroll
      for (int r = 0; r < DstTile::kRows; ++r) dst(r, j) = out;
    }
  }
};

struct FAdd {
  DEVICE float operator()(float a, float b) const { return a + b; }
};
struct FMax {
  DEVICE float operator()(float a, float b) const { return fmaxf(a, b); }
};

}  // namespace detail

template <typename RegTile, tl::Layout kLayout>
struct SumReduce {
  using DType = typename RegTile::DType::DType;
  template <typename DstTile>
  DEVICE void operator()(const RegTile& src, DstTile& dst) {
    detail::Reduce<RegTile, kLayout> reduce;
    reduce(src, dst, detail::FAdd{});
  }
};

template <typename RegTile, tl::Layout kLayout>
struct MaxReduce {
  using DType = typename RegTile::DType::DType;
  template <typename DstTile>
  DEVICE void operator()(const RegTile& src, DstTile& dst) {
    detail::Reduce<RegTile, kLayout> reduce;
    reduce(src, dst, detail::FMax{});
  }
};

}  // namespace tilefusion::cell::compute
