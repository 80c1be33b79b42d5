// Row / column reductions of accumulator register tiles (counterpart of
// include/cell/compute/reduce.hpp:16-152) for the MFMA accumulator layout.
//
// Row-major accumulator base tile: lane l holds column l%16 and rows 4*(l/16) .. +3, so the 16
// lanes that share a row are exactly one DPP row of the wavefront.  Reducing along a row is
//   1. fold the base tiles of a tile row inside the lane,
//   2. one 4-step rotate-and-combine over the DPP row (no LDS crossbar traffic),
// after which every lane of the DPP row holds the result.  The result vector of a tile with
// kRows base-tile rows is RegTile<T, RowMajor<kRows, 4>>: element (i, r) belongs to tile row
// 16*i + 4*(l/16) + r.  (On the reference's mma.m16n8k16 layout the vector is kRows x 2.)
// The column-major form reduces column-major accumulator tiles along columns symmetrically
// into RegTile<T, ColMajor<4, kCols>>.
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
  static_assert(BaseTile::kNumel == 4 && BaseTile::kType == tl::Layout::kRowMajor,
                "row reduction works on row-major accumulator base tiles");
  static constexpr int kRows = RegTile::kRows, kCols = RegTile::kCols;

  template <typename DstTile, typename Op>
  DEVICE void operator()(const RegTile& src, DstTile& dst, Op op) {
    static_assert(DstTile::kRows == kRows && DstTile::kCols == 4, "the result vector is kRows x 4");
#pragma unroll
    for (int i = 0; i < kRows; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = to_float(src(i, 0)(r, 0));
#pragma unroll
        for (int j = 1; j < kCols; ++j) v = op(v, to_float(src(i, j)(r, 0)));
        dst(i, r) = from_float<DType>(row16_allreduce(v, op));
      }
  }
};

template <typename RegTile>
struct Reduce<RegTile, tl::Layout::kColMajor> {
  using BaseTile = typename RegTile::DType;
  using DType = typename BaseTile::DType;
  static_assert(BaseTile::kNumel == 4 && BaseTile::kType == tl::Layout::kColMajor,
                "column reduction works on column-major accumulator base tiles");
  static constexpr int kRows = RegTile::kRows, kCols = RegTile::kCols;

  template <typename DstTile, typename Op>
  DEVICE void operator()(const RegTile& src, DstTile& dst, Op op) {
    static_assert(DstTile::kRows == 4 && DstTile::kCols == kCols, "the result vector is 4 x kCols");
#pragma unroll
    for (int j = 0; j < kCols; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = to_float(src(0, j)(0, r));
#pragma unroll
        for (int i = 1; i < kRows; ++i) v = op(v, to_float(src(i, j)(0, r)));
        dst(r, j) = from_float<DType>(row16_allreduce(v, op));
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
