// Broadcast of a reduced vector (or a scalar) over a register tile (counterpart of
// include/cell/compute/broadcast.hpp:14-187).  Row-major: src is the vector SumReduce /
// MaxReduce produce - one value per base-tile row, in column 0 - and element (i, 0) meets all
// the lane's elements of tile row 16*i + l%16.  The fused forms compute dst = f(dst, src) in
// place.
#pragma once

#include "cell/compute/math_functor.hpp"
#include "types/register.hpp"

namespace tilefusion::cell::compute {
namespace tl = tile_layout;

template <typename SrcTile, typename DstTile, tl::Layout kLayout>
struct Broadcast {
  using DType = typename DstTile::DType::DType;
  static_assert(BaseTileTraits<typename DstTile::DType>::kIsRowMajor == (kLayout == tl::Layout::kRowMajor),
                "a row vector is broadcast over row-major base tiles, a column vector over column-major ones");
  static constexpr int kRows = DstTile::kRows, kCols = DstTile::kCols;
  DEVICE void operator()(const SrcTile& src, DstTile& dst) {
#pragma unroll
    for (int i = 0; i < kRows; ++i)
#pragma unroll
      for (int j = 0; j < kCols; ++j)
#pragma unroll
        for (int e = 0; e < DstTile::DType::kNumel; ++e) {
          if constexpr (kLayout == tl::Layout::kRowMajor) {
            dst(i, j).mutable_data()[e] = src(i, 0);
          } else {
            dst(i, j).mutable_data()[e] = src(0, j);
          }
        }
  }
};

template <typename SrcTile, typename DstTile, typename Functor, tl::Layout kLayout>
struct BroadcastFuse {
  using DType = typename DstTile::DType::DType;
  static_assert(BaseTileTraits<typename DstTile::DType>::kIsRowMajor == (kLayout == tl::Layout::kRowMajor),
                "a row vector is broadcast over row-major base tiles, a column vector over column-major ones");
  static constexpr int kRows = DstTile::kRows, kCols = DstTile::kCols;
  DEVICE void operator()(const SrcTile& src, DstTile& dst) {
    Functor f;
#pragma unroll
    for (int i = 0; i < kRows; ++i)
#pragma unroll
      for (int j = 0; j < kCols; ++j)
#pragma unroll
        for (int e = 0; e < DstTile::DType::kNumel; ++e) {
          auto& d = dst(i, j).mutable_data()[e];
          if constexpr (kLayout == tl::Layout::kRowMajor) {
            f(d, src(i, 0), d);
          } else {
            f(d, src(0, j), d);
          }
        }
  }
};

// dst = f(src, scalar) element-wise, on a base tile or on a tile of base tiles
template <typename RegTile, typename Functor>
struct BroadcastScalar {
  template <typename Element>
  DEVICE void operator()(const RegTile& src, Element scalar, RegTile& dst) {
    if constexpr (requires(const typename RegTile::DType& d) { d.data(); }) {
      BroadcastScalar<typename RegTile::DType, Functor> inner;
#pragma unroll
      for (int i = 0; i < RegTile::kNumel; ++i) inner(src.data()[i], scalar, dst.mutable_data()[i]);
    } else {
      Functor f;
#pragma unroll
      for (int i = 0; i < RegTile::kNumel; ++i) f(src.data()[i], scalar, dst.mutable_data()[i]);
    }
  }
};

template <typename SrcTile, typename DstTile, tl::Layout kLayout>
using BroadcastAdd = BroadcastFuse<SrcTile, DstTile, Add<typename DstTile::DType::DType>, kLayout>;
template <typename SrcTile, typename DstTile, tl::Layout kLayout>
using BroadcastSub = BroadcastFuse<SrcTile, DstTile, Sub<typename DstTile::DType::DType>, kLayout>;
template <typename SrcTile, typename DstTile, tl::Layout kLayout>
using BroadcastMul = BroadcastFuse<SrcTile, DstTile, Mul<typename DstTile::DType::DType>, kLayout>;
template <typename SrcTile, typename DstTile, tl::Layout kLayout>
using BroadcastDiv = BroadcastFuse<SrcTile, DstTile, Div<typename DstTile::DType::DType>, kLayout>;

template <typename RegTile>
using BaseBroadcastScalarMul = BroadcastScalar<RegTile, Mul<typename RegTile::DType>>;
template <typename RegTile>
using BroadcastScalarMul = BroadcastScalar<RegTile, Mul<typename RegTile::DType::DType>>;

}  // namespace tilefusion::cell::compute
