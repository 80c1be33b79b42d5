// Element-wise maps over register tiles (counterpart of include/cell/compute/map.hpp:20-135).
// They are layout-agnostic: the same per-lane element index means the same matrix element in
// source and destination, so they simply walk the per-lane arrays, recursing through tiles of
// base tiles.
#pragma once

#include "cell/compute/math_functor.hpp"
#include "types/register.hpp"

namespace tilefusion::cell::compute {

namespace detail {

template <typename T>
inline constexpr bool kIsTile = requires(const T& t) { t.data(); };

template <typename RegTile, typename Functor>
struct ElementWise {
  using DType = typename RegTile::DType;
  DEVICE void operator()(const RegTile& src, RegTile& dst) {
#pragma unroll
    for (int i = 0; i < RegTile::kNumel; ++i) {
      if constexpr (kIsTile<DType>) {
        ElementWise<DType, Functor> inner;
        inner(src.data()[i], dst.mutable_data()[i]);
      } else {
        Functor f;
        f(src.data()[i], dst.mutable_data()[i]);
      }
    }
  }
};

template <typename SrcRegTile, typename DstRegTile, typename Functor>
struct ElementWise2 {
  static_assert(SrcRegTile::kNumel == DstRegTile::kNumel, "source and destination must have the same shape");
  DEVICE void operator()(const SrcRegTile& src, DstRegTile& dst) {
#pragma unroll
    for (int i = 0; i < SrcRegTile::kNumel; ++i) {
      if constexpr (kIsTile<typename SrcRegTile::DType>) {
        ElementWise2<typename SrcRegTile::DType, typename DstRegTile::DType, Functor> inner;
        inner(src.data()[i], dst.mutable_data()[i]);
      } else {
        Functor f;
        f(src.data()[i], dst.mutable_data()[i]);
      }
    }
  }
};

template <typename RegTile, typename Functor>
struct Binary {
  using DType = typename RegTile::DType;
  DEVICE void operator()(const RegTile& lhs, const RegTile& rhs, RegTile& dst) {
#pragma unroll
    for (int i = 0; i < RegTile::kNumel; ++i) {
      if constexpr (kIsTile<DType>) {
        Binary<DType, Functor> inner;
        inner(lhs.data()[i], rhs.data()[i], dst.mutable_data()[i]);
      } else {
        Functor f;
        f(lhs.data()[i], rhs.data()[i], dst.mutable_data()[i]);
      }
    }
  }
};

template <typename T>
struct ScalarOf {
  using type = T;
};
template <typename T>
  requires kIsTile<T>
struct ScalarOf<T> {
  using type = typename ScalarOf<typename T::DType>::type;
};

}  // namespace detail

template <typename T>
using scalar_of_t = typename detail::ScalarOf<T>::type;

template <typename RegTile>
using BaseTileExp = detail::ElementWise<RegTile, Exp<scalar_of_t<RegTile>>>;
template <typename RegTile>
using RegTileExp = detail::ElementWise<RegTile, Exp<scalar_of_t<RegTile>>>;
template <typename RegTile>
using BaseTileLog = detail::ElementWise<RegTile, Log<scalar_of_t<RegTile>>>;
template <typename RegTile>
using RegTileLog = detail::ElementWise<RegTile, Log<scalar_of_t<RegTile>>>;

template <typename RegTile>
using BaseTileRelu = detail::ElementWise<RegTile, Relu<scalar_of_t<RegTile>>>;
template <typename RegTile>
using RegTileRelu = detail::ElementWise<RegTile, Relu<scalar_of_t<RegTile>>>;

template <typename Src, typename Dst>
using BaseTileConvert = detail::ElementWise2<Src, Dst, Convert<scalar_of_t<Src>, scalar_of_t<Dst>>>;
template <typename Src, typename Dst>
using RegTileConvert = detail::ElementWise2<Src, Dst, Convert<scalar_of_t<Src>, scalar_of_t<Dst>>>;

#define TILEFUSION_BINARY_MAP(Name)                                                  \
  template <typename RegTile>                                                        \
  using BaseTile##Name = detail::Binary<RegTile, Name<scalar_of_t<RegTile>>>;        \
  template <typename RegTile>                                                        \
  using RegTile##Name = detail::Binary<RegTile, Name<scalar_of_t<RegTile>>>;
TILEFUSION_BINARY_MAP(Add)
TILEFUSION_BINARY_MAP(Sub)
TILEFUSION_BINARY_MAP(Mul)
TILEFUSION_BINARY_MAP(Div)
TILEFUSION_BINARY_MAP(Max)
TILEFUSION_BINARY_MAP(Min)
#undef TILEFUSION_BINARY_MAP

}  // namespace tilefusion::cell::compute
