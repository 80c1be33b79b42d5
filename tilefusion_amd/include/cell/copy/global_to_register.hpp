// Global <-> register tile movers (counterpart of include/cell/copy/global_to_register.hpp:217-270)
// in the lane order of the base tiles (types/register.hpp).
//
// For every base tile of the RegTile a lane moves its 4 (wide tiles: 8) elements of row or
// column l%16 of the block: as one 8- or 16-byte vector when the memory layout runs the same
// way as the base tile (row-major tile from row-major memory, column-major from column-major),
// element by element otherwise.
// The WarpReuse mode is honoured as documented (include/cell/copy/constants.hpp:7-14): with
// kRowReuseCont the wavefronts of a row share the row block and each reads ALL its columns.
#pragma once

#include "cell/copy/constants.hpp"
#include "cell/copy/warp.hpp"
#include "types/global.hpp"
#include "types/register.hpp"

namespace tilefusion::cell::copy {
namespace tl = tile_layout;

namespace detail {

template <typename BaseTile>
using FragmentMap = BaseTileTraits<BaseTile>;

// extent of the block one base tile covers in memory, in the form warp::ExecCounter takes
template <typename BaseTile>
struct BaseExtent {
  static constexpr int kRows = BaseTileTraits<BaseTile>::kRows;
  static constexpr int kCols = BaseTileTraits<BaseTile>::kCols;
};

// a lane's elements of one base tile as one vector
template <int kBytes>
struct VecOfBytes;
template <>
struct VecOfBytes<8> {
  using type = uint2;
};
template <>
struct VecOfBytes<16> {
  using type = uint4;
};
template <>
struct VecOfBytes<32> {
  struct type {
    uint4 lo, hi;
  };
};

// the lane's elements are contiguous in a tile with these strides
template <typename BaseTile, typename Tile>
inline constexpr bool kLaneContiguous =
    (BaseTileTraits<BaseTile>::kIsRowMajor && Tile::kColStride == 1) ||
    (!BaseTileTraits<BaseTile>::kIsRowMajor && Tile::kRowStride == 1);

// The register tile must be exactly the base tiles a wavefront walks over in its share.
template <typename Tile, typename Reg, typename WarpLayout, WarpReuse kMode>
struct GlobalRegCheck {
  using Exec = warp::ExecCounter<BaseExtent<typename Reg::DType>, Tile, WarpLayout, kMode>;
  static_assert(Exec::kRowExec == Reg::kRows && Exec::kColExec == Reg::kCols,
                "the register tile does not cover the wavefront's share of the tile");
};

}  // namespace detail

template <typename Reg_, typename WarpLayout_, WarpReuse kMode_>
struct GlobalToRegLoader {
  using Reg = Reg_;
  using WarpLayout = WarpLayout_;
  using BaseTile = typename Reg::DType;
  using DType = typename BaseTile::DType;
  using Traits = BaseTileTraits<BaseTile>;
  static constexpr WarpReuse kMode = kMode_;

  template <typename Global>
  DEVICE void operator()(const Global& src, Reg& dst) {
    [[maybe_unused]] detail::GlobalRegCheck<Global, Reg, WarpLayout, kMode> check;
    const int lane = warp::lane_id();
    const DType* base = src.data() + warp::GlobalOffsetHelper<WarpLayout, kMode>{}.template get_warp_offset<Global>();
#pragma unroll
    for (int i = 0; i < Reg::kRows; ++i)
#pragma unroll
      for (int j = 0; j < Reg::kCols; ++j) {
        DType* out = dst(i, j).mutable_data();
        int r, c;
        detail::FragmentMap<BaseTile>::coord(lane, 0, r, c);
        r += i * Traits::kRows;
        c += j * Traits::kCols;
        if constexpr (detail::kLaneContiguous<BaseTile, Global>) {
          using Vec = typename detail::VecOfBytes<sizeof(BaseTile)>::type;
          *reinterpret_cast<Vec*>(out) =
              *reinterpret_cast<const Vec*>(base + ptrdiff_t(r) * Global::kRowStride + ptrdiff_t(c) * Global::kColStride);
        } else {
#pragma unroll
          for (int e = 0; e < BaseTile::kNumel; ++e) {
            int rr, cc;
            detail::FragmentMap<BaseTile>::coord(lane, e, rr, cc);
            rr += i * Traits::kRows;
            cc += j * Traits::kCols;
            out[e] = base[ptrdiff_t(rr) * Global::kRowStride + ptrdiff_t(cc) * Global::kColStride];
          }
        }
      }
  }
};

template <typename Global_, typename Reg_, typename WarpLayout_>
struct RegToGlobalStorer {
  using Global = Global_;
  using Reg = Reg_;
  using WarpLayout = WarpLayout_;
  using BaseTile = typename Reg::DType;
  using DType = typename BaseTile::DType;
  using Traits = BaseTileTraits<BaseTile>;

  DEVICE void operator()(const Reg& src, Global& dst) {
    [[maybe_unused]] detail::GlobalRegCheck<Global, Reg, WarpLayout, WarpReuse::kCont> check;
    const int lane = warp::lane_id();
    DType* base = dst.mutable_data() +
                  warp::GlobalOffsetHelper<WarpLayout, WarpReuse::kCont>{}.template get_warp_offset<Global>();
#pragma unroll
    for (int i = 0; i < Reg::kRows; ++i)
#pragma unroll
      for (int j = 0; j < Reg::kCols; ++j) {
        const DType* in = src(i, j).data();
        if constexpr (detail::kLaneContiguous<BaseTile, Global>) {
          using Vec = typename detail::VecOfBytes<sizeof(BaseTile)>::type;
          int r, c;
          detail::FragmentMap<BaseTile>::coord(lane, 0, r, c);
          r += i * Traits::kRows;
          c += j * Traits::kCols;
          *reinterpret_cast<Vec*>(base + ptrdiff_t(r) * Global::kRowStride + ptrdiff_t(c) * Global::kColStride) =
              *reinterpret_cast<const Vec*>(in);
        } else {
#pragma unroll
          for (int e = 0; e < BaseTile::kNumel; ++e) {
            int rr, cc;
            detail::FragmentMap<BaseTile>::coord(lane, e, rr, cc);
            rr += i * Traits::kRows;
            cc += j * Traits::kCols;
            base[ptrdiff_t(rr) * Global::kRowStride + ptrdiff_t(cc) * Global::kColStride] = in[e];
          }
        }
      }
  }
};

}  // namespace tilefusion::cell::copy
