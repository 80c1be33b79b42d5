// LDS <-> register tile movers in the lane order of the base tiles (counterpart of
// include/cell/copy/shared_to_register.hpp:248-367; there is no ldmatrix on CDNA - a lane's part
// of a base tile is one ds_read_b64 (wide tiles: ds_read_b128) when the LDS layout runs the same
// way as the base tile, because both MFMA operands are contiguous in k).  The swizzle moves
// whole 16-byte vectors, so a lane's 8 or 16 aligned bytes stay together.
#pragma once

#include "cell/copy/global_to_register.hpp"
#include "types/register.hpp"
#include "types/shared.hpp"

namespace tilefusion::cell::copy {
namespace tl = tile_layout;

template <typename Reg_, typename WarpLayout_, WarpReuse kMode_>
struct SharedToRegLoader {
  using Reg = Reg_;
  using WarpLayout = WarpLayout_;
  using BaseTile = typename Reg::DType;
  using DType = typename BaseTile::DType;
  using Traits = BaseTileTraits<BaseTile>;
  static constexpr WarpReuse kMode = kMode_;

  template <typename Shared>
  DEVICE void operator()(const Shared& src, Reg& dst) {
    [[maybe_unused]] detail::GlobalRegCheck<Shared, Reg, WarpLayout, kMode> check;
    const int warp_off =
        warp::SharedOffsetHelper<WarpLayout, detail::BaseExtent<BaseTile>, Shared, kMode>{}.get_warp_offset();
    const int lane = warp::lane_id();
    const DType* base = src.data();
#pragma unroll
    for (int i = 0; i < Reg::kRows; ++i)
#pragma unroll
      for (int j = 0; j < Reg::kCols; ++j) {
        DType* out = dst(i, j).mutable_data();
        if constexpr (detail::kLaneContiguous<BaseTile, Shared> && sizeof(BaseTile) <= 16) {
          using Vec = typename detail::VecOfBytes<sizeof(BaseTile)>::type;
          int r, c;
          detail::FragmentMap<BaseTile>::coord(lane, 0, r, c);
          r += i * Traits::kRows;
          c += j * Traits::kCols;
          *reinterpret_cast<Vec*>(out) = *reinterpret_cast<const Vec*>(
              base + src.fetch_physical_offset(warp_off + r * Shared::kRowStride + c * Shared::kColStride));
        } else {
#pragma unroll
          for (int e = 0; e < BaseTile::kNumel; ++e) {
            int rr, cc;
            detail::FragmentMap<BaseTile>::coord(lane, e, rr, cc);
            rr += i * Traits::kRows;
            cc += j * Traits::kCols;
            out[e] = base[src.fetch_physical_offset(warp_off + rr * Shared::kRowStride + cc * Shared::kColStride)];
          }
        }
      }
  }
};

template <typename Reg_, typename WarpLayout_>
struct RegToSharedStorer {
  using Reg = Reg_;
  using WarpLayout = WarpLayout_;
  using BaseTile = typename Reg::DType;
  using DType = typename BaseTile::DType;
  using Traits = BaseTileTraits<BaseTile>;

  template <typename Shared>
  DEVICE void operator()(const Reg& src, Shared& dst) {
    [[maybe_unused]] detail::GlobalRegCheck<Shared, Reg, WarpLayout, WarpReuse::kCont> check;
    const int warp_off = warp::SharedOffsetHelper<WarpLayout, detail::BaseExtent<BaseTile>, Shared,
                                                  WarpReuse::kCont>{}.get_warp_offset();
    const int lane = warp::lane_id();
    DType* base = dst.mutable_data();
#pragma unroll
    for (int i = 0; i < Reg::kRows; ++i)
#pragma unroll
      for (int j = 0; j < Reg::kCols; ++j) {
        const DType* in = src(i, j).data();
        if constexpr (detail::kLaneContiguous<BaseTile, Shared> && sizeof(BaseTile) <= 16) {
          using Vec = typename detail::VecOfBytes<sizeof(BaseTile)>::type;
          int r, c;
          detail::FragmentMap<BaseTile>::coord(lane, 0, r, c);
          r += i * Traits::kRows;
          c += j * Traits::kCols;
          *reinterpret_cast<Vec*>(
              base + dst.fetch_physical_offset(warp_off + r * Shared::kRowStride + c * Shared::kColStride)) =
              *reinterpret_cast<const Vec*>(in);
        } else {
#pragma unroll
          for (int e = 0; e < BaseTile::kNumel; ++e) {
            int rr, cc;
            detail::FragmentMap<BaseTile>::coord(lane, e, rr, cc);
            rr += i * Traits::kRows;
            cc += j * Traits::kCols;
            base[dst.fetch_physical_offset(warp_off + rr * Shared::kRowStride + cc * Shared::kColStride)] = in[e];
          }
        }
      }
  }
};

}  // namespace tilefusion::cell::copy
