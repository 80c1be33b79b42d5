// LDS <-> register tile movers in MFMA fragment order (counterpart of
// include/cell/copy/shared_to_register.hpp:248-367; there is no ldmatrix on CDNA - an operand
// fragment is simply one ds_read_b128 per lane because both MFMA operands are contiguous in k).
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
        constexpr bool kContig = Traits::kIsOperand && ((Traits::kIsRowMajor && Shared::kColStride == 1) ||
                                                        (!Traits::kIsRowMajor && Shared::kRowStride == 1));
        if constexpr (kContig) {
          int r, c;
          detail::FragmentMap<BaseTile>::coord(lane, 0, r, c);
          r += i * Traits::kRows;
          c += j * Traits::kCols;
          *reinterpret_cast<uint4*>(out) = *reinterpret_cast<const uint4*>(
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
};

}  // namespace tilefusion::cell::copy
