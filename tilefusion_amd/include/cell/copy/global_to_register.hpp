// Global <-> register tile movers (counterpart of include/cell/copy/global_to_register.hpp:217-270)
// in MFMA fragment order.
//
// For every base tile of the RegTile a lane moves
//   * operand, row-major global:    one 16-byte vector  - row l%16, columns 8*(l/16) .. +7 of the
//                                   16 x 32 block;
//   * operand, column-major global: one 16-byte vector  - column l%16, rows 8*(l/16) .. +7 of the
//                                   32 x 16 block;
//   * accumulator, row-major:       4 scalars           - column l%16, rows 4*(l/16) .. +3 of the
//                                   16 x 16 block;
//   * accumulator, column-major:    4 scalars           - row l%16, columns 4*(l/16) .. +3.
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

// element coordinates (row, col) inside a base tile's block and the contiguity of a lane's
// elements, for lane `lane` and per-lane element index e
template <typename BaseTile>
struct FragmentMap {
  using Traits = BaseTileTraits<BaseTile>;
  DEVICE static void coord(int lane, int e, int& r, int& c) {
    if constexpr (Traits::kIsOperand) {
      if constexpr (Traits::kIsRowMajor) {
        r = lane % 16;
        c = 8 * (lane / 16) + e;
      } else {
        r = 8 * (lane / 16) + e;
        c = lane % 16;
      }
    } else {
      if constexpr (Traits::kIsRowMajor) {
        r = 4 * (lane / 16) + e;
        c = lane % 16;
      } else {
        r = lane % 16;
        c = 4 * (lane / 16) + e;
      }
    }
  }
};

// extent of the block one base tile covers in memory, in the form warp::ExecCounter takes
template <typename BaseTile>
struct BaseExtent {
  static constexpr int kRows = BaseTileTraits<BaseTile>::kRows;
  static constexpr int kCols = BaseTileTraits<BaseTile>::kCols;
};

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
        constexpr bool kContig = Traits::kIsOperand && ((Traits::kIsRowMajor && Global::kColStride == 1) ||
                                                        (!Traits::kIsRowMajor && Global::kRowStride == 1));
        if constexpr (kContig) {
          *reinterpret_cast<uint4*>(out) =
              *reinterpret_cast<const uint4*>(base + ptrdiff_t(r) * Global::kRowStride + ptrdiff_t(c) * Global::kColStride);
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
};

}  // namespace tilefusion::cell::copy
