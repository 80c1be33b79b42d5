// Register tiles (counterpart of include/types/register.hpp:84-131), re-sized for CDNA4.
//
// A RegTile is a per-lane array; a RegTile OF RegTiles tiles a wavefront-level matrix with
// MFMA base tiles.  For v_mfma_f32_16x16x32_{f16,bf16} a lane l of the 64 holds
//   * row-major operand base tile (16 rows x 32 k):   row l%16, k = 8*(l/16) .. +7   -> 1 x 8
//   * col-major operand base tile (32 k x 16 cols):   col l%16, k = 8*(l/16) .. +7   -> 8 x 1
//   * accumulator base tile (16 x 16), row-major:     col l%16, rows 4*(l/16) .. +3  -> 4 x 1
//   * accumulator base tile, column-major view:       row l%16, cols 4*(l/16) .. +3  -> 1 x 4
// BaseTileRowMajor<T> / BaseTileColMajor<T> pick the operand tile for 16-bit T and the
// accumulator tile for float; BaseTileAccRowMajor<T> is the accumulator tile for any T (e.g.
// scores converted to fp16 before they are stored).
#pragma once

#include "types/layout.hpp"

namespace tilefusion {
namespace tl = tile_layout;

template <typename Element_, typename Layout_>
class RegTile {
 public:
  using DType = Element_;
  using Layout = Layout_;
  static constexpr int kNumel = tl::get_numel<Layout>;
  static constexpr int kRows = tl::num_rows<Layout>;
  static constexpr int kCols = tl::num_cols<Layout>;
  static constexpr tl::Layout kType = tl::layout_type<Layout>;

  DEVICE RegTile() { clear(); }

  DEVICE DType* mutable_data() { return data_; }
  DEVICE const DType* data() const { return data_; }
  HOST_DEVICE constexpr Layout layout() const { return Layout{}; }

  DEVICE DType& operator()(int x, int y) { return data_[Layout{}(x, y)]; }
  DEVICE const DType& operator()(int x, int y) const { return data_[Layout{}(x, y)]; }

  // zero every element (recursively for tiles of tiles)
  DEVICE void clear() {
#pragma unroll
    for (int i = 0; i < kNumel; ++i) {
      if constexpr (requires(DType& d) { d.clear(); }) {
        data_[i].clear();
      } else {
        data_[i] = DType(0.f);
      }
    }
  }

  DEVICE void dump_value() const {
    if constexpr (requires(const DType& d) { d.dump_value(); }) {
      for (int i = 0; i < kNumel; ++i) data_[i].dump_value();
    } else {
      for (int i = 0; i < kNumel; ++i) printf("%.3f, ", to_float(data_[i]));
      printf("\n");
    }
  }

 private:
  DType data_[kNumel];
};

template <typename T>
inline constexpr bool kIsOperandType = sizeof(T) == 2;

template <typename T>
using BaseTileRowMajor =
    std::conditional_t<kIsOperandType<T>, RegTile<T, tl::RowMajor<1, 8>>, RegTile<T, tl::RowMajor<4, 1>>>;
template <typename T>
using BaseTileColMajor =
    std::conditional_t<kIsOperandType<T>, RegTile<T, tl::ColMajor<8, 1>>, RegTile<T, tl::ColMajor<1, 4>>>;
template <typename T>
using BaseTileAccRowMajor = RegTile<T, tl::RowMajor<4, 1>>;
template <typename T>
using BaseTileAccColMajor = RegTile<T, tl::ColMajor<1, 4>>;

// What a base tile covers at wavefront level, from its per-lane shape.
template <typename BaseTile>
struct BaseTileTraits {
  using DType = typename BaseTile::DType;
  static constexpr bool kIsOperand = BaseTile::kNumel == 8;
  static constexpr bool kIsRowMajor = BaseTile::kType == tl::Layout::kRowMajor;
  static_assert(BaseTile::kNumel == 8 || BaseTile::kNumel == 4, "not an MFMA base tile");
  // rows x cols of the matrix block one base tile holds across the 64 lanes
  static constexpr int kRows = kIsOperand ? (kIsRowMajor ? 16 : 32) : 16;
  static constexpr int kCols = kIsOperand ? (kIsRowMajor ? 32 : 16) : 16;
};

}  // namespace tilefusion
