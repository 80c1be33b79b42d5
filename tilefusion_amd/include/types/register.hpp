// Register tiles (counterpart of include/types/register.hpp:84-131) on a 64-lane wavefront.
//
// A RegTile is a per-lane array; a RegTile OF RegTiles tiles a wavefront-level matrix with
// base tiles.  A base tile covers the reference's 16 x 16 block; lane l of the 64 holds
//   * BaseTileRowMajor<T> = RegTile<T, RowMajor<1, 4>>:  row l%16,    columns 4*(l/16) .. +3
//   * BaseTileColMajor<T> = RegTile<T, ColMajor<4, 1>>:  column l%16, rows    4*(l/16) .. +3
// for every element type.  These are the A and B operand layouts of v_mfma_*_16x16x16 (two
// tiles adjacent in k feed one 16x16x32 instruction, see cell/compute/gemm.hpp), and the
// row-major tile is also the layout of an accumulator block computed with the two operands
// swapped - so, as with the reference's mma.m16n8k16 tiles, the accumulator of one gemm()
// becomes the A operand of the next after an element-wise conversion, and the same
// BaseTileRowMajor<float> the reference's kernels declare their accumulators with works here.
//
// Extension: a wide operand tile takes the whole 16 x 32 (32 x 16) block of the 16x16x32
// instruction in one piece, one 16-byte access per lane:
//   * WideBaseTileRowMajor<T> = RegTile<T, RowMajor<1, 8>>:  row l%16,    columns 8*(l/16) .. +7
//   * WideBaseTileColMajor<T> = RegTile<T, ColMajor<8, 1>>:  column l%16, rows    8*(l/16) .. +7
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
using BaseTileRowMajor = RegTile<T, tl::RowMajor<1, 4>>;
template <typename T>
using BaseTileColMajor = RegTile<T, tl::ColMajor<4, 1>>;
template <typename T>
  requires HalfType<T>
using WideBaseTileRowMajor = RegTile<T, tl::RowMajor<1, 8>>;
template <typename T>
  requires HalfType<T>
using WideBaseTileColMajor = RegTile<T, tl::ColMajor<8, 1>>;

// What a base tile covers at wavefront level, from its per-lane shape.
template <typename BaseTile>
struct BaseTileTraits {
  using DType = typename BaseTile::DType;
  static_assert((BaseTile::kRows == 1 && (BaseTile::kCols == 4 || BaseTile::kCols == 8)) ||
                    (BaseTile::kCols == 1 && (BaseTile::kRows == 4 || BaseTile::kRows == 8)),
                "not a base tile: use BaseTileRowMajor / BaseTileColMajor (or the wide forms)");
  static constexpr bool kIsWide = BaseTile::kNumel == 8;
  // a lane owns (part of) a row of the block, or (part of) a column
  static constexpr bool kIsRowMajor = BaseTile::kRows == 1;
  static constexpr int kNumelPerLane = BaseTile::kNumel;
  // rows x cols of the matrix block one base tile holds across the 64 lanes
  static constexpr int kRows = kIsRowMajor ? 16 : 4 * kNumelPerLane;
  static constexpr int kCols = kIsRowMajor ? 4 * kNumelPerLane : 16;

  // (row, col) inside the block of per-lane element e of lane `lane`
  DEVICE static void coord(int lane, int e, int& r, int& c) {
    if constexpr (kIsRowMajor) {
      r = lane % 16;
      c = kNumelPerLane * (lane / 16) + e;
    } else {
      r = kNumelPerLane * (lane / 16) + e;
      c = lane % 16;
    }
  }
};

}  // namespace tilefusion
