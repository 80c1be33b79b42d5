// GEMM with operands going straight from global memory to register tiles (counterpart of
// examples/101_gemm/01_gemm_global_reg/gemm.hpp): every wavefront loads the fragments of its
// rows of A and columns of B with GlobalToRegLoader, chunk by chunk along K, and multiplies
// them with gemm(); no LDS is used.  One workgroup per [kTM, kTN] tile of C.
#pragma once

#include "cell/mod.hpp"
#include "types/mod.hpp"

using namespace tilefusion;
using namespace tilefusion::cell;
using namespace tilefusion::cell::copy;
namespace tl = tile_layout;

template <typename InType, typename AccType, typename WarpLayout_, int kM, int kN, int kK, int kTM, int kTN, int kTK>
struct GemmTraits {
  using WarpLayout = WarpLayout_;
  static constexpr int kWarpRows = tl::num_rows<WarpLayout>, kWarpCols = tl::num_cols<WarpLayout>;
  static constexpr int kThreads = tl::get_numel<WarpLayout> * WARP_SIZE;
  using BaseShape = BaseTileShape<InType>;  // the 16 x 16 block one base tile covers
  static_assert(kTK % BaseShape::kCols == 0, "a chunk is a whole number of base tiles deep");

  // A: rows of one C tile, all of K, walked in [kTM, kTK] chunks
  using GlobalA = GlobalTile<InType, tl::RowMajor<kTM, kK>>;
  using IteratorA = TileIterator<GlobalA, TileShape<kTM, kTK>>;
  using RegA = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kTM / kWarpRows / BaseShape::kRows, kTK / BaseShape::kCols>>;
  using ALoader = GlobalToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;

  // B: column-major K x kTN
  using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kTN>>;
  using IteratorB = TileIterator<GlobalB, TileShape<kTK, kTN>>;
  using RegB = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kTK / BaseShape::kRows, kTN / kWarpCols / BaseShape::kCols>>;
  using BLoader = GlobalToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;

  // C: a [kTM, kTN] window of the row-major [kM, kN] output
  using GlobalC = GlobalTile<AccType, tl::RowMajor<kTM, kTN, kN>>;
  using RegC = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kTM / kWarpRows / BaseShape::kRows, kTN / kWarpCols / BaseShape::kCols>>;
  using CStorer = RegToGlobalStorer<GlobalC, RegC, WarpLayout>;
};

template <typename InType, typename AccType, typename Traits, int kN, int kK, int kTM, int kTN>
__global__ void gemm_global_reg(const InType* dA, const InType* dB, AccType* dC) {
  const InType* a = dA + (size_t)blockIdx.x * kTM * kK;
  const InType* b = dB + (size_t)blockIdx.y * kTN * kK;
  AccType* c = dC + (size_t)blockIdx.x * kTM * kN + blockIdx.y * kTN;

  typename Traits::IteratorA gAs(a);
  typename Traits::IteratorB gBs(b);
  typename Traits::RegA rA;
  typename Traits::RegB rB;
  typename Traits::RegC acc;
  typename Traits::ALoader load_a;
  typename Traits::BLoader load_b;
  for (int k = 0; k < Traits::IteratorA::sc1; ++k) {
    load_a(gAs(k), rA);
    load_b(gBs(k), rB);
    compute::gemm(rA, rB, acc);
  }
  typename Traits::GlobalC gC(c);
  typename Traits::CStorer store_c;
  store_c(acc, gC);
}
