// GEMM through all three memory levels (counterpart of examples/101_gemm/02_gemm_all_mem/
// gemm.hpp): global -> LDS with GlobalToSharedLoader into swizzled SharedTiles, LDS ->
// registers with SharedToRegLoader in base-tile lane order, gemm() on the register tiles, and
// the accumulator back to global memory.  One workgroup per [kTM, kTN] tile of C; K is walked
// in kTK chunks through LDS and in kRK steps through registers.
#pragma once

#include "cell/mod.hpp"
#include "types/mod.hpp"

using namespace tilefusion;
using namespace tilefusion::cell;
using namespace tilefusion::cell::copy;
namespace tl = tile_layout;

template <typename InType, typename AccType, typename WarpLayout_, int kM, int kN, int kK, int kTM, int kTN, int kTK,
          int kRK>
struct GemmTraits {
  using WarpLayout = WarpLayout_;
  static constexpr int kWarpRows = tl::num_rows<WarpLayout>, kWarpCols = tl::num_cols<WarpLayout>;
  static constexpr int kThreads = tl::get_numel<WarpLayout> * WARP_SIZE;
  using BaseShape = BaseTileShape<InType>;  // the 16 x 16 block one base tile covers
  static_assert(kRK % BaseShape::kCols == 0 && kTK % kRK == 0, "kRK is whole base tiles and divides kTK");

  using GlobalA = GlobalTile<InType, tl::RowMajor<kTM, kK>>;
  using GIteratorA = GTileIterator<GlobalA, TileShape<kTM, kTK>>;
  using SharedA = SharedTile<InType, tl::RowMajor<kTM, kTK>, /*swizzled=*/true, /*bytes=*/64>;
  using SIteratorA = STileIterator<SharedA, TileShape<kTM, kRK>>;
  using RegA = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kTM / kWarpRows / BaseShape::kRows, kRK / BaseShape::kCols>>;
  using G2SLoaderA = GlobalToSharedLoader<SharedA, WarpLayout>;
  using S2RLoaderA = SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;

  using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kTN>>;
  using GIteratorB = GTileIterator<GlobalB, TileShape<kTK, kTN>>;
  using SharedB = SharedTile<InType, tl::ColMajor<kTK, kTN>, true, 64>;
  using SIteratorB = STileIterator<SharedB, TileShape<kRK, kTN>>;
  using RegB = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kRK / BaseShape::kRows, kTN / kWarpCols / BaseShape::kCols>>;
  using G2SLoaderB = GlobalToSharedLoader<SharedB, WarpLayout>;
  using S2RLoaderB = SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;

  using GlobalC = GlobalTile<AccType, tl::RowMajor<kTM, kTN, kN>>;
  using RegC = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kTM / kWarpRows / BaseShape::kRows, kTN / kWarpCols / BaseShape::kCols>>;
  using R2GStorerC = RegToGlobalStorer<GlobalC, RegC, WarpLayout>;

  static constexpr int kSharedBytes = (SharedA::kNumel + SharedB::kNumel) * (int)sizeof(InType);
};

template <typename InType, typename AccType, typename Traits, int kN, int kK, int kTM, int kTN>
__global__ void gemm_all_mem(const InType* dA, const InType* dB, AccType* dC) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_bytes[];
  InType* lds = reinterpret_cast<InType*>(lds_bytes);
  const InType* a = dA + (size_t)blockIdx.x * kTM * kK;
  const InType* b = dB + (size_t)blockIdx.y * kTN * kK;
  AccType* c = dC + (size_t)blockIdx.x * kTM * kN + blockIdx.y * kTN;

  typename Traits::GIteratorA gAs(a);
  typename Traits::GIteratorB gBs(b);
  typename Traits::SharedA sA(lds);
  typename Traits::SharedB sB(lds + Traits::SharedA::kNumel);
  typename Traits::SIteratorA sAs(lds);
  typename Traits::SIteratorB sBs(lds + Traits::SharedA::kNumel);
  typename Traits::RegA rA;
  typename Traits::RegB rB;
  typename Traits::RegC acc;
  typename Traits::G2SLoaderA g2s_a;
  typename Traits::G2SLoaderB g2s_b;
  typename Traits::S2RLoaderA s2r_a;
  typename Traits::S2RLoaderB s2r_b;

  for (int k1 = 0; k1 < Traits::GIteratorA::sc1; ++k1) {
    g2s_a(gAs(k1), sA);
    g2s_b(gBs(k1), sB);
    __copy_async();
    __syncthreads();
    for (int k2 = 0; k2 < Traits::SIteratorA::sc1; ++k2) {
      s2r_a(sAs(k2), rA);
      s2r_b(sBs(k2), rB);
      compute::gemm(rA, rB, acc);
    }
    __syncthreads();  // the next chunk overwrites the LDS tiles
  }
  typename Traits::GlobalC gC(c);
  typename Traits::R2GStorerC store_c;
  store_c(acc, gC);
}
