// Fused back-to-back GEMM composed from the tile primitives (counterpart of
// include/kernels/fused_two_gemms_device.cuh:16-214): D[M,P] = (A[M,K] * B[K,N]) * C[N,P] with A,
// D row-major and B, C column-major; one workgroup per [kTM, kTP] tile of D; the intermediate
// A*B tile never leaves the chip.
//
// The first product arrives in the MFMA accumulator layout (a lane owns a column), the second
// MFMA wants it in the row-major operand layout (a lane owns a row): the fp16-rounded tile is
// re-laid-out through an LDS tile with RegToSharedStorer / SharedToRegLoader.  (The library's
// tuned entry point tf_fused_two_gemms_f16 avoids that round trip by computing the first
// product transposed.)
#pragma once

#include "cell/mod.hpp"
#include "types/mod.hpp"

namespace tilefusion::kernels {
using namespace tilefusion::cell;
using namespace tilefusion::cell::copy;
namespace tl = tile_layout;

template <typename InType_, typename AccType_, typename WarpLayout_, int kM_, int kN_, int kK_, int kP_, int kTM_,
          int kTN_, int kTK_, int kTP_>
struct FusedTwoGemmsTraits {
  using InType = InType_;
  using AccType = AccType_;
  using WarpLayout = WarpLayout_;
  using BaseShape = BaseTileShape<InType>;
  static constexpr int kThreads = tl::get_numel<WarpLayout> * WARP_SIZE;
  static constexpr int kWarpPerRow = tl::num_rows<WarpLayout>;
  static constexpr int kWarpPerCol = tl::num_cols<WarpLayout>;
  static_assert(kWarpPerCol == 1, "wavefronts must be arranged as a column vector");
  static constexpr int kM = kM_, kN = kN_, kK = kK_, kP = kP_;
  static constexpr int kTM = kTM_, kTN = kTN_, kTK = kTK_, kTP = kTP_;
  static constexpr int kSharedAccess = 64;
  static_assert(kTK % 32 == 0 && kTN % 32 == 0 && kTP % 16 == 0 && (kTM / kWarpPerRow) % 16 == 0,
                "tile sizes must be whole MFMA base tiles");

  using GlobalA = GlobalTile<InType, tl::RowMajor<kTM, kK>>;
  using GIteratorA = GTileIterator<GlobalA, TileShape<kTM, kTK>>;
  using SharedA = SharedTile<InType, tl::RowMajor<kTM, kTK>, true, kSharedAccess>;
  using RegA = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kTM / kWarpPerRow / 16, kTK / 32>>;
  using SharedALoader = GlobalToSharedLoader<SharedA, WarpLayout>;
  using RegALoader = SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;

  using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kN>>;
  using GIteratorB = GTileIterator<GlobalB, TileShape<kTK, kTN>>;
  using SharedB = SharedTile<InType, tl::ColMajor<kTK, kTN>, true, kSharedAccess>;
  using RegB = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kTK / 32, kTN / 16>>;
  using SharedBLoader = GlobalToSharedLoader<SharedB, WarpLayout>;
  using RegBLoader = SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;

  using GlobalC = GlobalTile<InType, tl::ColMajor<kN, kTP>>;
  using GIteratorC = GTileIterator<GlobalC, TileShape<kTN, kTP>>;
  using SharedC = SharedTile<InType, tl::ColMajor<kTN, kTP>, true, kSharedAccess>;
  using RegC = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kTN / 32, kTP / 16>>;
  using SharedCLoader = GlobalToSharedLoader<SharedC, WarpLayout>;
  using RegCLoader = SharedToRegLoader<RegC, WarpLayout, WarpReuse::kColReuseCont>;

  // intermediate tile: fp32 accumulators -> fp16 in accumulator layout -> LDS -> operand layout
  using RegAcc = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kTM / kWarpPerRow / 16, kTN / 16>>;
  using RegAccCast = RegTile<BaseTileAccRowMajor<InType>, tl::RowMajor<kTM / kWarpPerRow / 16, kTN / 16>>;
  using ConvertHalf = compute::RegTileConvert<RegAcc, RegAccCast>;
  using SharedP = SharedTile<InType, tl::RowMajor<kTM, kTN>, true, kSharedAccess>;
  using RegP = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kTM / kWarpPerRow / 16, kTN / 32>>;
  using StorerP = RegToSharedStorer<RegAccCast, WarpLayout>;
  using LoaderP = SharedToRegLoader<RegP, WarpLayout, WarpReuse::kRowReuseCont>;

  using GlobalD = GlobalTile<InType, tl::RowMajor<kTM, kTP, kP>>;
  using SharedD = SharedTile<InType, tl::RowMajor<kTM, kTP>, false>;
  using RegD = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kTM / kWarpPerRow / 16, kTP / 16>>;
  using RegDCast = RegTile<BaseTileAccRowMajor<InType>, tl::RowMajor<kTM / kWarpPerRow / 16, kTP / 16>>;
  using ConvertD = compute::RegTileConvert<RegD, RegDCast>;
  using StorerD = RegToGlobalStorer<GlobalD, RegDCast, WarpLayout>;

  static constexpr int kSharedBytes =
      (SharedA::kNumel + SharedB::kNumel + SharedC::kNumel + SharedP::kNumel) * (int)sizeof(InType);
};

template <typename InType, typename AccType, typename KeTraits>
DEVICE void ke_fused_two_gemms(const InType* dA, const InType* dB, const InType* dC, InType* dD) {
  using T = KeTraits;
  constexpr int kM = T::kM, kN = T::kN, kK = T::kK, kP = T::kP, kTM = T::kTM, kTP = T::kTP;
  const InType* A = dA + ptrdiff_t(blockIdx.z) * kM * kK + ptrdiff_t(blockIdx.x) * kTM * kK;
  const InType* B = dB + ptrdiff_t(blockIdx.z) * kK * kN;
  const InType* C = dC + ptrdiff_t(blockIdx.z) * kN * kP + ptrdiff_t(blockIdx.y) * kTP * kN;
  InType* D = dD + ptrdiff_t(blockIdx.z) * kM * kP + ptrdiff_t(blockIdx.x) * kTM * kP + blockIdx.y * kTP;

  extern __shared__ __attribute__((aligned(16))) unsigned char tilefusion_lds[];
  InType* lds = reinterpret_cast<InType*>(tilefusion_lds);
  typename T::SharedA sA(lds);
  typename T::SharedB sB(lds + T::SharedA::kNumel);
  typename T::SharedC sC(lds + T::SharedA::kNumel + T::SharedB::kNumel);
  typename T::SharedP sP(lds + T::SharedA::kNumel + T::SharedB::kNumel + T::SharedC::kNumel);

  typename T::GIteratorA gAs(A);
  typename T::GIteratorB gBs(B);
  typename T::GIteratorC gCs(C);
  typename T::SharedALoader load_sa;
  typename T::SharedBLoader load_sb;
  typename T::SharedCLoader load_sc;
  typename T::RegALoader load_ra;
  typename T::RegBLoader load_rb;
  typename T::RegCLoader load_rc;
  typename T::RegA rA;
  typename T::RegB rB;
  typename T::RegC rC;
  typename T::RegP rP;
  typename T::RegAcc acc;
  typename T::RegAccCast acc_half;
  typename T::RegD rD;

  for (int n = 0; n < T::GIteratorC::sc0; ++n) {
    load_sc(gCs(n), sC);
    for (int k = 0; k < T::GIteratorA::sc1; ++k) {
      load_sa(gAs(k), sA);
      load_sb(gBs(k, n), sB);
      __copy_async();
      __syncthreads();
      load_ra(sA, rA);
      load_rb(sB, rB);
      compute::gemm(rA, rB, acc);
      __syncthreads();  // sA / sB are overwritten by the next chunk
    }
    typename T::ConvertHalf to_half;
    to_half(acc, acc_half);
    typename T::StorerP store_p;
    store_p(acc_half, sP);
    __copy_async();
    __syncthreads();
    typename T::LoaderP load_p;
    load_p(sP, rP);
    load_rc(sC, rC);
    compute::gemm(rP, rC, rD);
    acc.clear();
    __syncthreads();  // sP / sC are overwritten by the next n-chunk
  }
  typename T::RegDCast out;
  typename T::ConvertD to_out;
  to_out(rD, out);
  typename T::GlobalD gD(D);
  typename T::StorerD store_d;
  store_d(out, gD);
}

}  // namespace tilefusion::kernels
