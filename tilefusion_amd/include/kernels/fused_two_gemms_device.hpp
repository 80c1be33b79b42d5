// Fused back-to-back GEMM composed from the tile primitives (counterpart of
// include/kernels/fused_two_gemms_device.cuh:16-214): D[M,P] = (A[M,K] * B[K,N]) * C[N,P] with A,
// D row-major and B, C column-major; one workgroup per [kTM, kTP] tile of D; the intermediate
// A*B tile never leaves the chip.
//
// The accumulator tile of the first product is a tile of row-major base tiles - the layout of an
// A operand (types/register.hpp) - so, as in the reference, it is converted to fp16 element by
// element and fed to the second gemm() straight from registers.  The first product's own
// operands are held as wide 16 x 32 base tiles when kTK is a multiple of 32.
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
  using BaseShape = BaseTileShape<InType>;  // 16 x 16
  static constexpr int kThreads = tl::get_numel<WarpLayout> * WARP_SIZE;
  static constexpr int kWarpPerRow = tl::num_rows<WarpLayout>;
  static constexpr int kWarpPerCol = tl::num_cols<WarpLayout>;
  static_assert(kWarpPerCol == 1, "wavefronts must be arranged as a column vector");
  static constexpr int kM = kM_, kN = kN_, kK = kK_, kP = kP_;
  static constexpr int kTM = kTM_, kTN = kTN_, kTK = kTK_, kTP = kTP_;
  static constexpr int kSharedAccess = 64;
  static_assert(kTK % 16 == 0 && kTN % 16 == 0 && kTP % 16 == 0 && (kTM / kWarpPerRow) % 16 == 0,
                "tile sizes must be whole base tiles");
  static constexpr bool kWideOperands = kTK % 32 == 0;
  static constexpr int kOperandK = kWideOperands ? 32 : BaseShape::kCols;
  template <typename T>
  using OperandRowMajor = std::conditional_t<kWideOperands, RegTile<T, tl::RowMajor<1, 8>>, BaseTileRowMajor<T>>;
  template <typename T>
  using OperandColMajor = std::conditional_t<kWideOperands, RegTile<T, tl::ColMajor<8, 1>>, BaseTileColMajor<T>>;

  using GlobalA = GlobalTile<InType, tl::RowMajor<kTM, kK>>;
  using GIteratorA = GTileIterator<GlobalA, TileShape<kTM, kTK>>;
  using SharedA = SharedTile<InType, tl::RowMajor<kTM, kTK>, true, kSharedAccess>;
  static constexpr int kAMs = kTM / kWarpPerRow / BaseShape::kRows;
  static constexpr int kAKs = kTK / kOperandK;
  using RegA = RegTile<OperandRowMajor<InType>, tl::RowMajor<kAMs, kAKs>>;
  using SharedALoader = GlobalToSharedLoader<SharedA, WarpLayout>;
  using RegALoader = SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;

  using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kN>>;
  using GIteratorB = GTileIterator<GlobalB, TileShape<kTK, kTN>>;
  using SharedB = SharedTile<InType, tl::ColMajor<kTK, kTN>, true, kSharedAccess>;
  static constexpr int kBKs = kTK / kOperandK;
  static constexpr int kBNs = kTN / kWarpPerCol / BaseShape::kCols;
  using RegB = RegTile<OperandColMajor<InType>, tl::ColMajor<kBKs, kBNs>>;
  using SharedBLoader = GlobalToSharedLoader<SharedB, WarpLayout>;
  using RegBLoader = SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;

  using GlobalC = GlobalTile<InType, tl::ColMajor<kN, kTP>>;
  using GIteratorC = GTileIterator<GlobalC, TileShape<kTN, kTP>>;
  using SharedC = SharedTile<InType, tl::ColMajor<kTN, kTP>, true, kSharedAccess>;
  static constexpr int kCNs = kTN / BaseShape::kRows;
  static constexpr int kCPs = kTP / kWarpPerCol / BaseShape::kCols;
  using RegC = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kCNs, kCPs>>;
  using SharedCLoader = GlobalToSharedLoader<SharedC, WarpLayout>;
  using RegCLoader = SharedToRegLoader<RegC, WarpLayout, WarpReuse::kColReuseCont>;

  // intermediate tile: fp32 accumulators, converted in place to the A operand of the second product
  static constexpr int kAccMs = kTM / kWarpPerRow / BaseShape::kRows;
  static constexpr int kAccNs = kTN / kWarpPerCol / BaseShape::kCols;
  using RegAcc = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kAccMs, kAccNs>>;
  using RegAccCast = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kAccMs, kAccNs>>;
  using ConvertHalf = compute::RegTileConvert<RegAcc, RegAccCast>;

  using GlobalD = GlobalTile<InType, tl::RowMajor<kTM, kTP, kP>>;
  static constexpr int kDMs = kTM / kWarpPerRow / BaseShape::kRows;
  static constexpr int kDPs = kTP / kWarpPerCol / BaseShape::kCols;
  using RegD = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kDMs, kDPs>>;
  using RegDHalf = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kDMs, kDPs>>;
  using ConvertD = compute::RegTileConvert<RegD, RegDHalf>;
  using StorerD = RegToGlobalStorer<GlobalD, RegDHalf, WarpLayout>;

  static constexpr int kSharedBytes = (SharedA::kNumel + SharedB::kNumel + SharedC::kNumel) * (int)sizeof(InType);
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
    load_rc(sC, rC);
    compute::gemm(acc_half, rC, rD);
    acc.clear();
    __syncthreads();  // sC is overwritten by the next n-chunk
  }
  typename T::RegDHalf out;
  typename T::ConvertD to_out;
  to_out(rD, out);
  typename T::GlobalD gD(D);
  typename T::StorerD store_d;
  store_d(out, gD);
}

}  // namespace tilefusion::kernels
