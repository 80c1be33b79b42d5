// Flash-attention forward composed from the tile primitives (counterpart of
// include/kernels/flash_attention_device.cuh:16-312): O[M,P] = softmax(scale * Q[M,K] K[K,N]
// (+ causal mask)) V[N,P]; Q, O row-major, K and V column-major (V is handed over transposed,
// as a [P][N] buffer); one workgroup per [kTM, kTP] tile of O, wavefronts stacked along M.
//
// Differences from the reference: running max / sum are fp32 and start at -inf / 0 (the
// reference keeps them in fp16 and starts the max at 0); the output stays un-normalised until
// the end (one divide instead of one per key tile); the causal mask skips key tiles that lie
// entirely above the diagonal.  The score tile is a tile of row-major base tiles, which is the
// layout of an A operand (types/register.hpp): exp(S - max) is rounded to fp16 element by element
// and fed to the second gemm() straight from registers, as in the reference.  Q and K are held as
// wide 16 x 32 base tiles when kTK is a multiple of 32.
//
// When one k-chunk covers the whole head dimension (kTK == kK) the Q tile is fetched once and
// stays in registers (the reference reloads it per key tile,
// include/kernels/flash_attention_device.cuh:231-262).  K / V tiles keep one LDS buffer each:
// double-buffering them was measured and loses more to the lower occupancy (two instead of three
// workgroups per CU at a head dimension of 96) than the overlap gains, because co-resident
// workgroups already cover each other's loads.
#pragma once

#include "cell/mod.hpp"
#include "types/mod.hpp"

namespace tilefusion::kernels {
using namespace tilefusion::cell;
using namespace tilefusion::cell::copy;
namespace tl = tile_layout;

template <typename InType_, typename AccType_, typename OutType_, typename WholeShape, typename CtaTileShape,
          typename WarpLayout_, double kSoftmaxScale_, bool kIsCausal_>
struct FlashAttentionTraits {
  using InType = InType_;
  using AccType = AccType_;
  using OutType = OutType_;
  using WarpLayout = WarpLayout_;
  static constexpr int kWarpPerRow = tl::num_rows<WarpLayout>;
  static constexpr int kWarpPerCol = tl::num_cols<WarpLayout>;
  static_assert(kWarpPerCol == 1, "wavefronts must be arranged as a column vector");
  static constexpr int kThreads = tl::get_numel<WarpLayout> * WARP_SIZE;
  static constexpr int kSharedAccess = 64;
  using BaseShape = BaseTileShape<InType>;

  static constexpr int kM = dim_size<0, WholeShape>;  // query length
  static constexpr int kN = dim_size<1, WholeShape>;  // key / value length
  static constexpr int kK = dim_size<2, WholeShape>;  // query / key hidden dim
  static constexpr int kP = dim_size<3, WholeShape>;  // value hidden dim
  static constexpr int kTM = dim_size<0, CtaTileShape>;
  static constexpr int kTN = dim_size<1, CtaTileShape>;
  static constexpr int kTK = dim_size<2, CtaTileShape>;
  static constexpr int kTP = dim_size<3, CtaTileShape>;
  static_assert(kTK % 16 == 0 && kTN % 16 == 0 && kTP % 16 == 0 && (kTM / kWarpPerRow) % 16 == 0,
                "tile sizes must be whole base tiles");
  static constexpr double kSoftmaxScale = kSoftmaxScale_;
  static constexpr bool kIsCausal = kIsCausal_;
  static constexpr bool kWideOperands = kTK % 32 == 0;
  static constexpr int kOperandK = kWideOperands ? 32 : BaseShape::kCols;
  template <typename T>
  using OperandRowMajor = std::conditional_t<kWideOperands, RegTile<T, tl::RowMajor<1, 8>>, BaseTileRowMajor<T>>;
  template <typename T>
  using OperandColMajor = std::conditional_t<kWideOperands, RegTile<T, tl::ColMajor<8, 1>>, BaseTileColMajor<T>>;

  using GlobalQ = GlobalTile<InType, tl::RowMajor<kTM, kK>>;
  using GIteratorQ = GTileIterator<GlobalQ, TileShape<kTM, kTK>>;
  using SharedQ = SharedTile<InType, tl::RowMajor<kTM, kTK>, true, kSharedAccess>;
  static constexpr int kQMs = kTM / kWarpPerRow / BaseShape::kRows;
  static constexpr int kQKs = kTK / kOperandK;
  using RegQ = RegTile<OperandRowMajor<InType>, tl::RowMajor<kQMs, kQKs>>;
  using SharedQLoader = GlobalToSharedLoader<SharedQ, WarpLayout>;
  using RegQLoader = SharedToRegLoader<RegQ, WarpLayout, WarpReuse::kRowReuseCont>;

  using GlobalK = GlobalTile<InType, tl::ColMajor<kK, kN>>;
  using GIteratorK = GTileIterator<GlobalK, TileShape<kTK, kTN>>;
  using SharedK = SharedTile<InType, tl::ColMajor<kTK, kTN>, true, kSharedAccess>;
  static constexpr int kKKs = kTK / kOperandK;
  static constexpr int kKNs = kTN / kWarpPerCol / BaseShape::kCols;
  using RegK = RegTile<OperandColMajor<InType>, tl::ColMajor<kKKs, kKNs>>;
  using SharedKLoader = GlobalToSharedLoader<SharedK, WarpLayout>;
  using RegKLoader = SharedToRegLoader<RegK, WarpLayout, WarpReuse::kColReuseCont>;

  using GlobalV = GlobalTile<InType, tl::ColMajor<kN, kTP>>;
  using GIteratorV = GTileIterator<GlobalV, TileShape<kTN, kTP>>;
  using SharedV = SharedTile<InType, tl::ColMajor<kTN, kTP>, true, kSharedAccess>;
  static constexpr int kVNs = kTN / BaseShape::kRows;
  static constexpr int kVPs = kTP / kWarpPerCol / BaseShape::kCols;
  using RegV = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kVNs, kVPs>>;
  using SharedVLoader = GlobalToSharedLoader<SharedV, WarpLayout>;
  using RegVLoader = SharedToRegLoader<RegV, WarpLayout, WarpReuse::kColReuseCont>;

  using GlobalO = GlobalTile<OutType, tl::RowMajor<kTM, kTP, kP>>;
  static constexpr int kOMs = kTM / kWarpPerRow / BaseShape::kRows;
  static constexpr int kOPs = kTP / kWarpPerCol / BaseShape::kCols;
  using RegO = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kOMs, kOPs>>;
  using RegOCast = RegTile<BaseTileRowMajor<OutType>, tl::RowMajor<kOMs, kOPs>>;
  using ConvertO = compute::RegTileConvert<RegO, RegOCast>;
  using OStorer = RegToGlobalStorer<GlobalO, RegOCast, WarpLayout>;

  static constexpr int kAccMs = kTM / kWarpPerRow / BaseShape::kRows;
  static constexpr int kAccNs = kTN / kWarpPerCol / BaseShape::kCols;
  using RegAcc = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kAccMs, kAccNs>>;
  using RegAccCast = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kAccMs, kAccNs>>;
  using ConvertAcc = compute::RegTileConvert<RegAcc, RegAccCast>;

  // one statistic per row a lane owns: one per base-tile row (fp32)
  using RegVec = RegTile<AccType, tl::RowMajor<kAccMs, 1>>;
  using RowMax = compute::MaxReduce<RegAcc, tl::Layout::kRowMajor>;
  using RowSum = compute::SumReduce<RegAcc, tl::Layout::kRowMajor>;
  using BroadcastSub = compute::BroadcastSub<RegVec, RegAcc, tl::Layout::kRowMajor>;
  using BroadcastMul = compute::BroadcastMul<RegVec, RegO, tl::Layout::kRowMajor>;
  using BroadcastDiv = compute::BroadcastDiv<RegVec, RegO, tl::Layout::kRowMajor>;
  using BlockExp = compute::RegTileExp<RegAcc>;
  using VecMax = compute::BaseTileMax<RegVec>;
  using VecAdd = compute::BaseTileAdd<RegVec>;
  using VecSub = compute::BaseTileSub<RegVec>;
  using VecMul = compute::BaseTileMul<RegVec>;
  using VecExp = compute::BaseTileExp<RegVec>;
  using ApplyMask = cell::ApplyMask<RegAcc, WarpLayout, BaseShape, MaskMode::kCausal>;
  using ApplyScoreScale = compute::BroadcastScalarMul<RegAcc>;

  // the whole head dimension in one chunk: Q is fetched once (see above)
  static constexpr bool kWholeK = kTK == kK;
  static constexpr int kSharedBytes = (SharedQ::kNumel + SharedK::kNumel + SharedV::kNumel) * (int)sizeof(InType);
};

template <typename InType, typename AccType, typename OutType, typename KeTraits>
DEVICE void ke_flash_attention(const InType* dQ, const InType* dK, const InType* dV, OutType* dO) {
  using T = KeTraits;
  constexpr int kM = T::kM, kN = T::kN, kK = T::kK, kP = T::kP;
  constexpr int kTM = T::kTM, kTN = T::kTN, kTP = T::kTP;
  const InType* Q = dQ + ptrdiff_t(blockIdx.z) * kM * kK + ptrdiff_t(blockIdx.x) * kTM * kK;
  const InType* K = dK + ptrdiff_t(blockIdx.z) * kK * kN;
  const InType* V = dV + ptrdiff_t(blockIdx.z) * kN * kP + ptrdiff_t(blockIdx.y) * kTP * kN;
  OutType* O = dO + ptrdiff_t(blockIdx.z) * kM * kP + ptrdiff_t(blockIdx.x) * kTM * kP + blockIdx.y * kTP;

  extern __shared__ __attribute__((aligned(16))) unsigned char tilefusion_lds[];
  InType* lds = reinterpret_cast<InType*>(tilefusion_lds);
  typename T::SharedQ sQ(lds);
  typename T::SharedK sK(lds + T::SharedQ::kNumel);
  typename T::SharedV sV(lds + T::SharedQ::kNumel + T::SharedK::kNumel);

  typename T::GIteratorQ gQs(Q);
  typename T::GIteratorK gKs(K);
  typename T::GIteratorV gVs(V);
  typename T::SharedQLoader load_sq;
  typename T::SharedKLoader load_sk;
  typename T::SharedVLoader load_sv;
  typename T::RegQLoader load_rq;
  typename T::RegKLoader load_rk;
  typename T::RegVLoader load_rv;
  typename T::RegQ rQ;
  typename T::RegK rK;
  typename T::RegV rV;
  typename T::RegAcc s;
  typename T::RegAccCast p_half;
  typename T::RegO o;
  typename T::RegVec run_max, run_sum, cur_max, cur_sum, new_max, alpha;
#pragma unroll
  for (int i = 0; i < T::RegVec::kNumel; ++i) run_max.mutable_data()[i] = -INFINITY;

  const int row_base = blockIdx.x * kTM;
  // causal: key tiles that start after the last row of this workgroup contribute nothing
  const int n_tiles = T::kIsCausal ? min((int)T::GIteratorV::sc0, (row_base + kTM + kTN - 1) / kTN)
                                   : (int)T::GIteratorV::sc0;
  // scale, mask, online softmax of the score tile `s` of key tile n; leaves the fp16 weights in p_half
  auto softmax_tile = [&](int n) {
    typename T::ApplyScoreScale scale;
    scale(s, AccType(T::kSoftmaxScale), s);
    if constexpr (T::kIsCausal) {
      typename T::ApplyMask mask;
      mask(s, row_base, n * kTN, -INFINITY);
    }
    typename T::RowMax row_max;
    row_max(s, cur_max);
    typename T::VecMax vmax;
    vmax(cur_max, run_max, new_max);
    // a row that is still fully masked keeps max = -inf; shift by 0 there so exp() sees -inf, not nan
#pragma unroll
    for (int i = 0; i < T::RegVec::kNumel; ++i) {
      const AccType m = new_max.data()[i];
      const AccType safe = (m == -INFINITY) ? AccType(0) : m;
      alpha.mutable_data()[i] = __expf(run_max.data()[i] - safe);
      cur_max.mutable_data()[i] = safe;
    }
    typename T::BroadcastSub sub;
    sub(cur_max, s);
    typename T::BlockExp block_exp;
    block_exp(s, s);
    typename T::RowSum row_sum;
    row_sum(s, cur_sum);
    typename T::VecMul vmul;
    vmul(run_sum, alpha, run_sum);
    typename T::VecAdd vadd;
    vadd(run_sum, cur_sum, run_sum);
    typename T::BroadcastMul rescale;
    rescale(alpha, o);
    copy_tile(new_max, run_max);

    typename T::ConvertAcc to_half;
    to_half(s, p_half);
  };

  if constexpr (T::kWholeK) {
    load_sq(gQs(0), sQ);
    for (int n = 0; n < n_tiles; ++n) {
      load_sk(gKs(0, n), sK);
      load_sv(gVs(n), sV);
      __copy_async();
      __syncthreads();
      if (n == 0) load_rq(sQ, rQ);   // stays in registers for every key tile
      load_rk(sK, rK);
      compute::gemm(rQ, rK, s);
      softmax_tile(n);
      load_rv(sV, rV);
      compute::gemm(p_half, rV, o);
      s.clear();
      __syncthreads();   // nobody still reads this tile
    }
  } else {
    for (int n = 0; n < n_tiles; ++n) {
      load_sv(gVs(n), sV);
      for (int k = 0; k < T::GIteratorQ::sc1; ++k) {
        load_sq(gQs(k), sQ);
        load_sk(gKs(k, n), sK);
        __copy_async();
        __syncthreads();
        load_rq(sQ, rQ);
        load_rk(sK, rK);
        compute::gemm(rQ, rK, s);
        __syncthreads();
      }
      softmax_tile(n);
      load_rv(sV, rV);
      compute::gemm(p_half, rV, o);
      s.clear();
      __syncthreads();
    }
  }
  typename T::BroadcastDiv normalise;
  normalise(run_sum, o);
  typename T::RegOCast out;
  typename T::ConvertO to_out;
  to_out(o, out);
  typename T::GlobalO gO(O);
  typename T::OStorer store_o;
  store_o(out, gO);
}

}  // namespace tilefusion::kernels
