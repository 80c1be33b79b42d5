// GEMM macro kernel composed from the tile primitives (counterpart of
// include/kernels/gemm_device.cuh:16-419): C[M,N] = A[M,K] * B[K,N], A row-major, B column-major,
// one workgroup per [kTM, kTN] tile of C, K walked in kTK chunks through LDS and in kRK steps
// through registers.
//
// This is the portable, shape-generic form of the kernel - every shape is a template
// parameter and any kernel written against the tile API composes the same way.  The library's
// own tuned GEMM entry point (tf_gemm_f16) is a separate hand-scheduled kernel.
//
// The traits are the reference's, formula for formula (base tiles are 16 x 16, a register step
// kRK is a multiple of 16); what follows from the hardware: a wavefront has 64 lanes
// (kThreads = |WarpLayout| * 64), and when kRK is a multiple of 32 the operand fragments are
// held as wide 16 x 32 base tiles (one 16-byte LDS read per lane and MFMA instead of two
// 8-byte ones; same arithmetic).
//
// Three schedules, as in the reference:
//   ke_gemm                  load chunk, wait, multiply (kNumStages >= 2: two LDS buffers, the
//                            next chunk is requested before the current one is multiplied);
//   ke_gemm_level1_pipeline  a global -> LDS Pipeline with asynchronous (LDS-direct) copies and
//                            kNumStages ring slots;
//   ke_gemm_level2_pipeline  the same ring plus a second Pipeline LDS -> registers that fetches
//                            the fragments of step n + 1 while step n multiplies (with three
//                            slots a chunk's copy has the whole previous chunk's multiply to
//                            land).
#pragma once

#include "cell/mod.hpp"
#include "types/mod.hpp"

namespace tilefusion::kernels {
using namespace tilefusion::cell;
using namespace tilefusion::cell::copy;
namespace tl = tile_layout;

template <typename InType_, typename AccType_, typename WarpLayout_, int kM_, int kN_, int kK_, int kTM_,
          int kTN_, int kTK_, int kRK_, int kNumStages_, int kSharedAccess = 64>
struct KeGemmTraits {
  using InType = InType_;
  using AccType = AccType_;
  using WarpLayout = WarpLayout_;
  using BaseShape = BaseTileShape<InType>;  // 16 x 16
  static constexpr int kNumStages = kNumStages_;

  static constexpr int kThreads = tl::get_numel<WarpLayout> * WARP_SIZE;
  static constexpr int kWarpPerRow = tl::num_rows<WarpLayout>;
  static constexpr int kWarpPerCol = tl::num_cols<WarpLayout>;

  static constexpr int kM = kM_, kN = kN_, kK = kK_;
  static constexpr int kTM = kTM_, kTN = kTN_, kTK = kTK_, kRK = kRK_;
  static_assert(kTK % kRK == 0 && kRK % BaseShape::kCols == 0, "kTK must be a multiple of kRK (a multiple of 16)");
  static constexpr bool kSwizzled = true;
  // operand fragments as wide base tiles when a register step is whole 32-deep blocks
  static constexpr bool kWideOperands = kRK % 32 == 0;
  static constexpr int kOperandK = kWideOperands ? 32 : BaseShape::kCols;
  template <typename T>
  using OperandRowMajor = std::conditional_t<kWideOperands, RegTile<T, tl::RowMajor<1, 8>>, BaseTileRowMajor<T>>;
  template <typename T>
  using OperandColMajor = std::conditional_t<kWideOperands, RegTile<T, tl::ColMajor<8, 1>>, BaseTileColMajor<T>>;

  using GlobalA = GlobalTile<InType, tl::RowMajor<kTM, kK, kK>>;
  using GIteratorA = GTileIterator<GlobalA, TileShape<kTM, kTK>>;
  using SharedA = SharedTile<InType, tl::RowMajor<kTM, kTK>, kSwizzled, kSharedAccess>;
  using SIteratorA = STileIterator<SharedA, TileShape<kTM, kRK>>;
  static constexpr int kAMs = kTM / kWarpPerRow / BaseShape::kRows;
  static constexpr int kAKs = kRK / kOperandK;
  using RegA = RegTile<OperandRowMajor<InType>, tl::RowMajor<kAMs, kAKs>>;
  using G2SLoaderA = GlobalToSharedLoader<SharedA, WarpLayout>;
  using S2RLoaderA = SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;

  using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kTN, kK>>;
  using GIteratorB = GTileIterator<GlobalB, TileShape<kTK, kTN>>;
  using SharedB = SharedTile<InType, tl::ColMajor<kTK, kTN>, kSwizzled, kSharedAccess>;
  using SIteratorB = STileIterator<SharedB, TileShape<kRK, kTN>>;
  static_assert(GIteratorA::sc1 == GIteratorB::sc0 && SIteratorA::sc1 == SIteratorB::sc0, "mismatched K dimension");
  static constexpr int kBKs = kRK / kOperandK;
  static constexpr int kBNs = kTN / kWarpPerCol / BaseShape::kCols;
  using RegB = RegTile<OperandColMajor<InType>, tl::ColMajor<kBKs, kBNs>>;
  using G2SLoaderB = GlobalToSharedLoader<SharedB, WarpLayout>;
  using S2RLoaderB = SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;

  using GlobalC = GlobalTile<AccType, tl::RowMajor<kTM, kTN, kN>>;
  using SharedC = SharedTile<AccType, tl::RowMajor<kTM, kTN>, false>;
  static constexpr int kCMs = kTM / kWarpPerRow / BaseShape::kRows;
  static constexpr int kCNs = kTN / kWarpPerCol / BaseShape::kCols;
  using RegC = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kCMs, kCNs>>;
  using RegAcc = RegTile<BaseTileRowMajor<float>, tl::RowMajor<kCMs, kCNs>>;
  using R2GStorerC = RegToGlobalStorer<GlobalC, RegC, WarpLayout>;
  using R2SStorerC = RegToSharedStorer<RegC, WarpLayout>;
  using S2GStorerC = SharedToGlobalStorer<SharedC, WarpLayout>;

  static constexpr int kStageElems = SharedA::kNumel + SharedB::kNumel;
  static constexpr int kLdsStages = kNumStages >= 2 ? 2 : 1;
  static constexpr int kSharedBytes = kStageElems * kLdsStages * (int)sizeof(InType);   // ke_gemm

  // The pipelined kernels keep kNumStages slots of A back to back, then kNumStages slots of B.
  using PipelineG2SA = Pipeline<InType, GlobalA, SharedA, GIteratorA, G2SLoaderA, kNumStages, GIteratorA::sc1>;
  using PipelineG2SB = Pipeline<InType, GlobalB, SharedB, GIteratorB, G2SLoaderB, kNumStages, GIteratorA::sc1>;
  // two register slots: the fragments in use and the ones being fetched
  using PipelineS2RA = Pipeline<InType, SharedA, RegA, SIteratorA, S2RLoaderA, 2, SIteratorA::sc1>;
  using PipelineS2RB = Pipeline<InType, SharedB, RegB, SIteratorB, S2RLoaderB, 2, SIteratorA::sc1>;
  static constexpr int kPipelineSharedBytes = kStageElems * kNumStages * (int)sizeof(InType);
  // vector-memory loads every wavefront issues for one k-chunk (what wait_group counts in)
  static constexpr int kLoadsPerChunk = G2SLoaderA::kLoadsPerLane + G2SLoaderB::kLoadsPerLane;
};

namespace detail {
template <typename KeTraits, typename InType, typename AccType>
DEVICE void store_acc(const typename KeTraits::RegAcc& acc, AccType* dC) {
  typename KeTraits::GlobalC gC(dC);
  typename KeTraits::R2GStorerC r2g;
  if constexpr (std::is_same_v<AccType, float>) {
    r2g(acc, gC);
  } else {
    typename KeTraits::RegC out;
    compute::RegTileConvert<typename KeTraits::RegAcc, typename KeTraits::RegC> cast;
    cast(acc, out);
    r2g(out, gC);
  }
}
}  // namespace detail

// kNumStages == 1: load chunk, synchronise, multiply.  kNumStages >= 2: double-buffered LDS.
template <typename InType, typename AccType, typename KeTraits>
DEVICE void ke_gemm(const InType* dA, const InType* dB, AccType* dC) {
  constexpr int kN = KeTraits::kN, kK = KeTraits::kK, kTM = KeTraits::kTM, kTN = KeTraits::kTN;
  const InType* gA_ptr = dA + ptrdiff_t(blockIdx.x) * kTM * kK;
  const InType* gB_ptr = dB + ptrdiff_t(blockIdx.y) * kTN * kK;
  AccType* gC_ptr = dC + ptrdiff_t(blockIdx.x) * kTM * kN + ptrdiff_t(blockIdx.y) * kTN;

  extern __shared__ __attribute__((aligned(16))) unsigned char tilefusion_lds[];
  InType* lds = reinterpret_cast<InType*>(tilefusion_lds);

  typename KeTraits::GIteratorA gAs(gA_ptr);
  typename KeTraits::GIteratorB gBs(gB_ptr);
  typename KeTraits::RegA rA;
  typename KeTraits::RegB rB;
  typename KeTraits::RegAcc acc;
  typename KeTraits::G2SLoaderA g2s_a;
  typename KeTraits::G2SLoaderB g2s_b;
  typename KeTraits::S2RLoaderA s2r_a;
  typename KeTraits::S2RLoaderB s2r_b;

  constexpr int kChunks = KeTraits::GIteratorA::sc1;
  constexpr int kStages = KeTraits::kLdsStages;
  auto stage_a = [&](int s) { return typename KeTraits::SharedA(lds + s * KeTraits::kStageElems); };
  auto stage_b = [&](int s) {
    return typename KeTraits::SharedB(lds + s * KeTraits::kStageElems + KeTraits::SharedA::kNumel);
  };

  if constexpr (kStages == 2) {
    auto sA0 = stage_a(0);
    auto sB0 = stage_b(0);
    g2s_a(gAs(0), sA0);
    g2s_b(gBs(0), sB0);
    __copy_async();
    __syncthreads();
  }
  for (int k1 = 0; k1 < kChunks; ++k1) {
    const int cur = kStages == 2 ? (k1 & 1) : 0;
    if constexpr (kStages == 2) {
      if (k1 + 1 < kChunks) {
        auto sAn = stage_a(cur ^ 1);
        auto sBn = stage_b(cur ^ 1);
        g2s_a(gAs(k1 + 1), sAn);
        g2s_b(gBs(k1 + 1), sBn);
      }
    } else {
      auto sA0 = stage_a(0);
      auto sB0 = stage_b(0);
      g2s_a(gAs(k1), sA0);
      g2s_b(gBs(k1), sB0);
      __copy_async();
      __syncthreads();
    }
    typename KeTraits::SIteratorA sAs(lds + cur * KeTraits::kStageElems);
    typename KeTraits::SIteratorB sBs(lds + cur * KeTraits::kStageElems + KeTraits::SharedA::kNumel);
#pragma unroll
    for (int k2 = 0; k2 < KeTraits::SIteratorA::sc1; ++k2) {
      s2r_a(sAs(k2), rA);
      s2r_b(sBs(k2), rB);
      compute::gemm(rA, rB, acc);
    }
    __copy_async();
    __syncthreads();
  }
  detail::store_acc<KeTraits, InType, AccType>(acc, gC_ptr);
}

// Level 1: global -> LDS through a Pipeline of kNumStages slots with asynchronous copies
// (counterpart of include/kernels/gemm_device.cuh:170-250).  kAhead = kNumStages - 1 chunks
// are in flight ahead of the one being multiplied.
template <typename InType, typename AccType, typename KeTraits>
DEVICE void ke_gemm_level1_pipeline(const InType* dA, const InType* dB, AccType* dC) {
  static_assert(KeTraits::kNumStages >= 2, "the pipelined kernels need kNumStages >= 2");
  constexpr int kN = KeTraits::kN, kK = KeTraits::kK, kTM = KeTraits::kTM, kTN = KeTraits::kTN;
  constexpr int kStages = KeTraits::kNumStages, kAhead = kStages - 1;
  constexpr int kChunks = KeTraits::GIteratorA::sc1, kLoads = KeTraits::kLoadsPerChunk;
  const InType* gA_ptr = dA + ptrdiff_t(blockIdx.x) * kTM * kK;
  const InType* gB_ptr = dB + ptrdiff_t(blockIdx.y) * kTN * kK;
  AccType* gC_ptr = dC + ptrdiff_t(blockIdx.x) * kTM * kN + ptrdiff_t(blockIdx.y) * kTN;

  extern __shared__ __attribute__((aligned(1024))) unsigned char tilefusion_lds[];
  InType* sA_ptr = reinterpret_cast<InType*>(tilefusion_lds);
  InType* sB_ptr = sA_ptr + KeTraits::SharedA::kNumel * kStages;

  typename KeTraits::RegA rA;
  typename KeTraits::RegB rB;
  typename KeTraits::RegAcc acc;
  typename KeTraits::S2RLoaderA s2r_a;
  typename KeTraits::S2RLoaderB s2r_b;
  typename KeTraits::PipelineG2SA pipeline_g2s_a(gA_ptr, sA_ptr);
  typename KeTraits::PipelineG2SB pipeline_g2s_b(gB_ptr, sB_ptr);

  // chunks 0 .. kAhead-1 before the loop, one copy group each
#pragma unroll
  for (int i = 0; i < kAhead && i < kChunks; ++i) {
    pipeline_g2s_a.commit();
    pipeline_g2s_b.commit();
    commit_copy_group();
  }
  for (int k = 0; k < kChunks; ++k) {
    // chunk k must have landed; the groups of chunks k+1 .. k+kAhead-1 may stay in flight
    // (near the end fewer have been issued: wait for everything)
    if (k + kAhead <= kChunks) wait_group<kAhead - 1, kLoads>();
    else wait_group<0>();
    // also the point where every wavefront is done with chunk k-1, whose slot is refilled next
    sync_threads_keep_copies();
    if (k + kAhead < kChunks) {
      pipeline_g2s_a.commit();
      pipeline_g2s_b.commit();
      commit_copy_group();
    }
    typename KeTraits::SIteratorA sAs(pipeline_g2s_a.get_dst_ptr_by_index(k));
    typename KeTraits::SIteratorB sBs(pipeline_g2s_b.get_dst_ptr_by_index(k));
#pragma unroll
    for (int k2 = 0; k2 < KeTraits::SIteratorA::sc1; ++k2) {
      s2r_a(sAs(k2), rA);
      s2r_b(sBs(k2), rB);
      compute::gemm(rA, rB, acc);
    }
  }
  detail::store_acc<KeTraits, InType, AccType>(acc, gC_ptr);
}

// Level 2: the level-1 ring plus a register-level Pipeline - the fragments of step n + 1 are
// read from LDS while step n multiplies (counterpart of include/kernels/gemm_device.cuh:252-419).
template <typename InType, typename AccType, typename KeTraits>
DEVICE void ke_gemm_level2_pipeline(const InType* dA, const InType* dB, AccType* dC) {
  static_assert(KeTraits::kNumStages >= 2, "the pipelined kernels need kNumStages >= 2");
  constexpr int kN = KeTraits::kN, kK = KeTraits::kK, kTM = KeTraits::kTM, kTN = KeTraits::kTN;
  constexpr int kStages = KeTraits::kNumStages, kAhead = kStages - 1;
  constexpr int kChunks = KeTraits::GIteratorA::sc1, kSteps = KeTraits::SIteratorA::sc1;
  constexpr int kLoads = KeTraits::kLoadsPerChunk;
  const InType* gA_ptr = dA + ptrdiff_t(blockIdx.x) * kTM * kK;
  const InType* gB_ptr = dB + ptrdiff_t(blockIdx.y) * kTN * kK;
  AccType* gC_ptr = dC + ptrdiff_t(blockIdx.x) * kTM * kN + ptrdiff_t(blockIdx.y) * kTN;

  extern __shared__ __attribute__((aligned(1024))) unsigned char tilefusion_lds[];
  InType* sA_ptr = reinterpret_cast<InType*>(tilefusion_lds);
  InType* sB_ptr = sA_ptr + KeTraits::SharedA::kNumel * kStages;

  typename KeTraits::RegAcc acc;
  typename KeTraits::PipelineG2SA pipeline_g2s_a(gA_ptr, sA_ptr);
  typename KeTraits::PipelineG2SB pipeline_g2s_b(gB_ptr, sB_ptr);

#pragma unroll
  for (int i = 0; i < kAhead && i < kChunks; ++i) {
    pipeline_g2s_a.commit();
    pipeline_g2s_b.commit();
    commit_copy_group();
  }
  // Transition from chunk k to chunk k + 1 (k = -1: from the prologue into chunk 0).  Chunks
  // 0 .. k + kAhead have been issued; chunk k + 1 must have landed, so kAhead - 1 groups may
  // stay in flight (fewer near the end: wait for everything).  After the barrier every
  // wavefront is done with chunk k, whose slot takes chunk k + 1 + kAhead.
  auto advance = [&](int k) {
    if (k + kAhead < kChunks) wait_group<kAhead - 1, kLoads>();
    else wait_group<0>();
    sync_threads_keep_copies();
    if (k + 1 + kAhead < kChunks) {
      pipeline_g2s_a.commit();
      pipeline_g2s_b.commit();
      commit_copy_group();
    }
  };
  advance(-1);

  typename KeTraits::RegA rA_ring[2];
  typename KeTraits::RegB rB_ring[2];
  typename KeTraits::PipelineS2RA pipeline_s2r_a(typename KeTraits::SharedA(pipeline_g2s_a.get_dst_ptr_by_index(0)),
                                                 rA_ring);
  typename KeTraits::PipelineS2RB pipeline_s2r_b(typename KeTraits::SharedB(pipeline_g2s_b.get_dst_ptr_by_index(0)),
                                                 rB_ring);
  pipeline_s2r_a.template commit_to<0>();   // fragments of step 0 -> register slot 0
  pipeline_s2r_b.template commit_to<0>();

  // One chunk: kSteps multiply steps, each fetching the fragments of the step after it into the
  // other register slot.  Step n of the whole run uses slot n % 2; the slots are named at
  // compile time (kFirst = slot of the chunk's first step), so with an odd kSteps consecutive
  // chunks alternate between the two instantiations.
  auto chunk = [&]<int kFirst>(int k) {
#pragma unroll
    for (int k2 = 0; k2 < kSteps; ++k2) {
      constexpr int kDummy = 0;
      (void)kDummy;
      auto step = [&]<int kSlot>() {
        if (k2 + 1 < kSteps) {
          pipeline_s2r_a.template commit_to<kSlot ^ 1>();   // next step of this chunk
          pipeline_s2r_b.template commit_to<kSlot ^ 1>();
        } else if (k + 1 < kChunks) {
          // last step of chunk k: its fragments are in registers already, so the next
          // fragments come from chunk k + 1
          advance(k);
          pipeline_s2r_a.reset_src_tile(pipeline_g2s_a.get_dst_ptr_by_index(k + 1));
          pipeline_s2r_b.reset_src_tile(pipeline_g2s_b.get_dst_ptr_by_index(k + 1));
          pipeline_s2r_a.template commit_to<kSlot ^ 1>();
          pipeline_s2r_b.template commit_to<kSlot ^ 1>();
        }
        compute::gemm(pipeline_s2r_a.template get_dst_tile<kSlot>(), pipeline_s2r_b.template get_dst_tile<kSlot>(),
                      acc);
      };
      if ((kFirst + k2) % 2 == 0) step.template operator()<0>();
      else step.template operator()<1>();
    }
  };
  if constexpr (kSteps % 2 == 0) {
    for (int k = 0; k < kChunks; ++k) chunk.template operator()<0>(k);
  } else {
    int k = 0;
    for (; k + 1 < kChunks; k += 2) {
      chunk.template operator()<0>(k);
      chunk.template operator()<1>(k + 1);
    }
    if (k < kChunks) chunk.template operator()<0>(k);
  }
  detail::store_acc<KeTraits, InType, AccType>(acc, gC_ptr);
}

}  // namespace tilefusion::kernels
