// Wavefront-level matrix multiply on register tiles (counterpart of
// include/cell/compute/gemm.hpp:18-201): c(i, j) += sum_k a(i, k) * b(k, j) over MFMA base tiles.
//
// The hardware atom is v_mfma_f32_16x16x32_{f16,bf16}: A base tile 16 x 32, B base tile 32 x 16,
// C base tile 16 x 16 (see types/register.hpp for the lane maps).  The reference's default
// atom tag MMA_ATOM_16x16x16 is kept as a name and selects this instruction.
#pragma once

#include "types/register.hpp"

namespace tilefusion::cell::compute {
namespace tl = tile_layout;

struct MMA_ATOM_16x16x32 {};
using MMA_ATOM_16x16x16 = MMA_ATOM_16x16x32;

namespace detail {
using half8_v = _Float16 __attribute__((ext_vector_type(8)));
using bf16x8_v = __bf16 __attribute__((ext_vector_type(8)));
using float4_v = float __attribute__((ext_vector_type(4)));
}  // namespace detail

template <typename InTypeA, typename InTypeB, typename AccType, typename AtomicShape = MMA_ATOM_16x16x16>
struct MmaAtom;

template <>
struct MmaAtom<__half, __half, float, MMA_ATOM_16x16x32> {
  using BaseTileA = BaseTileRowMajor<__half>;
  using BaseTileB = BaseTileColMajor<__half>;
  using BaseTileC = BaseTileRowMajor<float>;
  using BaseTile = BaseTileShape<__half>;
  DEVICE void operator()(const BaseTileA& a, const BaseTileB& b, BaseTileC& c) const {
    const auto va = *reinterpret_cast<const detail::half8_v*>(a.data());
    const auto vb = *reinterpret_cast<const detail::half8_v*>(b.data());
    auto vc = *reinterpret_cast<detail::float4_v*>(c.mutable_data());
    vc = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, vb, vc, 0, 0, 0);
    *reinterpret_cast<detail::float4_v*>(c.mutable_data()) = vc;
  }
};

template <>
struct MmaAtom<__bfloat16, __bfloat16, float, MMA_ATOM_16x16x32> {
  using BaseTileA = BaseTileRowMajor<__bfloat16>;
  using BaseTileB = BaseTileColMajor<__bfloat16>;
  using BaseTileC = BaseTileRowMajor<float>;
  using BaseTile = BaseTileShape<__bfloat16>;
  DEVICE void operator()(const BaseTileA& a, const BaseTileB& b, BaseTileC& c) const {
    const auto va = *reinterpret_cast<const detail::bf16x8_v*>(a.data());
    const auto vb = *reinterpret_cast<const detail::bf16x8_v*>(b.data());
    auto vc = *reinterpret_cast<detail::float4_v*>(c.mutable_data());
    vc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, vb, vc, 0, 0, 0);
    *reinterpret_cast<detail::float4_v*>(c.mutable_data()) = vc;
  }
};

// fp16 accumulator tile (counterpart of MmaAtom<__half, __half, __half>, include/cell/compute/
// gemm.hpp:63-105).  CDNA4 has no MFMA that accumulates in fp16: the product is accumulated in
// fp32 by the same instruction and rounded to fp16 once per atom, which is at least as
// accurate as the reference's fp16-accumulating mma.sync.
template <>
struct MmaAtom<__half, __half, __half, MMA_ATOM_16x16x32> {
  using BaseTileA = BaseTileRowMajor<__half>;
  using BaseTileB = BaseTileColMajor<__half>;
  using BaseTileC = BaseTileAccRowMajor<__half>;
  using BaseTile = BaseTileShape<__half>;
  DEVICE void operator()(const BaseTileA& a, const BaseTileB& b, BaseTileC& c) const {
    const auto va = *reinterpret_cast<const detail::half8_v*>(a.data());
    const auto vb = *reinterpret_cast<const detail::half8_v*>(b.data());
    detail::float4_v vc;
#pragma unroll
    for (int r = 0; r < 4; ++r) vc[r] = to_float(c.data()[r]);
    vc = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, vb, vc, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) c.mutable_data()[r] = from_float<__half>(vc[r]);
  }
};

template <typename RegTileA, typename RegTileB, typename RegTileC, typename AtomicShape = MMA_ATOM_16x16x16>
struct Gemm {
  using InTypeA = typename RegTileA::DType::DType;
  using InTypeB = typename RegTileB::DType::DType;
  using OutType = typename RegTileC::DType::DType;
  using Atom = MmaAtom<InTypeA, InTypeB, OutType, AtomicShape>;
  static_assert(std::is_same_v<typename RegTileA::DType, typename Atom::BaseTileA> &&
                    std::is_same_v<typename RegTileB::DType, typename Atom::BaseTileB> &&
                    std::is_same_v<typename RegTileC::DType, typename Atom::BaseTileC>,
                "A must be tiled by row-major operand base tiles, B by column-major operand base tiles, "
                "C by accumulator base tiles");
  static constexpr int kMs = RegTileA::kRows, kKs = RegTileA::kCols, kNs = RegTileB::kCols;
  static_assert(RegTileB::kRows == kKs && RegTileC::kRows == kMs && RegTileC::kCols == kNs,
                "base-tile counts of A [Ms x Ks], B [Ks x Ns], C [Ms x Ns] do not match");

  DEVICE void operator()(const RegTileA& a, const RegTileB& b, RegTileC& c) const {
    Atom mma;
#pragma unroll
    for (int i = 0; i < kMs; ++i)
#pragma unroll
      for (int j = 0; j < kNs; ++j)
#pragma unroll
        for (int k = 0; k < kKs; ++k) mma(a(i, k), b(k, j), c(i, j));
  }
};

template <typename RegTileA, typename RegTileB, typename RegTileC>
DEVICE void gemm(const RegTileA& a, const RegTileB& b, RegTileC& c) {
  Gemm<RegTileA, RegTileB, RegTileC> op;
  op(a, b, c);
}

}  // namespace tilefusion::cell::compute
