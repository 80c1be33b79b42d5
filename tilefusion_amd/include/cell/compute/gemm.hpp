// Wavefront-level matrix multiply on register tiles (counterpart of
// include/cell/compute/gemm.hpp:18-201): c(i, j) += sum_k a(i, k) * b(k, j) over base tiles.
//
// A is tiled by row-major base tiles, B by column-major ones (types/register.hpp): lane l holds
// 4 (wide tiles: 8) consecutive values of k of row / column l%16, which is what the MFMA
// operands want.  One 16 x 16 base tile of k is a v_mfma_f32_16x16x16_*; two base tiles that
// are adjacent in k are handed to ONE v_mfma_f32_16x16x32_* - the instruction sums over its
// (lane group, element) pairs, so any assignment of k values to them is valid as long as A and
// B use the same one, and the concatenation of two 4-element fragments is such an assignment.
// An odd tile count ends with one 16x16x16.
//
// The accumulator tile may be row-major (lane l: row l%16, columns 4*(l/16)..+3 - the same
// layout as an A operand tile, obtained by issuing the instruction with the operands swapped,
// which computes the transposed block) or column-major (the instruction's native result).
#pragma once

#include "types/register.hpp"

namespace tilefusion::cell::compute {
namespace tl = tile_layout;

struct MMA_ATOM_16x16x16 {};
struct MMA_ATOM_16x16x32 {};

namespace detail {
using half4_v = _Float16 __attribute__((ext_vector_type(4)));
using half8_v = _Float16 __attribute__((ext_vector_type(8)));
using bf16x4_v = __bf16 __attribute__((ext_vector_type(4)));
using bf16x8_v = __bf16 __attribute__((ext_vector_type(8)));
using short4_v = short __attribute__((ext_vector_type(4)));
using float4_v = float __attribute__((ext_vector_type(4)));

template <typename V, typename T>
DEVICE V load_vec(const T* p) {
  V v;
  __builtin_memcpy(&v, p, sizeof(V));
  return v;
}

// d += a * b over 16 (4 values of k per lane) or 32 (8 per lane) values of k; `a` holds rows,
// `b` columns of the 16 x 16 result, which comes out with lane l owning column l%16.
template <typename In>
struct Mfma;
template <>
struct Mfma<__half> {
  using V4 = half4_v;
  using V8 = half8_v;
  DEVICE static float4_v k16(V4 a, V4 b, float4_v c) { return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0); }
  DEVICE static float4_v k32(V8 a, V8 b, float4_v c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};
template <>
struct Mfma<__bfloat16> {
  using V4 = bf16x4_v;
  using V8 = bf16x8_v;
  DEVICE static float4_v k16(V4 a, V4 b, float4_v c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_v, a), __builtin_bit_cast(short4_v, b),
                                                    c, 0, 0, 0);
  }
  DEVICE static float4_v k32(V8 a, V8 b, float4_v c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};

template <typename BaseTileC>
DEVICE float4_v load_acc(const BaseTileC& c) {
  using T = typename BaseTileC::DType;
  float4_v v;
  if constexpr (std::is_same_v<T, float>) {
    v = load_vec<float4_v>(c.data());
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] = to_float(c.data()[r]);
  }
  return v;
}
template <typename BaseTileC>
DEVICE void store_acc(float4_v v, BaseTileC& c) {
  using T = typename BaseTileC::DType;
  if constexpr (std::is_same_v<T, float>) {
    __builtin_memcpy(c.mutable_data(), &v, sizeof(v));
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r) c.mutable_data()[r] = from_float<T>(v[r]);
  }
}

// `a` rows x `b` columns into an accumulator of either orientation
template <typename In, bool kRowMajorC, typename Frag>
DEVICE float4_v mfma(Frag a, Frag b, float4_v c) {
  if constexpr (sizeof(Frag) == 8) {
    return kRowMajorC ? Mfma<In>::k16(b, a, c) : Mfma<In>::k16(a, b, c);
  } else {
    return kRowMajorC ? Mfma<In>::k32(b, a, c) : Mfma<In>::k32(a, b, c);
  }
}
}  // namespace detail

// One base tile of A times one base tile of B (counterpart of the MmaAtom specialisations,
// include/cell/compute/gemm.hpp:18-150): MMA_ATOM_16x16x16 on the square tiles, MMA_ATOM_16x16x32
// on the wide ones.  The accumulator element type may be float or, for the reference's
// half-accumulating atom, __half: CDNA4 has no MFMA that accumulates in fp16, so the block is
// accumulated in fp32 and rounded once when it is written back - at least as accurate.
template <typename InTypeA, typename InTypeB, typename AccType, typename AtomicShape = MMA_ATOM_16x16x16>
struct MmaAtom {
  static_assert(std::is_same_v<InTypeA, InTypeB> && HalfType<InTypeA>, "operands are both __half or both __bfloat16");
  static_assert(std::is_same_v<AccType, float> || std::is_same_v<AccType, InTypeA>,
                "the accumulator is float or the operand type");
  static constexpr bool kWide = std::is_same_v<AtomicShape, MMA_ATOM_16x16x32>;
  using BaseTileA = std::conditional_t<kWide, RegTile<InTypeA, tl::RowMajor<1, 8>>, BaseTileRowMajor<InTypeA>>;
  using BaseTileB = std::conditional_t<kWide, RegTile<InTypeB, tl::ColMajor<8, 1>>, BaseTileColMajor<InTypeB>>;
  using BaseTileC = BaseTileRowMajor<AccType>;
  using BaseTile = BaseTileShape<InTypeA>;

  template <typename TileC>
  DEVICE void operator()(const BaseTileA& a, const BaseTileB& b, TileC& c) const {
    static_assert(std::is_same_v<typename TileC::DType, AccType> && TileC::kNumel == 4, "not an accumulator base tile");
    using V = std::conditional_t<kWide, typename detail::Mfma<InTypeA>::V8, typename detail::Mfma<InTypeA>::V4>;
    auto vc = detail::load_acc(c);
    vc = detail::mfma<InTypeA, BaseTileTraits<TileC>::kIsRowMajor>(detail::load_vec<V>(a.data()),
                                                                  detail::load_vec<V>(b.data()), vc);
    detail::store_acc(vc, c);
  }
};

// The atom tag is accepted for source compatibility (include/cell/compute/gemm.hpp:155-201); the
// instruction is chosen from the tiles: wide operand tiles take 16x16x32, square ones are paired.
template <typename RegTileA, typename RegTileB, typename RegTileC, typename AtomicShape = MMA_ATOM_16x16x16>
struct Gemm {
  using BaseA = typename RegTileA::DType;
  using BaseB = typename RegTileB::DType;
  using BaseC = typename RegTileC::DType;
  using InTypeA = typename BaseA::DType;
  using InTypeB = typename BaseB::DType;
  using OutType = typename BaseC::DType;
  using TraitsA = BaseTileTraits<BaseA>;
  using TraitsB = BaseTileTraits<BaseB>;
  using TraitsC = BaseTileTraits<BaseC>;
  static_assert(std::is_same_v<InTypeA, InTypeB> && HalfType<InTypeA>, "operands are both __half or both __bfloat16");
  static_assert(TraitsA::kIsRowMajor && !TraitsB::kIsRowMajor && TraitsA::kIsWide == TraitsB::kIsWide,
                "A must be tiled by row-major base tiles and B by column-major base tiles of the same width");
  static_assert(!TraitsC::kIsWide && (std::is_same_v<OutType, float> || std::is_same_v<OutType, InTypeA>),
                "C must be tiled by 16 x 16 base tiles of float (or of the operand type)");
  static constexpr bool kWide = TraitsA::kIsWide;
  static constexpr bool kRowMajorC = TraitsC::kIsRowMajor;
  static constexpr int kMs = RegTileA::kRows, kKs = RegTileA::kCols, kNs = RegTileB::kCols;
  static_assert(RegTileB::kRows == kKs && RegTileC::kRows == kMs && RegTileC::kCols == kNs,
                "base-tile counts of A [Ms x Ks], B [Ks x Ns], C [Ms x Ns] do not match");
  using M = detail::Mfma<InTypeA>;

  DEVICE void operator()(const RegTileA& a, const RegTileB& b, RegTileC& c) const {
#pragma unroll
    for (int i = 0; i < kMs; ++i)
#pragma unroll
      for (int j = 0; j < kNs; ++j) {
        auto vc = detail::load_acc(c(i, j));
        if constexpr (kWide) {
#pragma unroll
          for (int k = 0; k < kKs; ++k)
            vc = detail::mfma<InTypeA, kRowMajorC>(detail::load_vec<typename M::V8>(a(i, k).data()),
                                                   detail::load_vec<typename M::V8>(b(k, j).data()), vc);
        } else {
#pragma unroll
          for (int k = 0; k + 1 < kKs; k += 2) {
            const auto a0 = detail::load_vec<typename M::V4>(a(i, k).data());
            const auto a1 = detail::load_vec<typename M::V4>(a(i, k + 1).data());
            const auto b0 = detail::load_vec<typename M::V4>(b(k, j).data());
            const auto b1 = detail::load_vec<typename M::V4>(b(k + 1, j).data());
            vc = detail::mfma<InTypeA, kRowMajorC>(__builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7),
                                                   __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7), vc);
          }
          if constexpr (kKs % 2 == 1)
            vc = detail::mfma<InTypeA, kRowMajorC>(detail::load_vec<typename M::V4>(a(i, kKs - 1).data()),
                                                   detail::load_vec<typename M::V4>(b(kKs - 1, j).data()), vc);
        }
        detail::store_acc(vc, c(i, j));
      }
  }
};

template <typename RegTileA, typename RegTileB, typename RegTileC, typename AtomicShape = MMA_ATOM_16x16x16,
          typename GemmOp = Gemm<RegTileA, RegTileB, RegTileC, AtomicShape>>
DEVICE void gemm(const RegTileA& a, const RegTileB& b, RegTileC& c) {
  GemmOp op;
  op(a, b, c);
}

}  // namespace tilefusion::cell::compute
