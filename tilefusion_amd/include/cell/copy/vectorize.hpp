// Fixed-width vector moves (counterpart of include/cell/copy/vectorize.hpp:14-59): kVecNums
// elements travel as one 32-, 64- or 128-bit access, so the pointers must be aligned to that.
#pragma once

#include "types/base.hpp"

namespace tilefusion::cell::copy {

namespace detail {
template <int kBits>
struct VectorOfBits;
template <>
struct VectorOfBits<32> { using type = unsigned; };
template <>
struct VectorOfBits<64> { using type = uint2; };
template <>
struct VectorOfBits<128> { using type = uint4; };
}  // namespace detail

template <typename Element, int kVecNums>
struct Vectorize {
  using UnVecType = Element;
  static constexpr int vectorize_nums = kVecNums;
  static constexpr int vectorize_bits = sizeof(Element) * 8 * kVecNums;
  static_assert(vectorize_bits == 32 || vectorize_bits == 64 || vectorize_bits == 128,
                "a vector is one 32-, 64- or 128-bit access");
  using VecType = typename detail::VectorOfBits<vectorize_bits>::type;

  DEVICE void operator()(const UnVecType* src, UnVecType* dst) const {
    *reinterpret_cast<VecType*>(dst) = *reinterpret_cast<const VecType*>(src);
  }
  DEVICE void copy(const UnVecType* src, UnVecType* dst) const { (*this)(src, dst); }
};

}  // namespace tilefusion::cell::copy
