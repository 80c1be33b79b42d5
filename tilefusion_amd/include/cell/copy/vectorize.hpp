// Fixed-width vector moves between registers (counterpart of include/cell/copy/vectorize.hpp:14-59).
#pragma once

#include "types/base.hpp"

namespace tilefusion::cell::copy {

template <typename Element, int kVecNums>
struct Vectorize {
  static constexpr int vectorize_bits = sizeof(Element) * 8 * kVecNums;
  static_assert(vectorize_bits % 32 == 0, "vectors move in whole dwords");
  DEVICE void copy(const Element* src, Element* dst) const {
    const unsigned* s = reinterpret_cast<const unsigned*>(src);
    unsigned* d = reinterpret_cast<unsigned*>(dst);
#pragma unroll
    for (int i = 0; i < vectorize_bits / 32; ++i) d[i] = s[i];
  }
};

}  // namespace tilefusion::cell::copy
