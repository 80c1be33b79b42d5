// Packed pairs of 16-bit elements (counterpart of include/types/packing.hpp:7-22).
#pragma once

#include "types/base.hpp"

namespace tilefusion {

template <typename Element, int kN>
struct Packing;

template <>
struct Packing<__half, 2> {
  using PackedType = __half2;
};
template <>
struct Packing<__bfloat16, 2> {
  using PackedType = __hip_bfloat162;
};
template <>
struct Packing<float, 2> {
  using PackedType = float2;
};

}  // namespace tilefusion
