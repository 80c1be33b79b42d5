// Integer helpers used by the layouts (counterpart of include/util/math_utils.hpp:9-72 and of
// CeilDiv / ceil_div in include/cuda_utils.hpp).
#pragma once

#include "config.hpp"

namespace tilefusion {

template <int a, int b>
inline constexpr int CeilDiv = (a + b - 1) / b;

template <typename T>
HOST_DEVICE constexpr T ceil_div(T a, T b) {
  return (a + b - 1) / b;
}

template <int kN>
consteval bool is_power_of_2() {
  return kN > 0 && (kN & (kN - 1)) == 0;
}

template <int kN>
HOST_DEVICE constexpr int log2_exact() {
  static_assert(is_power_of_2<kN>(), "kN must be a power of 2");
  int n = 0;
  for (int v = kN; v > 1; v >>= 1) ++n;
  return n;
}

// div / mod by a compile-time constant; shifts and masks when it is a power of two.
template <bool kIsPow2, int kN>
struct DivModSelector {
  static HOST_DEVICE constexpr int div(int x) { return x / kN; }
  static HOST_DEVICE constexpr int mod(int x) { return x % kN; }
};
template <int kN>
struct DivModSelector<true, kN> {
  static HOST_DEVICE constexpr int div(int x) { return x >> log2_exact<kN>(); }
  static HOST_DEVICE constexpr int mod(int x) { return x & (kN - 1); }
};

}  // namespace tilefusion
