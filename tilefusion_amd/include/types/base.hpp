// Element types and the machine constants the tile types are sized by.
//
// Counterpart of include/types/base.hpp:20-68.  A base tile is the reference's square 16 x 16
// block for every element type, so the tile-count arithmetic of kernels written against the
// reference (kTM / kWarpPerRow / BaseShape::kRows, kRK / BaseShape::kCols, ...) carries over
// unchanged; what differs is how the block is spread over the lanes: 64 lanes hold 4 elements
// each (types/register.hpp) instead of 32 threads holding 8.  The matrix instructions behind
// it are v_mfma_f32_16x16x16_{f16,bf16} for one base tile of k and v_mfma_f32_16x16x32_* for
// two adjacent ones.  WideBaseTileShape is the 16 x 32 operand block of the 16x16x32
// instruction taken in one piece (an extension, see types/register.hpp).
#pragma once

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <type_traits>

#include "config.hpp"

typedef __hip_bfloat16 __bfloat16;

namespace tilefusion {

template <typename Element>
concept BaseType = std::is_same_v<Element, float> || std::is_same_v<Element, __half> ||
                   std::is_same_v<Element, __bfloat16>;

template <typename Element>
concept HalfType = std::is_same_v<Element, __half> || std::is_same_v<Element, __bfloat16>;

// Widest per-lane access (128 bits) and the contiguous run a group of lanes should cover
// (one 128-byte L2 line).
template <typename Element>
struct AccessBase {
  static constexpr int kAccessInBits = 128;
  static constexpr int kAccessInBytes = kAccessInBits / 8;
  static constexpr int kElementBits = sizeof(Element) * 8;
  static constexpr int kNumPerAccess = kAccessInBits / kElementBits;
  static constexpr int kMemTransWidth = 1024;  // bits
  static constexpr int kExpectedSize = kMemTransWidth / kElementBits;
};

// The block of a matrix one base tile covers: 16 x 16 for every element type, operands and
// accumulators alike (include/types/base.hpp:62-68).
template <typename Element>
  requires BaseType<Element>
struct BaseTileShape {
  static constexpr int kRows = 16;
  static constexpr int kCols = 16;
  static constexpr int kNumel = kRows * kCols;
  static constexpr int kNumelPerLane = kNumel / WARP_SIZE;
};

// The 16 x 32 block (in its contiguous orientation; 32 x 16 for a column-major operand) a
// wide 16-bit operand base tile covers.
template <typename Element>
  requires HalfType<Element>
struct WideBaseTileShape {
  static constexpr int kRows = 16;
  static constexpr int kCols = 32;
  static constexpr int kNumel = kRows * kCols;
  static constexpr int kNumelPerLane = kNumel / WARP_SIZE;
};

// Kernels written against earlier revisions of the reference spell traits::BaseTileShape (its
// own examples/101_gemm still do); the name resolves here.
namespace traits = ::tilefusion;

template <typename T>
HOST_DEVICE T from_float(float v) {
  if constexpr (std::is_same_v<T, __half>) {
    return __float2half(v);
  } else if constexpr (std::is_same_v<T, __bfloat16>) {
    return __float2bfloat16(v);
  } else {
    static_assert(std::is_same_v<T, float>, "unsupported element type");
    return v;
  }
}

template <typename T>
HOST_DEVICE float to_float(const T& v) {
  if constexpr (std::is_same_v<T, __half>) {
    return __half2float(v);
  } else if constexpr (std::is_same_v<T, __bfloat16>) {
    return __bfloat162float(v);
  } else {
    static_assert(std::is_same_v<T, float>, "unsupported element type");
    return v;
  }
}

}  // namespace tilefusion
