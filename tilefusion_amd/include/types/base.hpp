// Element types and the machine constants the tile types are sized by.
//
// Counterpart of include/types/base.hpp:20-68, re-derived for CDNA4: the matrix instruction the
// tiles are built around is v_mfma_f32_16x16x32_{f16,bf16}.  A 16-bit OPERAND base tile is
// therefore 16 x 32 (row-major A) or 32 x 16 (column-major B) with 8 contiguous-in-k elements
// per lane, and an ACCUMULATOR base tile is 16 x 16 with 4 elements per lane - not the 16 x 16
// / 8-per-thread tile of mma.m16n8k16 on a 32-lane warp.
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

// Shape of the tile one MFMA base tile of `Element`s covers, in its contiguous orientation:
// 16 x 32 for 16-bit operands (16 x 16 x 32 instruction), 16 x 16 for fp32 accumulators.
// For a column-major operand the roles of rows and columns swap (32 x 16).
template <typename Element>
  requires BaseType<Element>
struct BaseTileShape {
  static constexpr int kRows = 16;
  static constexpr int kCols = sizeof(Element) == 2 ? 32 : 16;
  static constexpr int kNumel = kRows * kCols;
  static constexpr int kNumelPerLane = kNumel / WARP_SIZE;
};

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
