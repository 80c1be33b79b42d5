// Cross-lane primitives on a 64-lane wavefront (counterpart of include/cell/warp.hpp:10-29).
#pragma once

#include <cstdint>

#include "config.hpp"

namespace tilefusion::cell {

// all 64 lanes
inline constexpr uint64_t MASK_ALL = ~uint64_t(0);

template <typename T>
DEVICE T shuffle_sync(uint64_t /*mask*/, T value, int src_lane) {
  return __shfl(value, src_lane, WARP_SIZE);
}
template <typename T>
DEVICE T shuffle_down_sync(uint64_t /*mask*/, T value, int delta) {
  return __shfl_down(value, delta, WARP_SIZE);
}

// DPP move inside a row of 16 lanes (no LDS crossbar round trip).
template <int kCtrl>
DEVICE float dpp_move(float x) {
  return __builtin_bit_cast(float,
                            __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), kCtrl, 0xf, 0xf, false));
}
// Combine a value over the 16 lanes of each DPP row; every lane receives the result.
template <typename Op>
DEVICE float row16_allreduce(float x, Op op) {
  x = op(x, dpp_move<0x128>(x));  // row_ror:8
  x = op(x, dpp_move<0x124>(x));  // row_ror:4
  x = op(x, dpp_move<0x122>(x));  // row_ror:2
  x = op(x, dpp_move<0x121>(x));  // row_ror:1
  return x;
}

}  // namespace tilefusion::cell
