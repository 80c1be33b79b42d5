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

// Combine a value over the four lanes l%16, l%16 + 16, l%16 + 32, l%16 + 48 (the lanes that
// share a row of a row-major base tile, or a column of a column-major one); every lane
// receives the result.  v_permlane16_swap / v_permlane32_swap exchange 16- and 32-lane halves
// between two registers in one instruction, without the LDS crossbar.
template <typename Op>
DEVICE float quad16_allreduce(float x, Op op) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  auto s16 = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  x = op(__builtin_bit_cast(float, (unsigned)s16[0]), __builtin_bit_cast(float, (unsigned)s16[1]));
  const unsigned v = __builtin_bit_cast(unsigned, x);
  auto s32 = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return op(__builtin_bit_cast(float, (unsigned)s32[0]), __builtin_bit_cast(float, (unsigned)s32[1]));
}

}  // namespace tilefusion::cell
