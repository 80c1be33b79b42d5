// Compile-time shape tuple (counterpart of include/types/tile_shape.hpp:11-31, on std::array
// instead of cute::array).
#pragma once

#include <array>
#include <cstddef>
#include <cstdint>

#include "config.hpp"

namespace tilefusion {

template <size_t... Ns>
struct TileShape {
  static constexpr std::array<size_t, sizeof...(Ns)> shape = {Ns...};
  static constexpr size_t kRank = sizeof...(Ns);
  static constexpr size_t kNumel = (size_t(1) * ... * Ns);
  static constexpr size_t get_numel() { return kNumel; }
};

template <typename Shape>
inline constexpr int64_t get_numel = Shape::kNumel;

template <size_t I, typename Shape>
inline constexpr size_t dim_size = std::get<I>(Shape::shape);

struct Underscore {};           // placeholder index: "the whole extent" when slicing
inline constexpr Underscore _;  // usable on host and device

}  // namespace tilefusion
