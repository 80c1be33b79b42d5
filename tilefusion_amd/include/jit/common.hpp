// Type names for source generators (counterpart of include/jit/common.hpp:9-26).
#pragma once

#include <string>
#include <type_traits>

#include "types/base.hpp"

namespace tilefusion::jit {

template <typename T>
inline std::string get_type_string() {
  if constexpr (std::is_same_v<T, float>) return "float";
  else if constexpr (std::is_same_v<T, double>) return "double";
  else if constexpr (std::is_same_v<T, int>) return "int";
  else if constexpr (std::is_same_v<T, __half>) return "__half";
  else if constexpr (std::is_same_v<T, __bfloat16>) return "__bfloat16";
  else static_assert(sizeof(T) == 0, "no source-level name registered for this type");
}

}  // namespace tilefusion::jit
