// Runtime dtype -> compile-time type switch for host launchers (counterpart of
// include/kernels/dispatch_macros.hpp:6-23).  `TYPE` is an at::ScalarType; the body sees the
// element type as `scalar_t` (__half / __bfloat16 / float).
//
// A host-only translation unit that cannot include the device headers defines
// TILEFUSION_DISPATCH_HOST_TYPES and provides the three type names itself.
#pragma once

#ifndef TILEFUSION_DISPATCH_HOST_TYPES
#include "types/base.hpp"
#endif

#define TILEFUSION_DISPATCH_CASE(ENUM, CTYPE, ...) \
  case ENUM: {                                     \
    using scalar_t = CTYPE;                        \
    __VA_ARGS__();                                 \
    break;                                         \
  }

#define TILEFUSION_DISPATCH_ALL_TYPES(TYPE, ...)                                   \
  switch (TYPE) {                                                                  \
    TILEFUSION_DISPATCH_CASE(at::ScalarType::Half, __half, __VA_ARGS__)            \
    TILEFUSION_DISPATCH_CASE(at::ScalarType::BFloat16, __bfloat16, __VA_ARGS__)    \
    TILEFUSION_DISPATCH_CASE(at::ScalarType::Float, float, __VA_ARGS__)            \
    default:                                                                       \
      TORCH_CHECK(false, "tilefusion: unsupported dtype ", toString(TYPE));        \
  }
