// Scalar functors (counterpart of include/cell/compute/math_functor.hpp:10-214).  They work on
// float, __half and __bfloat16; 16-bit types are computed in fp32 and rounded once.
#pragma once

#include <cmath>

#include "types/base.hpp"

namespace tilefusion::cell::compute {

#define TILEFUSION_BINARY_FUNCTOR(Name, expr)                          \
  template <typename Element>                                          \
  struct Name {                                                        \
    DEVICE Element operator()(Element a_, Element b_) const {          \
      const float a = to_float(a_), b = to_float(b_);                  \
      return from_float<Element>(expr);                                \
    }                                                                  \
    DEVICE void operator()(const Element& a_, const Element& b_, Element& out) const { \
      out = (*this)(a_, b_);                                           \
    }                                                                  \
  };
TILEFUSION_BINARY_FUNCTOR(Add, a + b)
TILEFUSION_BINARY_FUNCTOR(Sub, a - b)
TILEFUSION_BINARY_FUNCTOR(Mul, a* b)
TILEFUSION_BINARY_FUNCTOR(Div, a / b)
TILEFUSION_BINARY_FUNCTOR(Max, fmaxf(a, b))
TILEFUSION_BINARY_FUNCTOR(Min, fminf(a, b))
#undef TILEFUSION_BINARY_FUNCTOR

#define TILEFUSION_UNARY_FUNCTOR(Name, expr)                           \
  template <typename Element>                                          \
  struct Name {                                                        \
    DEVICE Element operator()(Element a_) const {                      \
      const float a = to_float(a_);                                    \
      return from_float<Element>(expr);                                \
    }                                                                  \
    DEVICE void operator()(const Element& a_, Element& out) const { out = (*this)(a_); } \
  };
TILEFUSION_UNARY_FUNCTOR(Exp, __expf(a))
TILEFUSION_UNARY_FUNCTOR(Log, __logf(a))
TILEFUSION_UNARY_FUNCTOR(Relu, fmaxf(a, 0.f))
#undef TILEFUSION_UNARY_FUNCTOR

template <typename SrcType, typename DstType>
struct Convert {
  DEVICE DstType operator()(SrcType a) const { return from_float<DstType>(to_float(a)); }
  DEVICE void operator()(const SrcType& a, DstType& out) const { out = (*this)(a); }
};

}  // namespace tilefusion::cell::compute
