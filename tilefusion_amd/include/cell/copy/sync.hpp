// Fences for asynchronous global -> LDS copies (counterpart of include/cell/copy/sync.hpp:10-26).
// The loaders of this library stage through registers, so a copy is complete once the
// wavefront's outstanding vector-memory and LDS operations have drained.
#pragma once

#include "config.hpp"

namespace tilefusion::cell::copy {

DEVICE void commit_copy_group() {}

template <int N>
DEVICE void wait_group() {
  static_assert(N >= 0, "N is the number of copy groups that may stay in flight");
  if constexpr (N == 0) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
}

DEVICE void __copy_async() {
  commit_copy_group();
  wait_group<0>();
}

}  // namespace tilefusion::cell::copy
