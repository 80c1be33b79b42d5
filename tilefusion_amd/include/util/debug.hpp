// Predicates for guarded debug printing (counterpart of include/util/debug.hpp:12-33).
#pragma once

#include "config.hpp"

namespace tilefusion {
DEVICE bool block(int bid) {
  return (int)(blockIdx.x + blockIdx.y * gridDim.x + blockIdx.z * gridDim.x * gridDim.y) == bid;
}
DEVICE bool thread(int tid, int bid) {
  const int id = threadIdx.x + threadIdx.y * blockDim.x + threadIdx.z * blockDim.x * blockDim.y;
  return id == tid && block(bid);
}
DEVICE bool thread(int tid) { return thread(tid, 0); }
DEVICE bool thread0() { return thread(0, 0); }
DEVICE bool block0() { return block(0); }
}  // namespace tilefusion
