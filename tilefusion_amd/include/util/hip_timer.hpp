// Event-pair GPU stopwatch (counterpart of CudaTimer, include/util/cuda_timer.hpp:11-45).
#pragma once

#include <hip/hip_runtime.h>

namespace tilefusion {

class HipTimer {
 public:
  HipTimer() {
    (void)hipEventCreate(&start_);
    (void)hipEventCreate(&stop_);
  }
  ~HipTimer() {
    (void)hipEventDestroy(start_);
    (void)hipEventDestroy(stop_);
  }
  HipTimer(const HipTimer&) = delete;
  HipTimer& operator=(const HipTimer&) = delete;

  void start(hipStream_t st = nullptr) {
    stream_ = st;
    (void)hipEventRecord(start_, stream_);
  }
  // milliseconds since start(); waits for the work enqueued in between
  float stop() {
    (void)hipEventRecord(stop_, stream_);
    (void)hipEventSynchronize(stop_);
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, start_, stop_);
    return ms;
  }

 private:
  hipEvent_t start_{}, stop_{};
  hipStream_t stream_ = nullptr;
};
using CudaTimer = HipTimer;  // the reference's name, for sources written against it

}  // namespace tilefusion
