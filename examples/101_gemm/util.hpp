// Shared helpers of the GEMM examples: seeded inputs, a CPU reference, a comparison and a
// timing loop (counterpart of examples/101_gemm/util.hpp in the reference).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "util/hip_timer.hpp"

#define HIP_OK(expr)                                                                          \
  do {                                                                                        \
    hipError_t e_ = (expr);                                                                   \
    if (e_ != hipSuccess) {                                                                   \
      std::fprintf(stderr, "%s failed: %s (%s:%d)\n", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
      std::exit(2);                                                                           \
    }                                                                                         \
  } while (0)

// uniform in [-1, 1) from a small LCG: the same numbers on every run and every host
inline void fill_uniform(std::vector<__half>& v, unsigned seed) {
  unsigned s = seed * 2654435761u + 12345u;
  for (auto& x : v) {
    s = s * 1664525u + 1013904223u;
    x = __float2half(((s >> 8) & 0xffff) / 32768.0f - 1.0f);
  }
}

// C[m][n] = sum_k A[m][k] * B[k][n], A row-major [M,K], B column-major (a row-major [N,K] buffer)
inline void gemm_cpu(const std::vector<__half>& a, const std::vector<__half>& b, std::vector<float>& c, int m,
                     int n, int k) {
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) {
      float s = 0.f;
      for (int p = 0; p < k; ++p) s += __half2float(a[(size_t)i * k + p]) * __half2float(b[(size_t)j * k + p]);
      c[(size_t)i * n + j] = s;
    }
}

// relative L2 error; prints and returns whether it is within 1e-3
inline bool check(const std::vector<float>& got, const std::vector<float>& want) {
  double num = 0, den = 0;
  for (size_t i = 0; i < got.size(); ++i) {
    num += (double)(got[i] - want[i]) * (got[i] - want[i]);
    den += (double)want[i] * want[i];
  }
  const double rel = std::sqrt(num / (den > 0 ? den : 1));
  std::printf("relative L2 error vs CPU fp32: %.3e %s\n", rel, rel <= 1e-3 ? "(ok)" : "(MISMATCH)");
  return rel <= 1e-3;
}
