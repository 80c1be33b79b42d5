/* Naive fp32 triple-loop GEMM, test infrastructure only.
 * Restates the checker of the reference's tests/cpp/cell/test_single_wmma.cu:20-33:
 * A [m,k] row-major, B col-major k x n (an [n,k] buffer), C [m,n] row-major, one fp32
 * accumulator per output summed in k order.  Inputs arrive as fp32 (already rounded to
 * fp16 by the caller).  Built by oracle/Makefile into oracle/liboracle_naive.so. */
#include <stddef.h>

void oracle_naive_gemm(int m, int n, int k, const float* a, const float* b, float* c) {
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) {
      float s = 0.f;
      for (int kk = 0; kk < k; ++kk) s += a[(size_t)i * k + kk] * b[(size_t)j * k + kk];
      c[(size_t)i * n + j] = s;
    }
}

/* Direct single-query attention for one (batch, head) slice, double accumulation.
 * No reference counterpart; used to pin oracle.flash_decode_ref independently of torch. */
#include <math.h>
void oracle_naive_decode(int lkv, int d, int dv, const float* q, const float* k, const float* v,
                         double scale, float* out) {
  double mx = -INFINITY;
  for (int n = 0; n < lkv; ++n) {
    double s = 0;
    for (int i = 0; i < d; ++i) s += (double)q[i] * k[(size_t)n * d + i];
    s *= scale;
    if (s > mx) mx = s;
  }
  double den = 0;
  for (int j = 0; j < dv; ++j) out[j] = 0.f;
  double acc[1024];
  for (int j = 0; j < dv; ++j) acc[j] = 0;
  for (int n = 0; n < lkv; ++n) {
    double s = 0;
    for (int i = 0; i < d; ++i) s += (double)q[i] * k[(size_t)n * d + i];
    double e = exp(s * scale - mx);
    den += e;
    for (int j = 0; j < dv; ++j) acc[j] += e * v[(size_t)n * dv + j];
  }
  for (int j = 0; j < dv; ++j) out[j] = (float)(acc[j] / den);
}
