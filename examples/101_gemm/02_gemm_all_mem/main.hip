#include "../util.hpp"
#include "gemm.hpp"

int main() {
  constexpr int kM = 1024, kN = 1024, kK = 512;
  constexpr int kTM = 128, kTN = 128, kTK = 64, kRK = 32;
  using WarpLayout = tl::RowMajor<2, 2>;
  using Traits = GemmTraits<__half, float, WarpLayout, kM, kN, kK, kTM, kTN, kTK, kRK>;

  std::vector<__half> a(kM * kK), b(kN * kK);
  fill_uniform(a, 3);
  fill_uniform(b, 4);
  __half *dA, *dB;
  float* dC;
  HIP_OK(hipMalloc(&dA, a.size() * 2));
  HIP_OK(hipMalloc(&dB, b.size() * 2));
  HIP_OK(hipMalloc(&dC, kM * kN * 4));
  HIP_OK(hipMemcpy(dA, a.data(), a.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dB, b.data(), b.size() * 2, hipMemcpyHostToDevice));

  auto kernel = gemm_all_mem<__half, float, Traits, kN, kK, kTM, kTN>;
  const dim3 grid(kM / kTM, kN / kTN), block(Traits::kThreads);
  hipLaunchKernelGGL(kernel, grid, block, Traits::kSharedBytes, 0, dA, dB, dC);
  HIP_OK(hipGetLastError());
  HIP_OK(hipDeviceSynchronize());

  std::vector<float> c(kM * kN), ref(kM * kN);
  HIP_OK(hipMemcpy(c.data(), dC, c.size() * 4, hipMemcpyDeviceToHost));
  gemm_cpu(a, b, ref, kM, kN, kK);
  const bool ok = check(c, ref);

  tilefusion::HipTimer timer;
  timer.start();
  for (int i = 0; i < 20; ++i) hipLaunchKernelGGL(kernel, grid, block, Traits::kSharedBytes, 0, dA, dB, dC);
  const float ms = timer.stop() / 20;
  std::printf("[%d, %d, %d] tiles [%d, %d, %d] rk %d: %.3f ms, %.2f TFLOP/s, %d bytes of LDS\n", kM, kN, kK, kTM, kTN,
              kTK, kRK, ms, 2.0 * kM * kN * kK / ms / 1e9, Traits::kSharedBytes);
  return ok ? 0 : 1;
}
