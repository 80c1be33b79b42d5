// Drop-in check, part 2: the kernel of the REFERENCE's own examples/101_gemm/02_gemm_all_mem/
// gemm.hpp (global -> LDS -> registers, accumulator back through a swizzled fp32 LDS tile),
// found through the include path the build recipe passes, instantiated against the tile headers
// of this repository.  It runs on ONE wavefront per workgroup: the reference's kernel refills its
// LDS tiles, and then overlays them with the C tile, without a barrier after the last fragment
// reads (examples/101_gemm/02_gemm_all_mem/gemm.hpp:140-156 there), which only a single
// wavefront makes well defined.
#include <hip/hip_runtime.h>

#include "gemm.hpp"   // the reference's file

#define DROPIN_API extern "C" __attribute__((visibility("default")))

namespace {
template <typename WholeShape, typename CtaTileShape, int kRK, typename WarpLayout>
int run(const void* a, const void* b, void* c) {
  using InType = __half;
  using AccType = float;
  using Config = KeGemmTraits<InType, AccType, WholeShape, CtaTileShape, kRK, WarpLayout>;
  constexpr int kM = Config::kM, kN = Config::kN, kK = Config::kK;
  constexpr int kTM = Config::kTM, kTN = Config::kTN, kTK = Config::kTK;
  auto kernel = &gemm<InType, AccType, kM, kN, kK, kTM, kTN, kTK, typename Config::GIteratorA, typename Config::SIteratorA,
                      typename Config::SharedA, typename Config::RegA, typename Config::G2SLoaderA,
                      typename Config::S2RLoaderA, typename Config::GIteratorB, typename Config::SIteratorB,
                      typename Config::SharedB, typename Config::RegB, typename Config::G2SLoaderB,
                      typename Config::S2RLoaderB, typename Config::GlobalC, typename Config::SharedC,
                      typename Config::RegC, typename Config::R2SStorerC, typename Config::S2GStorerC>;
  constexpr int kInputs = (kTM * kTK + kTK * kTN) * (int)sizeof(InType);
  constexpr int kOutput = kTM * kTN * (int)sizeof(AccType);
  constexpr int kLds = kInputs > kOutput ? kInputs : kOutput;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLds) != hipSuccess)
    return -2;
  hipLaunchKernelGGL(kernel, dim3(kM / kTM, kN / kTN), dim3(tl::get_numel<WarpLayout> * WARP_SIZE), kLds, 0,
                     static_cast<const InType*>(a), static_cast<const InType*>(b), static_cast<AccType*>(c));
  hipError_t e = hipGetLastError();
  return e != hipSuccess ? (int)e : (int)hipDeviceSynchronize();
}
}  // namespace

// variant 0: [128, 128, 256] in [64, 64, 64] tiles, register steps of 16; variant 1: [64, 128, 128]
// in [32, 64, 128] tiles, register steps of 32
DROPIN_API int dropin_example_02(int variant, const void* a, const void* b, void* c) {
  switch (variant) {
    case 0: return run<GemmShape<128, 128, 256>, GemmShape<64, 64, 64>, 16, tl::RowMajor<1, 1>>(a, b, c);
    case 1: return run<GemmShape<64, 128, 128>, GemmShape<32, 64, 128>, 32, tl::RowMajor<1, 1>>(a, b, c);
    default: return -1;
  }
}
DROPIN_API void dropin_example_02_shape(int variant, int* m, int* n, int* k) {
  static const int t[2][3] = {{128, 128, 256}, {64, 128, 128}};
  *m = t[variant][0]; *n = t[variant][1]; *k = t[variant][2];
}
