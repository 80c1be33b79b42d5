// Drop-in check, part 1: instantiates the kernel of the REFERENCE's own
// examples/101_gemm/01_gemm_global_reg/gemm.hpp - found through the include path the build recipe
// passes, never copied - against the tile headers of this repository, and launches it behind a
// C ABI.  Only the launch is written here: 64 lanes per wavefront instead of the 32 threads per
// warp the reference's host code multiplies by (examples/101_gemm/01_gemm_global_reg/main.cu:62).
#include <hip/hip_runtime.h>

#include "gemm.hpp"   // the reference's file

#define DROPIN_API extern "C" __attribute__((visibility("default")))

namespace {
template <typename WholeShape, int kTM, int kTN, typename WarpLayout>
int run(const void* a, const void* b, void* c) {
  using InType = __half;
  using AccType = float;
  using Config = GemmTraits<InType, AccType, WholeShape, kTM, kTN, WarpLayout>;
  constexpr int kM = dim_size<0, WholeShape>, kN = dim_size<1, WholeShape>, kK = dim_size<2, WholeShape>;
  auto kernel = simple_gemm<InType, AccType, kM, kN, kK, kTM, kTN, typename Config::IteratorA, typename Config::RegA,
                            typename Config::ALoader, typename Config::IteratorB, typename Config::RegB,
                            typename Config::BLoader, typename Config::GlobalC, typename Config::RegC,
                            typename Config::CStorer>;
  hipLaunchKernelGGL(kernel, dim3(kM / kTM, kN / kTN), dim3(tl::get_numel<WarpLayout> * WARP_SIZE), 0, 0,
                     static_cast<const InType*>(a), static_cast<const InType*>(b), static_cast<AccType*>(c));
  hipError_t e = hipGetLastError();
  return e != hipSuccess ? (int)e : (int)hipDeviceSynchronize();
}
}  // namespace

// variant 0: the README's single tile (A 128 x 256, B 256 x 64 column-major, C 128 x 64, 2 x 2
// wavefronts); variant 1: a grid of tiles, [256, 256, 512] with [128, 64] tiles, 2 x 2 wavefronts;
// variant 2: [128, 128, 128] with [64, 32] tiles on 4 x 1 wavefronts
DROPIN_API int dropin_example_01(int variant, const void* a, const void* b, void* c) {
  switch (variant) {
    case 0: return run<GemmShape<128, 64, 256>, 128, 64, tl::RowMajor<2, 2>>(a, b, c);
    case 1: return run<GemmShape<256, 256, 512>, 128, 64, tl::RowMajor<2, 2>>(a, b, c);
    case 2: return run<GemmShape<128, 128, 128>, 64, 32, tl::RowMajor<4, 1>>(a, b, c);
    default: return -1;
  }
}
DROPIN_API void dropin_example_01_shape(int variant, int* m, int* n, int* k) {
  static const int t[3][3] = {{128, 64, 256}, {256, 256, 512}, {128, 128, 128}};
  *m = t[variant][0]; *n = t[variant][1]; *k = t[variant][2];
}
