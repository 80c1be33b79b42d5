// Drop-in check, part 4: the kernel of the REFERENCE's global -> shared -> global copy benchmark
// (benchmarks/cpp/g2s_copy/tilefusion_copy.cuh, found through the include path of the build
// recipe, never copied) instantiated against the tile headers of this repository, with the tile
// and wavefront layouts its main program sweeps (benchmarks/cpp/g2s_copy/main.cu:36-71,143-165).
// Only the launch is written here: 64 lanes per wavefront where the reference's host code
// multiplies by 32, and loader / storer objects that live in device memory (the reference hands
// the kernel references to host objects; they are stateless, but a reference has to point
// somewhere the GPU may read).
#include <hip/hip_runtime.h>

#include "cell/copy/mod.hpp"
#include "types/mod.hpp"

#include "tilefusion_copy.cuh"   // the reference's file

#define DROPIN_API extern "C" __attribute__((visibility("default")))

using namespace tilefusion;
using namespace tilefusion::cell;
using namespace tilefusion::cell::copy;
namespace tl = tile_layout;

namespace {
template <typename Layout, typename WarpLayout, int kRepeat>
int run(const void* src, void* dst) {
  using Element = __half;
  using Global = GlobalTile<Element, Layout>;
  using Shared = SharedTile<Element, Layout, true /*kSwizzled*/>;
  using Loader = GlobalToSharedLoader<Shared, WarpLayout>;
  using Storer = SharedToGlobalStorer<Shared, WarpLayout>;
  auto kernel = &g2s_data_transfer<Element, Global, Shared, Loader, Storer, kRepeat>;
  const int shm_size = Shared::kNumel * (int)sizeof(Element);
  if (shm_size > 48 * 1024)
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, shm_size);
  void* objects = nullptr;   // one byte each for the two empty functors
  hipError_t e = hipMalloc(&objects, 256);
  if (e != hipSuccess) return (int)e;
  Loader& loader = *static_cast<Loader*>(objects);
  Storer& storer = *reinterpret_cast<Storer*>(static_cast<char*>(objects) + 128);
  hipLaunchKernelGGL(kernel, dim3(1), dim3(WarpLayout::kNumel * WARP_SIZE), shm_size, 0,
                     static_cast<const Element*>(src), static_cast<Element*>(dst), loader, storer);
  e = hipGetLastError();
  if (e == hipSuccess) e = hipDeviceSynchronize();
  (void)hipFree(objects);
  return (int)e;
}
}  // namespace

// the eleven (tile, wavefront layout) pairs of the reference's main(), in its order
DROPIN_API int dropin_g2s_copy(int variant, const void* src, void* dst) {
  switch (variant) {
    case 0: return run<tl::RowMajor<16, 64>, tl::RowMajor<1, 1>, 3>(src, dst);
    case 1: return run<tl::RowMajor<64, 64>, tl::RowMajor<1, 1>, 3>(src, dst);
    case 2: return run<tl::RowMajor<64, 64>, tl::RowMajor<2, 1>, 3>(src, dst);
    case 3: return run<tl::RowMajor<64, 64>, tl::RowMajor<4, 1>, 3>(src, dst);
    case 4: return run<tl::RowMajor<128, 128>, tl::RowMajor<1, 1>, 3>(src, dst);
    case 5: return run<tl::RowMajor<128, 128>, tl::RowMajor<2, 2>, 3>(src, dst);
    case 6: return run<tl::RowMajor<128, 128>, tl::RowMajor<4, 2>, 3>(src, dst);
    case 7: return run<tl::RowMajor<128, 256>, tl::RowMajor<1, 1>, 3>(src, dst);
    case 8: return run<tl::RowMajor<128, 256>, tl::RowMajor<2, 2>, 3>(src, dst);
    case 9: return run<tl::RowMajor<128, 256>, tl::RowMajor<2, 4>, 3>(src, dst);
    case 10: return run<tl::RowMajor<128, 256>, tl::RowMajor<4, 4>, 3>(src, dst);
    default: return -1;
  }
}
DROPIN_API void dropin_g2s_copy_shape(int variant, int* rows, int* cols) {
  static const int t[11][2] = {{16, 64}, {64, 64}, {64, 64}, {64, 64}, {128, 128}, {128, 128},
                               {128, 128}, {128, 256}, {128, 256}, {128, 256}, {128, 256}};
  *rows = t[variant][0]; *cols = t[variant][1];
}
