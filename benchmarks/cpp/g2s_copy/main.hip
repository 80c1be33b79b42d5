// Global <-> LDS copy micro-benchmark (counterpart of benchmarks/cpp/g2s_copy/main.cu:20-165 in
// the reference): one workgroup loads a row-major fp16 tile into LDS with GlobalToSharedLoader
// and stores it back with SharedToGlobalStorer, kRepeat times, for the reference's tile shapes
// and wavefront layouts.  The baseline column is a hand-written copy with the best access
// pattern a single workgroup has (every lane moves 16 bytes, consecutive lanes consecutive
// addresses, no swizzle).  Both results must equal the source bit for bit.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#include "cell/mod.hpp"
#include "types/mod.hpp"
#include "util/hip_timer.hpp"

using namespace tilefusion;
using namespace tilefusion::cell;
using namespace tilefusion::cell::copy;
namespace tl = tile_layout;

#define HIP_OK(expr)                                                                               \
  do {                                                                                             \
    hipError_t e_ = (expr);                                                                        \
    if (e_ != hipSuccess) {                                                                        \
      std::fprintf(stderr, "%s failed: %s (%s:%d)\n", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
      std::exit(2);                                                                                \
    }                                                                                              \
  } while (0)

template <typename Element, typename Global, typename Shared, typename WarpLayout, int kRepeat>
__global__ void g2s_data_transfer(const Element* src_ptr, Element* dst_ptr) {
  extern __shared__ __attribute__((aligned(16))) unsigned char buf_[];
  Global src(src_ptr + (size_t)blockIdx.x * Global::kNumel);   // every workgroup has a tile of its own
  Shared inter(reinterpret_cast<Element*>(buf_));
  Global dst(dst_ptr + (size_t)blockIdx.x * Global::kNumel);
  GlobalToSharedLoader<Shared, WarpLayout> loader;
  SharedToGlobalStorer<Shared, WarpLayout> storer;
  for (int i = 0; i < kRepeat; ++i) {
    loader(src, inter);
    __copy_async();
    __syncthreads();
    storer(inter, dst);
    __syncthreads();
  }
}

template <typename Element, int kNumel, int kThreads, int kRepeat>
__global__ void baseline_transfer(const Element* src, Element* dst) {
  extern __shared__ __attribute__((aligned(16))) unsigned char buf_[];
  using Vec = uint4;
  constexpr int kVecs = kNumel * (int)sizeof(Element) / (int)sizeof(Vec);
  Vec* lds = reinterpret_cast<Vec*>(buf_);
  src += (size_t)blockIdx.x * kNumel;
  dst += (size_t)blockIdx.x * kNumel;
  for (int i = 0; i < kRepeat; ++i) {
    for (int v = threadIdx.x; v < kVecs; v += kThreads) lds[v] = reinterpret_cast<const Vec*>(src)[v];
    __syncthreads();
    for (int v = threadIdx.x; v < kVecs; v += kThreads) reinterpret_cast<Vec*>(dst)[v] = lds[v];
    __syncthreads();
  }
}

template <typename F>
static float time_ms(F&& launch) {
  launch();  // warm-up
  HIP_OK(hipDeviceSynchronize());
  HipTimer timer;
  timer.start();
  for (int i = 0; i < 20; ++i) launch();
  const float ms = timer.stop() / 20;
  HIP_OK(hipGetLastError());
  return ms;
}

static int failures = 0;

// kGrid workgroups, each round-tripping a tile of its own: 1 is the reference's measurement (the
// latency of one tile through one CU), one workgroup per CU shows what the chip sustains.
template <typename Element, typename Layout, typename WarpLayout>
void run_test_rowmajor(int kGrid) {
  constexpr int kRepeat = 100;
  constexpr int kNumel = Layout::kNumel;
  constexpr int kThreads = tl::get_numel<WarpLayout> * WARP_SIZE;
  using Global = GlobalTile<Element, Layout>;
  using Shared = SharedTile<Element, Layout, true>;

  const size_t total = (size_t)kNumel * kGrid;
  std::vector<Element> h_src(total), h1(total), h2(total);
  for (size_t i = 0; i < total; ++i) h_src[i] = __float2half((float)((i + i / kNumel) % 2048));
  Element *src, *dst1, *dst2;
  HIP_OK(hipMalloc(&src, total * sizeof(Element)));
  HIP_OK(hipMalloc(&dst1, total * sizeof(Element)));
  HIP_OK(hipMalloc(&dst2, total * sizeof(Element)));
  HIP_OK(hipMemcpy(src, h_src.data(), total * sizeof(Element), hipMemcpyHostToDevice));
  HIP_OK(hipMemset(dst1, 0, total * sizeof(Element)));
  HIP_OK(hipMemset(dst2, 0, total * sizeof(Element)));
  constexpr int kLds = kNumel * sizeof(Element);

  const float t1 = time_ms([&] {
    hipLaunchKernelGGL((g2s_data_transfer<Element, Global, Shared, WarpLayout, kRepeat>), dim3(kGrid), dim3(kThreads),
                       kLds, 0, src, dst1);
  });
  const float t2 = time_ms([&] {
    hipLaunchKernelGGL((baseline_transfer<Element, kNumel, kThreads, kRepeat>), dim3(kGrid), dim3(kThreads), kLds, 0,
                       src, dst2);
  });
  HIP_OK(hipMemcpy(h1.data(), dst1, total * sizeof(Element), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(h2.data(), dst2, total * sizeof(Element), hipMemcpyDeviceToHost));
  bool ok = true;
  for (size_t i = 0; i < total; ++i)
    ok &= __half2float(h1[i]) == __half2float(h_src[i]) && __half2float(h2[i]) == __half2float(h_src[i]);
  if (!ok) ++failures;
  // bytes through LDS per launch: kRepeat x (load + store) of the tile
  const double gbs = 2.0 * kRepeat * total * sizeof(Element) / (t1 * 1e-3) / 1e9;
  // one CU's LDS moves 128 bytes per clock; at the 2.4 GHz peak clock that is 307 GB/s
  const double lds_frac = gbs / (128.0 * 2.4 * kGrid);
  std::printf("|RowMajor(%d, %d)|(%d, %d)|%.4f|%.4f|%.4f|%.1f|%.2f|%s|\n", (int)Layout::kRows, (int)Layout::kCols,
              (int)tl::num_rows<WarpLayout>, (int)tl::num_cols<WarpLayout>, t1, t2, t1 / t2, gbs, lds_frac,
              ok ? "ok" : "MISMATCH");
  HIP_OK(hipFree(src));
  HIP_OK(hipFree(dst1));
  HIP_OK(hipFree(dst2));
}

static void table(int grid) {
  std::printf("\n%d workgroup%s:\n\n", grid, grid == 1 ? " (the reference's measurement)" : "s, one tile each");
  std::printf("|Shape|Wavefront Layout|tile API(ms)|baseline(ms)|Ratio|tile API GB/s|of the LDS peak of the CUs used|check|\n");
  std::printf("|:---|:---:|:---:|:---:|:---:|:---:|:---:|:---:|\n");
  using DType = __half;
  run_test_rowmajor<DType, tl::RowMajor<16, 64>, tl::RowMajor<1, 1>>(grid);
  run_test_rowmajor<DType, tl::RowMajor<64, 64>, tl::RowMajor<1, 1>>(grid);
  run_test_rowmajor<DType, tl::RowMajor<64, 64>, tl::RowMajor<2, 1>>(grid);
  run_test_rowmajor<DType, tl::RowMajor<64, 64>, tl::RowMajor<4, 1>>(grid);
  run_test_rowmajor<DType, tl::RowMajor<128, 128>, tl::RowMajor<1, 1>>(grid);
  run_test_rowmajor<DType, tl::RowMajor<128, 128>, tl::RowMajor<2, 2>>(grid);
  run_test_rowmajor<DType, tl::RowMajor<128, 128>, tl::RowMajor<4, 2>>(grid);
  run_test_rowmajor<DType, tl::RowMajor<128, 256>, tl::RowMajor<1, 1>>(grid);
  run_test_rowmajor<DType, tl::RowMajor<128, 256>, tl::RowMajor<2, 2>>(grid);
  run_test_rowmajor<DType, tl::RowMajor<128, 256>, tl::RowMajor<2, 4>>(grid);
  run_test_rowmajor<DType, tl::RowMajor<128, 256>, tl::RowMajor<4, 4>>(grid);
}

int main() {
  table(1);
  table(256);
  if (failures) std::printf("%d configuration(s) FAILED\n", failures);
  else std::printf("all configurations ok\n");
  return failures ? 1 : 0;
}
