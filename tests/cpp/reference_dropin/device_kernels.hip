// Drop-in check, part 3: the REFERENCE's three macro kernels - include/kernels/gemm_device.cuh
// (ke_gemm and both pipelined forms), fused_two_gemms_device.cuh and flash_attention_device.cuh,
// found through the include path the build recipe passes, never copied - instantiated against
// the tile headers of this repository with the shapes of the reference's own Python tests, and
// launched behind a C ABI.  The reference's traits size the thread block as warps x 32
// (include/kernels/gemm_device.cuh:26); the launches here use 64 lanes per wavefront.
#include <hip/hip_runtime.h>

#include "kernels/flash_attention_device.cuh"   // the reference's files
#include "kernels/fused_two_gemms_device.cuh"
#include "kernels/gemm_device.cuh"

#define DROPIN_API extern "C" __attribute__((visibility("default")))

namespace {
using namespace tilefusion::kernels;

int finish() {
  hipError_t e = hipGetLastError();
  return e != hipSuccess ? (int)e : (int)hipDeviceSynchronize();
}

template <typename Traits, int kLevel>
__global__ void k_gemm(const __half* a, const __half* b, float* c) {
  if constexpr (kLevel == 0) ke_gemm<__half, float, Traits>(a, b, c);
  else if constexpr (kLevel == 1) ke_gemm_level1_pipeline<__half, float, Traits>(a, b, c);
  else ke_gemm_level2_pipeline<__half, float, Traits>(a, b, c);
}
// LDS as the reference's launcher sizes it (src/kernels/gemm.cu:116-121): the staged inputs or the C tile
template <typename WarpLayout, int kLevel, int M, int N, int K, int TM, int TN, int TK, int RK, int kStages>
int run_gemm(const void* a, const void* b, void* c) {
  using Traits = KeGemmTraits<__half, float, WarpLayout, M, N, K, TM, TN, TK, RK, kStages, 64>;
  constexpr int kInputs = (TM * TK + TK * TN) * kStages * (int)sizeof(__half);
  constexpr int kOutput = TM * TN * (int)sizeof(float);
  constexpr int kLds = kInputs > kOutput ? kInputs : kOutput;
  auto kernel = k_gemm<Traits, kLevel>;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLds) != hipSuccess)
    return -2;
  hipLaunchKernelGGL(kernel, dim3(M / TM, N / TN), dim3(tl::get_numel<WarpLayout> * WARP_SIZE), kLds, 0,
                     static_cast<const __half*>(a), static_cast<const __half*>(b), static_cast<float*>(c));
  return finish();
}

template <typename Traits>
__global__ void k_fused(const __half* a, const __half* b, const __half* c, __half* d) {
  ke_fused_two_gemms<__half, float, Traits>(a, b, c, d);
}
template <typename WarpLayout, int M, int N, int K, int P, int TM, int TN, int TK, int TP>
int run_fused(const void* a, const void* b, const void* c, void* d) {
  using Traits = FusedTwoGemmsTraits<__half, float, WarpLayout, M, N, K, P, TM, TN, TK, TP>;
  constexpr int kInputs = (TM * TK + TK * TN + TN * TP) * (int)sizeof(__half);
  constexpr int kOutput = TM * TP * (int)sizeof(__half);
  constexpr int kLds = kInputs > kOutput ? kInputs : kOutput;
  auto kernel = k_fused<Traits>;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLds) != hipSuccess)
    return -2;
  hipLaunchKernelGGL(kernel, dim3(M / TM, P / TP, 1), dim3(tl::get_numel<WarpLayout> * WARP_SIZE), kLds, 0,
                     static_cast<const __half*>(a), static_cast<const __half*>(b), static_cast<const __half*>(c),
                     static_cast<__half*>(d));
  return finish();
}

template <typename Traits>
__global__ void k_flash(const __half* q, const __half* k, const __half* v, __half* o) {
  ke_flash_attention<__half, float, __half, Traits>(q, k, v, o);
}
template <int M, int N, int K, int P, int TM, int TN, int TK, int TP, bool kCausal>
int run_flash(const void* q, const void* k, const void* v, void* o) {
  using WarpLayout = tl::RowMajor<4, 1>;   // src/kernels/flash_attn.cu:81
  constexpr double kScale = 0.08838834764831845;   // 1 / sqrt(128)
  static_assert(K == 128, "the softmax scale above is for a head dimension of 128");
  using Traits = FlashAttentionTraits<__half, float, __half, TileShape<M, N, K, P>, TileShape<TM, TN, TK, TP>, WarpLayout,
                                      kScale, kCausal>;
  constexpr int kLds = (TM * TK + TK * TN + TN * TP) * (int)sizeof(__half);
  auto kernel = k_flash<Traits>;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLds) != hipSuccess)
    return -2;
  hipLaunchKernelGGL(kernel, dim3(M / TM, P / TP, 1), dim3(tl::get_numel<WarpLayout> * WARP_SIZE), kLds, 0,
                     static_cast<const __half*>(q), static_cast<const __half*>(k), static_cast<const __half*>(v),
                     static_cast<__half*>(o));
  return finish();
}
}  // namespace

// GEMM, 64 x 64 x 64 tiles, register steps of 16 (tests/python/test_gemm.py:75-135).
// variant 0: ke_gemm on one wavefront per workgroup (its loop refills the LDS tiles without a
//            barrier after the fragment reads, include/kernels/gemm_device.cuh:153-165, which is
//            only well defined for a single wavefront), [128, 128, 128];
// variant 1: level-1 pipeline, 2 stages, 2 x 2 wavefronts, [256, 256, 256];
// variant 2: level-2 pipeline, 3 stages, 2 x 2 wavefronts, [256, 256, 256];
// variant 3: level-2 pipeline, 3 stages, 2 x 2 wavefronts, [512, 512, 512].
DROPIN_API int dropin_ke_gemm(int variant, const void* a, const void* b, void* c) {
  switch (variant) {
    case 0: return run_gemm<tl::RowMajor<1, 1>, 0, 128, 128, 128, 64, 64, 64, 16, 1>(a, b, c);
    case 1: return run_gemm<tl::RowMajor<2, 2>, 1, 256, 256, 256, 64, 64, 64, 16, 2>(a, b, c);
    case 2: return run_gemm<tl::RowMajor<2, 2>, 2, 256, 256, 256, 64, 64, 64, 16, 3>(a, b, c);
    case 3: return run_gemm<tl::RowMajor<2, 2>, 2, 512, 512, 512, 64, 64, 64, 16, 3>(a, b, c);
    default: return -1;
  }
}
DROPIN_API void dropin_ke_gemm_shape(int variant, int* m, int* n, int* k) {
  static const int t[4][3] = {{128, 128, 128}, {256, 256, 256}, {256, 256, 256}, {512, 512, 512}};
  *m = t[variant][0]; *n = t[variant][1]; *k = t[variant][2];
}

// fused two GEMMs: the reference's test case M, N, K, P = 256, 128, 64, 64 with 64-wide tiles
// (tests/python/test_fused_two_gemms.py) on 2 x 1 wavefronts.  kTP equals kP: the reference
// declares its D tile with a row stride of kTP (include/kernels/fused_two_gemms_device.cuh:91).
DROPIN_API int dropin_ke_fused(const void* a, const void* b, const void* c, void* d) {
  return run_fused<tl::RowMajor<2, 1>, 256, 128, 64, 64, 64, 64, 64, 64>(a, b, c, d);
}

// flash attention: the reference's two test cases (tests/python/test_flash_attn.py:202-232),
// tiles (64, 128, 128, 128): variant 0 (64, 128, 128, 128) plain, variant 1 (128, 128, 128, 128) causal
DROPIN_API int dropin_ke_flash(int variant, const void* q, const void* k, const void* v, void* o) {
  switch (variant) {
    case 0: return run_flash<64, 128, 128, 128, 64, 128, 128, 128, false>(q, k, v, o);
    case 1: return run_flash<128, 128, 128, 128, 64, 128, 128, 128, true>(q, k, v, o);
    default: return -1;
  }
}
