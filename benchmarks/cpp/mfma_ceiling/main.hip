// What the matrix cores of this GPU sustain with nothing else going on: every SIMD of every CU
// runs a loop of back-to-back fp16 MFMAs on random operands held in registers (no LDS, no memory
// traffic), long enough for the power management to settle.  The result is the ceiling any fp16
// GEMM-shaped kernel on the same box is under: the clock a kernel gets follows the power it
// draws, so a kernel that also moves data through LDS, L2 and the fabric runs at a lower clock
// than this loop.  Two MFMA shapes with the same flops per loop iteration are compared.
//
// Printed per shape: time per launch, TFLOP/s, shader cycles per iteration (256 = the matrix
// pipe never idles) and the shader clock the loop ran at (cycles counted by s_memtime / time).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));

#define HIP_OK(expr)                                                                        \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    if (e_ != hipSuccess) {                                                                 \
      std::fprintf(stderr, "%s failed: %s\n", #expr, hipGetErrorString(e_));                \
      std::exit(2);                                                                         \
    }                                                                                       \
  } while (0)

#define M16(acc, a, b) "v_mfma_f32_16x16x32_f16 %" #acc ", %" #a ", %" #b ", %" #acc "\n\t"
#define M32(acc, a, b) "v_mfma_f32_32x32x16_f16 %" #acc ", %" #a ", %" #b ", %" #acc "\n\t"

// kShape 16: 16 x v_mfma_f32_16x16x32_f16 per iteration; kShape 32: 8 x v_mfma_f32_32x32x16_f16.
// The instruction order is fixed in assembly so that no compiler scheduling enters the figure.
template <int kShape>
__global__ __launch_bounds__(256) void mfma_loop(int iters, const half8* src, float* out) {
  const half8 a0 = src[threadIdx.x], a1 = src[threadIdx.x + 256], a2 = src[threadIdx.x + 512],
              a3 = src[threadIdx.x + 768];
  const half8 b0 = src[(threadIdx.x * 7 + 3) % 1024], b1 = src[(threadIdx.x * 5 + 11) % 1024];
  const long long t0 = __builtin_amdgcn_s_memtime();
  float r = 0;
  if constexpr (kShape == 16) {
    float4v c0{}, c1{}, c2{}, c3{}, c4{}, c5{}, c6{}, c7{};
    for (int it = 0; it < iters; ++it)
      asm volatile(M16(0, 8, 12) M16(1, 9, 12) M16(2, 10, 12) M16(3, 11, 12) M16(4, 8, 13) M16(5, 9, 13)
                   M16(6, 10, 13) M16(7, 11, 13) M16(0, 9, 13) M16(1, 10, 13) M16(2, 11, 13) M16(3, 8, 13)
                   M16(4, 9, 12) M16(5, 10, 12) M16(6, 11, 12) M16(7, 8, 12)
                   : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3), "+v"(c4), "+v"(c5), "+v"(c6), "+v"(c7)
                   : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(b0), "v"(b1));
    r = c0[0] + c1[1] + c2[2] + c3[3] + c4[0] + c5[1] + c6[2] + c7[3];
  } else {
    float16v c0{}, c1{}, c2{}, c3{};
    for (int it = 0; it < iters; ++it)
      asm volatile(M32(0, 4, 8) M32(1, 5, 8) M32(2, 6, 9) M32(3, 7, 9) M32(0, 5, 9) M32(1, 6, 9) M32(2, 7, 8)
                   M32(3, 4, 8)
                   : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3)
                   : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(b0), "v"(b1));
    r = c0[0] + c1[1] + c2[2] + c3[3];
  }
  const long long t1 = __builtin_amdgcn_s_memtime();
  if (threadIdx.x == 0 && blockIdx.x == 5) out[1] = (float)(t1 - t0) / iters;
  if (r == 123.456f) out[0] = r;   // keeps the accumulators alive
}

template <int kShape>
static double run(const half8* src, float* out, int cus) {
  const int iters = 10000;   // ~1.3 ms per launch
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0));
  HIP_OK(hipEventCreate(&e1));
  for (int w = 0; w < 300; ++w) hipLaunchKernelGGL(mfma_loop<kShape>, dim3(cus), dim3(256), 0, 0, iters, src, out);
  HIP_OK(hipDeviceSynchronize());
  const int reps = 100;
  HIP_OK(hipEventRecord(e0));
  for (int rep = 0; rep < reps; ++rep)
    hipLaunchKernelGGL(mfma_loop<kShape>, dim3(cus), dim3(256), 0, 0, iters, src, out);
  HIP_OK(hipEventRecord(e1));
  HIP_OK(hipEventSynchronize(e1));
  float ms;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  ms /= reps;
  const double flops = (double)cus * 4 * iters * 16 * (2.0 * 16 * 16 * 32);
  float h[2];
  HIP_OK(hipMemcpy(h, out, sizeof(h), hipMemcpyDeviceToHost));
  const double tflops = flops / ms / 1e9;
  std::printf("|%s|%.3f|%.0f|%.2f|%.1f|%.2f|\n", kShape == 16 ? "v_mfma_f32_16x16x32_f16" : "v_mfma_f32_32x32x16_f16", ms,
              tflops, tflops / 2500.0, h[1], h[1] * iters / (ms * 1e6));
  return tflops;
}

int main() {
  hipDeviceProp_t prop;
  HIP_OK(hipGetDeviceProperties(&prop, 0));
  const int cus = prop.multiProcessorCount;
  half8* src;
  float* out;
  HIP_OK(hipMalloc(&src, 1024 * sizeof(half8)));
  HIP_OK(hipMalloc(&out, 64));
  static _Float16 h[8192];
  std::srand(1);
  for (auto& x : h) x = (_Float16)((std::rand() / (float)RAND_MAX - 0.5f) * 2.f);
  HIP_OK(hipMemcpy(src, h, sizeof(h), hipMemcpyHostToDevice));
  std::printf("%d CUs, one workgroup of 4 wavefronts each, ~0.5 s per row\n\n", cus);
  std::printf("|instruction|ms per launch|TFLOP/s|of the 2500 TFLOP/s peak|cycles per iteration (256 = pipe never idle)|shader clock (GHz)|\n");
  std::printf("|:---|:---:|:---:|:---:|:---:|:---:|\n");
  const double t16 = run<16>(src, out, cus);
  const double t32 = run<32>(src, out, cus);
  return t16 > 0 && t32 > 0 ? 0 : 1;
}
