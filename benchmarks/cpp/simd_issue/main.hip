// What one SIMD of a gfx950 compute unit issues per cycle when two wavefronts share it: the cost
// of VALU / transcendental / dot / LDS instructions of one wavefront while the other streams
// MFMAs, and the cost of an attention-like MFMA block next to a softmax-like VALU block.
// These figures decide how the flash-attention kernel arranges its two wavefronts per SIMD.
// No counterpart in the reference (its kernels are compiler-scheduled).
//
// Every kernel is 256 workgroups x 8 wavefronts; wavefronts w and w + 4 share a SIMD.  Wavefronts
// 0-3 ("first", the older ones for the issue arbiter) run one role, 4-7 another.  A role that
// only provides the background runs three times as many iterations as the measured one, so that
// it is active for the whole measurement.  Times are shader cycles (s_memtime) per iteration.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef unsigned uint4v __attribute__((ext_vector_type(4)));
typedef unsigned uint2v __attribute__((ext_vector_type(2)));
#define CK(x)                                                       \
  do {                                                              \
    hipError_t e = (x);                                             \
    if (e != hipSuccess) {                                          \
      printf("%s: %s\n", #x, hipGetErrorString(e));                 \
      exit(1);                                                      \
    }                                                               \
  } while (0)

enum Role {
  kIdle = 0,
  kMfma,      // 32 x v_mfma_f32_16x16x32_f16, 8 independent accumulators
  kFma,       // 96 x v_fma_f32
  kCvt,       // 96 x v_cvt_pk_f16_f32
  kMax3,      // 96 x v_max3_f32
  kExp,       // 96 x v_exp_f32
  kDot2,      // 96 x v_dot2c_f32_f16
  kFmaLds,    // 96 x v_fma_f32 with 32 x ds_read_b128 in between
  kMfmaLds,   // 32 x MFMA with 32 x ds_read_b128 in between
  kBlock16,   // attention MFMA block, 16x16x32: 68 MFMA, 36 ds_read_b64_tr_b16 pairs... (see below)
  kBlock32,   // the same work with 34 x v_mfma_f32_32x32x16_f16
  kSoftmax,   // 32 exp, 16 cvt_pk, 20 max3 (one tile of 32 queries x 64 keys)
};

// ---- single-instruction streams: operands %0-%7 eight independent registers, %8 / %9 sources
#define R8(OP) OP(0) OP(1) OP(2) OP(3) OP(4) OP(5) OP(6) OP(7)
#define FMA(i) "v_fma_f32 %" #i ", %" #i ", %8, %9\n\t"
#define CVT(i) "v_cvt_pk_f16_f32 %" #i ", %8, %9\n\t"
#define MAX3(i) "v_max3_f32 %" #i ", %" #i ", %8, %9\n\t"
#define EXPI(i) "v_exp_f32 %" #i ", %" #i "\n\t"
#define DOT2(i) "v_dot2c_f32_f16 %" #i ", 0x3c003c00, %8\n\t"
#define X12(S) S S S S S S S S S S S S

// ---- MFMA streams: %0-%7 accumulators, %8-%11 fragment registers (LDS destinations), %12 / %13
//      operands, %14 LDS address, %15-%22 destinations of the transposing reads
#define M16(i, a) "v_mfma_f32_16x16x32_f16 %" #i ", %" #a ", %13, %" #i "\n\t"
#define B128(d, off) "ds_read_b128 %" #d ", %14 offset:" #off "\n\t"
#define TRR(d, off) "ds_read_b64_tr_b16 %" #d ", %14 offset:" #off "\n\t"
#define W(n) "s_waitcnt lgkmcnt(" #n ")\n\t"
#define VADD "v_add_u32 %14, 0, %14\n\t"
#define M8 M16(0, 8) M16(1, 9) M16(2, 10) M16(3, 11) M16(4, 8) M16(5, 9) M16(6, 10) M16(7, 11)
#define ML(i, f, off) M16(i, f) B128(f, off)
#define ML8 ML(0, 8, 0) ML(1, 9, 4096) ML(2, 10, 8192) ML(3, 11, 12288) ML(4, 8, 1024) ML(5, 9, 5120) ML(6, 10, 9216) ML(7, 11, 13312)
// The MFMA block of one 64-key tile for 32 queries, as the attention kernel issues it:
//   second product: 36 MFMAs (32 + 4 for the row sums), a pair of transposing reads and a wait
//   per MFMA pair, then the four K fragment reads of the next tile;
//   first product: 4 reduction steps of 8 MFMAs with the next step's 4 fragment reads and waits.
#define PV16(i, j, f, lo, hi) M16(i, f) M16(j, f) TRR(lo, 0) TRR(hi, 2048) W(6)
#define PVBLK16                                                                               \
  PV16(0, 1, 8, 15, 16) PV16(2, 3, 9, 17, 18) PV16(4, 5, 10, 19, 20) PV16(6, 7, 11, 21, 22) VADD \
  PV16(0, 1, 8, 15, 16) PV16(2, 3, 9, 17, 18) PV16(4, 5, 10, 19, 20) PV16(6, 7, 11, 21, 22) VADD \
  PV16(0, 1, 8, 15, 16)
#define QK16                                                                                      \
  M16(0, 8) M16(1, 8) B128(8, 4096) W(4) M16(2, 9) M16(3, 9) B128(9, 8192) W(4) M16(4, 10) M16(5, 10) \
  B128(10, 12288) W(4) M16(6, 11) M16(7, 11) B128(11, 0) W(4) VADD
#define BLOCK16 PVBLK16 PVBLK16 B128(8, 0) B128(9, 4096) B128(10, 8192) B128(11, 12288) QK16 QK16 QK16 QK16 W(0)
// the same with 32x32x16 MFMAs: %0-%3 accumulators, %4-%7 fragments, %8 / %9 operands, %10 address
#define M32(i, a) "v_mfma_f32_32x32x16_f16 %" #i ", %" #a ", %9, %" #i "\n\t"
#define TRR2(d, off) "ds_read_b64_tr_b16 %" #d ", %10 offset:" #off "\n\t"
#define B1282(d, off) "ds_read_b128 %" #d ", %10 offset:" #off "\n\t"
#define VADD2 "v_add_u32 %10, 0, %10\n\t"
#define PV32(i, f, lo, hi) M32(i, f) TRR2(lo, 0) TRR2(hi, 2048) W(6)
#define PVBLK32                                                                                  \
  PV32(0, 4, 11, 12) PV32(1, 5, 13, 14) PV32(2, 6, 15, 16) PV32(3, 7, 17, 18) VADD2 PV32(0, 4, 11, 12) \
  PV32(1, 5, 13, 14) PV32(2, 6, 15, 16) PV32(3, 7, 17, 18) VADD2 PV32(0, 4, 11, 12)
#define QK32 \
  M32(0, 4) B1282(4, 4096) W(4) M32(1, 5) B1282(5, 8192) W(4) M32(2, 6) B1282(6, 12288) W(4) M32(3, 7) B1282(7, 0) W(4) VADD2
#define BLOCK32 PVBLK32 PVBLK32 B1282(4, 0) B1282(5, 4096) B1282(6, 8192) B1282(7, 12288) QK32 QK32 QK32 QK32 W(0)
// softmax of one tile: %0-%7 scores, %8 / %9 running maxima, %10 / %11 packed weights
#define SEX(i) "v_exp_f32 %" #i ", %" #i "\n\t"
#define SCV(d, a, b) "v_cvt_pk_f16_f32 %" #d ", %" #a ", %" #b "\n\t"
#define SMX(d, a, b) "v_max3_f32 %" #d ", %" #d ", %" #a ", %" #b "\n\t"
#define SMQ                                                                                      \
  SMX(8, 0, 1) SMX(9, 2, 3) SMX(8, 4, 5) SMX(9, 6, 7) SMX(8, 0, 2) SEX(0) SEX(1) SCV(10, 0, 1) SEX(2) \
  SEX(3) SCV(11, 2, 3) SEX(4) SEX(5) SCV(10, 4, 5) SEX(6) SEX(7) SCV(11, 6, 7)

template <int ROLE>
__device__ void run_role(int iters, float* out, char* lds, int prio, int slot) {
  half8 x, y;
  for (int t = 0; t < 8; ++t) {
    x[t] = (_Float16)(0.001f * (threadIdx.x + t));
    y[t] = (_Float16)(0.002f * (threadIdx.x * 3 + t));
  }
  unsigned addr = (unsigned)(size_t)(__attribute__((address_space(3))) char*)lds + (threadIdx.x & 63) * 16 +
                  ((threadIdx.x >> 6) & 3) * 16384;
  if (prio) __builtin_amdgcn_s_setprio(2);
  float r = 0.f;
  __syncthreads();
  const long long t0 = __builtin_amdgcn_s_memtime();
  if constexpr (ROLE == kFma || ROLE == kCvt || ROLE == kMax3 || ROLE == kExp || ROLE == kDot2) {
    float f0 = threadIdx.x * 0.01f, f1 = f0 + 1, f2 = f0 + 2, f3 = f0 + 3, f4 = f0 + 4, f5 = f0 + 5, f6 = f0 + 6,
          f7 = f0 + 7, c1 = 0.999f, c2 = 0.001f;
    for (int i = 0; i < iters; ++i) {
#define STREAM(OP)                                                                                        \
  asm volatile(X12(R8(OP)) : "+v"(f0), "+v"(f1), "+v"(f2), "+v"(f3), "+v"(f4), "+v"(f5), "+v"(f6), "+v"(f7) \
               : "v"(c1), "v"(c2))
      if constexpr (ROLE == kFma) STREAM(FMA);
      if constexpr (ROLE == kCvt) STREAM(CVT);
      if constexpr (ROLE == kMax3) STREAM(MAX3);
      if constexpr (ROLE == kExp) STREAM(EXPI);
      if constexpr (ROLE == kDot2) STREAM(DOT2);
    }
    r = f0 + f1 + f2 + f3 + f4 + f5 + f6 + f7;
  } else if constexpr (ROLE == kSoftmax) {
    float s0 = threadIdx.x * 0.01f, s1 = s0 + 1, s2 = s0 + 2, s3 = s0 + 3, s4 = s0 + 4, s5 = s0 + 5, s6 = s0 + 6,
          s7 = s0 + 7, m0 = 0, m1 = 0, p0 = 0, p1 = 0;
    for (int i = 0; i < iters; ++i)
      asm volatile(SMQ SMQ SMQ SMQ
                   : "+v"(s0), "+v"(s1), "+v"(s2), "+v"(s3), "+v"(s4), "+v"(s5), "+v"(s6), "+v"(s7), "+v"(m0),
                     "+v"(m1), "+v"(p0), "+v"(p1));
    r = s0 + s1 + s2 + s3 + s4 + s5 + s6 + s7 + m0 + m1 + p0 + p1;
  } else if constexpr (ROLE == kBlock32) {
    float16v a0{}, a1{}, a2{}, a3{};
    a0[0] = 1; a1[1] = 2; a2[2] = 3; a3[3] = 4;
    uint4v f0{}, f1{}, f2{}, f3{};
    uint2v d0{}, d1{}, d2{}, d3{}, d4{}, d5{}, d6{}, d7{};
    for (int i = 0; i < iters; ++i)
      asm volatile(BLOCK32
                   : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(f0), "+v"(f1), "+v"(f2), "+v"(f3), "+v"(x), "+v"(y),
                     "+v"(addr), "+v"(d0), "+v"(d1), "+v"(d2), "+v"(d3), "+v"(d4), "+v"(d5), "+v"(d6), "+v"(d7));
    r = a0[0] + a1[1] + a2[2] + a3[3] + (float)(f0[0] + f1[0] + f2[0] + f3[0] + d0[0] + d1[0] + d2[0] + d3[0] +
                                               d4[0] + d5[0] + d6[0] + d7[0]);
  } else if constexpr (ROLE != kIdle) {
    float4v a0{1, 2, 3, 4}, a1 = a0, a2 = a0, a3 = a0, a4 = a0, a5 = a0, a6 = a0, a7 = a0;
    uint4v f0{1, 2, 3, 4}, f1 = f0, f2 = f0, f3 = f0;
    uint2v d0{}, d1{}, d2{}, d3{}, d4{}, d5{}, d6{}, d7{};
    float g0 = threadIdx.x * 0.01f, g1 = g0 + 1;
    for (int i = 0; i < iters; ++i) {
#define MSTREAM(S)                                                                                               \
  asm volatile(S : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7), "+v"(f0),      \
               "+v"(f1), "+v"(f2), "+v"(f3), "+v"(x), "+v"(y), "+v"(addr), "+v"(d0), "+v"(d1), "+v"(d2), "+v"(d3), \
               "+v"(d4), "+v"(d5), "+v"(d6), "+v"(d7), "+v"(g0), "+v"(g1))
      if constexpr (ROLE == kMfma) MSTREAM(M8 M8 M8 M8);
      if constexpr (ROLE == kMfmaLds) MSTREAM(ML8 ML8 ML8 ML8 W(0));
      if constexpr (ROLE == kBlock16) MSTREAM(BLOCK16);
      if constexpr (ROLE == kFmaLds) {
#define FL(d, off) "v_fma_f32 %23, %23, %24, %24\n\tv_fma_f32 %24, %24, %23, %23\n\tv_fma_f32 %23, %23, %24, %24\n\t" B128(d, off)
        MSTREAM(FL(8, 0) FL(9, 4096) FL(10, 8192) FL(11, 12288) FL(8, 1024) FL(9, 5120) FL(10, 9216) FL(11, 13312)
                FL(8, 0) FL(9, 4096) FL(10, 8192) FL(11, 12288) FL(8, 1024) FL(9, 5120) FL(10, 9216) FL(11, 13312)
                FL(8, 0) FL(9, 4096) FL(10, 8192) FL(11, 12288) FL(8, 1024) FL(9, 5120) FL(10, 9216) FL(11, 13312)
                FL(8, 0) FL(9, 4096) FL(10, 8192) FL(11, 12288) FL(8, 1024) FL(9, 5120) FL(10, 9216) FL(11, 13312) W(0));
      }
    }
    r = a0[0] + a1[1] + a2[2] + a3[3] + a4[0] + a5[0] + a6[0] + a7[0] + g0 + g1 +
        (float)(f0[0] + f1[0] + f2[0] + f3[0] + d0[0] + d1[0] + d2[0] + d3[0] + d4[0] + d5[0] + d6[0] + d7[0]);
  }
  const long long t1 = __builtin_amdgcn_s_memtime();
  if (blockIdx.x == 17 && (threadIdx.x & 255) == 0) out[1024 + slot] = (float)(t1 - t0) / iters;
  if (r == 12345.678f) out[threadIdx.x] = r;  // keeps the results alive
}

template <int FIRST, int SECOND>
__global__ __launch_bounds__(512) void probe(int iters_first, int iters_second, float* out, int prio_first,
                                             int prio_second) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  for (int i = threadIdx.x; i < 81920 / 4; i += 512) ((unsigned*)smem)[i] = i * 2654435761u;
  if (threadIdx.x < 256) run_role<FIRST>(iters_first, out, smem, prio_first, 0);
  else run_role<SECOND>(iters_second, out, smem, prio_second, 1);
}

struct Result { float first, second; };
// bg: 0 = both roles run `iters` iterations, 1 = the first role is background (3x), 2 = the second
template <int FIRST, int SECOND>
Result run(int bg = 0, int prio_first = 0, int prio_second = 0) {
  float* out;
  CK(hipMalloc(&out, 8192));
  CK(hipMemset(out, 0, 8192));
  const int iters = 3000;
  CK(hipFuncSetAttribute((const void*)probe<FIRST, SECOND>, hipFuncAttributeMaxDynamicSharedMemorySize, 81920));
  for (int w = 0; w < 2; ++w)
    hipLaunchKernelGGL((probe<FIRST, SECOND>), dim3(256), dim3(512), 81920, 0, bg == 1 ? 3 * iters : iters,
                       bg == 2 ? 3 * iters : iters, out, prio_first, prio_second);
  CK(hipDeviceSynchronize());
  float h[2];
  CK(hipMemcpy(h, out + 1024, 8, hipMemcpyDeviceToHost));
  CK(hipFree(out));
  return {h[0], h[1]};
}

template <int ROLE>
void stream_row(const char* name, int n) {
  const float alone = run<ROLE, kIdle>().first;
  const float under_old = run<kMfma, ROLE>(1).second;   // MFMA stream in the older wavefront
  const float under_young = run<ROLE, kMfma>(2).first;  // MFMA stream in the younger wavefront
  printf("|%s|%.1f|%.1f|%.1f|\n", name, alone / n, under_old / n, under_young / n);
}

int main() {
  printf("16x16x32 MFMA stream alone: %.1f cycles per MFMA; two wavefronts of one SIMD both streaming: %.1f per MFMA and SIMD\n\n",
         run<kMfma, kIdle>().first / 32, run<kMfma, kMfma>().second / 64);
  printf("|instruction stream of one wavefront|cycles per instruction, alone|while an older wavefront of the SIMD streams MFMAs|while a younger one does|\n");
  printf("|:---|:---:|:---:|:---:|\n");
  stream_row<kFma>("v_fma_f32", 96);
  stream_row<kCvt>("v_cvt_pk_f16_f32", 96);
  stream_row<kMax3>("v_max3_f32", 96);
  stream_row<kExp>("v_exp_f32", 96);
  stream_row<kDot2>("v_dot2c_f32_f16", 96);
  printf("\n|stream|cycles per iteration|\n|:---|:---:|\n");
  printf("|96 v_fma_f32|%.0f|\n", run<kFma, kIdle>().first);
  printf("|96 v_fma_f32 + 32 ds_read_b128|%.0f|\n", run<kFmaLds, kIdle>().first);
  printf("|32 MFMA|%.0f|\n", run<kMfma, kIdle>().first);
  printf("|32 MFMA + 32 ds_read_b128|%.0f|\n", run<kMfmaLds, kIdle>().first);
  printf("\n|MFMA block of one attention tile (32 queries x 64 keys, D = 128)|16x16x32 (68 MFMAs)|32x32x16 (34 MFMAs)|\n|:---|:---:|:---:|\n");
  printf("|alone|%.0f|%.0f|\n", run<kBlock16, kIdle>().first, run<kBlock32, kIdle>().first);
  printf("|next to the softmax block of a younger wavefront|%.0f|%.0f|\n", run<kBlock16, kSoftmax>(2).first,
         run<kBlock32, kSoftmax>(2).first);
  printf("|next to the softmax block of an older wavefront|%.0f|%.0f|\n", run<kSoftmax, kBlock16>(1).second,
         run<kSoftmax, kBlock32>(1).second);
  printf("|the same with raised priority (s_setprio 2) for the MFMA block|%.0f|%.0f|\n",
         run<kSoftmax, kBlock16>(1, 0, 1).second, run<kSoftmax, kBlock32>(1, 0, 1).second);
  printf("\n|softmax block of one tile (32 exp2, 16 convert, 20 max3)|cycles|\n|:---|:---:|\n");
  printf("|alone|%.0f|\n", run<kSoftmax, kIdle>().first);
  printf("|next to the MFMA block (16x16x32) of an older wavefront|%.0f|\n", run<kBlock16, kSoftmax>(1).second);
  printf("|next to the MFMA block of a younger wavefront|%.0f|\n", run<kSoftmax, kBlock16>(2).first);
  printf("\ndone\n");
  return 0;
}
