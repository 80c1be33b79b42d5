// Shared host/device helpers for the gfx950 kernels: vector types, MFMA wrappers,
// direct global->LDS loads, error reporting for the C ABI.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "tilefusion_c.h"

namespace tfk {

using half_t = _Float16;
using bf16_t = __bf16;
using half2_t = _Float16 __attribute__((ext_vector_type(2)));
using half4_t = _Float16 __attribute__((ext_vector_type(4)));
using half8_t = _Float16 __attribute__((ext_vector_type(8)));
using float4_t = float __attribute__((ext_vector_type(4)));
using float16_t = float __attribute__((ext_vector_type(16)));
using uint4_t = unsigned __attribute__((ext_vector_type(4)));
using uint2_t = unsigned __attribute__((ext_vector_type(2)));

constexpr int kWaveSize = 64;
constexpr int kMaxLdsBytes = 160 * 1024;

#define TFK_DEVICE __device__ __forceinline__

// D(32x32) += A(32x16) * B(16x32).  Lane l supplies A[l%32][8*(l/32)+t] and
// B[8*(l/32)+t][l%32], t = 0..7; accumulator register r of lane l is
// D[8*(r/4) + 4*(l/32) + r%4][l%32].
TFK_DEVICE float16_t mfma_32x32x16(half8_t a, half8_t b, float16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
// D(16x16) += A(16x32) * B(32x16).  Lane l supplies A[l%16][8*(l/16)+t] and
// B[8*(l/16)+t][l%16]; accumulator register r of lane l is D[4*(l/16)+r][l%16].
TFK_DEVICE float4_t mfma_16x16x32(half8_t a, half8_t b, float4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// 16 bytes per lane straight from global memory into LDS, bypassing VGPRs.  `lds_wave_base`
// must be wave-uniform; lane l's 16 bytes land at lds_wave_base + 16*l.
TFK_DEVICE void load_global_to_lds_16B(const void* gptr, void* lds_wave_base) {
  __builtin_amdgcn_global_load_lds(
      (const __attribute__((address_space(1))) void*)gptr,
      (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}

// Same transfer issued from inline assembly.  The compiler then does not model the write into
// LDS at all, so it never drains these loads on its own (with the builtin it inserts
// vmcnt(0) at every control-flow join after a load); ordering against LDS reads is entirely
// the caller's job (wait_vmem / barrier_keep_vmem below).  `lds_addr` is the wave-uniform LDS
// byte address of the 1 KiB destination.
TFK_DEVICE void lds_dma_16B(const void* gptr, unsigned lds_addr) {
  // M0 (the LDS destination) is an INPUT of the statement: the compiler writes it and cannot use the
  // register for anything else between that write and the load; the s_nop is the wait state an
  // M0 write needs in front of an LDS-direct load
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(gptr), "{m0}"(lds_addr)
               : "memory");
}
TFK_DEVICE unsigned lds_address(const void* p) {
  return (unsigned)(size_t)((__attribute__((address_space(3))) const char*)p);
}

TFK_DEVICE void wait_vmem_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// Wait until at most N of this wavefront's vector-memory loads are still outstanding
// (loads complete in issue order, so the oldest ones are the ones that have landed).
template <int N>
TFK_DEVICE void wait_vmem() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// Workgroup barrier for a direct-to-LDS pipeline: waits for this wavefront's LDS reads and
// for all but its N youngest vector-memory loads, then synchronises.  __syncthreads() would
// drain every outstanding load (vmcnt(0)) and with it the tiles still in flight.
template <int N>
TFK_DEVICE void barrier_keep_vmem() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// Bare workgroup barrier: nothing of this wavefront is drained (LDS reads and vector-memory loads
// stay in flight; the caller knows that nothing another wavefront does behind it depends on them).
TFK_DEVICE void barrier_only() { asm volatile("s_barrier" ::: "memory"); }

// Workgroup barrier that only drains this wavefront's LDS traffic (reads and writes), leaving
// global loads into registers in flight.
TFK_DEVICE void barrier_lds_only() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---- host side ---------------------------------------------------------------------------
void set_error(const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);

#define TFK_HIP_TRY(expr)                                   \
  do {                                                      \
    hipError_t e__ = (expr);                                \
    if (e__ != hipSuccess) return ::tfk::hip_fail(e__, #expr); \
  } while (0)

// Opts `kern` in to `lds` bytes of dynamic LDS.  The attribute is per device and sticky, so the
// runtime call is made once per kernel and device (a bit per device ordinal in a static of the
// calling template instantiation, i.e. of the kernel), not on every launch.
#define TFK_LDS_OPT_IN(kern, lds)                                                              \
  do {                                                                                         \
    static std::atomic<unsigned long long> done__{0};                                          \
    int dev__ = 0;                                                                             \
    TFK_HIP_TRY(hipGetDevice(&dev__));                                                         \
    const unsigned long long bit__ = (dev__ >= 0 && dev__ < 64) ? (1ull << dev__) : 0ull;      \
    if (!(done__.load(std::memory_order_acquire) & bit__) || bit__ == 0) {                     \
      TFK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                     \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (lds)));     \
      done__.fetch_or(bit__, std::memory_order_release);                                       \
    }                                                                                          \
  } while (0)

#define TFK_REQUIRE(cond, code, ...)  \
  do {                                \
    if (!(cond)) {                    \
      ::tfk::set_error(__VA_ARGS__);  \
      return (code);                  \
    }                                 \
  } while (0)

}  // namespace tfk
