// Run-time instantiations of the header macro kernels, used behind the C ABI for shapes and
// element types that have no ahead-of-time kernel (see jit_ops.cpp).
#pragma once

#include <cstdint>

#include "common.hpp"

namespace tfk {

// c_kind: 0 = fp32 output, 1 = output in the input type
bool jit_gemm_supports(int64_t M, int64_t N, int64_t K);
int jit_gemm(const void* A, const void* B, void* C, int dtype, int c_kind, int64_t M, int64_t N, int64_t K, int tm,
             int tn, int tk, int num_stages, int pipeline_level, hipStream_t st);

// V must be handed over transposed ([batch, Dv, Lkv])
bool jit_flash_attention_supports(int64_t Lq, int64_t Lkv, int64_t D, int64_t Dv, int v_is_transposed);
int jit_flash_attention(const void* Q, const void* K, const void* Vt, void* O, int dtype, int64_t batch, int64_t Lq,
                        int64_t Lkv, int64_t D, int64_t Dv, int tq, int tkv, int thqk, int thv, double scale,
                        int causal, hipStream_t st);

}  // namespace tfk
