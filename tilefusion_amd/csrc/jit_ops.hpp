// Run-time instantiation of the header attention kernel, used behind the C ABI for head dimensions
// that have no ahead-of-time kernel (see jit_ops.cpp).
#pragma once

#include <cstdint>

#include "common.hpp"

namespace tfk {

// V must be handed over transposed ([batch, Dv, Lkv])
bool jit_flash_attention_supports(int64_t Lq, int64_t Lkv, int64_t D, int64_t Dv, int v_is_transposed);
int jit_flash_attention(const void* Q, const void* K, const void* Vt, void* O, int dtype, int64_t batch, int64_t Lq,
                        int64_t Lkv, int64_t D, int64_t Dv, int tq, int tkv, int thqk, int thv, double scale,
                        int causal, hipStream_t st);

}  // namespace tfk
