// Flash-attention forward for gfx950: O = softmax(scale * Q K^T (+ causal mask)) V per
// (batch x head) slice, fp16 in/out, fp32 scores and fp32 running max / sum.
//
// Counterpart of ke_flash_attention (include/kernels/flash_attention_device.cuh:130-312, mask
// include/cell/mask.hpp:75-82) and its host launcher (src/kernels/flash_attn.cu:58-152).
// CDNA4 design (FA-2 style, un-normalised O with one divide at the end):
//   * one workgroup = 128 queries (4 wavefronts x 32), key/value tiles of 64 rows,
//     v_mfma_f32_32x32x16_f16 throughout;
//   * Q stays in registers for the whole workgroup (the reference reloads it per KV tile);
//   * scores are computed transposed, S^T = K Q^T, so a lane owns ONE query row: its 32
//     score values per tile are plain registers, the row max / sum is an in-lane reduction
//     plus a single v_permlane32_swap with the partner lane, and exp2(S^T) converted to fp16
//     is already the B-operand fragment of the second MFMA O^T = V^T P^T;
//   * K and V tiles go global -> LDS directly (global_load_lds_dwordx4), double-buffered;
//     V is kept [key][dim] in LDS and transposed on the way to registers with
//     ds_read_b64_tr_b16; both tiles are XOR-swizzled against bank conflicts;
//   * causal: tiles right of the diagonal are skipped, only tiles crossing it are masked.
#include "common.hpp"

namespace tfk {
namespace {

constexpr int kBM = 128;  // queries per workgroup
constexpr int kBN = 64;   // keys per tile
constexpr int kFaWaves = 4;
constexpr int kFaThreads = kFaWaves * kWaveSize;

// K tile [kBN][D]: 16 consecutive rows reading one logical chunk hit 16 bank groups.
template <int CH>
__host__ __device__ constexpr int swz_k(int row, int c) {
  constexpr int kRowsPer256B = CH >= 16 ? 1 : 16 / CH;
  return c ^ ((row / kRowsPer256B) % CH);
}
// V tile [kBN][DV] read by transposing 4-row x 16-column blocks: 4 consecutive rows must land
// in different 64-byte quarters of the bank space.
template <int CH>
__host__ __device__ constexpr int swz_v(int row, int c) {
  if constexpr (CH >= 16) return c ^ ((row & 3) << 2);
  return c ^ (((row >> 1) & 1) << 2);
}

// v_permlane32_swap hands every lane its own value and the value of lane l ^ 32 (in an order
// that depends on the half the lane sits in), which is all a symmetric reduction needs.
TFK_DEVICE float pair_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, x),
                                            __builtin_bit_cast(unsigned, x), false, false);
  const unsigned a = r[0], b = r[1];  // copy out: bit_cast of a vector element is unreliable
  return fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}
TFK_DEVICE float pair_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, x),
                                            __builtin_bit_cast(unsigned, x), false, false);
  const unsigned a = r[0], b = r[1];
  return __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
}

typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));

TFK_DEVICE half4_t lds_read_tr4(const char* p) {
  fp16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
      (__attribute__((address_space(3))) fp16x4_t*)(p));
  return __builtin_bit_cast(half4_t, v);
}

template <int D, int DV, bool kVT, bool kCausal>
__global__ __launch_bounds__(kFaThreads, 2) void flash_attention_fwd_kernel(
    const half_t* __restrict__ Q, const half_t* __restrict__ K, const half_t* __restrict__ V,
    half_t* __restrict__ O, int Lq, int Lkv, float scale_log2, int q_tiles) {
  constexpr int kKChunks = D / 8;
  constexpr int kVChunks = kVT ? kBN / 8 : DV / 8;
  constexpr int kKBytes = kBN * D * 2;
  constexpr int kVBytes = kBN * DV * 2;
  constexpr int kStageBytes = kKBytes + kVBytes;
  constexpr int kNT = kBN / 32;
  constexpr int kDT = DV / 32;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 31, lg = lane >> 5;
  // heavy (late) query tiles first when causal
  const int qt = kCausal ? (q_tiles - 1 - (int)blockIdx.x) : (int)blockIdx.x;
  const size_t bh = blockIdx.y;
  Q += bh * (size_t)Lq * D;
  K += bh * (size_t)Lkv * D;
  V += bh * (size_t)Lkv * DV;
  O += bh * (size_t)Lq * DV;

  const int q_row0 = qt * kBM + wave * 32;   // first query row of this wavefront
  const int m_row = q_row0 + lr;             // this lane's query row
  const int m_ld = min(m_row, Lq - 1);

  half8_t qf[D / 16];
#pragma unroll
  for (int kk = 0; kk < D / 16; ++kk)
    qf[kk] = *reinterpret_cast<const half8_t*>(Q + (size_t)m_ld * D + kk * 16 + lg * 8);

  int n_end = Lkv;
  if (kCausal) n_end = min(Lkv, qt * kBM + kBM);
  const int num_tiles = (n_end + kBN - 1) / kBN;

  auto issue_tile_loads = [&](int stage, int n0) {
    char* sk = smem + stage * kStageBytes;
    char* sv = sk + kKBytes;
    {  // K tile: [kBN][D]
      constexpr int kRowsPerInstr = 64 / kKChunks;
      constexpr int kInstr = kBN * kKChunks / 64;
      for (int i = wave; i < kInstr; i += kFaWaves) {
        const int row = i * kRowsPerInstr + lane / kKChunks;
        const int c = swz_k<kKChunks>(row, lane % kKChunks);
        const int gr = min(n0 + row, Lkv - 1);
        load_global_to_lds_16B(K + (size_t)gr * D + c * 8, sk + i * 1024);
      }
    }
    if constexpr (!kVT) {  // V tile: [kBN][DV]
      constexpr int kRowsPerInstr = 64 / kVChunks;
      constexpr int kInstr = kBN * kVChunks / 64;
      for (int i = wave; i < kInstr; i += kFaWaves) {
        const int row = i * kRowsPerInstr + lane / kVChunks;
        const int c = swz_v<kVChunks>(row, lane % kVChunks);
        const int gr = min(n0 + row, Lkv - 1);
        load_global_to_lds_16B(V + (size_t)gr * DV + c * 8, sv + i * 1024);
      }
    } else {  // V^T tile: [DV][kBN] out of a [DV][Lkv] matrix
      constexpr int kRowsPerInstr = 64 / kVChunks;
      constexpr int kInstr = DV * kVChunks / 64;
      for (int i = wave; i < kInstr; i += kFaWaves) {
        const int row = i * kRowsPerInstr + lane / kVChunks;
        const int c = swz_k<kVChunks>(row, lane % kVChunks);
        const int gc = min(n0 + c * 8, Lkv - 8);
        load_global_to_lds_16B(V + (size_t)row * Lkv + gc, sv + i * 1024);
      }
    }
  };

  float16_t o_acc[kDT];
#pragma unroll
  for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.f;
  float m_run = -INFINITY;  // running max of scale*log2(e)*score
  float l_run = 0.f;        // this lane's share of the running sum

  issue_tile_loads(0, 0);
  wait_vmem_all();
  __syncthreads();

  for (int it = 0; it < num_tiles; ++it) {
    if (it + 1 < num_tiles) issue_tile_loads((it + 1) & 1, (it + 1) * kBN);
    const char* sk = smem + (it & 1) * kStageBytes;
    const char* sv = sk + kKBytes;
    const int n0 = it * kBN;

    // ---- S^T = K Q^T ------------------------------------------------------------------
    float16_t s[kNT];
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[nt][r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < D / 16; ++kk)
#pragma unroll
      for (int nt = 0; nt < kNT; ++nt) {
        const int row = nt * 32 + lr;
        const half8_t kf = *reinterpret_cast<const half8_t*>(
            sk + row * D * 2 + swz_k<kKChunks>(row, 2 * kk + lg) * 16);
        s[nt] = mfma_32x32x16(kf, qf[kk], s[nt]);
      }

    // ---- scale, mask ------------------------------------------------------------------
    // s[nt][r] is the score of key n0 + 32*nt + 8*(r/4) + 4*lg + r%4 against query m_row
    const bool need_mask = (kCausal && (n0 + kBN - 1 > q_row0)) || (n0 + kBN > Lkv);
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[nt][r] *= scale_log2;
    if (need_mask) {
#pragma unroll
      for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int n = n0 + nt * 32 + 8 * (r / 4) + 4 * lg + (r % 4);
          if (n >= Lkv || (kCausal && n > m_row)) s[nt][r] = -INFINITY;
        }
    }

    // ---- online softmax ---------------------------------------------------------------
    float mx = s[0][0];
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[nt][r]);
    mx = pair_max(mx);
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    float psum = 0.f;
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        s[nt][r] = __builtin_amdgcn_exp2f(s[nt][r] - m_new);
        psum += s[nt][r];
      }
    l_run = l_run * alpha + psum;
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) o_acc[dt][r] *= alpha;

    // ---- O^T += V^T P^T ---------------------------------------------------------------
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        // reduction step over keys nk .. nk+15; slot t of lane group lg is key
        // nk + 4*lg + t (t < 4) or nk + 8 + 4*lg + (t - 4)
        half8_t pb;
#pragma unroll
        for (int t = 0; t < 8; ++t) pb[t] = (half_t)s[nt][8 * j + t];
        const int nk = nt * 32 + 16 * j;
#pragma unroll
        for (int dt = 0; dt < kDT; ++dt) {
          half8_t vf;
          if constexpr (!kVT) {
            const int r16 = lane & 15;
            const int col = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (r16 & 3);
            const int row_lo = nk + 4 * lg + (r16 >> 2);
            const int row_hi = row_lo + 8;
            const half4_t lo = lds_read_tr4(sv + row_lo * DV * 2 + swz_v<kVChunks>(row_lo, col / 8) * 16 + (col % 8) * 2);
            const half4_t hi = lds_read_tr4(sv + row_hi * DV * 2 + swz_v<kVChunks>(row_hi, col / 8) * 16 + (col % 8) * 2);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              vf[t] = lo[t];
              vf[4 + t] = hi[t];
            }
          } else {
            const int row = dt * 32 + lr;
            const int c0 = nk / 8;  // keys nk + 4*lg .. +3 live in chunk c0, half lg
            const half4_t lo = *reinterpret_cast<const half4_t*>(
                sv + row * kBN * 2 + swz_k<kVChunks>(row, c0) * 16 + lg * 8);
            const half4_t hi = *reinterpret_cast<const half4_t*>(
                sv + row * kBN * 2 + swz_k<kVChunks>(row, c0 + 1) * 16 + lg * 8);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              vf[t] = lo[t];
              vf[4 + t] = hi[t];
            }
          }
          o_acc[dt] = mfma_32x32x16(vf, pb, o_acc[dt]);
        }
      }

    wait_vmem_all();
    __syncthreads();
  }

  // ---- epilogue: O[m][d] = O^T[d][m] / l --------------------------------------------------
  const float l_tot = pair_sum(l_run);
  const float inv = 1.f / l_tot;
  if (m_row < Lq) {
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        half4_t out;
#pragma unroll
        for (int t = 0; t < 4; ++t) out[t] = (half_t)(o_acc[dt][4 * q + t] * inv);
        *reinterpret_cast<half4_t*>(O + (size_t)m_row * DV + dt * 32 + 8 * q + 4 * lg) = out;
      }
  }
}

template <int D, int DV, bool kVT, bool kCausal>
int launch(const void* Q, const void* K, const void* V, void* O, int batch, int Lq, int Lkv,
           float scale_log2, hipStream_t st) {
  auto kern = flash_attention_fwd_kernel<D, DV, kVT, kCausal>;
  constexpr int lds = 2 * (kBN * D * 2 + kBN * DV * 2);
  static_assert(lds <= kMaxLdsBytes, "tiles do not fit in LDS");
  TFK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  const int q_tiles = (Lq + kBM - 1) / kBM;
  hipLaunchKernelGGL(kern, dim3(q_tiles, batch), dim3(kFaThreads), lds, st,
                     static_cast<const half_t*>(Q), static_cast<const half_t*>(K),
                     static_cast<const half_t*>(V), static_cast<half_t*>(O), Lq, Lkv, scale_log2,
                     q_tiles);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}

template <int D, int DV>
int pick(const void* Q, const void* K, const void* V, void* O, int batch, int Lq, int Lkv,
         float scale_log2, bool vt, bool causal, hipStream_t st) {
  if (vt) {
    if (causal) return launch<D, DV, true, true>(Q, K, V, O, batch, Lq, Lkv, scale_log2, st);
    return launch<D, DV, true, false>(Q, K, V, O, batch, Lq, Lkv, scale_log2, st);
  }
  if (causal) return launch<D, DV, false, true>(Q, K, V, O, batch, Lq, Lkv, scale_log2, st);
  return launch<D, DV, false, false>(Q, K, V, O, batch, Lq, Lkv, scale_log2, st);
}

}  // namespace
}  // namespace tfk

extern "C" int tf_flash_attention_fwd_f16(const void* Q, const void* K, const void* V, void* O,
                                          int64_t batch, int64_t Lq, int64_t Lkv, int64_t D,
                                          int64_t Dv, int v_is_transposed, int tile_length_q,
                                          int tile_length_kv, int tile_hidden_qk,
                                          int tile_hidden_v, double softmax_scale, int causal,
                                          void* stream) {
  using namespace tfk;
  TFK_REQUIRE(Q && K && V && O, TF_ERR_INVALID_ARG, "tf_flash_attention_fwd_f16: null pointer");
  TFK_REQUIRE(batch > 0 && Lq > 0 && Lkv > 0 && D > 0 && Dv > 0, TF_ERR_INVALID_ARG,
              "tf_flash_attention_fwd_f16: sizes must be positive");
  TFK_REQUIRE(batch < 65536 && Lq < (1 << 24) && Lkv < (1 << 24), TF_ERR_INVALID_ARG,
              "tf_flash_attention_fwd_f16: dimension too large");
  TFK_REQUIRE(tile_length_q > 0 && tile_length_kv > 0 && tile_hidden_qk > 0 && tile_hidden_v > 0,
              TF_ERR_INVALID_ARG, "tf_flash_attention_fwd_f16: tile sizes must be positive");
  TFK_REQUIRE(Lq % tile_length_q == 0 && Lkv % tile_length_kv == 0 && D % tile_hidden_qk == 0 &&
                  Dv % tile_hidden_v == 0,
              TF_ERR_INVALID_ARG,
              "tf_flash_attention_fwd_f16: tile [%d,%d,%d,%d] does not divide problem [%lld,%lld,%lld,%lld]",
              tile_length_q, tile_length_kv, tile_hidden_qk, tile_hidden_v, (long long)Lq,
              (long long)Lkv, (long long)D, (long long)Dv);
  TFK_REQUIRE(softmax_scale == softmax_scale && softmax_scale - softmax_scale == 0.0,
              TF_ERR_INVALID_ARG, "tf_flash_attention_fwd_f16: softmax_scale must be finite");
  TFK_REQUIRE((D == 128 && Dv == 128) || (D == 64 && Dv == 64), TF_ERR_UNSUPPORTED,
              "tf_flash_attention_fwd_f16: head dims (D=%lld, Dv=%lld) must be 128/128 or 64/64",
              (long long)D, (long long)Dv);
  TFK_REQUIRE(!v_is_transposed || Lkv % 8 == 0, TF_ERR_UNSUPPORTED,
              "tf_flash_attention_fwd_f16: transposed V needs Lkv %% 8 == 0");
  const float scale_log2 = (float)(softmax_scale * 1.4426950408889634);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (D == 128)
    return pick<128, 128>(Q, K, V, O, (int)batch, (int)Lq, (int)Lkv, scale_log2,
                          v_is_transposed != 0, causal != 0, st);
  return pick<64, 64>(Q, K, V, O, (int)batch, (int)Lq, (int)Lkv, scale_log2,
                      v_is_transposed != 0, causal != 0, st);
}
