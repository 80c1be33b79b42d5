// Flash-attention forward for gfx950: O = softmax(scale * Q K^T (+ causal mask)) V per
// (batch x head) slice, fp16 in/out, fp32 scores and fp32 running max / sum.
//
// Counterpart of ke_flash_attention (include/kernels/flash_attention_device.cuh:130-312, mask
// include/cell/mask.hpp:75-82) and its host launcher (src/kernels/flash_attn.cu:58-152).
// CDNA4 design (FA-2 style, un-normalised O with one divide at the end):
//   * one workgroup = 256 queries (8 wavefronts x 32; 4 x 32 for short query ranges),
//     key/value tiles of 64 rows, v_mfma_f32_32x32x16_f16 throughout;
//   * Q stays in registers for the whole workgroup (the reference reloads it per KV tile);
//   * scores are computed transposed, S^T = K Q^T, so a lane owns ONE query row: its 32
//     score values per tile are plain registers, the row max / sum is an in-lane reduction
//     plus a single v_permlane32_swap with the partner lane, and exp2(S^T) converted to fp16
//     is already the B-operand fragment of the second MFMA O^T = V^T P^T;
//   * K and V tiles go global -> LDS directly (global_load_lds_dwordx4) into a 3-stage ring;
//     V is kept [key][dim] in LDS and transposed on the way to registers with
//     ds_read_b64_tr_b16; both tiles are XOR-swizzled against bank conflicts;
//   * causal: tiles right of the diagonal are skipped, only tiles crossing it are masked.
#include <type_traits>

#include "common.hpp"

namespace tfk {
namespace {

constexpr int kBN = 64;   // keys per tile
constexpr int kStages = 3;

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

// `addr` is a 32-bit LDS byte address: integer arithmetic on it (base register + constant)
// folds into the instruction's offset field, pointer arithmetic through a generic pointer
// does not.
TFK_DEVICE half4_t lds_read_tr4(unsigned addr) {
  fp16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
      (__attribute__((address_space(3))) fp16x4_t*)(size_t)addr);
  return __builtin_bit_cast(half4_t, v);
}
TFK_DEVICE half4_t lds_read_b64(unsigned addr) {
  return *(__attribute__((address_space(3))) const half4_t*)(size_t)addr;
}
TFK_DEVICE half8_t lds_read_b128(unsigned addr) {
  return *(__attribute__((address_space(3))) const half8_t*)(size_t)addr;
}
// Hides how `x` was computed from the optimiser.  Without it the loop-invariant part of
// (stage base + lane offset + constant) is hoisted as one register per read and the constant
// never reaches the offset field.
TFK_DEVICE unsigned opaque(unsigned x) {
  asm volatile("" : "+v"(x));
  return x;
}

// kWavesT wavefronts x 32 queries per workgroup.  8 wavefronts (256 queries) halve the
// K/V traffic per query and put two wavefronts on every SIMD, so one wavefront's softmax
// (VALU) overlaps the other's MFMAs; 4 wavefronts serve short query ranges.
template <int D, int DV, bool kVT, bool kCausal, int kWavesT>
__global__ __launch_bounds__(kWavesT * 64) void flash_attention_fwd_kernel(
    const half_t* __restrict__ Q, const half_t* __restrict__ K, const half_t* __restrict__ V,
    half_t* __restrict__ O, int Lq, int Lkv, float scale_log2, int q_tiles, int total_items) {
  constexpr int kBMq = kWavesT * 32;
  constexpr int kKChunks = D / 8;
  constexpr int kVChunks = kVT ? kBN / 8 : DV / 8;
  constexpr int kKBytes = kBN * D * 2;
  constexpr int kVBytes = kBN * DV * 2;
  constexpr int kStageBytes = kKBytes + kVBytes;
  constexpr int kNT = kBN / 32;
  constexpr int kDT = DV / 32;
  constexpr int kKInstr = kKBytes / 1024;            // 1 KiB wavefront loads per K tile
  constexpr int kVInstr = kVBytes / 1024;
  constexpr int kKPerWave = (kKInstr + kWavesT - 1) / kWavesT;
  constexpr int kVPerWave = (kVInstr + kWavesT - 1) / kWavesT;
  constexpr int kLoadsPerTile = kKPerWave + kVPerWave;  // per wavefront (idle slots re-load)
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 31, lg = lane >> 5;
  // Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2: id % 8 is the XCD,
  // id / 8 the position in that XCD's queue.  Work is arranged so that the query tiles of a
  // slice stream the same K/V through ONE L2 instead of eight.
  //   non-causal: items in slice-major order, cut into 8 contiguous chunks (the last one may
  //               be short; its surplus workgroups exit at once);
  //   causal:     work per query tile varies 1..q_tiles, so every queue is sorted
  //               heaviest (latest) tile first across the slices it owns; with a slice count
  //               that is not a multiple of 8 the queues would be unequal, so the order falls
  //               back to heaviest-first over all slices.
  int qt;
  size_t bh;
  if (!kCausal) {
    const int per_xcd = (total_items + 7) / 8;
    const int item = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (item >= total_items) return;
    qt = item % q_tiles;
    bh = item / q_tiles;
  } else {
    if ((int)blockIdx.x >= total_items) return;
    const int slices = total_items / q_tiles;
    if (slices % 8 == 0) {
      const int per = slices / 8, slot = blockIdx.x / 8;
      qt = q_tiles - 1 - slot / per;
      bh = (blockIdx.x % 8) * per + slot % per;
    } else {
      qt = q_tiles - 1 - (int)blockIdx.x / slices;
      bh = blockIdx.x % slices;
    }
  }
  Q += bh * (size_t)Lq * D;
  K += bh * (size_t)Lkv * D;
  V += bh * (size_t)Lkv * DV;
  O += bh * (size_t)Lq * DV;

  const int q_row0 = qt * kBMq + wave * 32;  // first query row of this wavefront
  const int m_row = q_row0 + lr;             // this lane's query row
  const int m_ld = min(m_row, Lq - 1);

  // A negative scale is folded into Q (scores change sign, the scale becomes positive), so
  // that the running maximum can be taken on raw scores and scaled once per row.
  const float c = fmaxf(fabsf(scale_log2), 1e-30f);  // (a zero scale still yields uniform weights)
  half8_t qf[D / 16];
#pragma unroll
  for (int kk = 0; kk < D / 16; ++kk) {
    qf[kk] = *reinterpret_cast<const half8_t*>(Q + (size_t)m_ld * D + kk * 16 + lg * 8);
    if (scale_log2 < 0.f) qf[kk] = -qf[kk];
  }

  int n_end = Lkv;
  if (kCausal) n_end = min(Lkv, qt * kBMq + kBMq);
  const int num_tiles = (n_end + kBN - 1) / kBN;

  // ---- global -> LDS plan: wavefront instruction i of a tile covers 1 KiB of it ------------
  const unsigned smem_base = lds_address(smem);
  auto issue_tile_loads = [&](int tile) __attribute__((always_inline)) {
    const int n0 = min(tile, num_tiles - 1) * kBN;  // clamped past the end (never read)
    const unsigned sk = smem_base + (tile % kStages) * kStageBytes;
    const unsigned sv = sk + kKBytes;
#pragma unroll
    for (int t = 0; t < kKPerWave; ++t) {  // K tile: [kBN][D]
      const int i = (wave + kWavesT * t) % kKInstr;
      constexpr int kRowsPerInstr = 64 / kKChunks;
      const int row = i * kRowsPerInstr + lane / kKChunks;
      const int cc = swz_k<kKChunks>(row, lane % kKChunks);
      const int gr = min(n0 + row, Lkv - 1);
      lds_dma_16B(K + (size_t)gr * D + cc * 8, sk + i * 1024);
    }
#pragma unroll
    for (int t = 0; t < kVPerWave; ++t) {
      const int i = (wave + kWavesT * t) % kVInstr;
      constexpr int kRowsPerInstr = 64 / kVChunks;
      const int row = i * kRowsPerInstr + lane / kVChunks;
      if constexpr (!kVT) {  // V tile: [kBN][DV]
        const int cc = swz_v<kVChunks>(row, lane % kVChunks);
        const int gr = min(n0 + row, Lkv - 1);
        lds_dma_16B(V + (size_t)gr * DV + cc * 8, sv + i * 1024);
      } else {  // V^T tile: [DV][kBN] out of a [DV][Lkv] matrix
        const int cc = swz_k<kVChunks>(row, lane % kVChunks);
        const int gc = min(n0 + cc * 8, Lkv - 8);
        lds_dma_16B(V + (size_t)row * Lkv + gc, sv + i * 1024);
      }
    }
  };

  // ---- LDS -> register plan -----------------------------------------------------------------
  // Every fragment read is (stage base) + (per-lane offset) + (compile-time immediate): the
  // swizzles only XOR lane-dependent bits into the chunk index, so the lane part is computed
  // once here and the tile loop spends no VALU on addresses beyond adding the stage base.
  //   K fragment (nt, kk): row 32*nt + lr, logical chunk 2*kk + lg.
  unsigned k_off[D / 16];
#pragma unroll
  for (int kk = 0; kk < D / 16; ++kk) k_off[kk] = lr * D * 2 + swz_k<kKChunks>(lr, 2 * kk + lg) * 16;
  //   V fragment (dt, keys nk..nk+15), V kept [key][dim]: a 16-lane group transposes the 4 x 16
  //   block of rows nk + 4*lg (+8) .. +3, columns 32*dt + 16*((lane>>4)&1) .. +15; lane r of the
  //   group addresses row r/4, columns 4*(r%4) .. +3 of that block.
  //   V^T fragment, V kept [dim][key]: row 32*dt + lr, keys nk + 4*lg (+8) .. +3.
  constexpr int kVOffs = kVT ? 8 : kDT;
  unsigned v_off[kVOffs];
  if constexpr (!kVT) {
    const int r16 = lane & 15;
    const int row_l = 4 * lg + (r16 >> 2);
    const int col_l = 16 * ((lane >> 4) & 1) + 4 * (r16 & 3);
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt) {
      const int col = dt * 32 + col_l;
      v_off[dt] = row_l * DV * 2 + swz_v<kVChunks>(row_l, col / 8) * 16 + (col % 8) * 2;
    }
  } else {
#pragma unroll
    for (int cc = 0; cc < 8; ++cc) v_off[cc] = lr * kBN * 2 + swz_k<kVChunks>(lr, cc) * 16 + lg * 8;
  }

  float16_t o_acc[kDT];
#pragma unroll
  for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.f;
  float m_run = -INFINITY;  // reference max of the raw (sign-adjusted) scores (see below)
  float l_run = 0.f;        // this lane's share of the running sum

  // Ring of kStages tiles: tile it+kStages-1 is requested at the top of iteration it.
#pragma unroll
  for (int t = 0; t < kStages - 1; ++t) issue_tile_loads(t);

  // Every iteration starts with the ring step: tile `it` has landed once only the younger
  // tiles' loads are outstanding; the barrier also tells us every wavefront is done with
  // tile it-1, whose stage is re-filled next.
  auto ring_step = [&](int it) __attribute__((always_inline)) {
    barrier_keep_vmem<(kStages - 2) * kLoadsPerTile>();
    issue_tile_loads(it + kStages - 1);
  };
  auto process_tile = [&](int it, auto mask_c) __attribute__((always_inline)) {
    constexpr bool kMask = decltype(mask_c)::value;
    const unsigned stage_base = smem_base + (it % kStages) * kStageBytes;
    const int n0 = it * kBN;
    // ---- S^T = K Q^T ------------------------------------------------------------------
    float16_t s[kNT];
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[nt][r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < D / 16; ++kk) {
      const unsigned kb = opaque(stage_base + k_off[kk]);
#pragma unroll
      for (int nt = 0; nt < kNT; ++nt) {
        const half8_t kf = lds_read_b128(kb + nt * 32 * D * 2);
        s[nt] = mfma_32x32x16(kf, qf[kk], s[nt]);
      }
    }

    // ---- mask -------------------------------------------------------------------------
    // s[nt][r] is the score of key n0 + 32*nt + 8*(r/4) + 4*lg + r%4 against query m_row
    if constexpr (kMask) {
#pragma unroll
      for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int n = n0 + nt * 32 + 8 * (r / 4) + 4 * lg + (r % 4);
          if (n >= Lkv || (kCausal && n > m_row)) s[nt][r] = -INFINITY;
        }
    }

    // ---- online softmax: p = exp2(c*s - c*m) -------------------------------------------
    float mx = s[0][0];
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[nt][r]);
    mx = pair_max(mx);
    // Lazy rescale: exponents are taken against a reference m_run that is only raised when a
    // row's maximum has grown by more than kLazy (in log2 units) since the reference was set.
    // Until then p = 2^(c*(s - m_run)) may reach 2^kLazy, which fp16 P and the fp32 sums hold
    // easily, and the final O / l is unchanged because O and l share the reference.  Raising
    // it costs a multiply of every O accumulator, so this skips it on almost every tile.
    constexpr float kLazy = 8.f;
    if (__builtin_amdgcn_ballot_w64((mx - m_run) * c > kLazy) != 0) {
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c);
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[dt][r] *= alpha;
      m_run = m_new;
    }
    const float mc = m_run * c;
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[nt][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[nt][r], c, -mc));

    // ---- O^T += V^T P^T ---------------------------------------------------------------
    // The row sum is taken over the fp16-rounded weights, the values that actually multiply
    // V (v_dot2_f32_f16 against (1, 1): two weights per instruction, fp32 accumulate).
    unsigned vb[kVOffs];
#pragma unroll
    for (int x = 0; x < kVOffs; ++x) vb[x] = opaque(stage_base + v_off[x]) + kKBytes;
    const half2_t ones = {(half_t)1.f, (half_t)1.f};
    float psum = 0.f;
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        // reduction step over keys nk .. nk+15; slot t of lane group lg is key
        // nk + 4*lg + t (t < 4) or nk + 8 + 4*lg + (t - 4)
        half8_t pb;
#pragma unroll
        for (int t = 0; t < 8; ++t) pb[t] = (half_t)s[nt][8 * j + t];
        psum = __builtin_amdgcn_fdot2(__builtin_shufflevector(pb, pb, 0, 1), ones, psum, false);
        psum = __builtin_amdgcn_fdot2(__builtin_shufflevector(pb, pb, 2, 3), ones, psum, false);
        psum = __builtin_amdgcn_fdot2(__builtin_shufflevector(pb, pb, 4, 5), ones, psum, false);
        psum = __builtin_amdgcn_fdot2(__builtin_shufflevector(pb, pb, 6, 7), ones, psum, false);
        const int nk = nt * 32 + 16 * j;
#pragma unroll
        for (int dt = 0; dt < kDT; ++dt) {
          half4_t lo, hi;
          if constexpr (!kVT) {
            lo = lds_read_tr4(vb[dt] + nk * DV * 2);
            hi = lds_read_tr4(vb[dt] + (nk + 8) * DV * 2);
          } else {
            lo = lds_read_b64(vb[nk / 8] + dt * 32 * kBN * 2);
            hi = lds_read_b64(vb[nk / 8 + 1] + dt * 32 * kBN * 2);
          }
          half8_t vf;
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            vf[t] = lo[t];
            vf[4 + t] = hi[t];
          }
          o_acc[dt] = mfma_32x32x16(vf, pb, o_acc[dt]);
        }
      }
    l_run += psum;
  };

  // Tiles [0, n_plain) need no mask for this wavefront's 32 rows, [n_plain, n_compute) cross
  // the diagonal or the end of the keys, and [n_compute, num_tiles) lie above the diagonal:
  // the wavefront only keeps the ring (barrier + loads) going for its workgroup.
  int n_plain = min(num_tiles, Lkv / kBN);
  int n_compute = num_tiles;
  if (kCausal) {
    n_plain = max(0, min(n_plain, (q_row0 + 1) / kBN));
    n_compute = min(num_tiles, (q_row0 + 31) / kBN + 1);
  }
  int it = 0;
  for (; it < n_plain; ++it) {
    ring_step(it);
    process_tile(it, std::false_type{});
  }
  for (; it < n_compute; ++it) {
    ring_step(it);
    process_tile(it, std::true_type{});
  }
  for (; it < num_tiles; ++it) ring_step(it);
  wait_vmem_all();  // the clamped tail loads must not outlive the workgroup's LDS

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

template <int D, int DV, bool kVT, bool kCausal, int kWavesT>
int launch_w(const void* Q, const void* K, const void* V, void* O, int batch, int Lq, int Lkv,
             float scale_log2, hipStream_t st) {
  auto kern = flash_attention_fwd_kernel<D, DV, kVT, kCausal, kWavesT>;
  constexpr int lds = kStages * (kBN * D * 2 + kBN * DV * 2);
  static_assert(lds <= kMaxLdsBytes, "tiles do not fit in LDS");
  TFK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  constexpr int bm = kWavesT * 32;
  const int q_tiles = (Lq + bm - 1) / bm;
  const int total_items = q_tiles * batch;
  const dim3 grid(8 * ((total_items + 7) / 8));
  hipLaunchKernelGGL(kern, grid, dim3(kWavesT * 64), lds, st,
                     static_cast<const half_t*>(Q), static_cast<const half_t*>(K),
                     static_cast<const half_t*>(V), static_cast<half_t*>(O), Lq, Lkv, scale_log2,
                     q_tiles, total_items);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}

template <int D, int DV, bool kVT, bool kCausal>
int launch(const void* Q, const void* K, const void* V, void* O, int batch, int Lq, int Lkv,
           float scale_log2, hipStream_t st) {
  if (Lq > 128) return launch_w<D, DV, kVT, kCausal, 8>(Q, K, V, O, batch, Lq, Lkv, scale_log2, st);
  return launch_w<D, DV, kVT, kCausal, 4>(Q, K, V, O, batch, Lq, Lkv, scale_log2, st);
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
  TFK_REQUIRE(batch < 65536 && Lq < (1 << 21) && Lkv < (1 << 24), TF_ERR_INVALID_ARG,
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
