// Flash-attention forward for gfx950: O = softmax(scale * Q K^T (+ causal mask)) V per
// (batch x head) slice, fp16 or bf16 in/out, fp32 scores and fp32 running max / sum.
//
// Counterpart of ke_flash_attention (include/kernels/flash_attention_device.cuh:130-312, mask
// include/cell/mask.hpp:75-82) and its host launcher (src/kernels/flash_attn.cu:58-152).
// CDNA4 design (FA-2 style, un-normalised O with one divide at the end):
//   * one workgroup = 256 queries (8 wavefronts x 32; 4 x 32 for short query ranges),
//     key/value tiles of 64 rows, v_mfma_f32_16x16x32_f16 throughout (the most
//     power-efficient fp16 MFMA shape: the kernel runs at the power limit, so energy per
//     flop sets its speed);
//   * Q stays in registers for the whole workgroup (the reference reloads it per KV tile);
//   * scores are computed transposed, S^T = K Q^T, so a lane owns one query row per 16-query
//     block: its score values are plain registers, the running max is an in-lane
//     reduction (the 4 lanes that share a query only talk when the reference max moves),
//     and exp2(S^T) converted to fp16 is already the B-operand fragment of the second MFMA
//     O^T = V^T P^T;
//   * K and V tiles go global -> LDS directly (global_load_lds_dwordx4) into a ring of 5 tiles
//     (4 for the 4-wavefront workgroup);
//     V is kept [key][dim] in LDS and transposed on the way to registers with
//     ds_read_b64_tr_b16; both tiles are XOR-swizzled against bank conflicts;
//   * causal: tiles right of the diagonal are skipped, only tiles crossing it are masked.
#include <type_traits>

#include "common.hpp"
#include "jit_ops.hpp"

namespace tfk {
namespace {

constexpr int kBN = 64;   // keys per tile
// LDS ring depth: the 8-wavefront kernel keeps two tiles live (its two wavefront sets are half a
// tile apart) and three in flight; the 4-wavefront kernel one live and three in flight.
__host__ __device__ constexpr int ring_stages(int waves) { return waves == 8 ? 5 : 4; }
// Row pitch (in elements) of a [key][dim] tile in LDS: the next power of two.  The swizzles XOR
// chunk indices, which needs a power-of-two chunk count, and a 1 KiB request must cover whole
// rows.  A head dimension of 96 is kept in 128-element rows whose last quarter is never read.
__host__ __device__ constexpr int lds_pitch(int d) { return d <= 64 ? 64 : 128; }

// K tile [kBN][D] (and a transposed V tile [DV][kBN]): 16 consecutive rows reading one logical
// 16-byte chunk hit 16 different bank groups.
template <int CH>
__host__ __device__ constexpr int swz_k(int row, int c) {
  constexpr int kRowsPer256B = CH >= 16 ? 1 : 16 / CH;
  return c ^ ((row / kRowsPer256B) % CH);
}
// V tile [kBN][DV] read by transposing 4-row x 16-column blocks: a half wavefront touches 8
// rows x 32 bytes at the same column, which must land in 8 different 32-byte bank windows.
template <int CH>
__host__ __device__ constexpr int swz_v(int row, int c) {
  if constexpr (CH >= 16) return c ^ ((row & 7) << 1);
  return c ^ (((row >> 1) & 3) << 1);
}

typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));

// The kernel moves 16-bit elements without looking at them; the element type T (half_t or bf16_t)
// only selects the MFMA and the float -> T conversion.
template <typename T>
struct Vec {
  using v2 = T __attribute__((ext_vector_type(2)));
  using v4 = T __attribute__((ext_vector_type(4)));
  using v8 = T __attribute__((ext_vector_type(8)));
};
template <typename T>
TFK_DEVICE float4_t mfma_t(typename Vec<T>::v8 a, typename Vec<T>::v8 b, float4_t c) {
  if constexpr (std::is_same_v<T, bf16_t>) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  else return mfma_16x16x32(a, b, c);
}
// fp16 saturates at its largest finite value (an absurd |Q * scale| must not become inf); bf16
// has the range of fp32.
template <typename T>
TFK_DEVICE T to_elem_saturating(float x) {
  if constexpr (std::is_same_v<T, bf16_t>) return (T)x;
  else return (T)__builtin_amdgcn_fmed3f(x, -65504.f, 65504.f);
}

// `addr` is a 32-bit LDS byte address: integer arithmetic on it (base register + constant)
// folds into the instruction's offset field, pointer arithmetic through a generic pointer
// does not.
template <typename V4>
TFK_DEVICE V4 lds_read_tr4(unsigned addr) {
  fp16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
      (__attribute__((address_space(3))) fp16x4_t*)(size_t)addr);
  return __builtin_bit_cast(V4, v);
}
template <typename V4>
TFK_DEVICE V4 lds_read_b64(unsigned addr) {
  return *(__attribute__((address_space(3))) const V4*)(size_t)addr;
}
template <typename V8>
TFK_DEVICE V8 lds_read_b128(unsigned addr) {
  return *(__attribute__((address_space(3))) const V8*)(size_t)addr;
}
// Hides how `x` was computed from the optimiser.  Without it the loop-invariant part of
// (stage base + lane offset + constant) is hoisted as one register per read and the constant
// never reaches the offset field.
TFK_DEVICE unsigned opaque(unsigned x) {
  asm volatile("" : "+v"(x));
  return x;
}
// Reduction over the 4 lanes l, l^16, l^32, l^48 that share a query (rare path).
TFK_DEVICE float quad_max(float x) {
  x = fmaxf(x, __shfl_xor(x, 16));
  return fmaxf(x, __shfl_xor(x, 32));
}

// kWavesT wavefronts x 32 queries per workgroup.  8 wavefronts (256 queries) halve the
// K/V traffic per query and put two wavefronts on every SIMD, so one wavefront's softmax
// (VALU) overlaps the other's MFMAs; 4 wavefronts serve short query ranges.
template <typename T, int D, int DV, bool kVT, bool kCausal, int kWavesT, int kQB>
__global__ __launch_bounds__(kWavesT * 64) void flash_attention_fwd_kernel(
    const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
    T* __restrict__ O, int Lq, int Lkv, float scale_log2, int q_tiles, int total_items) {
  using V2 = typename Vec<T>::v2;
  using V4 = typename Vec<T>::v4;
  using V8 = typename Vec<T>::v8;
  constexpr int kStages = ring_stages(kWavesT);
  constexpr int kRowsPerWave = 16 * kQB;  // kQB 16-query blocks per wavefront
  constexpr int kBMq = kWavesT * kRowsPerWave;
  constexpr int DP = lds_pitch(D), DVP = lds_pitch(DV);   // LDS row pitch of the K / natural V tile
  constexpr int kKChunks = DP / 8;
  constexpr int kVChunks = kVT ? kBN / 8 : DVP / 8;
  constexpr int kKBytes = kBN * DP * 2;
  constexpr int kVBytes = kVT ? DV * kBN * 2 : kBN * DVP * 2;
  constexpr int kStageBytes = kKBytes + kVBytes;
  constexpr int kKB = kBN / 16;   // 16-key blocks per tile (rows of S^T)
  constexpr int kKK = D / 32;     // reduction steps of S^T = K Q^T
  constexpr int kDB = DV / 16;    // 16-wide blocks of the head dimension (rows of O^T)
  constexpr int kJ = kBN / 32;    // reduction steps of O^T += V^T P^T
  constexpr int kKInstr = kKBytes / 1024;            // 1 KiB wavefront loads per K tile
  constexpr int kVInstr = kVBytes / 1024;
  constexpr int kKPerWave = (kKInstr + kWavesT - 1) / kWavesT;
  constexpr int kVPerWave = (kVInstr + kWavesT - 1) / kWavesT;
  constexpr int kLoadsPerTile = kKPerWave + kVPerWave;  // per wavefront (idle slots re-load)
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, lg = lane >> 4;
  // Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2: id % 8 is the XCD,
  // id / 8 the position in that XCD's queue.  Work is arranged so that the query tiles of a
  // slice stream the same K/V through ONE L2 instead of eight.
  //   non-causal: items in slice-major order, cut into 8 contiguous chunks (the last one may
  //               be short; its surplus workgroups exit at once);
  //   causal:     work per query tile grows with its position, so a workgroup takes query
  //               tile q_tiles-1-p and then tile p of the same slice: every workgroup does the
  //               same amount of work, no sorting by weight is needed and the slice-major
  //               order (with its L2 locality) is kept.  An odd number of query tiles falls
  //               back to one tile per workgroup, heaviest tiles first over all slices.
  int qt_of_pass[2] = {0, 0};
  int num_passes = 1;
  size_t bh;
  if (!kCausal || q_tiles % 2 == 0) {
    const int per_slice = kCausal ? q_tiles / 2 : q_tiles;
    const int per_xcd = (total_items + 7) / 8;
    const int item = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (item >= total_items) return;
    const int p = item % per_slice;
    bh = item / per_slice;
    if (kCausal) {
      qt_of_pass[0] = q_tiles - 1 - p;
      qt_of_pass[1] = p;
      num_passes = 2;
    } else {
      qt_of_pass[0] = p;
    }
  } else {
    if ((int)blockIdx.x >= total_items) return;
    const int slices = total_items / q_tiles;
    qt_of_pass[0] = q_tiles - 1 - (int)blockIdx.x / slices;
    bh = blockIdx.x % slices;
  }
  Q += bh * (size_t)Lq * D;
  K += bh * (size_t)Lkv * D;
  V += bh * (size_t)Lkv * DV;
  O += bh * (size_t)Lq * DV;

  for (int pass = 0; pass < num_passes; ++pass) {
  const int qt = qt_of_pass[pass];
  const int q_row0 = qt * kBMq + wave * kRowsPerWave;  // first query row of this wavefront
  // this lane's query rows: block qb holds row q_row0 + 16*qb + lr

  // The softmax scale (times log2 e) is folded into Q once: Q' = fp16(Q * scale_log2), so the
  // MFMA result is already in log2 units; and each score accumulator starts at minus the
  // row's reference maximum instead of zero, so the MFMA result IS the exp2 argument - no
  // per-score multiply or subtract is left in the tile loop.
  // Q^T fragments (B operand): lane holds Q'[row][32*kk + 8*lg .. +7]
  V8 qf[kKK][kQB];
#pragma unroll
  for (int qb = 0; qb < kQB; ++qb) {
    const int m_ld = min(q_row0 + 16 * qb + lr, Lq - 1);
#pragma unroll
    for (int kk = 0; kk < kKK; ++kk) {
      const V8 raw = *reinterpret_cast<const V8*>(Q + (size_t)m_ld * D + kk * 32 + lg * 8);
#pragma unroll
      for (int t = 0; t < 8; ++t) qf[kk][qb][t] = to_elem_saturating<T>((float)raw[t] * scale_log2);
    }
  }

  int n_end = Lkv;
  if (kCausal) n_end = min(Lkv, qt * kBMq + kBMq);
  const int num_tiles = (n_end + kBN - 1) / kBN;

  // ---- global -> LDS plan: wavefront instruction i of a tile covers 1 KiB of it ------------
  // Request r of a wavefront (r < kKPerWave: K tile, else V tile) is one instruction: scalar
  // base (start of the tile in global memory) + a per-lane 32-bit offset computed once here.
  // Only a tile that crosses the end of the keys takes the slow form with clamped addresses.
  const unsigned smem_base = lds_address(smem);
  unsigned req_off[kLoadsPerTile];   // per-lane byte offset inside the tile (global side)
  unsigned req_lds[kLoadsPerTile];   // wave-uniform byte offset inside the stage (LDS side)
#pragma unroll
  for (int t = 0; t < kKPerWave; ++t) {  // K tile: [kBN][D]
    const int i = (wave + kWavesT * t) % kKInstr;
    constexpr int kRowsPerInstr = 64 / kKChunks;
    const int row = i * kRowsPerInstr + lane / kKChunks;
    // (a physical chunk whose logical chunk lies beyond D is never read: it re-fetches the last one)
    req_off[t] = (unsigned)(row * D + min(swz_k<kKChunks>(row, lane % kKChunks), D / 8 - 1) * 8) * 2u;
    req_lds[t] = i * 1024;
  }
#pragma unroll
  for (int t = 0; t < kVPerWave; ++t) {
    const int i = (wave + kWavesT * t) % kVInstr;
    constexpr int kRowsPerInstr = 64 / kVChunks;
    const int row = i * kRowsPerInstr + lane / kVChunks;
    if constexpr (!kVT)  // V tile: [kBN][DV]
      req_off[kKPerWave + t] = (unsigned)(row * DV + min(swz_v<kVChunks>(row, lane % kVChunks), DV / 8 - 1) * 8) * 2u;
    else                 // V^T tile: [DV][kBN] out of a [DV][Lkv] matrix
      req_off[kKPerWave + t] = ((unsigned)row * (unsigned)Lkv + swz_k<kVChunks>(row, lane % kVChunks) * 8) * 2u;
    req_lds[kKPerWave + t] = kKBytes + i * 1024;
  }
  auto issue_request = [&](int tile, int r) __attribute__((always_inline)) {
    const int n0 = min(tile, num_tiles - 1) * kBN;  // clamped past the end (never read)
    const unsigned dst = smem_base + (tile % kStages) * kStageBytes + req_lds[r];
    if (n0 + kBN <= Lkv) {
      const char* base = r < kKPerWave ? reinterpret_cast<const char*>(K + (size_t)n0 * D)
                         : kVT         ? reinterpret_cast<const char*>(V + n0)
                                       : reinterpret_cast<const char*>(V + (size_t)n0 * DV);
      // the LDS destination is an M0 INPUT of the statement: the compiler writes M0 itself and
      // cannot use the register for anything else between that write and the request; the
      // s_nop is the wait state an M0 write needs in front of an LDS-direct load
      asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :
                   : "v"(req_off[r]), "s"(base), "{m0}"(dst)
                   : "memory");
      return;
    }
    if (r < kKPerWave) {
      const int i = (wave + kWavesT * r) % kKInstr;
      constexpr int kRowsPerInstr = 64 / kKChunks;
      const int row = i * kRowsPerInstr + lane / kKChunks;
      const int cc = min(swz_k<kKChunks>(row, lane % kKChunks), D / 8 - 1);
      const int gr = min(n0 + row, Lkv - 1);
      lds_dma_16B(K + (size_t)gr * D + cc * 8, dst);
    } else {
      const int i = (wave + kWavesT * (r - kKPerWave)) % kVInstr;
      constexpr int kRowsPerInstr = 64 / kVChunks;
      const int row = i * kRowsPerInstr + lane / kVChunks;
      if constexpr (!kVT) {
        const int cc = min(swz_v<kVChunks>(row, lane % kVChunks), DV / 8 - 1);
        const int gr = min(n0 + row, Lkv - 1);
        lds_dma_16B(V + (size_t)gr * DV + cc * 8, dst);
      } else {
        const int cc = swz_k<kVChunks>(row, lane % kVChunks);
        const int gc = min(n0 + cc * 8, Lkv - 8);
        lds_dma_16B(V + (size_t)row * Lkv + gc, dst);
      }
    }
  };
  // The same request for a tile known to lie wholly inside the key range: no clamping, no
  // branch.  The tile loop uses this form wherever it can, because the bookkeeping of the
  // general form (~30 scalar instructions and two branches per request) is issued between
  // MFMAs of a wavefront that has the matrix pipe to itself at that moment: it cost ~100
  // cycles per request with the pipe idle.
  auto issue_request_lean = [&](int tile, int r) __attribute__((always_inline)) {
    const unsigned dst = smem_base + (tile % kStages) * kStageBytes + req_lds[r];
    const char* base = r < kKPerWave ? reinterpret_cast<const char*>(K) + (size_t)tile * (kBN * D * 2)
                       : kVT         ? reinterpret_cast<const char*>(V) + (size_t)tile * (kBN * 2)
                                     : reinterpret_cast<const char*>(V) + (size_t)tile * (kBN * DV * 2);
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(req_off[r]), "s"(base), "{m0}"(dst)
                 : "memory");
  };
  auto issue_tile_loads = [&](int tile) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < kLoadsPerTile; ++r) issue_request(tile, r);
  };

  // ---- LDS -> register plan -----------------------------------------------------------------
  // Every fragment read is (stage base) + (per-lane offset) + (compile-time immediate): the
  // swizzles only XOR lane-dependent bits into the chunk index, so the lane part is computed
  // once here and the tile loop spends no VALU on addresses beyond adding the stage base.
  //   K fragment (kb, kk) - A operand, 16 keys x 32 dims: row 16*kb + lr, logical chunk 4*kk + lg.
  unsigned k_off[kKK];
#pragma unroll
  for (int kk = 0; kk < kKK; ++kk) k_off[kk] = lr * DP * 2 + swz_k<kKChunks>(lr, 4 * kk + lg) * 16;
  //   Reduction step j of the second product covers keys 32*j .. +31; slot t of lane group lg
  //   is key 32*j + 4*lg + t (t < 4) or 32*j + 16 + 4*lg + (t - 4): exactly the keys whose
  //   scores the lane already holds in its accumulators of key blocks 2*j and 2*j + 1.
  //   V fragment (db, j) - A operand, 16 dims x 32 keys.
  //     V kept [key][dim]: each 16-lane group transposes the 4 x 16 block of rows
  //     32*j + 4*lg (+16) .. +3, columns 16*db .. +15; lane r of the group addresses row r/4,
  //     columns 4*(r%4) .. +3 of that block.  One offset per (db & 1, db / 2 via XOR) would not
  //     be constant, so the lane part is kept per db.
  //     V kept [dim][key]: row 16*db + lr, keys 32*j + 4*lg (+16) .. +3 (8 bytes each).
  constexpr int kVOffs = kVT ? 2 * kJ : kDB;
  unsigned v_off[kVOffs];
  if constexpr (!kVT) {
    const int row_l = 4 * lg + (lr >> 2);
#pragma unroll
    for (int db = 0; db < kDB; ++db) {
      const int col = db * 16 + 4 * (lr & 3);
      v_off[db] = row_l * DVP * 2 + swz_v<kVChunks>(row_l, col / 8) * 16 + (col % 8) * 2;
    }
  } else {
#pragma unroll
    for (int x = 0; x < 2 * kJ; ++x) {  // x = 2*j + half: keys 32*j + 16*half + 4*lg .. +3
      const int key = 16 * x + 4 * lg;
      v_off[x] = lr * kBN * 2 + swz_k<kVChunks>(lr, key / 8) * 16 + (key % 8) * 2;
    }
  }

  float4_t o_acc[kDB][kQB];
#pragma unroll
  for (int db = 0; db < kDB; ++db)
#pragma unroll
    for (int qb = 0; qb < kQB; ++qb) o_acc[db][qb] = float4_t{0.f, 0.f, 0.f, 0.f};
  // neg_m: minus the reference maximum of a row's scaled scores (the accumulator start value);
  // l_acc: the running sum of a row's weights, kept as one more accumulator block of the second
  // product (a block of V^T whose 16 rows are all ones): the matrix pipe adds up the 16-bit
  // weights that actually multiply V.  Every register of l_acc[qb] holds the sum of row lr.
  // (A v_dot2 per pair of weights, the obvious VALU form, takes ~20 cycles per instruction while
  // another wavefront of the SIMD streams MFMAs - against 8 for an ordinary VALU instruction.)
  float neg_m[kQB];
  float4_t l_acc[kQB];
#pragma unroll
  for (int qb = 0; qb < kQB; ++qb) {
    neg_m[qb] = 0.f;  // reference 0 until the first tile raises it
    l_acc[qb] = float4_t{0.f, 0.f, 0.f, 0.f};
  }
  V8 ones_frag;
#pragma unroll
  for (int t = 0; t < 8; ++t) ones_frag[t] = (T)1.f;

  float4_t s[kKB][kQB];  // scores of the tile in flight
  // Operand fragments are requested from LDS one step ahead of the MFMAs that use them, into
  // ping-pong registers, so that LDS latency is covered by the previous step's MFMAs (or by
  // the softmax arithmetic) instead of stalling the wavefront in front of every MFMA group.
  V8 kf[2][kKB];   // K fragments of reduction step kk (buffer kk & 1)
  V8 vf[2][kDB];   // V fragments of reduction step j (buffer j & 1)
  auto k_reads = [&](int buf, int it, int kk) __attribute__((always_inline)) {
    const unsigned ka = opaque(smem_base + (it % kStages) * kStageBytes + k_off[kk]);
#pragma unroll
    for (int kb = 0; kb < kKB; ++kb) kf[buf][kb] = lds_read_b128<V8>(ka + kb * 16 * DP * 2);
  };
  auto v_reads = [&](int buf, int it, int j) __attribute__((always_inline)) {
    const unsigned stage_base = smem_base + (it % kStages) * kStageBytes;
#pragma unroll
    for (int db = 0; db < kDB; ++db) {
      V4 lo, hi;
      if constexpr (!kVT) {
        const unsigned va = opaque(stage_base + v_off[db]) + kKBytes;
        lo = lds_read_tr4<V4>(va + (32 * j) * DVP * 2);
        hi = lds_read_tr4<V4>(va + (32 * j + 16) * DVP * 2);
      } else {
        lo = lds_read_b64<V4>(opaque(stage_base + v_off[2 * j]) + kKBytes + db * 16 * kBN * 2);
        hi = lds_read_b64<V4>(opaque(stage_base + v_off[2 * j + 1]) + kKBytes + db * 16 * kBN * 2);
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        vf[buf][db][t] = lo[t];
        vf[buf][db][4 + t] = hi[t];
      }
    }
  };
  // ---- S^T = K Q'^T - m: s[kb][qb][r] = log2-scaled score of key 64*it + 16*kb + 4*lg + r
  //      against row lr of query block qb, minus that row's reference maximum.  Expects the
  //      fragments of step kk = 0 to be on their way into kf[0]. ---------------------------
  //      req_tile >= 0: that tile's requests are issued between the reduction steps.
  //      lean_c: the requested tile is a whole tile inside the key range (lean request form).
  //      The fragment reads of the next reduction step and the requests sit BETWEEN the MFMAs
  //      (one piece behind each pair): a wavefront issues in order, so anything clustered
  //      between two reduction steps runs with the matrix pipe drained.
  auto qk_tile = [&](int it, int req_tile, auto lean_c) __attribute__((always_inline)) {
    constexpr bool kLean = decltype(lean_c)::value;
#pragma unroll
    for (int kb = 0; kb < kKB; ++kb)
#pragma unroll
      for (int qb = 0; qb < kQB; ++qb) s[kb][qb] = float4_t{neg_m[qb], neg_m[qb], neg_m[qb], neg_m[qb]};
#pragma unroll
    for (int kk = 0; kk < kKK; ++kk) {
      const unsigned ka = kk + 1 < kKK ? opaque(smem_base + (it % kStages) * kStageBytes + k_off[kk + 1]) : 0u;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kb = 0; kb < kKB; ++kb) {
#pragma unroll
        for (int qb = 0; qb < kQB; ++qb) s[kb][qb] = mfma_t<T>(kf[kk & 1][kb], qf[kk][qb], s[kb][qb]);
        if (kk + 1 < kKK) kf[(kk + 1) & 1][kb] = lds_read_b128<V8>(ka + kb * 16 * DP * 2);
        if (req_tile >= 0) {
#pragma unroll
          for (int r = 0; r < kLoadsPerTile; ++r)
            if ((r * kKK * kKB) / kLoadsPerTile == kk * kKB + kb) {
              if constexpr (kLean) issue_request_lean(req_tile, r);
              else issue_request(req_tile, r);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  V8 pb[kJ][kQB];  // 16-bit weights, B operand of the second product
  // ---- mask, online softmax, fp16 weights.  Requests the V fragments of step j = 0. -------
  auto softmax_tile = [&](int it, auto mask_c) __attribute__((always_inline)) {
    constexpr bool kMask = decltype(mask_c)::value;
    const int n0 = it * kBN;
    v_reads(0, it, 0);
    __builtin_amdgcn_sched_barrier(0);
    // ---- mask -------------------------------------------------------------------------
    if constexpr (kMask) {
#pragma unroll
      for (int kb = 0; kb < kKB; ++kb)
#pragma unroll
        for (int qb = 0; qb < kQB; ++qb)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int n = n0 + kb * 16 + 4 * lg + r;
            if (n >= Lkv || (kCausal && n > q_row0 + 16 * qb + lr)) s[kb][qb][r] = -INFINITY;
          }
    }

    // ---- online softmax: p = exp2(s) ---------------------------------------------------
    // Lazy reference: the reference maximum is only raised when some lane sees a score more
    // than kLazy (log2 units) above it.  Until then p may reach 2^kLazy, which fp16 P and the
    // fp32 sums hold easily, and the final O / l is unchanged because O and l share the
    // reference.  The check needs no cross-lane traffic: it looks at each lane's own 16 keys;
    // only when it fires are the 4 lanes that share a query reduced, every O accumulator
    // multiplied and this tile's scores re-based.
    constexpr float kLazy = 8.f;
    float mx[kQB];
    bool grow = false;
#pragma unroll
    for (int qb = 0; qb < kQB; ++qb) {
      mx[qb] = s[0][qb][0];
#pragma unroll
      for (int kb = 0; kb < kKB; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r) mx[qb] = fmaxf(mx[qb], s[kb][qb][r]);
      grow |= mx[qb] > kLazy;
    }
    // The first tile sets the reference to the row's true maximum, whichever way that is from
    // the initial 0 (every row has at least key 0 unmasked there; nothing is accumulated yet).
    const bool first = it == 0;
    if (first || __builtin_amdgcn_ballot_w64(grow) != 0) {
#pragma unroll
      for (int qb = 0; qb < kQB; ++qb) {
        const float qmax = quad_max(mx[qb]);
        const float shift = first ? qmax : fmaxf(0.f, qmax);  // afterwards the reference only rises
        const float alpha = first ? 1.f : __builtin_amdgcn_exp2f(-shift);
        l_acc[qb] *= alpha;
#pragma unroll
        for (int db = 0; db < kDB; ++db) o_acc[db][qb] *= alpha;
#pragma unroll
        for (int kb = 0; kb < kKB; ++kb) s[kb][qb] -= shift;
        neg_m[qb] -= shift;
      }
    }
#pragma unroll
    for (int qb = 0; qb < kQB; ++qb)
#pragma unroll
      for (int kb = 0; kb < kKB; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r) s[kb][qb][r] = __builtin_amdgcn_exp2f(s[kb][qb][r]);

#pragma unroll
    for (int j = 0; j < kJ; ++j)
#pragma unroll
      for (int qb = 0; qb < kQB; ++qb) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          pb[j][qb][t] = (T)s[2 * j][qb][t];
          pb[j][qb][4 + t] = (T)s[2 * j + 1][qb][t];
        }
      }
    __builtin_amdgcn_sched_barrier(0);
  };
  // ---- O^T += V^T P^T; during its last step the K fragments (kk = 0) of tile `it_next`
  //      are requested for the QK phase that follows ------------------------------------------
  auto pv_tile = [&](int it, int it_next) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < kJ; ++j) {
      if (j + 1 < kJ) v_reads((j + 1) & 1, it, j + 1);
      else k_reads(0, it_next, 0);
#pragma unroll
      for (int db = 0; db < kDB; ++db)
#pragma unroll
        for (int qb = 0; qb < kQB; ++qb) o_acc[db][qb] = mfma_t<T>(vf[j & 1][db], pb[j][qb], o_acc[db][qb]);
#pragma unroll
      for (int qb = 0; qb < kQB; ++qb) l_acc[qb] = mfma_t<T>(ones_frag, pb[j][qb], l_acc[qb]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Tiles [0, n_plain) need no mask for this wavefront's rows, [n_plain, n_compute) cross
  // the diagonal or the end of the keys, and [n_compute, num_tiles) lie above the diagonal:
  // the wavefront only keeps the ring (barrier + loads) going for its workgroup.
  int n_plain = min(num_tiles, Lkv / kBN);
  int n_compute = num_tiles;
  if (kCausal) {
    n_plain = max(0, min(n_plain, (q_row0 + 1) / kBN));
    n_compute = min(num_tiles, (q_row0 + kRowsPerWave - 1) / kBN + 1);
  }
  const int n_fast = min(num_tiles, Lkv / kBN);  // whole tiles of this pass (lean request form)
  if constexpr (kWavesT == 8) {
    // Two wavefronts share a SIMD (w and w + 4) and a SIMD has one matrix pipe and one VALU, so
    // the two SETS of wavefronts (0-3, 4-7) run the same loop half a tile apart, in time slots
    // fenced by two workgroup barriers per tile:
    //     slot 2t   : set 0: PV(t-1), QK(t)  [MFMA]      set 1: softmax(t-1)     [VALU]
    //     slot 2t+1 : set 0: softmax(t)      [VALU]      set 1: PV(t-1), QK(t)   [MFMA]
    // While one wavefront of a SIMD streams its 64 MFMAs the other one does its exp2 / convert
    // work, and neither pipe waits for the other: measured per tile, a wavefront's MFMA block
    // takes ~1100-1200 cycles and its softmax ~1000 while the partner's MFMAs run (VALU
    // instructions issue at half rate then), against ~3500 for an arrangement that lets the
    // phases of the two wavefronts drift (QK, softmax and PV of both then run one after another).
    // Without the second barrier the sets do drift: the hardware issues from the older wavefront
    // first and whichever set gets ahead keeps the matrix pipe.
    // Ring of 5 tiles: tile t is read from slot 2t (QK by set 0) to slot 2t+3 (PV by set 1), so
    // two tiles are live and three are in flight.  QK(t) carries the requests of tile t+3, which
    // go into the stage of tile t-2 (last read in slot 2t-1).  The barrier behind an MFMA block
    // (after QK(t+1) has requested tile t+4) waits until only tiles t+3, t+4 are in flight: tile
    // t+2 has then landed, one slot before the first wavefront reads it.
#pragma unroll
    for (int t = 0; t < 3; ++t) issue_tile_loads(t);
    barrier_keep_vmem<2 * kLoadsPerTile>();  // tile 0 has landed
    const bool second_set = wave >= 4;
    if (second_set) barrier_only();  // slot 0: set 0 alone
    k_reads(0, 0, 0);
    if (n_compute > 0) qk_tile(0, 3, std::false_type{});
    else issue_tile_loads(3);
    auto tile_step = [&](int t, auto mask_c, auto lean_c) __attribute__((always_inline)) {
      barrier_keep_vmem<2 * kLoadsPerTile>();  // tile t+1 has landed (own loads; then everyone's)
      softmax_tile(t, mask_c);
      barrier_only();  // the V fragments requested by softmax_tile stay in flight across it
      // Raised issue priority for the MFMA block: the arbiter serves the older wavefront first, so
      // without it the MFMA blocks of set 1 lose issue slots to the softmax of set 0 (~1700 against
      // ~1480 cycles per block).  It buys 7% in cycles and 1-2% in time: the kernel runs at the
      // power limit, and the shader clock gives back most of what a denser schedule saves.
      __builtin_amdgcn_s_setprio(2);
      pv_tile(t, t + 1);
      if (t + 1 < n_compute) qk_tile(t + 1, t + 4, lean_c);
      else issue_tile_loads(t + 4);
      __builtin_amdgcn_s_setprio(0);
    };
    // [0, n_lean): unmasked tile, a QK product follows and its requests (tile t+4) are whole tiles
    const int n_lean = min(min(n_plain, n_compute - 1), n_fast - 4);
    int t = 0;
    for (; t < n_lean; ++t) tile_step(t, std::false_type{}, std::true_type{});
    for (; t < n_plain; ++t) tile_step(t, std::false_type{}, std::false_type{});
    for (; t < n_compute; ++t) tile_step(t, std::true_type{}, std::false_type{});
    for (; t < num_tiles; ++t) {  // above the diagonal: keep the ring and the barriers going
      barrier_keep_vmem<2 * kLoadsPerTile>();
      barrier_only();
      issue_tile_loads(t + 4);
    }
    if (!second_set) barrier_only();  // the slot in which set 1 finishes its last tile
  } else {
    // One wavefront per SIMD.  Ring of 4 tiles: iteration `it` starts with the ring barrier (tile
    // it has landed, the stage of tile it-1 is free) and QK(it) carries the requests of tile it+3.
#pragma unroll
    for (int t = 0; t < kStages - 1; ++t) issue_tile_loads(t);
    barrier_keep_vmem<(kStages - 2) * kLoadsPerTile>();  // tile 0 has landed
    auto ring_barrier = [&]() __attribute__((always_inline)) {
      barrier_keep_vmem<(kStages - 3) * kLoadsPerTile>();
    };
    const int n_lean = min(n_plain, n_fast - (kStages - 1));
    int it = 0;
    k_reads(0, 0, 0);
    for (; it < n_lean; ++it) {
      ring_barrier();
      qk_tile(it, it + kStages - 1, std::true_type{});
      softmax_tile(it, std::false_type{});
      pv_tile(it, it + 1);
    }
    for (; it < n_plain; ++it) {
      ring_barrier();
      qk_tile(it, it + kStages - 1, std::false_type{});
      softmax_tile(it, std::false_type{});
      pv_tile(it, it + 1);
    }
    for (; it < n_compute; ++it) {
      ring_barrier();
      qk_tile(it, it + kStages - 1, std::false_type{});
      softmax_tile(it, std::true_type{});
      pv_tile(it, it + 1);
    }
    for (; it < num_tiles; ++it) {
      ring_barrier();
      issue_tile_loads(it + kStages - 1);
    }
  }
  wait_vmem_all();  // the clamped tail loads must not outlive the workgroup's LDS

  // ---- epilogue: O[m][16*db + 4*lg + r] = O^T / l ------------------------------------------
  // A lane holds 4 consecutive head dims of row lr for every 16-wide block db.  Stored as they
  // are, a store instruction writes 16 rows x 32 bytes with the four lanes of a row 16 lane
  // ids apart, and the address unit only merges ADJACENT lanes: 64 accesses per instruction.
  // The data is therefore re-dealt first, a pair of blocks (db, db+1) at a time: the 16-lane
  // groups g and g^1 trade halves (v_permlane16_swap), after which groups 0/2 hold dims 0-7 /
  // 8-15 of block db and groups 1/3 the same of block db+1, 16 bytes per lane; ds_bpermute then
  // moves the 16 bytes of (row r, segment s) to lane 4*r + s, and four adjacent lanes store 64
  // contiguous bytes of a row.
  {
    const int st_row = lane >> 2, st_seg = lane & 3;
    // segment s of a row lives in group {0, 2, 1, 3}[s] after the swap
    const int src_lane = st_row + 16 * (((st_seg & 1) << 1) | (st_seg >> 1));
#pragma unroll
    for (int qb = 0; qb < kQB; ++qb) {
      const float inv = 1.f / l_acc[qb][0];   // of this lane's own row lr
      const int m_row = q_row0 + 16 * qb + st_row;   // the row this lane stores
      T* o_lane = O + (size_t)m_row * DV + 8 * st_seg;
#pragma unroll
      for (int db = 0; db < kDB; db += 2) {
        unsigned x[2], y[2];
#pragma unroll
        for (int d = 0; d < 2; ++d) {
          const V2 hx = {(T)(o_acc[db][qb][2 * d] * inv), (T)(o_acc[db][qb][2 * d + 1] * inv)};
          const V2 hy = {(T)(o_acc[db + 1][qb][2 * d] * inv), (T)(o_acc[db + 1][qb][2 * d + 1] * inv)};
          x[d] = __builtin_bit_cast(unsigned, hx);
          y[d] = __builtin_bit_cast(unsigned, hy);
#if defined(__HIP_DEVICE_COMPILE__)
          // x of the odd groups <-> y of the even groups
          auto sw = __builtin_amdgcn_permlane16_swap(x[d], y[d], false, false);
          x[d] = sw[0];
          y[d] = sw[1];
#endif
        }
        uint4_t v;
        v[0] = (unsigned)__builtin_amdgcn_ds_bpermute(4 * src_lane, (int)x[0]);
        v[1] = (unsigned)__builtin_amdgcn_ds_bpermute(4 * src_lane, (int)x[1]);
        v[2] = (unsigned)__builtin_amdgcn_ds_bpermute(4 * src_lane, (int)y[0]);
        v[3] = (unsigned)__builtin_amdgcn_ds_bpermute(4 * src_lane, (int)y[1]);
        if (m_row < Lq) *reinterpret_cast<uint4_t*>(o_lane + 16 * db) = v;
      }
    }
  }
  // the next pass re-fills the ring: nobody may still be reading the last tiles
  if (pass + 1 < num_passes) __syncthreads();
  }  // pass
}

template <typename T, int D, int DV, bool kVT, bool kCausal, int kWavesT, int kQB>
int launch_w(const void* Q, const void* K, const void* V, void* O, int batch, int Lq, int Lkv,
             float scale_log2, hipStream_t st) {
  auto kern = flash_attention_fwd_kernel<T, D, DV, kVT, kCausal, kWavesT, kQB>;
  constexpr int lds = ring_stages(kWavesT) * (kBN * lds_pitch(D) * 2 + (kVT ? DV * kBN * 2 : kBN * lds_pitch(DV) * 2));
  static_assert(lds <= kMaxLdsBytes, "tiles do not fit in LDS");
  TFK_LDS_OPT_IN(kern, lds);
  constexpr int bm = kWavesT * 16 * kQB;
  const int q_tiles = (Lq + bm - 1) / bm;
  // causal with an even tile count: one workgroup per PAIR of query tiles (see the kernel)
  const int total_items = (kCausal && q_tiles % 2 == 0) ? (q_tiles / 2) * batch : q_tiles * batch;
  const dim3 grid(8 * ((total_items + 7) / 8));
  hipLaunchKernelGGL(kern, grid, dim3(kWavesT * 64), lds, st,
                     static_cast<const T*>(Q), static_cast<const T*>(K),
                     static_cast<const T*>(V), static_cast<T*>(O), Lq, Lkv, scale_log2,
                     q_tiles, total_items);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}

template <typename T, int D, int DV, bool kVT, bool kCausal>
int launch(const void* Q, const void* K, const void* V, void* O, int batch, int Lq, int Lkv,
           float scale_log2, hipStream_t st) {
  if (Lq > 128) return launch_w<T, D, DV, kVT, kCausal, 8, 2>(Q, K, V, O, batch, Lq, Lkv, scale_log2, st);
  return launch_w<T, D, DV, kVT, kCausal, 4, 2>(Q, K, V, O, batch, Lq, Lkv, scale_log2, st);
}

template <typename T, int D, int DV>
int pick(const void* Q, const void* K, const void* V, void* O, int batch, int Lq, int Lkv,
         float scale_log2, bool vt, bool causal, hipStream_t st) {
  if (vt) {
    if (causal) return launch<T, D, DV, true, true>(Q, K, V, O, batch, Lq, Lkv, scale_log2, st);
    return launch<T, D, DV, true, false>(Q, K, V, O, batch, Lq, Lkv, scale_log2, st);
  }
  if (causal) return launch<T, D, DV, false, true>(Q, K, V, O, batch, Lq, Lkv, scale_log2, st);
  return launch<T, D, DV, false, false>(Q, K, V, O, batch, Lq, Lkv, scale_log2, st);
}

}  // namespace
}  // namespace tfk

namespace tfk {
namespace {
int check_attention_args(const char* who, const void* Q, const void* K, const void* V, const void* O, int64_t batch,
                         int64_t Lq, int64_t Lkv, int64_t D, int64_t Dv, int tile_length_q, int tile_length_kv,
                         int tile_hidden_qk, int tile_hidden_v, double softmax_scale) {
  TFK_REQUIRE(Q && K && V && O, TF_ERR_INVALID_ARG, "%s: null pointer", who);
  TFK_REQUIRE(batch > 0 && Lq > 0 && Lkv > 0 && D > 0 && Dv > 0, TF_ERR_INVALID_ARG, "%s: sizes must be positive", who);
  TFK_REQUIRE(batch < 65536 && Lq < (1 << 21) && Lkv < (1 << 24), TF_ERR_INVALID_ARG, "%s: dimension too large", who);
  TFK_REQUIRE(tile_length_q > 0 && tile_length_kv > 0 && tile_hidden_qk > 0 && tile_hidden_v > 0,
              TF_ERR_INVALID_ARG, "%s: tile sizes must be positive", who);
  TFK_REQUIRE(Lq % tile_length_q == 0 && Lkv % tile_length_kv == 0 && D % tile_hidden_qk == 0 &&
                  Dv % tile_hidden_v == 0,
              TF_ERR_INVALID_ARG, "%s: tile [%d,%d,%d,%d] does not divide problem [%lld,%lld,%lld,%lld]", who,
              tile_length_q, tile_length_kv, tile_hidden_qk, tile_hidden_v, (long long)Lq,
              (long long)Lkv, (long long)D, (long long)Dv);
  TFK_REQUIRE(softmax_scale == softmax_scale && softmax_scale - softmax_scale == 0.0,
              TF_ERR_INVALID_ARG, "%s: softmax_scale must be finite", who);
  return TF_OK;
}

// Head dimensions without a tuned kernel go to a run-time instantiation of the header kernel
// (any D %% 32 == 0, Dv %% 16 == 0 with V transposed, Lq %% 16 == 0, Lkv %% 32 == 0).
int attention_fallback(const char* who, const void* Q, const void* K, const void* V, void* O, int dtype,
                       int64_t batch, int64_t Lq, int64_t Lkv, int64_t D, int64_t Dv, int v_is_transposed,
                       int tq, int tkv, int thqk, int thv, double softmax_scale, int causal, hipStream_t st) {
  TFK_REQUIRE(jit_flash_attention_supports(Lq, Lkv, D, Dv, v_is_transposed), TF_ERR_UNSUPPORTED,
              "%s: no tuned kernel for head dims (D=%lld, Dv=%lld) (128/128, 96/96 and 64/64 have one), and the run-time "
              "compiled kernel needs a transposed V, D %% 32 == 0, Dv %% 16 == 0, Lq %% 16 == 0, Lkv %% 32 == 0 "
              "(got Lq=%lld Lkv=%lld, V %s); the torch op pads and transposes as needed",
              who, (long long)D, (long long)Dv, (long long)Lq, (long long)Lkv,
              v_is_transposed ? "transposed" : "in natural layout");
  return jit_flash_attention(Q, K, V, O, dtype, batch, Lq, Lkv, D, Dv, tq, tkv, thqk, thv, softmax_scale, causal, st);
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
  if (int rc = check_attention_args("tf_flash_attention_fwd_f16", Q, K, V, O, batch, Lq, Lkv, D, Dv, tile_length_q,
                                    tile_length_kv, tile_hidden_qk, tile_hidden_v, softmax_scale))
    return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool tuned = D == Dv && (D == 128 || D == 96 || D == 64);
  if (!tuned)
    return attention_fallback("tf_flash_attention_fwd_f16", Q, K, V, O, TF_DTYPE_F16, batch, Lq, Lkv, D, Dv,
                              v_is_transposed, tile_length_q, tile_length_kv, tile_hidden_qk, tile_hidden_v,
                              softmax_scale, causal, st);
  TFK_REQUIRE(!v_is_transposed || Lkv % 8 == 0, TF_ERR_UNSUPPORTED,
              "tf_flash_attention_fwd_f16: transposed V needs Lkv %% 8 == 0");
  const float scale_log2 = (float)(softmax_scale * 1.4426950408889634);
  if (D == 128)
    return pick<half_t, 128, 128>(Q, K, V, O, (int)batch, (int)Lq, (int)Lkv, scale_log2,
                                  v_is_transposed != 0, causal != 0, st);
  if (D == 96)
    return pick<half_t, 96, 96>(Q, K, V, O, (int)batch, (int)Lq, (int)Lkv, scale_log2,
                                v_is_transposed != 0, causal != 0, st);
  return pick<half_t, 64, 64>(Q, K, V, O, (int)batch, (int)Lq, (int)Lkv, scale_log2,
                              v_is_transposed != 0, causal != 0, st);
}

extern "C" int tf_flash_attention_fwd(const void* Q, const void* K, const void* V, void* O, int dtype, int64_t batch,
                                      int64_t Lq, int64_t Lkv, int64_t D, int64_t Dv, int v_is_transposed,
                                      int tile_length_q, int tile_length_kv, int tile_hidden_qk, int tile_hidden_v,
                                      double softmax_scale, int causal, void* stream) {
  using namespace tfk;
  if (dtype == TF_DTYPE_F16)
    return tf_flash_attention_fwd_f16(Q, K, V, O, batch, Lq, Lkv, D, Dv, v_is_transposed, tile_length_q, tile_length_kv,
                                      tile_hidden_qk, tile_hidden_v, softmax_scale, causal, stream);
  TFK_REQUIRE(dtype == TF_DTYPE_BF16, TF_ERR_UNSUPPORTED,
              "tf_flash_attention_fwd: dtype must be TF_DTYPE_F16 or TF_DTYPE_BF16");
  if (int rc = check_attention_args("tf_flash_attention_fwd", Q, K, V, O, batch, Lq, Lkv, D, Dv, tile_length_q,
                                    tile_length_kv, tile_hidden_qk, tile_hidden_v, softmax_scale))
    return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool tuned = D == Dv && (D == 128 || D == 96 || D == 64) && (!v_is_transposed || Lkv % 8 == 0);
  if (!tuned)
    return attention_fallback("tf_flash_attention_fwd", Q, K, V, O, dtype, batch, Lq, Lkv, D, Dv, v_is_transposed,
                              tile_length_q, tile_length_kv, tile_hidden_qk, tile_hidden_v, softmax_scale, causal, st);
  // the tuned kernels with the bf16 MFMA, bf16 weights and bf16 output
  const float scale_log2 = (float)(softmax_scale * 1.4426950408889634);
  if (D == 128)
    return pick<bf16_t, 128, 128>(Q, K, V, O, (int)batch, (int)Lq, (int)Lkv, scale_log2,
                                  v_is_transposed != 0, causal != 0, st);
  if (D == 96)
    return pick<bf16_t, 96, 96>(Q, K, V, O, (int)batch, (int)Lq, (int)Lkv, scale_log2,
                                v_is_transposed != 0, causal != 0, st);
  return pick<bf16_t, 64, 64>(Q, K, V, O, (int)batch, (int)Lq, (int)Lkv, scale_log2,
                              v_is_transposed != 0, causal != 0, st);
}
