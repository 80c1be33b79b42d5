// Fused back-to-back GEMM for gfx950: D[M,P] = (A[M,K] * B[K,N]) * C[N,P], fp16 or bf16 in/out,
// fp32 accumulate; the intermediate A*B lives only in registers (rounded to the element type like
// the reference does, include/kernels/fused_two_gemms_device.cuh:200).
//
// Counterpart of ke_fused_two_gemms (include/kernels/fused_two_gemms_device.cuh:114-214) and its
// host launcher (src/kernels/fused_two_gemms.cu:66-144).  CDNA4 design:
//   * one workgroup = 64 rows of A (4 wavefronts x 16 rows), v_mfma_f32_16x16x32_f16;
//   * the first GEMM is computed transposed, S^T = B_buf * A^T, so that every lane ends up
//     holding one row m of A*B: the 16x16 accumulator layout (lane -> column m, registers ->
//     4 consecutive n) is, after fp16 conversion, exactly the A-operand fragment layout of
//     the second MFMA up to a permutation of the reduction index, which the C-operand loads
//     mirror.  No LDS round trip, no shuffles for the intermediate;
//   * B and C chunks go global -> LDS directly (global_load_lds_dwordx4) into XOR-swizzled
//     tiles shared by the 4 wavefronts; A fragments are private to a wavefront and are read
//     straight from global memory into registers;
//   * D is staged through LDS so that global stores are 16 bytes per lane along rows.
#include <algorithm>
#include <type_traits>

#include "common.hpp"

namespace tfk {
namespace {

// The kernels move 16-bit elements without looking at them; the element type T (half_t or bf16_t)
// only selects the MFMA and the float -> T conversions.
template <typename T> using vec2_t = T __attribute__((ext_vector_type(2)));
template <typename T> using vec4_t = T __attribute__((ext_vector_type(4)));
template <typename T> using vec8_t = T __attribute__((ext_vector_type(8)));
template <typename T>
TFK_DEVICE float4_t mfma_t(vec8_t<T> a, vec8_t<T> b, float4_t c) {
  if constexpr (std::is_same_v<T, bf16_t>) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  else return mfma_16x16x32(a, b, c);
}

constexpr int kRowsPerBlock = 64;
constexpr int kWaves = 4;
constexpr int kThreads = kWaves * kWaveSize;

// Physical 16-byte chunk for logical chunk c of `row` in a tile whose rows hold CH chunks.
template <int CH>
__host__ __device__ constexpr int swz(int row, int c) {
  constexpr int kRowsPer256B = CH >= 16 ? 1 : 16 / CH;
  return c ^ ((row / kRowsPer256B) % CH);
}

// Cooperative direct global->LDS copy of a [ROWS x COLS] fp16 tile (row stride `ld` elements
// in global memory) into a swizzled LDS tile with COLS-element rows.
template <typename T, int ROWS, int COLS>
TFK_DEVICE void tile_to_lds(const T* __restrict__ g, size_t ld, char* lds, int wave, int lane) {
  constexpr int CH = COLS / 8;
  constexpr int kRowsPerInstr = 64 / CH;
  constexpr int kInstr = ROWS * CH / 64;
  static_assert(ROWS * CH % 64 == 0, "tile must be a whole number of 1 KiB wavefront loads");
  for (int i = wave; i < kInstr; i += kWaves) {
    const int row = i * kRowsPerInstr + lane / CH;
    const int c = swz<CH>(row, lane % CH);
    load_global_to_lds_16B(g + (size_t)row * ld + c * 8, lds + i * 1024);
  }
}

// The two products of one n-tile for one wavefront, with the LDS fragment reads issued one
// step ahead of the MFMAs that use them (a wavefront alone on its SIMD has nobody to hide the
// LDS latency behind; requesting step s+1 before multiplying step s takes it off the critical
// path).  sB: [TN][KC] tile, sC: [TP][TN] tile, both XOR-swizzled.
//   first_product:  acc1[nt] += S^T tile (rows n from B, columns m from A) over the KC / 32 steps
//   second_product: acc2[pt] += (fp16 of acc1) * C over the TN / 32 steps; lane (m = lr, group
//                   lg) holds A*B[m][16*nt + 4*lg + r] in acc1[nt][r], and reduction step s uses
//                   n = 32*s + {4*lg + 0..3, 16 + 4*lg + 0..3} as its 8 slots.
template <typename T, int TN, int KC>
TFK_DEVICE void first_product(const char* sB, const vec8_t<T>* af, float4_t* acc1, int lr, int lg) {
  constexpr int kNT = TN / 16, kKSteps = KC / 32, kCh = KC / 8;
  vec8_t<T> bf[2][kNT];
  auto read_b = [&](int buf, int ks) __attribute__((always_inline)) {
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt) {
      const int row = nt * 16 + lr;
      bf[buf][nt] = *reinterpret_cast<const vec8_t<T>*>(sB + row * KC * 2 + swz<kCh>(row, ks * 4 + lg) * 16);
    }
  };
  read_b(0, 0);
#pragma unroll
  for (int ks = 0; ks < kKSteps; ++ks) {
    if (ks + 1 < kKSteps) read_b((ks + 1) & 1, ks + 1);
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt) acc1[nt] = mfma_t<T>(bf[ks & 1][nt], af[ks], acc1[nt]);
    __builtin_amdgcn_sched_barrier(0);
  }
}
template <typename T, int TN, int TP>
TFK_DEVICE void second_product(const char* sC, const float4_t* acc1, float4_t* acc2, int lr, int lg) {
  constexpr int kPT = TP / 16, kSteps = TN / 32, kCh = TN / 8;
  vec8_t<T> cf[2][kPT];
  auto read_c = [&](int buf, int s2) __attribute__((always_inline)) {
#pragma unroll
    for (int pt = 0; pt < kPT; ++pt) {
      const int row = pt * 16 + lr;
      const char* base = sC + row * TN * 2 + (lg & 1) * 8;
      const vec4_t<T> lo = *reinterpret_cast<const vec4_t<T>*>(base + swz<kCh>(row, 4 * s2 + (lg >> 1)) * 16);
      const vec4_t<T> hi = *reinterpret_cast<const vec4_t<T>*>(base + swz<kCh>(row, 4 * s2 + 2 + (lg >> 1)) * 16);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        cf[buf][pt][r] = lo[r];
        cf[buf][pt][4 + r] = hi[r];
      }
    }
  };
  read_c(0, 0);
#pragma unroll
  for (int s2 = 0; s2 < kSteps; ++s2) {
    if (s2 + 1 < kSteps) read_c((s2 + 1) & 1, s2 + 1);
    vec8_t<T> pa;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      pa[r] = (T)acc1[2 * s2][r];
      pa[4 + r] = (T)acc1[2 * s2 + 1][r];
    }
#pragma unroll
    for (int pt = 0; pt < kPT; ++pt) acc2[pt] = mfma_t<T>(pa, cf[s2 & 1][pt], acc2[pt]);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// ------------------------------------------------------------------------------------------
// Plain kernel: one workgroup = 64 rows (4 wavefronts x 16), n-tiles of TN, k-chunks of KC.
//
// Per n-tile and k-chunk the order of events is chosen for latency (at the benchmark shape
// the whole kernel is one n-tile and one k-chunk, 64 MFMAs per wavefront, so its run time is
// the sum of one trip to memory and one short dependent chain):
//   * A fragments are requested FIRST (they come from HBM, the tiles of B and C from the L2),
//     then the B tile, then the C tile, all asynchronously; the first product starts as soon
//     as A and B have landed, with the C tile still in flight;
//   * fragment reads run one step ahead of the MFMAs across both products;
//   * B rows are dealt to the 16-row MFMA fragments so that the fp16-rounded accumulators of
//     the first product are the second MFMA's operand fragment for EIGHT CONSECUTIVE n
//     (fragment nt takes rows 32*(nt/2) + 8*(i/4) + 4*(nt%2) + i%4, i = 0..15): the matching C
//     fragment is then one 16-byte read;
//   * the second product is computed transposed (D^T = C^T * S^T), which leaves a lane with
//     four consecutive columns of one row of D; pairs of tiles are re-dealt with
//     v_permlane16_swap + ds_bpermute so that four adjacent lanes store 64 contiguous bytes.
//     No LDS staging of D, no barrier in the epilogue.
// ------------------------------------------------------------------------------------------
// row of the B tile that element i of 16-row fragment nt multiplies
__host__ __device__ constexpr int b_frag_row(int nt, int i) { return 32 * (nt / 2) + 8 * (i / 4) + 4 * (nt % 2) + i % 4; }
// XOR key of a B-tile row: the sixteen rows of a fragment get sixteen different keys
template <int CH>
__host__ __device__ constexpr int b_key(int row) {
  if constexpr (CH >= 16) return ((row >> 3) & 3) << 2 | (row & 3);
  else return (row / (16 / CH)) % CH;
}

template <typename T, int TN, int TP, int KC>
__global__ __launch_bounds__(kThreads) void fused_two_gemms_kernel(
    const T* __restrict__ A, const T* __restrict__ B, const T* __restrict__ C,
    T* __restrict__ D, int M, int N, int K, int P) {
  constexpr int kBCh = KC / 8;       // 16-byte chunks per sB row
  constexpr int kCCh = TN / 8;       // per sC row
  constexpr int kKSteps = KC / 32;
  constexpr int kNT = TN / 16;       // 16-wide n tiles of the first GEMM
  constexpr int kPT = TP / 16;       // 16-wide p tiles of the second GEMM
  constexpr int kSteps2 = TN / 32;
  constexpr int kBInstr = TN * kBCh / 64, kCInstr = (TP * kCCh + 63) / 64;   // 1 KiB requests per tile
  constexpr int kBPerWave = (kBInstr + kWaves - 1) / kWaves, kCPerWave = (kCInstr + kWaves - 1) / kWaves;
  static_assert(TN % 32 == 0 && KC % 32 == 0 && TP % 16 == 0, "whole MFMA base tiles");
  __shared__ __attribute__((aligned(1024))) char sB[TN * KC * 2];
  __shared__ __attribute__((aligned(1024))) char sC[kCInstr * 1024];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, lg = lane >> 4;
  const int m0 = blockIdx.x * kRowsPerBlock;
  const int p0 = blockIdx.y * TP;
  const size_t batch = blockIdx.z;
  A += batch * (size_t)M * K;
  B += batch * (size_t)N * K;
  C += batch * (size_t)P * N;
  D += batch * (size_t)M * P;

  // Every global access is a scalar base (tile origin, 64-bit, computed on the scalar unit) plus
  // a 32-bit byte offset per lane that stays inside the tile: the address arithmetic in front of
  // the first request is on this kernel's critical path (per-lane 64-bit pointers for the 4 + 16
  // requests of a wavefront cost ~1 us of the ~3.5 us the kernel ran).
  const int a_row = min(wave * 16 + lr, M - 1 - m0);  // clamped: rows past M are never stored
  const char* a_base = reinterpret_cast<const char*>(A + (size_t)m0 * K);
  const unsigned a_off = ((unsigned)a_row * (unsigned)K + 8u * lg) * 2u;
  const unsigned sB_addr = lds_address(sB), sC_addr = lds_address(sC);
  auto dma = [](unsigned off, const char* base, unsigned lds_addr) __attribute__((always_inline)) {
    // the LDS destination is an M0 INPUT of the statement: the compiler writes M0 itself and
    // cannot use the register for anything else between that write and the request; the s_nop
    // is the wait state an M0 write needs in front of an LDS-direct load
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(off), "s"(base), "{m0}"(lds_addr)
                 : "memory");
  };

  // 1 KiB request i of the B tile covers rows 64 / kBCh * i ..; lane l fills physical chunk
  // l % kBCh of its row with the logical chunk the key maps there.  The same for C with the
  // plain key.  Requests beyond the tile (a C tile smaller than 1 KiB) re-fetch row 0.
  auto request_b = [&](int n0, int k0) __attribute__((always_inline)) {
    const char* b_base = reinterpret_cast<const char*>(B + (size_t)n0 * K + k0);
#pragma unroll
    for (int q = 0; q < kBPerWave; ++q) {
      const int i = wave + kWaves * q;
      if (kBInstr % kWaves != 0 && i >= kBInstr) break;
      const int row = i * (64 / kBCh) + lane / kBCh;
      const int c = (lane % kBCh) ^ b_key<kBCh>(row);
      dma(((unsigned)row * (unsigned)K + (unsigned)c * 8u) * 2u, b_base, sB_addr + i * 1024);
    }
  };
  auto request_c = [&](int n0) __attribute__((always_inline)) {
    const char* c_base = reinterpret_cast<const char*>(C + (size_t)p0 * N + n0);
#pragma unroll
    for (int q = 0; q < kCPerWave; ++q) {
      const int i = wave + kWaves * q;
      if (kCInstr % kWaves != 0 && i >= kCInstr) break;
      const int row = min(i * (64 / kCCh) + lane / kCCh, TP - 1);
      const int c = swz<kCCh>(row, lane % kCCh);
      dma(((unsigned)row * (unsigned)N + (unsigned)c * 8u) * 2u, c_base, sC_addr + i * 1024);
    }
  };
  // requests of this wavefront that are still allowed in flight when B (and A) must be there
  const int c_requests = (kCInstr % kWaves == 0 || wave < kCInstr % kWaves) ? kCPerWave : kCPerWave - 1;

  auto read_b = [&](vec8_t<T>* dst, int ks) __attribute__((always_inline)) {
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt) {
      const int row = b_frag_row(nt, lr);
      dst[nt] = *reinterpret_cast<const vec8_t<T>*>(sB + row * KC * 2 + ((ks * 4 + lg) ^ b_key<kBCh>(row)) * 16);
    }
  };
  auto read_c = [&](vec8_t<T>* dst, int s2) __attribute__((always_inline)) {
#pragma unroll
    for (int pt = 0; pt < kPT; ++pt) {
      const int row = pt * 16 + lr;
      dst[pt] = *reinterpret_cast<const vec8_t<T>*>(sC + row * TN * 2 + swz<kCCh>(row, 4 * s2 + lg) * 16);
    }
  };

  float4_t acc2[kPT];
#pragma unroll
  for (int pt = 0; pt < kPT; ++pt) acc2[pt] = float4_t{0.f, 0.f, 0.f, 0.f};

  for (int n0 = 0; n0 < N; n0 += TN) {
    float4_t acc1[kNT];
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt) acc1[nt] = float4_t{0.f, 0.f, 0.f, 0.f};

    for (int k0 = 0; k0 < K; k0 += KC) {
      const bool first_chunk = k0 == 0;
      // previous readers of sB (and, at a new n-tile, of sC) are done
      if (n0 != 0 || k0 != 0) barrier_lds_only();
      vec8_t<T> af[kKSteps];
      // All three kinds of request are issued from assembly, so that the compiler places no
      // vector-memory waits of its own (it would drain everything, the C tile included, in
      // front of the first LDS read or the first use of an A fragment).
      {
        const char* a_chunk = a_base + (size_t)k0 * 2;
#pragma unroll
        for (int ks = 0; ks < kKSteps; ++ks)
          // (early-clobber outputs: a fragment register never doubles as the address register of
          //  a later request)
          asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3"
                       : "=&v"(af[ks])
                       : "v"(a_off), "s"(a_chunk), "n"(ks * 64)
                       : "memory");
      }
      // the A requests are on their way before the arithmetic of the B and C requests starts.
      // Between here and the wait below the compiler believes the fragment registers written
      // although the data is still in flight: nothing in between reads them (only requests and
      // their scalar address arithmetic are issued), and tests/test_gpu_fused_two_gemms.py::
      // test_every_plain_kernel_instance_is_exact pins that, for every instance of this kernel and
      // both element types, on problems with several k-chunks and n-tiles.
      __builtin_amdgcn_sched_barrier(0);
      request_b(n0, k0);
      if (first_chunk) request_c(n0);
      // A and B have landed once at most this wavefront's C requests are outstanding (loads
      // retire in order); the fragment registers are re-defined behind the wait so that no use
      // of them can be scheduled in front of it.
      if (first_chunk && c_requests == kCPerWave) {
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(kCPerWave) : "memory");
      } else if (first_chunk && kCPerWave > 1) {
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(kCPerWave > 1 ? kCPerWave - 1 : 0) : "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) asm volatile("" : "+v"(af[ks]));
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");

      // first product, transposed: acc1[nt] += B rows (fragment nt) x A^T, reads one step ahead
      vec8_t<T> bf[2][kNT];
      read_b(bf[0], 0);
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) {
        if (ks + 1 < kKSteps) read_b(bf[(ks + 1) & 1], ks + 1);
#pragma unroll
        for (int nt = 0; nt < kNT; ++nt) acc1[nt] = mfma_t<T>(bf[ks & 1][nt], af[ks], acc1[nt]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // the C tile has landed for everybody
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // second product, transposed: lane (m = lr, group lg) holds A*B[m][32*s2 + 8*lg + 0..7] in
    // acc1[2*s2][0..3], acc1[2*s2 + 1][0..3]; acc2[pt] += C rows (p) x that
    vec8_t<T> cf[2][kPT];
    read_c(cf[0], 0);
#pragma unroll
    for (int s2 = 0; s2 < kSteps2; ++s2) {
      if (s2 + 1 < kSteps2) read_c(cf[(s2 + 1) & 1], s2 + 1);
      vec8_t<T> pa;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pa[r] = (T)acc1[2 * s2][r];
        pa[4 + r] = (T)acc1[2 * s2 + 1][r];
      }
#pragma unroll
      for (int pt = 0; pt < kPT; ++pt) acc2[pt] = mfma_t<T>(cf[s2 & 1][pt], pa, acc2[pt]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // Epilogue: acc2[pt][r] = D[m0 + 16*wave + lr][p0 + 16*pt + 4*lg + r].
  const int d_row0 = m0 + wave * 16;
  if constexpr (kPT % 2 == 0) {
    // Pairs of tiles: the 16-lane groups g and g^1 trade halves (v_permlane16_swap), after which
    // group 0/2 holds columns 0-7 / 8-15 of tile pt and group 1/3 the same of tile pt+1, 16 bytes
    // per lane; ds_bpermute then moves the 16 bytes of (row r, segment s) to lane 4*r + s, so
    // that a store writes 16 rows x 64 contiguous bytes with four adjacent lanes per row.
    const int st_row = lane >> 2, st_seg = lane & 3;
    const int src_lane = st_row + 16 * (((st_seg & 1) << 1) | (st_seg >> 1));
    T* d_lane = D + (size_t)(d_row0 + st_row) * P + p0 + 8 * st_seg;
    const bool row_ok = d_row0 + st_row < M;
    uint4_t v[kPT / 2];
#pragma unroll
    for (int pt = 0; pt < kPT; pt += 2) {
      typedef vec2_t<T> h2_t;
      unsigned x[2], y[2];
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        const h2_t hx = {(T)acc2[pt][2 * d], (T)acc2[pt][2 * d + 1]};
        const h2_t hy = {(T)acc2[pt + 1][2 * d], (T)acc2[pt + 1][2 * d + 1]};
        x[d] = __builtin_bit_cast(unsigned, hx);
        y[d] = __builtin_bit_cast(unsigned, hy);
#if defined(__HIP_DEVICE_COMPILE__)
        auto sw = __builtin_amdgcn_permlane16_swap(x[d], y[d], false, false);
        x[d] = sw[0];
        y[d] = sw[1];
#endif
      }
      v[pt / 2][0] = (unsigned)__builtin_amdgcn_ds_bpermute(4 * src_lane, (int)x[0]);
      v[pt / 2][1] = (unsigned)__builtin_amdgcn_ds_bpermute(4 * src_lane, (int)x[1]);
      v[pt / 2][2] = (unsigned)__builtin_amdgcn_ds_bpermute(4 * src_lane, (int)y[0]);
      v[pt / 2][3] = (unsigned)__builtin_amdgcn_ds_bpermute(4 * src_lane, (int)y[1]);
    }
    // streaming stores: D is written once and not read again here, and an ordinary store next
    // to the operand reads costs this latency-bound kernel 10%
    if (row_ok) {
#pragma unroll
      for (int pt = 0; pt < kPT; pt += 2)
        __builtin_nontemporal_store(v[pt / 2], reinterpret_cast<uint4_t*>(d_lane + 16 * pt));
    }
  } else {
    // a single 16-column tile: 8 bytes per lane
#pragma unroll
    for (int pt = 0; pt < kPT; ++pt) {
      vec4_t<T> v;
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] = (T)acc2[pt][r];
      if (d_row0 + lr < M)
        *reinterpret_cast<vec4_t<T>*>(D + (size_t)(d_row0 + lr) * P + p0 + 16 * pt + 4 * lg) = v;
    }
  }
}

template <typename T, int TN, int TP, int KC>
int launch(const void* A, const void* B, const void* C, void* D, int batch, int M, int N, int K,
           int P, hipStream_t st) {
  dim3 grid((M + kRowsPerBlock - 1) / kRowsPerBlock, P / TP, batch);
  hipLaunchKernelGGL((fused_two_gemms_kernel<T, TN, TP, KC>), grid, dim3(kThreads), 0, st,
                     static_cast<const T*>(A), static_cast<const T*>(B),
                     static_cast<const T*>(C), static_cast<T*>(D), M, N, K, P);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}

// ------------------------------------------------------------------------------------------
// Streaming variant for long N (K = P = 128, N a multiple of 64, at least four n-tiles): n-tiles
// of 64 (a B tile [64][128] and a C tile [128][64], whole 128-byte lines either way) go global ->
// LDS through a four-stage ring, three tiles ahead of the one being multiplied, one barrier per
// n-tile; A fragments are loaded once.  A workgroup alone on a CU has to hide the L2 latency
// with bytes in flight: two 64 KiB stages (one tile ahead) ran at a quarter of this speed.
// ------------------------------------------------------------------------------------------
// kSplit = 2: a second set of kWavesT wavefronts takes every other n-tile of the same rows (the
// pair w, w + kWavesT shares a SIMD), and the two partial D tiles are added through LDS at the
// end.  A wavefront's chain per tile - fragment reads, 16 MFMAs, fp16 conversion, 16 MFMAs that
// depend on it - leaves the matrix pipe idle most of the time; a second, independent chain on
// the same SIMD fills it.  Only the first set issues the tile requests.
// kPartial: blockIdx.y selects a part of `tiles_per_part` n-tiles, and the workgroup writes its fp32
// partial sums to part blockIdx.y of the workspace W [batch][parts][M][128] instead of D; a second
// kernel adds the parts up.  M / 64 workgroups do not fill the chip for the shapes this kernel is
// for, and a workgroup is bound by how many tile bytes its ring keeps in flight, not by arithmetic.
template <typename T, int kWavesT, int kSplit, bool kPartial>
__global__ __launch_bounds__(kWavesT * kSplit * 64) void fused_two_gemms_stream_kernel(
    const T* __restrict__ A, const T* __restrict__ B, const T* __restrict__ C,
    T* __restrict__ D, float* __restrict__ W, int M, int N, int tiles_per_part) {
  constexpr int K = 128, P = 128, TN = 64, kStagesS = 4;
  constexpr int kRows = 16 * kWavesT;
  constexpr int kBBytes = TN * K * 2;                // 16 KiB: B tile [n][k], 256-byte rows
  constexpr int kCBytes = P * TN * 2;                // 16 KiB: C tile [p][n], 128-byte rows
  constexpr int kStageBytes = kBBytes + kCBytes;
  constexpr int kBInstr = kBBytes / 1024, kCInstr = kCBytes / 1024;   // 1 KiB wavefront requests
  // the first kReqWaves wavefronts issue the tile requests (all of them when there are four)
  constexpr int kReqWaves = kWavesT > 4 ? 4 : kWavesT;
  constexpr int kReqPerWave = (kBInstr + kCInstr) / kReqWaves;
  static_assert((kBInstr / kReqWaves) % 4 == 0 && (kCInstr / kReqWaves) % 4 == 0,
                "a wavefront's requests of a tile come in groups of four consecutive instructions");
  // tiles requested ahead of the one being multiplied: the ring allows kStagesS - 1, the 6-bit
  // vmcnt allows 63 requests of one wavefront to stay in flight behind the awaited tile
  constexpr int kAhead = (kStagesS - 2) * kReqPerWave <= 63 ? kStagesS - 1 : 63 / kReqPerWave + 1;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  T* sD = reinterpret_cast<T*>(smem + kStagesS * kStageBytes);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_id = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave = wave_id % kWavesT;      // which 16 rows
  const int half = wave_id / kWavesT;      // which n-tiles (t % kSplit == half)
  const int lr = lane & 15, lg = lane >> 4;
  const int m0 = blockIdx.x * kRows;
  const size_t batch = blockIdx.z;
  A += batch * (size_t)M * K;
  B += batch * (size_t)N * K;
  C += batch * (size_t)P * N;
  D += batch * (size_t)M * P;
  const unsigned smem_base = lds_address(smem);

  const int a_row = min(m0 + wave * 16 + lr, M - 1);  // clamped: rows past M are never stored
  vec8_t<T> af[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks)
    af[ks] = *reinterpret_cast<const vec8_t<T>*>(A + (size_t)a_row * K + 8 * lg + ks * 32);

  // this workgroup's n-tiles: [t_begin, t_begin + n_tiles)
  const int t_begin = kPartial ? (int)blockIdx.y * tiles_per_part : 0;
  const int n_tiles = kPartial ? min(tiles_per_part, N / TN - t_begin) : N / TN;
  // Requests of n-tile t (clamped past the end: the surplus lands in a stage nobody reads
  // again).  Instruction i of the B tile covers rows 4i .. 4i+3 (16 chunks each), of the C tile
  // rows 8i .. 8i+7 (8 chunks each); lane l fills physical chunk l % 16 (l % 8) and fetches the
  // logical chunk the swizzle maps there.  The swizzle XORs row bits into the chunk index, so the
  // per-lane byte offsets of all instructions follow from one base by an XOR with a constant
  // (B: 4 variants, C: 2); everything else - the tile origin, the rows 4i or 8i, the part
  // cancelled by the immediate offset - is scalar.  Four instructions share one M0 value.
  const unsigned voff_b0 = (lane / 16) * (K * 2) + (((lane % 16) ^ (lane / 16)) << 4);
  const unsigned voff_c0 = (lane / 8) * (unsigned)N * 2u + (((lane % 8) ^ (lane / 16)) << 4);
  auto request_tile = [&](int t) __attribute__((always_inline)) {
    if (wave_id >= kReqWaves) return;
    const unsigned stage = smem_base + (t % kStagesS) * kStageBytes;
    const int n0 = (t_begin + min(t, n_tiles - 1)) * TN;
    const char* b_src = reinterpret_cast<const char*>(B) + (size_t)n0 * (K * 2);
    const char* c_src = reinterpret_cast<const char*>(C) + (size_t)n0 * 2;
#pragma unroll
    for (int q = 0; q < kBInstr / kReqWaves; ++q) {
      // instructions are dealt in blocks of kBInstr / kReqWaves consecutive ones per wavefront
      const int i_first = wave_id * (kBInstr / kReqWaves);
      const unsigned voff = voff_b0 ^ (unsigned)(((q % 4) * 4) << 4);        // row 4i: chunk ^= 4 * (i % 4)
      const char* src = b_src + (size_t)(i_first + q) * 1024 - (q % 4) * 1024;   // + rows, - what the immediate adds
      // four requests share one M0 value (an input of each statement, so the compiler keeps it
      // there) and differ in the immediate offset
      asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%2"
                   :
                   : "v"(voff), "s"(src), "n"(1024 * (q % 4)), "{m0}"(stage + (i_first + q - q % 4) * 1024)
                   : "memory");
    }
#pragma unroll
    for (int q = 0; q < kCInstr / kReqWaves; ++q) {
      const int i_first = wave_id * (kCInstr / kReqWaves);
      const unsigned voff = voff_c0 ^ (unsigned)(((q % 2) * 4) << 4);        // row 8i: chunk ^= 4 * (i % 2)
      const char* src = c_src + (size_t)(i_first + q) * 8 * (size_t)N * 2 - (q % 4) * 1024;
      asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%2"
                   :
                   : "v"(voff), "s"(src), "n"(1024 * (q % 4)), "{m0}"(stage + kBBytes + (i_first + q - q % 4) * 1024)
                   : "memory");
    }
  };

  float4_t acc2[8];
#pragma unroll
  for (int pt = 0; pt < 8; ++pt) acc2[pt] = float4_t{0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int t = 0; t < kAhead; ++t) request_tile(t);
  for (int t = 0; t < n_tiles; ++t) {
    // this wavefront's requests of tile t have landed (kAhead - 1 younger tiles stay in flight); after
    // the barrier everybody's have, and everybody is done with tile t-1, whose stage is refilled
    wait_vmem<(kAhead - 1) * kReqPerWave>();
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    request_tile(t + kAhead);
    const char* sB = smem + (t % kStagesS) * kStageBytes;
    const char* sC = sB + kBBytes;

    if (kSplit > 1 && t % kSplit != half) continue;
    float4_t acc1[TN / 16];
#pragma unroll
    for (int nt = 0; nt < TN / 16; ++nt) acc1[nt] = float4_t{0.f, 0.f, 0.f, 0.f};
    first_product<T, TN, K>(sB, af, acc1, lr, lg);
    second_product<T, TN, P>(sC, acc1, acc2, lr, lg);
  }
  wait_vmem_all();  // the surplus requests must not outlive the workgroup's LDS
  if constexpr (kSplit > 1) {
    // add the second set's partial sums to the first set's (the ring is free by now)
    __syncthreads();
    constexpr int kPartElems = kWavesT * 8 * 64;   // float4 per wavefront set
    static_assert((kSplit - 1) * kPartElems * 16 <= kStagesS * kStageBytes, "partial sums fit in the ring");
    float4_t* part = reinterpret_cast<float4_t*>(smem) + (size_t)wave * 8 * 64 + lane;
    if (half != 0) {
#pragma unroll
      for (int pt = 0; pt < 8; ++pt) part[(half - 1) * kPartElems + pt * 64] = acc2[pt];
    }
    __syncthreads();
    if (half == 0) {
#pragma unroll
      for (int h = 1; h < kSplit; ++h)
#pragma unroll
        for (int pt = 0; pt < 8; ++pt) acc2[pt] += part[(h - 1) * kPartElems + pt * 64];
    }
  }

  // Epilogue: acc2[pt][r] = D[m0 + 16*wave + 4*lg + r][16*pt + lr]
  if constexpr (kPartial) {
    // fp32 partial sums straight from the accumulators: 16 adjacent lanes write 64 contiguous bytes
    if (half == 0) {
      float* w = W + ((batch * gridDim.y + blockIdx.y) * (size_t)M + m0 + wave * 16 + 4 * lg) * P + lr;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (m0 + wave * 16 + 4 * lg + r < M) {
#pragma unroll
          for (int pt = 0; pt < 8; ++pt) __builtin_nontemporal_store(acc2[pt][r], w + (size_t)r * P + pt * 16);
        }
    }
    return;
  }
  // fp16 result, staged through LDS for 16-byte stores along rows
  if (half == 0) {
#pragma unroll
    for (int pt = 0; pt < 8; ++pt)
#pragma unroll
      for (int r = 0; r < 4; ++r) sD[(wave * 16 + 4 * lg + r) * P + pt * 16 + lr] = (T)acc2[pt][r];
  }
  __syncthreads();
  constexpr int kDChunks = P / 8;
  for (int f = tid; f < kRows * kDChunks; f += kWavesT * kSplit * 64) {
    const int row = f / kDChunks, c = f % kDChunks;
    if (m0 + row < M)
      __builtin_nontemporal_store(*reinterpret_cast<const uint4_t*>(sD + row * P + c * 8),
                                  reinterpret_cast<uint4_t*>(D + (size_t)(m0 + row) * P + c * 8));
  }
}

// D[b][i] = fp16(sum over parts of W[b][part][i]), i over the M * 128 elements of a problem
template <typename T>
__global__ __launch_bounds__(256) void fused_two_gemms_reduce_kernel(const float* __restrict__ W,
                                                                     T* __restrict__ D, int parts,
                                                                     size_t elems) {
  const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= elems) return;
  const float* w = W + (size_t)blockIdx.z * parts * elems + i;
  float4_t acc = __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(w));
  for (int part = 1; part < parts; ++part)
    acc += __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(w + (size_t)part * elems));
  vec4_t<T> h = {(T)acc[0], (T)acc[1], (T)acc[2], (T)acc[3]};
  *reinterpret_cast<vec4_t<T>*>(D + (size_t)blockIdx.z * elems + i) = h;
}

template <typename T, int kWavesT, int kSplit>
int launch_stream(const void* A, const void* B, const void* C, void* D, int batch, int M, int N,
                  hipStream_t st) {
  auto kern = fused_two_gemms_stream_kernel<T, kWavesT, kSplit, false>;
  constexpr int lds = 4 * (64 * 128 * 2 + 128 * 64 * 2) + 16 * kWavesT * 128 * 2;
  static_assert(lds <= kMaxLdsBytes, "ring does not fit in LDS");
  TFK_LDS_OPT_IN(kern, lds);
  dim3 grid((M + 16 * kWavesT - 1) / (16 * kWavesT), 1, batch);
  hipLaunchKernelGGL(kern, grid, dim3(kWavesT * kSplit * 64), lds, st, static_cast<const T*>(A),
                     static_cast<const T*>(B), static_cast<const T*>(C),
                     static_cast<T*>(D), static_cast<float*>(nullptr), M, N, 0);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}

// How a long-N problem (K = P = 128) is cut when a workspace is available: `parts` ranges of
// `tiles_per_part` 64-wide n-tiles for row blocks of `rows` rows.  A workgroup takes a CU to itself
// (the ring fills its LDS) and is bound by the tile bytes it keeps in flight, so the cut aims at one
// workgroup per CU (row blocks x parts <= 256) and keeps at least the four tiles per part that
// fill the ring.  Measured on the reference's sweep, a launch takes about 9.6 + 0.9 t us with
// 64-row blocks and 11.8 + 1.23 t us with 128-row blocks (eight wavefronts share every tile), t the
// tiles a workgroup walks, against 4 + 0.8 t uncut: the second launch and the trip of the partial
// sums through memory are in the constants.  The cheapest of the three is taken; 128-row blocks
// only from eight tiles per part on (shorter walks are dominated by filling the ring, and eight
// wavefronts fill it no faster than four).  parts == 1: no cut.
struct SplitPlan { int parts, tiles_per_part, rows; };
SplitPlan fused_split_plan(int64_t batch, int64_t M, int64_t N, int64_t K, int64_t P) {
  const SplitPlan uncut = {1, 0, 64};
  if (!(K == 128 && P == 128 && N % 64 == 0 && N >= 512)) return uncut;
  const int64_t n_tiles = N / 64;
  auto cut = [&](int rows) -> SplitPlan {
    const int64_t row_blocks = (M + rows - 1) / rows * batch;
    int64_t parts = std::min<int64_t>(256 / std::max<int64_t>(row_blocks, 1), n_tiles / 4);
    if (parts <= 1) return {1, 0, rows};
    const int64_t per = (n_tiles + parts - 1) / parts;
    return {(int)((n_tiles + per - 1) / per), (int)per, rows};
  };
  const SplitPlan p64 = cut(64), p128 = cut(128);
  double best = 4.0 + 0.8 * (double)n_tiles;
  SplitPlan plan = uncut;
  if (p64.parts > 1 && 9.6 + 0.9 * p64.tiles_per_part < best) {
    best = 9.6 + 0.9 * p64.tiles_per_part;
    plan = p64;
  }
  if (p128.parts > 1 && p128.tiles_per_part >= 8 && 11.8 + 1.23 * p128.tiles_per_part < best) plan = p128;
  return plan;
}

template <typename T, int kWavesT, int kSplit>
int launch_stream_split(const void* A, const void* B, const void* C, void* D, float* W, SplitPlan plan, int batch,
                        int M, int N, hipStream_t st) {
  auto kern = fused_two_gemms_stream_kernel<T, kWavesT, kSplit, true>;
  constexpr int lds = 4 * (64 * 128 * 2 + 128 * 64 * 2) + 16 * kWavesT * 128 * 2;
  TFK_LDS_OPT_IN(kern, lds);
  dim3 grid((M + 16 * kWavesT - 1) / (16 * kWavesT), plan.parts, batch);
  hipLaunchKernelGGL(kern, grid, dim3(kWavesT * kSplit * 64), lds, st, static_cast<const T*>(A),
                     static_cast<const T*>(B), static_cast<const T*>(C),
                     static_cast<T*>(D), W, M, N, plan.tiles_per_part);
  TFK_HIP_TRY(hipGetLastError());
  const size_t elems = (size_t)M * 128;
  hipLaunchKernelGGL(fused_two_gemms_reduce_kernel<T>, dim3((unsigned)((elems / 4 + 255) / 256), 1, batch), dim3(256), 0,
                     st, W, static_cast<T*>(D), plan.parts, elems);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}

template <typename T, int TN, int TP>
int pick_kc(const void* A, const void* B, const void* C, void* D, int batch, int M, int N, int K,
            int P, hipStream_t st) {
  if (K % 128 == 0) return launch<T, TN, TP, 128>(A, B, C, D, batch, M, N, K, P, st);
  return launch<T, TN, TP, 32>(A, B, C, D, batch, M, N, K, P, st);
}

template <typename T, int TN>
int pick_tp(const void* A, const void* B, const void* C, void* D, int batch, int M, int N, int K,
            int P, hipStream_t st) {
  if (P % 128 == 0) return pick_kc<T, TN, 128>(A, B, C, D, batch, M, N, K, P, st);
  if (P % 64 == 0) return pick_kc<T, TN, 64>(A, B, C, D, batch, M, N, K, P, st);
  return pick_kc<T, TN, 16>(A, B, C, D, batch, M, N, K, P, st);
}

}  // namespace
}  // namespace tfk

namespace tfk {
namespace {
int check_fused_args(const char* who, const void* A, const void* B, const void* C, const void* D, int64_t batch,
                     int64_t M, int64_t N, int64_t K, int64_t P, int tm, int tn, int tk, int tp) {
  TFK_REQUIRE(A && B && C && D, TF_ERR_INVALID_ARG, "%s: null pointer", who);
  TFK_REQUIRE(batch > 0 && M > 0 && N > 0 && K > 0 && P > 0, TF_ERR_INVALID_ARG, "%s: sizes must be positive", who);
  TFK_REQUIRE(batch < 65536 && M < (1 << 30) && N < (1 << 24) && K < (1 << 24) && P < (1 << 24),
              TF_ERR_INVALID_ARG, "%s: dimension too large", who);
  TFK_REQUIRE(tm > 0 && tn > 0 && tk > 0 && tp > 0, TF_ERR_INVALID_ARG, "%s: tile sizes must be positive", who);
  TFK_REQUIRE(M % tm == 0 && N % tn == 0 && K % tk == 0 && P % tp == 0, TF_ERR_INVALID_ARG,
              "%s: tile [%d,%d,%d,%d] does not divide problem [%lld,%lld,%lld,%lld]", who, tm, tn, tk, tp,
              (long long)M, (long long)N, (long long)K, (long long)P);
  TFK_REQUIRE(K % 32 == 0 && N % 32 == 0 && P % 16 == 0, TF_ERR_UNSUPPORTED,
              "%s: needs K %% 32 == 0, N %% 32 == 0, P %% 16 == 0 (got K=%lld N=%lld P=%lld); zero-pad K and N "
              "(the torch op does)", who, (long long)K, (long long)N, (long long)P);
  return TF_OK;
}
}  // namespace
}  // namespace tfk

namespace tfk {
namespace {
// the tuned kernels for element type T (arguments already checked)
template <typename T>
int run_fused(const void* A, const void* B, const void* C, void* D, int64_t batch, int64_t M, int64_t N, int64_t K,
              int64_t P, hipStream_t st) {
  // long N: stream the B / C tiles through the LDS ring (8-15% faster than the plain kernel's
  // load - wait - multiply per n-tile; both are bound by the latencies of one wavefront per SIMD)
  if (K == 128 && P == 128 && N % 64 == 0 && N >= 256) {
    // enough rows for a 128-row block per CU: eight wavefronts share every tile (1.23 us per tile
    // for 128 rows against 0.8 us for 64)
    if (N >= 512 && (M + 127) / 128 * batch >= 256)
      return launch_stream<T, 8, 1>(A, B, C, D, (int)batch, (int)M, (int)N, st);
    return launch_stream<T, 4, 2>(A, B, C, D, (int)batch, (int)M, (int)N, st);
  }
  if (N % 128 == 0) return pick_tp<T, 128>(A, B, C, D, (int)batch, (int)M, (int)N, (int)K, (int)P, st);
  return pick_tp<T, 32>(A, B, C, D, (int)batch, (int)M, (int)N, (int)K, (int)P, st);
}
template <typename T>
int run_fused_split(const void* A, const void* B, const void* C, void* D, float* W, SplitPlan plan, int64_t batch,
                    int64_t M, int64_t N, hipStream_t st) {
  if (plan.rows == 128) return launch_stream_split<T, 8, 1>(A, B, C, D, W, plan, (int)batch, (int)M, (int)N, st);
  return launch_stream_split<T, 4, 2>(A, B, C, D, W, plan, (int)batch, (int)M, (int)N, st);
}
}  // namespace
}  // namespace tfk

extern "C" int tf_fused_two_gemms_f16(const void* A, const void* B, const void* C, void* D,
                                      int64_t batch, int64_t M, int64_t N, int64_t K, int64_t P,
                                      int tm, int tn, int tk, int tp, void* stream) {
  using namespace tfk;
  if (int rc = check_fused_args("tf_fused_two_gemms_f16", A, B, C, D, batch, M, N, K, P, tm, tn, tk, tp)) return rc;
  return run_fused<half_t>(A, B, C, D, batch, M, N, K, P, static_cast<hipStream_t>(stream));
}

extern "C" size_t tf_fused_two_gemms_workspace_bytes(int dtype, int64_t batch, int64_t M, int64_t N, int64_t K,
                                                     int64_t P) {
  using namespace tfk;
  if ((dtype != TF_DTYPE_F16 && dtype != TF_DTYPE_BF16) || batch <= 0 || M <= 0 || N <= 0) return 0;
  const SplitPlan plan = fused_split_plan(batch, M, N, K, P);
  return plan.parts > 1 ? (size_t)plan.parts * (size_t)batch * (size_t)M * 128 * sizeof(float) : 0;
}

extern "C" int tf_fused_two_gemms_ws(const void* A, const void* B, const void* C, void* D, int dtype, int64_t batch,
                                     int64_t M, int64_t N, int64_t K, int64_t P, int tm, int tn, int tk, int tp,
                                     void* workspace, size_t workspace_bytes, void* stream) {
  using namespace tfk;
  const size_t want = tf_fused_two_gemms_workspace_bytes(dtype, batch, M, N, K, P);
  if (want == 0 || workspace == nullptr || workspace_bytes < want)
    return tf_fused_two_gemms(A, B, C, D, dtype, batch, M, N, K, P, tm, tn, tk, tp, stream);
  if (int rc = check_fused_args("tf_fused_two_gemms_ws", A, B, C, D, batch, M, N, K, P, tm, tn, tk, tp)) return rc;
  TFK_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, TF_ERR_INVALID_ARG,
              "tf_fused_two_gemms_ws: workspace must be 16-byte aligned");
  const SplitPlan plan = fused_split_plan(batch, M, N, K, P);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == TF_DTYPE_BF16)
    return run_fused_split<bf16_t>(A, B, C, D, static_cast<float*>(workspace), plan, batch, M, N, st);
  return run_fused_split<half_t>(A, B, C, D, static_cast<float*>(workspace), plan, batch, M, N, st);
}

extern "C" int tf_fused_two_gemms(const void* A, const void* B, const void* C, void* D, int dtype, int64_t batch,
                                  int64_t M, int64_t N, int64_t K, int64_t P, int tm, int tn, int tk, int tp,
                                  void* stream) {
  using namespace tfk;
  if (dtype == TF_DTYPE_F16) return tf_fused_two_gemms_f16(A, B, C, D, batch, M, N, K, P, tm, tn, tk, tp, stream);
  TFK_REQUIRE(dtype == TF_DTYPE_BF16, TF_ERR_UNSUPPORTED,
              "tf_fused_two_gemms: dtype must be TF_DTYPE_F16 or TF_DTYPE_BF16");
  // bf16: the same kernels with the bf16 MFMA, a bf16 intermediate and bf16 output
  if (int rc = check_fused_args("tf_fused_two_gemms", A, B, C, D, batch, M, N, K, P, tm, tn, tk, tp)) return rc;
  return run_fused<bf16_t>(A, B, C, D, batch, M, N, K, P, static_cast<hipStream_t>(stream));
}
