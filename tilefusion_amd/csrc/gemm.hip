// GEMM macro kernel for gfx950: C[M,N] = A[M,K] * B[K,N] with A row-major and B handed over
// as its [N,K] buffer (column-major K x N), fp16 in, fp32 accumulate, fp32 or fp16 out.
//
// Counterpart of the reference's ke_gemm / ke_gemm_level1_pipeline / ke_gemm_level2_pipeline
// (include/kernels/gemm_device.cuh:110-419) and its host launcher (src/kernels/gemm.cu:63-142),
// re-designed for CDNA4:
//   * 64-lane wavefronts, v_mfma_f32_16x16x32_f16 base tiles, accumulators in the unified
//     512-entry register file (one wavefront per SIMD, 128x128 per wavefront at the big tile);
//   * both operands are K-contiguous, so an MFMA operand fragment is one 16-byte LDS read;
//   * tiles go global -> LDS without passing through VGPRs (global_load_lds_dwordx4) into an
//     XOR-swizzled LDS ring: a wavefront instruction always writes 1 KiB of consecutive LDS,
//     so the swizzle is applied on the global (source) side;
//   * the main kernel (gemm_ring64_kernel) uses 64-deep k-tiles so that every request fetches
//     whole 128-byte lines, keeps the ring in units of one operand, and issues its MFMAs from
//     assembly with a hand-placed instruction order (a lone wavefront issues one instruction
//     per 4 cycles: at most three others fit behind a 16-cycle MFMA); it comes with 256 x 256
//     tiles and, for grids that those would leave most CUs idle on, with 128 x 128 tiles;
//     K % 64 != 0 falls back to the 32-deep direct-to-LDS kernel, other shapes to a
//     bounds-checked one;
//   * workgroup -> tile map keeps the workgroups of one XCD (one L2) on a compact block of
//     output tiles.
#include <type_traits>

#include "common.hpp"

namespace tfk {
namespace {

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, int STAGES_>
struct GemmShape {
  static constexpr int BM = BM_, BN = BN_, BK = BK_;
  static constexpr int kStages = STAGES_;  // LDS stages of the direct-load pipeline
  static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * kWaveSize;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // tile of one wavefront
  static constexpr int TM = WM / 32, TN = WN / 32;            // 32x32 MFMA tiles per wavefront
  static constexpr int kKSteps = BK / 16;
  static constexpr int kChunks = BK / 8;              // 16-byte chunks per tile row
  static constexpr int kRowsPer256B = 16 / kChunks;   // rows that share one pass over all banks
  static constexpr int kRowsPerInstr = 64 / kChunks;  // rows one wavefront load covers
  static constexpr int kABytes = BM * BK * 2;
  static constexpr int kBBytes = BN * BK * 2;
  static constexpr int kStageBytes = kABytes + kBBytes;
  static_assert(WM % 32 == 0 && WN % 32 == 0 && BK % 16 == 0, "wavefront tile must be MFMA-sized");
  static_assert((BM * kChunks) % (64 * kWaves) == 0 && (BN * kChunks) % (64 * kWaves) == 0,
                "tile rows must split evenly over the wavefronts' 1 KiB loads");

  // Physical 16-byte chunk of logical chunk `c` in tile row `row`.  Sixteen consecutive rows
  // reading the same logical chunk land in sixteen different 16-byte bank groups.
  __host__ __device__ static constexpr int swizzle(int row, int c) {
    return c ^ ((row / kRowsPer256B) % kChunks);
  }
};

// XCD-aware tile order.  Workgroup ids are dealt round-robin to the 8 XCDs, so ids that are
// equal mod 8 share an L2.  Give each XCD a run of consecutive positions in a grouped
// (4 tile-rows at a time) walk of the output so its workgroups re-use A and B panels.
TFK_DEVICE void tile_of_block(int bid, int nblocks, int tiles_m, int tiles_n, int& tm, int& tn) {
  int pid = bid;
  if ((nblocks & 7) == 0) pid = (bid & 7) * (nblocks >> 3) + (bid >> 3);
  constexpr int kGroup = 4;
  const int group_size = kGroup * tiles_n;
  const int gid = pid / group_size;
  const int first_m = gid * kGroup;
  const int rows = min(tiles_m - first_m, kGroup);
  const int in_group = pid - gid * group_size;
  tm = first_m + in_group % rows;
  tn = in_group / rows;
}

template <typename OutT>
TFK_DEVICE void store_out(OutT* p, float v) {
  if constexpr (sizeof(OutT) == 2) {
    *p = (OutT)v;
  } else {
    *p = v;
  }
}

// MFMAs by operand type (half_t or bf16_t) for the kernels that issue them through builtins
template <typename InT> using in8_t = InT __attribute__((ext_vector_type(8)));
template <typename InT>
TFK_DEVICE float4_t mfma16_t(in8_t<InT> a, in8_t<InT> b, float4_t c) {
  if constexpr (std::is_same_v<InT, bf16_t>) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  else return mfma_16x16x32(a, b, c);
}
template <typename InT>
TFK_DEVICE float16_t mfma32_t(in8_t<InT> a, in8_t<InT> b, float16_t c) {
  if constexpr (std::is_same_v<InT, bf16_t>) return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  else return mfma_32x32x16(a, b, c);
}

// ------------------------------------------------------------------------------------------
// Fast path: M % BM == 0, N % BN == 0, K % 32 == 0.  Direct global->LDS ring, 16x16x32 MFMA.
// ------------------------------------------------------------------------------------------
// Tile shape of the fast path.  BK is fixed at 32: one v_mfma_f32_16x16x32_f16 consumes a whole
// k-tile, a 16-row operand fragment is one contiguous 1 KiB of LDS, and a tile is 32 KiB at
// 256 x 256 so that four of them are in the ring.  (Under realistic operand data the MFMA
// rate on MI355X is set by power, and the 16x16x32 shape sustains ~17% more flop/s than
// 32x32x16 for the same 128 x 128 wavefront tile.)
template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, int STAGES_>
struct DirectShape {
  static constexpr int BM = BM_, BN = BN_, BK = BK_;
  static constexpr int kKSteps = BK / 32;                     // MFMA k-steps per tile
  static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr int kStages = STAGES_;
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * kWaveSize;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // tile of one wavefront
  static constexpr int TM = WM / 16, TN = WN / 16;            // 16x16 MFMA tiles per wavefront
  static constexpr int kChunks = BK / 8;                      // 16-byte chunks per tile row
  static constexpr int kRowsPer256B = 16 / kChunks;           // rows sharing one pass over the banks
  static constexpr int kRowsPerInstr = 64 / kChunks;          // rows one wavefront load covers
  static constexpr int kABytes = BM * BK * 2;
  static constexpr int kBBytes = BN * BK * 2;
  static constexpr int kStageBytes = kABytes + kBBytes;
  static constexpr int kAInstr = BM * kChunks / 64 / kWaves;  // 1 KiB loads per wavefront
  static constexpr int kBInstr = BN * kChunks / 64 / kWaves;
  static_assert(WM % 16 == 0 && WN % 16 == 0, "wavefront tile must be MFMA-sized");
  static_assert((BM * kChunks) % (64 * kWaves) == 0 && (BN * kChunks) % (64 * kWaves) == 0,
                "tile rows must split evenly over the wavefronts' 1 KiB loads");
  // XOR swizzle of the 16-byte chunk index against LDS bank conflicts of the fragment reads
  // (lane l reads row l % 16 of a 16-row block, logical chunk l / 16 of the k-step).
  // ds_read_b128 serves a wavefront in four passes of 16 lanes, and the passes are NOT runs of
  // consecutive lanes: measured on gfx950 they are {0-3, 12-15, 20-23, 24-27},
  // {4-7, 8-11, 16-19, 28-31} and the same two sets + 32.  Each pass must touch 16 different
  // 16-byte bank groups (address mod 256).
  //   128-byte rows and wider: chunk ^ (row / kRowsPer256B) % kChunks does that.
  //   64-byte rows: a row supplies address bits 6-7 itself (row % 4), the chunk the bits 4-5;
  //   a pass mixes row quads t = (row / 4) % 4 of two different chunk indices, {0, 3} of one
  //   with {1, 2} of the next, so the XOR mask per row quad has to be 0, 2, 3, 1 (a plain
  //   chunk ^ t leaves every pass with a two-way conflict).
  __host__ __device__ static constexpr int swizzle(int row, int c) {
    if constexpr (kChunks == 4) return c ^ ((0x78 >> (2 * ((row / 4) % 4))) & 3);
    return c ^ ((row / kRowsPer256B) % kChunks);
  }
};

template <typename S, typename OutT, typename InT>
__global__ __launch_bounds__(S::kThreads) void gemm_direct_lds_kernel(
    const InT* __restrict__ A, const InT* __restrict__ B, OutT* __restrict__ C, int M,
    int N, int K, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int tile_m, tile_n;
  tile_of_block(blockIdx.x, gridDim.x, tiles_m, tiles_n, tile_m, tile_n);
  const int m0 = tile_m * S::BM, n0 = tile_n * S::BN;
  const int wm = wave / S::WAVES_N, wn = wave % S::WAVES_N;

  // --- global -> LDS plan -----------------------------------------------------------------
  // Wavefront instruction i of a tile covers 16 rows; lane l fills physical chunk l % 4 of
  // row 16*i + l / 4 and fetches the logical chunk that the swizzle maps there.
  constexpr int kAInstr = S::kAInstr, kBInstr = S::kBInstr;
  const int ld_row = lane / S::kChunks;
  const int ld_pc = lane % S::kChunks;
  const char* a_tile = reinterpret_cast<const char*>(A + (size_t)m0 * K);
  const char* b_tile = reinterpret_cast<const char*>(B + (size_t)n0 * K);
  unsigned a_goff[kAInstr], b_goff[kBInstr];
#pragma unroll
  for (int t = 0; t < kAInstr; ++t) {
    const int row = (wave + S::kWaves * t) * S::kRowsPerInstr + ld_row;
    a_goff[t] = (unsigned)row * (unsigned)K * 2u + (unsigned)S::swizzle(row, ld_pc) * 16u;
  }
#pragma unroll
  for (int t = 0; t < kBInstr; ++t) {
    const int row = (wave + S::kWaves * t) * S::kRowsPerInstr + ld_row;
    b_goff[t] = (unsigned)row * (unsigned)K * 2u + (unsigned)S::swizzle(row, ld_pc) * 16u;
  }

  // --- LDS -> register plan ---------------------------------------------------------------
  // Fragment i of A at k-step ks: lane l reads row wm*WM + 16*i + l%16, logical chunk
  // 4*ks + l/16 (8 halves of k).
  const int fr = lane & 15, fg = lane >> 4;
  const int ra = wm * S::WM + fr, rb = wn * S::WN + fr;
  unsigned a_rd[S::kKSteps], b_rd[S::kKSteps];
#pragma unroll
  for (int ks = 0; ks < S::kKSteps; ++ks) {
    a_rd[ks] = ra * S::BK * 2 + S::swizzle(ra, 4 * ks + fg) * 16;
    b_rd[ks] = rb * S::BK * 2 + S::swizzle(rb, 4 * ks + fg) * 16;
  }

  // acc[i][j][r] = C[m0 + wm*WM + 16*i + l%16][n0 + wn*WN + 16*j + 4*(l/16) + r]: the MFMA is
  // issued with the B fragment as its row operand, so a lane owns 4 consecutive columns of
  // one row of C and stores them with one 8- or 16-byte instruction.
  float4_t acc[S::TM][S::TN];
#pragma unroll
  for (int i = 0; i < S::TM; ++i)
#pragma unroll
    for (int j = 0; j < S::TN; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

  // --- main loop --------------------------------------------------------------------------
  // kStages LDS stages, two sets of fragment registers, and an explicit issue schedule.
  // A loaded MI355X needs the better part of a microsecond from issuing a tile's global->LDS
  // loads to having it in LDS - about the MFMA time of a k-tile - so tile kt+kStages-1 is
  // requested while tile kt is multiplied.  A k-tile is TM "slots" of TN MFMAs.  Per slot the
  // wavefront also issues its share of the 1 KiB global->LDS loads of the far tile and the
  // LDS reads that fetch one A and one B fragment of the NEXT tile, so neither the LDS pipe
  // nor the texture-address path ever sees a burst (a burst of loads blocks the wavefront's
  // MFMA issue while the address FIFO drains).  One workgroup barrier per k-tile, at its
  // start: by then tile kt+1 has landed (s_waitcnt vmcnt leaves only the younger tiles'
  // loads outstanding) and every wavefront has read all of tile kt into registers, so stage
  // kt is free for the next iteration's loads.
  constexpr int kLoadsPerTile = kAInstr + kBInstr;
  constexpr int NS = S::kStages;
  constexpr int KS = S::kKSteps;
  constexpr int kSlots = KS * S::TM;
  constexpr int kBarrierSlot = (KS - 1) * S::TM;  // in front of the tile's last k-step
  static_assert(S::TN <= S::TM && (NS >= 3 || (NS == 2 && KS == 2)),
                "issue schedule: TN <= TM; >= 3 stages, or 2 stages of 2 k-steps");
  // NS >= 3: every slot of iteration kt requests a piece of tile kt+NS-1 (stage of tile kt-1,
  // free since the previous barrier).  NS == 2: the slots in front of the barrier request the
  // second half of tile kt+1, the slots behind it the first half of tile kt+2 (into the stage
  // this barrier frees).
  auto first_load = [](int slot) constexpr {
    if (NS >= 3) return slot * kLoadsPerTile / kSlots;
    return slot < kBarrierSlot ? kLoadsPerTile / 2 + slot * (kLoadsPerTile / 2) / kBarrierSlot
                               : (slot - kBarrierSlot) * (kLoadsPerTile / 2) / (kSlots - kBarrierSlot);
  };
  auto end_load = [&](int slot) constexpr {
    if (NS >= 3) return (slot + 1) * kLoadsPerTile / kSlots;
    return slot < kBarrierSlot ? kLoadsPerTile / 2 + (slot + 1) * (kLoadsPerTile / 2) / kBarrierSlot
                               : (slot + 1 - kBarrierSlot) * (kLoadsPerTile / 2) / (kSlots - kBarrierSlot);
  };
  // loads that may still be in flight when tile kt+1 is needed
  constexpr int kInFlightAtBarrier =
      NS >= 3 ? (NS - 3) * kLoadsPerTile + kBarrierSlot * kLoadsPerTile / kSlots : 0;
  const int num_k_tiles = K / S::BK;
  in8_t<InT> af[2][S::TM], bf[2][S::TN];

  auto issue_load = [&](int stage, int k0, int n) __attribute__((always_inline)) {
    char* sa = smem + stage * S::kStageBytes;
    if (n < kAInstr) {
      load_global_to_lds_16B(a_tile + (size_t)k0 * 2 + a_goff[n], sa + (wave + S::kWaves * n) * 1024);
    } else {
      const int t = n - kAInstr;
      load_global_to_lds_16B(b_tile + (size_t)k0 * 2 + b_goff[t],
                             sa + S::kABytes + (wave + S::kWaves * t) * 1024);
    }
  };
  // Slot i of a k-step fetches its share of the NEXT k-step's fragments.  Every slot of that
  // next step multiplies ALL B fragments with one A fragment, so B goes first (slots 0 ..
  // TM/2-1, two fragments each) and the A fragments follow in the order they are used: when
  // the next step starts, everything its first slots touch was requested at least TM/2 slots
  // earlier and no MFMA ever waits on a fragment read issued just in front of it.
  auto load_frags = [&](int stage, int ks, int buf, int i) __attribute__((always_inline)) {
    const char* sa = smem + stage * S::kStageBytes;
    const char* sb = sa + S::kABytes;
    constexpr int kTotal = S::TM + S::TN;               // fragments per k-step
    constexpr int kPerSlot = (kTotal + S::TM - 1) / S::TM;
#pragma unroll
    for (int f = i * kPerSlot; f < (i + 1) * kPerSlot && f < kTotal; ++f) {
      if (f < S::TN) bf[buf][f] = *reinterpret_cast<const in8_t<InT>*>(sb + b_rd[ks] + f * 16 * S::BK * 2);
      else af[buf][f - S::TN] = *reinterpret_cast<const in8_t<InT>*>(sa + a_rd[ks] + (f - S::TN) * 16 * S::BK * 2);
    }
  };
  // Past the end the schedule keeps running on a clamped tile index: the extra loads land in
  // a stage nobody reads again, which is cheaper than a branch per slot.
  auto tile_k = [&](int t) __attribute__((always_inline)) { return min(t, num_k_tiles - 1) * S::BK; };

  if constexpr (NS >= 3) {
#pragma unroll
    for (int t = 0; t < NS - 1; ++t)
#pragma unroll
      for (int n = 0; n < kLoadsPerTile; ++n) issue_load(t, tile_k(t), n);
    barrier_keep_vmem<(NS - 2) * kLoadsPerTile>();
  } else {
#pragma unroll
    for (int n = 0; n < kLoadsPerTile; ++n) issue_load(0, tile_k(0), n);
#pragma unroll
    for (int n = 0; n < kLoadsPerTile / 2; ++n) issue_load(1, tile_k(1), n);
    barrier_keep_vmem<kLoadsPerTile / 2>();
  }
#pragma unroll
  for (int i = 0; i < S::TM; ++i) load_frags(0, 0, 0, i);

  // (No branch may sit inside this loop: at every control-flow join the compiler drains the
  // LDS-direct loads with vmcnt(0), which serialises the whole pipeline.)
  auto iteration = [&](int kt, auto parity_c) __attribute__((always_inline)) {
    // fragment set used by k-step ks of this tile (steps alternate sets across tiles)
    constexpr int base = (KS % 2) ? decltype(parity_c)::value : 0;
    const int stage = kt % NS;
    const int stage_next = (kt + 1) % NS;
#pragma unroll
    for (int slot = 0; slot < kSlots; ++slot) {
      const int ks = slot / S::TM, i = slot % S::TM;
      const int cur = base ^ (ks & 1);
      __builtin_amdgcn_sched_barrier(0);
      if (slot == kBarrierSlot) barrier_keep_vmem<kInFlightAtBarrier>();
#pragma unroll
      for (int n = first_load(slot); n < end_load(slot); ++n) {
        if constexpr (NS >= 3) {
          issue_load((kt + NS - 1) % NS, tile_k(kt + NS - 1), n);
        } else {
          if (slot < kBarrierSlot) issue_load(stage_next, tile_k(kt + 1), n);
          else issue_load(stage, tile_k(kt + 2), n);
        }
      }
      if (ks + 1 < KS) load_frags(stage, ks + 1, cur ^ 1, i);
      else load_frags(stage_next, 0, cur ^ 1, i);
#pragma unroll
      for (int j = 0; j < S::TN; ++j) acc[i][j] = mfma16_t<InT>(bf[cur][j], af[cur][i], acc[i][j]);
    }
  };
  int kt = 0;
  for (; kt + 1 < num_k_tiles; kt += 2) {
    iteration(kt, std::integral_constant<int, 0>{});
    iteration(kt + 1, std::integral_constant<int, 1>{});
  }
  if (kt < num_k_tiles) iteration(kt, std::integral_constant<int, 0>{});
  __builtin_amdgcn_sched_barrier(0);
  wait_vmem_all();  // the clamped tail loads must not outlive the workgroup's LDS

  // --- epilogue ---------------------------------------------------------------------------
  const int c_row0 = m0 + wm * S::WM + fr;
  const int c_col0 = n0 + wn * S::WN + 4 * fg;
#pragma unroll
  for (int i = 0; i < S::TM; ++i)
#pragma unroll
    for (int j = 0; j < S::TN; ++j) {
      OutT* dst = C + (size_t)(c_row0 + 16 * i) * N + c_col0 + 16 * j;
      if constexpr (sizeof(OutT) == 2) {
        typedef OutT out4_t __attribute__((ext_vector_type(4)));
        out4_t v;
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = (OutT)acc[i][j][r];
        *reinterpret_cast<out4_t*>(dst) = v;
      } else {
        *reinterpret_cast<float4_t*>(dst) = acc[i][j];
      }
    }
}

// ------------------------------------------------------------------------------------------
// 256 x 256 x 64 path: same 2 x 2 wavefronts of 128 x 128, but k-tiles of 64 so that every
// global->LDS instruction fetches whole 128-byte lines (8 rows x 128 bytes).  The vector L1
// moves full lines, so the 64-byte row segments of a 32-deep tile spend half of the L2->L1
// bandwidth on bytes that are dropped and requested again one k-tile later.
//
// A 64-deep tile is 64 KiB and only 160 KiB of LDS exist, so the ring is kept in UNITS of one
// operand of one tile (32 KiB, five of them): unit u lives in ring slot u % 5, A of tile t is
// unit 2t and B of tile t unit 2t+1.  Iteration t:
//   k-step 0: multiplies fragments (t, 0), reads fragments (t, 1), requests A of tile t+2 into
//             the slot B of tile t-1 left;
//   barrier:  tile t is read out (both its units are free) and tile t+1 has landed
//             (vmcnt leaves only the 8 requests of k-step 0 outstanding);
//   k-step 1: multiplies (t, 1), reads fragments (t+1, 0), requests B of tile t+2 into the
//             slot A of tile t left.
// Every request has at least 8 MFMA slots (1024 MFMA cycles) to land.
// ------------------------------------------------------------------------------------------
//
// The same kernel serves 128 x 128 tiles (2 x 2 wavefronts of 64 x 64, units of 16 KiB) for
// grids that 256 x 256 tiles would leave most CUs idle on.  Its k-steps are four times
// shorter, so requests run kAhead = 4 tiles ahead (a ring of 2 * kAhead + 1 = 9 units).
template <int BM_, int WAVES_N_, int AHEAD_>
struct Ring64Shape {
  static constexpr int BM = BM_, BN = BM_, BK = 64;
  static constexpr int WAVES_M = 2, WAVES_N = WAVES_N_;
  static constexpr int kWaves = WAVES_M * WAVES_N, kThreads = kWaves * kWaveSize;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 16, TN = WN / 16;          // 16x16 MFMA tiles per wavefront
  static constexpr int kRowBytes = BK * 2;                  // 128
  static constexpr int kUnitBytes = BM * kRowBytes;         // one operand of one tile
  static constexpr int kAhead = AHEAD_;                     // tiles between a request and its use
  static constexpr int kUnits = 2 * kAhead + 1;
  static constexpr int kLoads = BM / 8 / kWaves;            // 1 KiB requests per wavefront and unit
  // slot schedule of a k-step (TM slots of TN MFMAs): the TM + TN fragment reads of the next
  // k-step are dealt to the first kReadSlots slots; the scalar bookkeeping runs in the gaps
  // without a read from slot kPrepSlot on
  static constexpr int kReads = TM + TN;
  static constexpr int kReadSlots = TM == 8 ? 6 : TM - 1;
  static constexpr int kPrepSlot = TM == 8 ? 6 : 0;
  static constexpr int reads_first(int i) { return i < kReadSlots ? (i * kReads) / kReadSlots : kReads; }
  static constexpr int reads_in(int i) { return reads_first(i + 1) - reads_first(i); }
  // read number d of a slot follows MFMA (d * TN) / n of that slot (gap j = that + 1)
  static constexpr bool gap_has_read(int i, int j) {
    const int n = reads_in(i);
    for (int d = 0; d < n; ++d)
      if (j == (d * TN) / n + 1) return true;
    return false;
  }
  // which bookkeeping piece runs in gap j of slot i (-1: none); a table, so that the unrolled
  // slots index it with constants
  struct PrepTable {
    int piece[TM * TN];
  };
  static constexpr PrepTable make_prep_table() {
    PrepTable t{};
    int rank = 0;
    for (int i = 0; i < TM; ++i)
      for (int j = 0; j < TN; ++j) t.piece[i * TN + j] = (i < kPrepSlot || gap_has_read(i, j)) ? -1 : rank++;
    return t;
  }
  static constexpr PrepTable kPrep = make_prep_table();
  static constexpr int free_gaps() { return kPrep.piece[TM * TN - 1] + 1; }
  static constexpr bool reads_fit() {
    for (int i = 0; i < TM; ++i) {
      if (reads_in(i) > TN - 1) return false;
      for (int d = 1; d < reads_in(i); ++d)   // two reads never share a gap
        if ((d * TN) / reads_in(i) == ((d - 1) * TN) / reads_in(i)) return false;
    }
    return true;
  }
  static_assert((TM == 8 || TM == 4) && (TN == 8 || TN == 4) && TM % kLoads == 0 && kLoads % 4 == 0,
                "slot schedule: a request every TM / kLoads slots, M0 shared by four requests");
  static_assert(reads_fit() && free_gaps() >= 7,
                "slot schedule: every read and bookkeeping piece needs its own gap");
  static_assert((2 * kAhead - 3) * kLoads < 64, "vmcnt is a 6-bit counter");
  // 128-byte rows: two rows per pass over the banks; chunk ^ (row / 2) % 8 keeps every
  // ds_read_b128 lane pass on 16 different bank groups
  __host__ __device__ static constexpr int swizzle(int row, int c) { return c ^ ((row / 2) % 8); }
};

// InT is half_t or bf16_t: the two differ in the MFMA mnemonic and in the conversion of the
// result, everything else moves 16-bit elements without looking at them.
template <typename S, typename InT, typename OutT>
__global__ __launch_bounds__(S::kThreads) void gemm_ring64_kernel(
    const InT* __restrict__ A, const InT* __restrict__ B, OutT* __restrict__ C, int M,
    int N, int K, int tiles_m, int tiles_n) {
  constexpr bool kBf16 = std::is_same_v<InT, bf16_t>;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int tile_m, tile_n;
  tile_of_block(blockIdx.x, gridDim.x, tiles_m, tiles_n, tile_m, tile_n);
  const int m0 = tile_m * S::BM, n0 = tile_n * S::BN;
  const int wm = wave / S::WAVES_N, wn = wave % S::WAVES_N;

  // global -> LDS plan: request n of a wavefront covers rows (wave * kLoads + n) * 8 .. +7 of a
  // unit (consecutive 1 KiB blocks of LDS, so four requests share one M0 base and differ in the
  // instruction's immediate offset); lane l fills physical chunk l % 8 of row l / 8 and fetches the logical chunk the
  // swizzle maps there.  A and B share the per-lane offsets (same row stride K); the address
  // is a scalar base (tile origin + k offset) plus this 32-bit per-lane offset, so a request
  // needs no vector arithmetic.
  const int ld_row = wave * 8 * S::kLoads + lane / 8, ld_c = lane % 8;
  const char* a_tile = reinterpret_cast<const char*>(A + (size_t)m0 * K);
  const char* b_tile = reinterpret_cast<const char*>(B + (size_t)n0 * K);
  unsigned g_off[S::kLoads];
#pragma unroll
  for (int n = 0; n < S::kLoads; ++n)
    g_off[n] = (unsigned)(ld_row + 8 * n) * (unsigned)K * 2u + (unsigned)S::swizzle(ld_row + 8 * n, ld_c) * 16u -
               1024u * (n % 4);   // the instruction's immediate offset (added to both addresses) gives it back
  // LDS -> fragment plan: fragment i of k-step ks: row 16*i + l%16 of the wavefront's rows,
  // logical chunk 4*ks + l/16
  const int fr = lane & 15, fg = lane >> 4;
  unsigned a_rd[2], b_rd[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    a_rd[ks] = (wm * S::WM + fr) * S::kRowBytes + S::swizzle(fr, 4 * ks + fg) * 16;
    b_rd[ks] = (wn * S::WN + fr) * S::kRowBytes + S::swizzle(fr, 4 * ks + fg) * 16;
  }

  float4_t acc[S::TM][S::TN];
#pragma unroll
  for (int i = 0; i < S::TM; ++i)
#pragma unroll
    for (int j = 0; j < S::TN; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

  const int num_k_tiles = K / S::BK;
  const unsigned smem_addr = lds_address(smem);
  // Slot i of a k-step multiplies A fragment i with all B fragments; both operands have two
  // register sets (this k-step's and the next one's).
  half8_t afx[2][S::TM], bf[2][S::TN];
  // The requests are issued from inline assembly: the compiler then keeps exact counts for the
  // fragment reads (a direct-to-LDS load it knows about makes every LDS wait a full drain),
  // and the vector-memory waits are placed by hand below.
  // src: tile origin + k offset (scalar); lds_unit: LDS byte address of this wavefront's first
  // 1 KiB block in the destination unit.
  // M0 - the LDS destination of requests n .. n+3 (n % 4 == 0), which differ in the immediate
  // offset - is an INPUT of every request statement: the compiler writes it (once per group of
  // four: the statements do not change it) and cannot use the register for anything else between
  // that write and a request.  The s_nop is the wait state an M0 write needs in front of an
  // LDS-direct load; next to a request at the head of a slot it costs no issue time.
  auto request = [&](const char* src, unsigned lds_unit, int n) __attribute__((always_inline)) {
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%2"
                 :
                 : "v"(g_off[n]), "s"(src), "n"(1024 * (n % 4)), "{m0}"(lds_unit + (n - n % 4) * 1024)
                 : "memory");
  };
  auto k_src = [&](const char* tile, int t) __attribute__((always_inline)) {
    return tile + (size_t)min(t, num_k_tiles - 1) * S::BK * 2;   // clamped past the end
  };
  const unsigned lds_wave = smem_addr + wave * S::kLoads * 1024;
  // Slot with the MFMAs issued from inline assembly, accumulators pinned to AGPRs, and the
  // slot's fragment reads placed by hand between them.  (With compiler-issued MFMAs the
  // register allocator, at exactly 256 live accumulators, shuffles accumulators through VGPRs
  // whenever the schedule changes slightly.)
  auto lds_read_b128 = [](unsigned addr) __attribute__((always_inline)) {
    return *(__attribute__((address_space(3))) const half8_t*)(size_t)addr;
  };
  // rd_a / rd_b: this lane's LDS byte address of fragment 0 of the next k-step's A / B operand
  // (unit base + row + swizzled chunk); fragment f is f * 2 KiB further, in the offset field.
  auto slot_pinned = [&](int buf, int i, unsigned rd_a, unsigned rd_b, auto&& between) __attribute__((always_inline)) {
    // The TN + TM fragment reads of the next k-step, B fragments first, are dealt to the first
    // kReadSlots slots; the last slot(s) read nothing, so the drain in front of the barrier
    // (and the one at the head of the next k-step) finds the reads already returned.
    const int first = S::reads_first(i);
    const int n_reads = S::reads_in(i);
    int done = 0;
#pragma unroll
    for (int j = 0; j < S::TN; ++j) {
      if constexpr (kBf16)
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(bf[buf][j]), "v"(afx[buf][i]));
      else
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(bf[buf][j]), "v"(afx[buf][i]));
      // after MFMA j: issue the next read if j is its position (reads spread evenly over the slot)
      if (done < n_reads && j == (done * S::TN) / n_reads + 1) {
        const int q = first + done;
        __builtin_amdgcn_sched_barrier(0);
        if (q < S::TN) bf[buf ^ 1][q] = lds_read_b128(rd_b + q * 16 * S::kRowBytes);
        else afx[buf ^ 1][q - S::TN] = lds_read_b128(rd_a + (q - S::TN) * 16 * S::kRowBytes);
        __builtin_amdgcn_sched_barrier(0);
        ++done;
      } else {
        between(j);   // a piece of scalar bookkeeping, if this gap has one
      }
    }
  };
  // Workgroup barrier in the middle of tile t: tile t+1 must have landed, the requests of
  // tiles t+2 .. t+kAhead-1 and of this tile's k-step 0 stay in flight.  The LDS wait and the
  // barrier are builtins so that the compiler knows every earlier fragment read has returned.
  constexpr int kInFlight = (2 * S::kAhead - 3) * S::kLoads;
  auto ring_barrier = [&]() __attribute__((always_inline)) {
    // one s_waitcnt: vmcnt(kInFlight) lgkmcnt(0); a builtin, so the compiler knows the LDS part
    __builtin_amdgcn_s_waitcnt((kInFlight & 15) | 0x70 | ((kInFlight >> 4) << 14));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  constexpr int kSlotsPerLoad = S::TM / S::kLoads;   // a request every so many slots

  // prologue: tiles 0 .. kAhead-1 into the first 2 * kAhead units; fragments (0, 0) once
  // tile 0 is there
#pragma unroll
  for (int u = 0; u < 2 * S::kAhead; ++u)
#pragma unroll
    for (int n = 0; n < S::kLoads; ++n) {
      request(k_src(u % 2 ? b_tile : a_tile, u / 2), lds_wave + u * S::kUnitBytes, n);
    }
  wait_vmem<2 * (S::kAhead - 1) * S::kLoads>();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
#pragma unroll
  for (int f = 0; f < S::TN; ++f)
    bf[0][f] = *reinterpret_cast<const half8_t*>(smem + S::kUnitBytes + b_rd[0] + f * 16 * S::kRowBytes);
#pragma unroll
  for (int i = 0; i < S::TM; ++i)
    afx[0][i] = *reinterpret_cast<const half8_t*>(smem + a_rd[0] + i * 16 * S::kRowBytes);
  // drained here, visibly to the compiler, so that the waits it places at the head of the loop
  // only have to cover the loop's own reads
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
  __builtin_amdgcn_sched_barrier(0);

  // Ring bookkeeping, in bytes: oa = LDS offset of the unit holding A of tile t; B of tile t is
  // one unit further, A of t+1 two, ... (mod kUnits units).  A wavefront alone on its SIMD issues one
  // instruction every 4 cycles, so a 16-cycle MFMA hides at most three other instructions:
  // everything an iteration needs (fragment read bases, request destinations and sources) is
  // therefore computed during the previous k-step in pieces of at most three instructions,
  // each pinned into its own gap between two MFMAs of the slots that carry no fragment reads.
  constexpr unsigned kRingBytes = S::kUnits * S::kUnitBytes;
  auto ring = [](unsigned o) __attribute__((always_inline)) { return o >= kRingBytes ? o - kRingBytes : o; };
  const unsigned rdbase_a0 = smem_addr + a_rd[0], rdbase_a1 = smem_addr + a_rd[1];
  const unsigned rdbase_b0 = smem_addr + b_rd[0], rdbase_b1 = smem_addr + b_rd[1];
  const int last_tile = num_k_tiles - 1;
  unsigned oa = 0;                                             // A of tile t
  unsigned oa1 = 2 * S::kUnitBytes, ob1 = 3 * S::kUnitBytes;   // A, B of tile t+1
  unsigned rd_a1 = rdbase_a1, rd_b1 = rdbase_b1 + S::kUnitBytes;   // reads of (t, k-step 1)
  unsigned req_a = lds_wave + 2 * S::kAhead * S::kUnitBytes;       // A of t+kAhead
  const char* src_a = k_src(a_tile, S::kAhead);
  unsigned rd_a0 = 0, rd_b0 = 0, req_b = 0;                        // set during k-step 0
  const char* src_b = b_tile;
  int kt = 0;
#define TFK_PIN_S(x) asm volatile("" : "+s"(x))
#define TFK_PIN_V(x) asm volatile("" : "+v"(x))
  // pieces run in the read-free gaps from slot kPrepSlot on of k-step 0 / k-step 1
  auto prep0 = [&](int step, int t) __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    switch (step) {
      case 0: TFK_PIN_S(oa); oa1 = ring(oa + 2 * S::kUnitBytes); TFK_PIN_S(oa1); break;
      case 1: ob1 = ring(oa1 + S::kUnitBytes); TFK_PIN_S(ob1); break;
      case 2: rd_a0 = rdbase_a0 + oa1; TFK_PIN_V(rd_a0); break;
      case 3: rd_b0 = rdbase_b0 + ob1; TFK_PIN_V(rd_b0); break;
      case 4: req_b = lds_wave + oa; TFK_PIN_S(req_b); break;
      case 5: kt = t; TFK_PIN_S(kt); kt = min(kt + S::kAhead, last_tile); TFK_PIN_S(kt); break;
      case 6: src_b = b_tile + (size_t)(unsigned)(kt * (S::BK * 2)); TFK_PIN_S(src_b); break;
      default: break;
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto prep1 = [&](int step, int t) __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    switch (step) {
      case 0: oa = oa1; TFK_PIN_S(oa); rd_a1 = rdbase_a1 + oa; TFK_PIN_V(rd_a1); break;
      case 1: rd_b1 = rdbase_b1 + ob1; TFK_PIN_V(rd_b1); break;
      case 2: req_a = ring(oa + 2 * S::kAhead * S::kUnitBytes); TFK_PIN_S(req_a); break;
      case 3: req_a += lds_wave; TFK_PIN_S(req_a); break;
      case 4: kt = t; TFK_PIN_S(kt); kt = min(kt + S::kAhead + 1, last_tile); TFK_PIN_S(kt); break;
      case 5: src_a = a_tile + (size_t)(unsigned)(kt * (S::BK * 2)); TFK_PIN_S(src_a); break;
      default: break;
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // request n of a k-step goes at the head of slot n * kSlotsPerLoad
  for (int t = 0; t < num_k_tiles; ++t) {
#pragma unroll
    for (int i = 0; i < S::TM; ++i) {
      __builtin_amdgcn_sched_barrier(0);
      if (i % kSlotsPerLoad == 0) request(src_a, req_a, i / kSlotsPerLoad);
      slot_pinned(0, i, rd_a1, rd_b1, [&](int j) __attribute__((always_inline)) {
        prep0(S::kPrep.piece[i * S::TN + j], t);
      });
    }
    __builtin_amdgcn_sched_barrier(0);
    ring_barrier();
#pragma unroll
    for (int i = 0; i < S::TM; ++i) {
      __builtin_amdgcn_sched_barrier(0);
      if (i % kSlotsPerLoad == 0) request(src_b, req_b, i / kSlotsPerLoad);
      slot_pinned(1, i, rd_a0, rd_b0, [&](int j) __attribute__((always_inline)) {
        prep1(S::kPrep.piece[i * S::TN + j], t);
      });
    }
    // The compiler does not know that the accumulators are written by MFMAs (they are issued
    // from assembly), so nothing would keep it from reading the youngest results right behind
    // the loop without the wait states the matrix pipe needs.  The delay therefore sits inside
    // the last iteration, in front of anything the register allocator may put on the exit
    // edge.  The iteration count is laundered through an empty asm so that the test is not
    // recognised as the exit condition and sunk out of the loop.
    int t_seen = t;
    asm volatile("" : "+s"(t_seen));
    if (t_seen + 1 == num_k_tiles) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  }
  __builtin_amdgcn_sched_barrier(0);
  wait_vmem_all();  // the clamped tail requests must not outlive the workgroup's LDS
  // --- epilogue -----------------------------------------------------------------------------
  // acc[i][j][r] = C[.. + 16*i + l%16][.. + 16*j + 4*(l/16) + r].  For fp16 output the data is
  // re-dealt so that a store instruction writes 16 rows x 64 contiguous bytes with FOUR
  // ADJACENT lanes per row: the address unit merges adjacent lanes into one 64-byte access,
  // whereas lanes 16 apart cost one access each (measured: 64 accesses per instruction and
  // 9 k cycles of epilogue per wavefront).  Step 1: the 16-lane groups g and g^1 trade halves
  // of a pair of tiles (v_permlane16_swap), after which group 0/2 holds columns 0-7 / 8-15 of
  // tile j and group 1/3 the same of tile j+1, 16 bytes per lane.  Step 2: ds_bpermute moves
  // the 16 bytes of (row r, segment s) to lane 4*r + s.
  const int c_row0 = m0 + wm * S::WM;
  if constexpr (sizeof(OutT) == 2) {
    const int st_row = lane >> 2, st_seg = lane & 3;
    // segment s of a row lives in group {0, 2, 1, 3}[s] after step 1
    const int src_lane = st_row + 16 * (((st_seg & 1) << 1) | (st_seg >> 1));
    OutT* c_lane = C + (size_t)(c_row0 + st_row) * N + n0 + wn * S::WN + 8 * st_seg;
#pragma unroll
    for (int i = 0; i < S::TM; ++i)
#pragma unroll
      for (int j = 0; j < S::TN; j += 2) {
        typedef InT h2_t __attribute__((ext_vector_type(2)));
        unsigned x[2], y[2];
#pragma unroll
        for (int d = 0; d < 2; ++d) {
          const h2_t hx = {(InT)acc[i][j][2 * d], (InT)acc[i][j][2 * d + 1]};
          const h2_t hy = {(InT)acc[i][j + 1][2 * d], (InT)acc[i][j + 1][2 * d + 1]};
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
        *reinterpret_cast<uint4_t*>(c_lane + (size_t)(16 * i) * N + 16 * j) = v;
      }
  } else {
    const int c_col0 = n0 + wn * S::WN + 4 * fg;
#pragma unroll
    for (int i = 0; i < S::TM; ++i)
#pragma unroll
      for (int j = 0; j < S::TN; ++j)
        *reinterpret_cast<float4_t*>(C + (size_t)(c_row0 + fr + 16 * i) * N + c_col0 + 16 * j) = acc[i][j];
  }
}

using RingBig = Ring64Shape<256, 2, 2>;   // 5 units of 32 KiB
using RingMid = Ring64Shape<128, 2, 4>;   // 9 units of 16 KiB: one workgroup per CU, requests 4 tiles ahead
using RingMid2 = Ring64Shape<128, 2, 2>;  // 5 units of 16 KiB: two workgroups per CU cover each other's stalls

template <typename S, typename OutT, typename InT = half_t>
int launch_ring64(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t st) {
  auto kern = gemm_ring64_kernel<S, InT, OutT>;
  constexpr int lds = S::kUnits * S::kUnitBytes;
  static_assert(lds <= kMaxLdsBytes, "ring does not fit in LDS");
  TFK_LDS_OPT_IN(kern, lds);
  const int tiles_m = M / S::BM, tiles_n = N / S::BN;
  hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(S::kThreads), lds, st,
                     static_cast<const InT*>(A), static_cast<const InT*>(B),
                     static_cast<OutT*>(C), M, N, K, tiles_m, tiles_n);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}

// ------------------------------------------------------------------------------------------
// General path: any M, N; K % 8 == 0.  Register-staged, bounds-checked, one LDS stage.
// ------------------------------------------------------------------------------------------
template <typename S, typename OutT, typename InT>
__global__ __launch_bounds__(S::kThreads) void gemm_guarded_kernel(
    const InT* __restrict__ A, const InT* __restrict__ B, OutT* __restrict__ C, int M,
    int N, int K) {
  __shared__ __attribute__((aligned(16))) char sa[S::kABytes];
  __shared__ __attribute__((aligned(16))) char sb[S::kBBytes];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int m0 = blockIdx.x * S::BM, n0 = blockIdx.y * S::BN;
  const int wm = wave / S::WAVES_N, wn = wave % S::WAVES_N;
  const int fr = lane & 31, fg = lane >> 5;

  float16_t acc[S::TM][S::TN];
#pragma unroll
  for (int i = 0; i < S::TM; ++i)
#pragma unroll
    for (int j = 0; j < S::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  for (int k0 = 0; k0 < K; k0 += S::BK) {
    for (int f = tid; f < S::BM * S::kChunks; f += S::kThreads) {
      const int row = f / S::kChunks, c = f % S::kChunks;
      const int gr = m0 + row, gk = k0 + c * 8;
      uint4_t v = {0u, 0u, 0u, 0u};
      if (gr < M && gk < K) v = *reinterpret_cast<const uint4_t*>(A + (size_t)gr * K + gk);
      *reinterpret_cast<uint4_t*>(sa + row * S::BK * 2 + S::swizzle(row, c) * 16) = v;
    }
    for (int f = tid; f < S::BN * S::kChunks; f += S::kThreads) {
      const int row = f / S::kChunks, c = f % S::kChunks;
      const int gr = n0 + row, gk = k0 + c * 8;
      uint4_t v = {0u, 0u, 0u, 0u};
      if (gr < N && gk < K) v = *reinterpret_cast<const uint4_t*>(B + (size_t)gr * K + gk);
      *reinterpret_cast<uint4_t*>(sb + row * S::BK * 2 + S::swizzle(row, c) * 16) = v;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < S::kKSteps; ++kk) {
      in8_t<InT> af[S::TM], bf[S::TN];
#pragma unroll
      for (int i = 0; i < S::TM; ++i) {
        const int row = wm * S::WM + i * 32 + fr;
        af[i] = *reinterpret_cast<const in8_t<InT>*>(sa + row * S::BK * 2 + S::swizzle(row, 2 * kk + fg) * 16);
      }
#pragma unroll
      for (int j = 0; j < S::TN; ++j) {
        const int row = wn * S::WN + j * 32 + fr;
        bf[j] = *reinterpret_cast<const in8_t<InT>*>(sb + row * S::BK * 2 + S::swizzle(row, 2 * kk + fg) * 16);
      }
#pragma unroll
      for (int i = 0; i < S::TM; ++i)
#pragma unroll
        for (int j = 0; j < S::TN; ++j) acc[i][j] = mfma32_t<InT>(af[i], bf[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < S::TM; ++i)
#pragma unroll
    for (int j = 0; j < S::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * S::WM + i * 32 + 8 * (r / 4) + 4 * fg + (r % 4);
        const int col = n0 + wn * S::WN + j * 32 + fr;
        if (row < M && col < N) store_out(C + (size_t)row * N + col, acc[i][j][r]);
      }
}

using ShapeBig = DirectShape<256, 256, 32, 2, 2, 4>;         // 4 x 32 KiB of LDS, 128x128 per wavefront
using ShapeMid = DirectShape<128, 128, 32, 2, 2, 4>;      // 4 x 16 KiB, 64x64 per wavefront
using ShapeSmall = GemmShape<64, 64, 32, 2, 2, 1>;    // bounds-checked path

template <typename S, typename OutT, typename InT>
int launch_direct(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t st) {
  auto kern = gemm_direct_lds_kernel<S, OutT, InT>;
  constexpr int lds = S::kStages * S::kStageBytes;
  static_assert(lds <= kMaxLdsBytes, "tile does not fit in LDS");
  TFK_LDS_OPT_IN(kern, lds);
  const int tiles_m = M / S::BM, tiles_n = N / S::BN;
  hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(S::kThreads), lds, st,
                     static_cast<const InT*>(A), static_cast<const InT*>(B),
                     static_cast<OutT*>(C), M, N, K, tiles_m, tiles_n);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}

template <typename S, typename OutT, typename InT>
int launch_guarded(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t st) {
  dim3 grid((M + S::BM - 1) / S::BM, (N + S::BN - 1) / S::BN);
  hipLaunchKernelGGL((gemm_guarded_kernel<S, OutT, InT>), grid, dim3(S::kThreads), 0, st,
                     static_cast<const InT*>(A), static_cast<const InT*>(B),
                     static_cast<OutT*>(C), M, N, K);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}

bool ring64_fits(int M, int N, int K) { return M % 128 == 0 && N % 128 == 0 && K % 64 == 0; }

template <typename OutT, typename InT>
int dispatch_ring64(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t st) {
  // 256 x 256 tiles do ~1.5x the work per cycle of 128 x 128 tiles (measured: 96 vs 146 us at
  // 4096^3) but come in quarters as many: compare the rounds of tiles the 256 CUs need, a round
  // of big tiles costing 4 units and a round of mid tiles 1.6.
  constexpr int64_t kCUs = 256;
  const bool big_fits = M % 256 == 0 && N % 256 == 0;
  const int64_t big_rounds = ((M / 256) * (N / 256) + kCUs - 1) / kCUs;
  const int64_t mid_rounds = ((M / 128) * (N / 128) + kCUs - 1) / kCUs;
  if (big_fits && 5 * big_rounds <= 2 * mid_rounds)
    return launch_ring64<RingBig, OutT, InT>(A, B, C, M, N, K, st);
  // more 128 x 128 tiles than CUs: the 80 KiB variant, so that two workgroups share a CU
  // (2048 x 4096 x 2048: 33.3 -> 30.5 us); otherwise the deep ring
  if ((M / 128) * (N / 128) > kCUs) return launch_ring64<RingMid2, OutT, InT>(A, B, C, M, N, K, st);
  return launch_ring64<RingMid, OutT, InT>(A, B, C, M, N, K, st);
}

template <typename OutT, typename InT>
int dispatch(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t st) {
  if (ring64_fits(M, N, K)) return dispatch_ring64<OutT, InT>(A, B, C, M, N, K, st);
  if (M % 256 == 0 && N % 256 == 0 && K % ShapeBig::BK == 0 && (int64_t)(M / 256) * (N / 256) >= 128)
    return launch_direct<ShapeBig, OutT, InT>(A, B, C, M, N, K, st);
  if (M % 128 == 0 && N % 128 == 0 && K % 32 == 0)
    return launch_direct<ShapeMid, OutT, InT>(A, B, C, M, N, K, st);
  return launch_guarded<ShapeSmall, OutT, InT>(A, B, C, M, N, K, st);
}

}  // namespace
}  // namespace tfk

namespace tfk {
namespace {
int check_gemm_args(const char* who, const void* A, const void* B, const void* C, int64_t M, int64_t N, int64_t K,
                    int tm, int tn, int tk, int num_stages, int pipeline_level) {
  TFK_REQUIRE(A && B && C, TF_ERR_INVALID_ARG, "%s: null pointer", who);
  TFK_REQUIRE(M > 0 && N > 0 && K > 0, TF_ERR_INVALID_ARG, "%s: M, N, K must be positive", who);
  TFK_REQUIRE(M < (1 << 30) && N < (1 << 30) && K < (1 << 22), TF_ERR_INVALID_ARG, "%s: dimension too large", who);
  TFK_REQUIRE(tm > 0 && tn > 0 && tk > 0, TF_ERR_INVALID_ARG, "%s: tile sizes must be positive", who);
  TFK_REQUIRE(M % tm == 0 && N % tn == 0 && K % tk == 0, TF_ERR_INVALID_ARG,
              "%s: tile [%d,%d,%d] does not divide problem [%lld,%lld,%lld]", who, tm, tn, tk,
              (long long)M, (long long)N, (long long)K);
  TFK_REQUIRE(num_stages >= 1 && num_stages <= 3, TF_ERR_INVALID_ARG, "%s: num_stages must be 1, 2 or 3", who);
  TFK_REQUIRE(pipeline_level >= 0 && pipeline_level <= 2, TF_ERR_INVALID_ARG,
              "%s: pipeline_level must be 0, 1 or 2", who);
  return TF_OK;
}
}  // namespace
}  // namespace tfk

extern "C" int tf_gemm_f16(const void* A, const void* B, void* C, int c_is_f16, int64_t M,
                           int64_t N, int64_t K, int tm, int tn, int tk, int num_stages,
                           int pipeline_level, void* stream) {
  using namespace tfk;
  if (int rc = check_gemm_args("tf_gemm_f16", A, B, C, M, N, K, tm, tn, tk, num_stages, pipeline_level)) return rc;
  TFK_REQUIRE(K % 8 == 0, TF_ERR_UNSUPPORTED, "tf_gemm_f16: K (%lld) must be a multiple of 8",
              (long long)K);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (c_is_f16) return dispatch<half_t, half_t>(A, B, C, (int)M, (int)N, (int)K, st);
  return dispatch<float, half_t>(A, B, C, (int)M, (int)N, (int)K, st);
}

extern "C" int tf_gemm(const void* A, const void* B, void* C, int dtype, int c_is_f32, int64_t M, int64_t N,
                       int64_t K, int tm, int tn, int tk, int num_stages, int pipeline_level, void* stream) {
  using namespace tfk;
  if (dtype == TF_DTYPE_F16)
    return tf_gemm_f16(A, B, C, c_is_f32 ? 0 : 1, M, N, K, tm, tn, tk, num_stages, pipeline_level, stream);
  TFK_REQUIRE(dtype == TF_DTYPE_BF16, TF_ERR_UNSUPPORTED, "tf_gemm: dtype must be TF_DTYPE_F16 or TF_DTYPE_BF16");
  if (int rc = check_gemm_args("tf_gemm", A, B, C, M, N, K, tm, tn, tk, num_stages, pipeline_level)) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // bf16: the same kernels with the bf16 MFMAs (every kernel of this file is a template of the
  // operand type)
  TFK_REQUIRE(K % 8 == 0, TF_ERR_UNSUPPORTED, "tf_gemm: K (%lld) must be a multiple of 8", (long long)K);
  if (c_is_f32) return dispatch<float, bf16_t>(A, B, C, (int)M, (int)N, (int)K, st);
  return dispatch<bf16_t, bf16_t>(A, B, C, (int)M, (int)N, (int)K, st);
}
