// GEMM macro kernel for gfx950: C[M,N] = A[M,K] * B[K,N] with A row-major and B handed over
// as its [N,K] buffer (column-major K x N), fp16 in, fp32 accumulate, fp32 or fp16 out.
//
// Counterpart of the reference's ke_gemm / ke_gemm_level1_pipeline / ke_gemm_level2_pipeline
// (include/kernels/gemm_device.cuh:110-419) and its host launcher (src/kernels/gemm.cu:63-142),
// re-designed for CDNA4:
//   * 64-lane wavefronts, v_mfma_f32_32x32x16_f16 base tiles, accumulators in the unified
//     512-entry register file (one wavefront per SIMD, 128x128 per wavefront at the big tile);
//   * both operands are K-contiguous, so an MFMA operand fragment is one 16-byte LDS read;
//   * tiles go global -> LDS without passing through VGPRs (global_load_lds_dwordx4) into a
//     double-buffered, XOR-swizzled LDS layout: a wavefront instruction always writes 1 KiB
//     of consecutive LDS, so the swizzle is applied on the global (source) side;
//   * workgroup -> tile map keeps the workgroups of one XCD (one L2) on a compact block of
//     output tiles.
#include "common.hpp"

namespace tfk {
namespace {

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_>
struct GemmShape {
  static constexpr int BM = BM_, BN = BN_, BK = BK_;
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

// ------------------------------------------------------------------------------------------
// Fast path: M % BM == 0, N % BN == 0, K % BK == 0.  Direct global->LDS, two LDS stages.
// ------------------------------------------------------------------------------------------
template <typename S, typename OutT>
__global__ __launch_bounds__(S::kThreads) void gemm_direct_lds_kernel(
    const half_t* __restrict__ A, const half_t* __restrict__ B, OutT* __restrict__ C, int M,
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
  // Wavefront instruction i of a tile covers rows [i*kRowsPerInstr, +kRowsPerInstr); lane l
  // fills physical chunk l % kChunks of row i*kRowsPerInstr + l / kChunks.
  constexpr int kAInstr = S::BM * S::kChunks / 64 / S::kWaves;  // per wavefront
  constexpr int kBInstr = S::BN * S::kChunks / 64 / S::kWaves;
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
  auto issue_tile_loads = [&](int stage, int k0) {
    char* sa = smem + stage * S::kStageBytes;
    char* sb = sa + S::kABytes;
    const char* ga = a_tile + (size_t)k0 * 2;
    const char* gb = b_tile + (size_t)k0 * 2;
#pragma unroll
    for (int t = 0; t < kAInstr; ++t)
      load_global_to_lds_16B(ga + a_goff[t], sa + (wave + S::kWaves * t) * 1024);
#pragma unroll
    for (int t = 0; t < kBInstr; ++t)
      load_global_to_lds_16B(gb + b_goff[t], sb + (wave + S::kWaves * t) * 1024);
  };

  // --- LDS -> register plan ---------------------------------------------------------------
  // Fragment (i, kk) of A: lane l reads row wm*WM + 32*i + l%32, logical chunk 2*kk + l/32.
  const int fr = lane & 31, fg = lane >> 5;
  unsigned a_rd[S::kKSteps], b_rd[S::kKSteps];
#pragma unroll
  for (int kk = 0; kk < S::kKSteps; ++kk) {
    const int ra = wm * S::WM + fr, rb = wn * S::WN + fr;
    a_rd[kk] = ra * S::BK * 2 + S::swizzle(ra, 2 * kk + fg) * 16;
    b_rd[kk] = rb * S::BK * 2 + S::swizzle(rb, 2 * kk + fg) * 16;
  }

  float16_t acc[S::TM][S::TN];
#pragma unroll
  for (int i = 0; i < S::TM; ++i)
#pragma unroll
    for (int j = 0; j < S::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int num_k_tiles = K / S::BK;
  issue_tile_loads(0, 0);
  wait_vmem_all();
  __syncthreads();

  for (int kt = 0; kt < num_k_tiles; ++kt) {
    if (kt + 1 < num_k_tiles) issue_tile_loads((kt + 1) & 1, (kt + 1) * S::BK);
    const char* sa = smem + (kt & 1) * S::kStageBytes;
    const char* sb = sa + S::kABytes;
#pragma unroll
    for (int kk = 0; kk < S::kKSteps; ++kk) {
      half8_t af[S::TM], bf[S::TN];
#pragma unroll
      for (int i = 0; i < S::TM; ++i)
        af[i] = *reinterpret_cast<const half8_t*>(sa + a_rd[kk] + i * 32 * S::BK * 2);
#pragma unroll
      for (int j = 0; j < S::TN; ++j)
        bf[j] = *reinterpret_cast<const half8_t*>(sb + b_rd[kk] + j * 32 * S::BK * 2);
#pragma unroll
      for (int i = 0; i < S::TM; ++i)
#pragma unroll
        for (int j = 0; j < S::TN; ++j) acc[i][j] = mfma_32x32x16(af[i], bf[j], acc[i][j]);
    }
    wait_vmem_all();
    __syncthreads();
  }

  // --- epilogue ---------------------------------------------------------------------------
  const int c_row0 = m0 + wm * S::WM + 4 * fg;
  const int c_col0 = n0 + wn * S::WN + fr;
#pragma unroll
  for (int i = 0; i < S::TM; ++i)
#pragma unroll
    for (int j = 0; j < S::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = c_row0 + i * 32 + 8 * (r / 4) + (r % 4);
        const int col = c_col0 + j * 32;
        store_out(C + (size_t)row * N + col, acc[i][j][r]);
      }
}

// ------------------------------------------------------------------------------------------
// General path: any M, N; K % 8 == 0.  Register-staged, bounds-checked, one LDS stage.
// ------------------------------------------------------------------------------------------
template <typename S, typename OutT>
__global__ __launch_bounds__(S::kThreads) void gemm_guarded_kernel(
    const half_t* __restrict__ A, const half_t* __restrict__ B, OutT* __restrict__ C, int M,
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
      half8_t af[S::TM], bf[S::TN];
#pragma unroll
      for (int i = 0; i < S::TM; ++i) {
        const int row = wm * S::WM + i * 32 + fr;
        af[i] = *reinterpret_cast<const half8_t*>(sa + row * S::BK * 2 + S::swizzle(row, 2 * kk + fg) * 16);
      }
#pragma unroll
      for (int j = 0; j < S::TN; ++j) {
        const int row = wn * S::WN + j * 32 + fr;
        bf[j] = *reinterpret_cast<const half8_t*>(sb + row * S::BK * 2 + S::swizzle(row, 2 * kk + fg) * 16);
      }
#pragma unroll
      for (int i = 0; i < S::TM; ++i)
#pragma unroll
        for (int j = 0; j < S::TN; ++j) acc[i][j] = mfma_32x32x16(af[i], bf[j], acc[i][j]);
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

using ShapeBig = GemmShape<256, 256, 64, 2, 2>;
using ShapeMid = GemmShape<128, 128, 64, 2, 2>;
using ShapeSmall = GemmShape<64, 64, 32, 2, 2>;

template <typename S, typename OutT>
int launch_direct(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t st) {
  auto kern = gemm_direct_lds_kernel<S, OutT>;
  constexpr int lds = 2 * S::kStageBytes;
  static_assert(lds <= kMaxLdsBytes, "tile does not fit in LDS");
  static thread_local int configured_dev = -1;
  int dev = 0;
  TFK_HIP_TRY(hipGetDevice(&dev));
  if (configured_dev != dev) {
    TFK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    configured_dev = dev;
  }
  const int tiles_m = M / S::BM, tiles_n = N / S::BN;
  hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(S::kThreads), lds, st,
                     static_cast<const half_t*>(A), static_cast<const half_t*>(B),
                     static_cast<OutT*>(C), M, N, K, tiles_m, tiles_n);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}

template <typename S, typename OutT>
int launch_guarded(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t st) {
  dim3 grid((M + S::BM - 1) / S::BM, (N + S::BN - 1) / S::BN);
  hipLaunchKernelGGL((gemm_guarded_kernel<S, OutT>), grid, dim3(S::kThreads), 0, st,
                     static_cast<const half_t*>(A), static_cast<const half_t*>(B),
                     static_cast<OutT*>(C), M, N, K);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}

template <typename OutT>
int dispatch(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t st) {
  if (M % 256 == 0 && N % 256 == 0 && K % 64 == 0 && (int64_t)(M / 256) * (N / 256) >= 128)
    return launch_direct<ShapeBig, OutT>(A, B, C, M, N, K, st);
  if (M % 128 == 0 && N % 128 == 0 && K % 64 == 0)
    return launch_direct<ShapeMid, OutT>(A, B, C, M, N, K, st);
  return launch_guarded<ShapeSmall, OutT>(A, B, C, M, N, K, st);
}

}  // namespace
}  // namespace tfk

extern "C" int tf_gemm_f16(const void* A, const void* B, void* C, int c_is_f16, int64_t M,
                           int64_t N, int64_t K, int tm, int tn, int tk, int num_stages,
                           int pipeline_level, void* stream) {
  using namespace tfk;
  TFK_REQUIRE(A && B && C, TF_ERR_INVALID_ARG, "tf_gemm_f16: null pointer");
  TFK_REQUIRE(M > 0 && N > 0 && K > 0, TF_ERR_INVALID_ARG, "tf_gemm_f16: M, N, K must be positive");
  TFK_REQUIRE(M < (1 << 30) && N < (1 << 30) && K < (1 << 22), TF_ERR_INVALID_ARG,
              "tf_gemm_f16: dimension too large");
  TFK_REQUIRE(K % 8 == 0, TF_ERR_UNSUPPORTED, "tf_gemm_f16: K (%lld) must be a multiple of 8",
              (long long)K);
  TFK_REQUIRE(tm > 0 && tn > 0 && tk > 0, TF_ERR_INVALID_ARG, "tf_gemm_f16: tile sizes must be positive");
  TFK_REQUIRE(M % tm == 0 && N % tn == 0 && K % tk == 0, TF_ERR_INVALID_ARG,
              "tf_gemm_f16: tile [%d,%d,%d] does not divide problem [%lld,%lld,%lld]", tm, tn, tk,
              (long long)M, (long long)N, (long long)K);
  TFK_REQUIRE(num_stages >= 1 && num_stages <= 3, TF_ERR_INVALID_ARG,
              "tf_gemm_f16: num_stages must be 1, 2 or 3");
  TFK_REQUIRE(pipeline_level >= 0 && pipeline_level <= 2, TF_ERR_INVALID_ARG,
              "tf_gemm_f16: pipeline_level must be 0, 1 or 2");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (c_is_f16) return dispatch<half_t>(A, B, C, (int)M, (int)N, (int)K, st);
  return dispatch<float>(A, B, C, (int)M, (int)N, (int)K, st);
}
