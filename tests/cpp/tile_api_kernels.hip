// GPU test kernels for the tile-programming headers, exported with a C ABI so the pytest
// files can drive them through ctypes.  They restate the asserted tests of the reference
// (tests/cpp/cell/test_g2s_load.cu, test_s2r_copy.cu, test_swizzled_copy.cu, test_gemm.cu) and
// add asserted tests for what the reference only prints (G2R/R2G, reduce, broadcast, mask).
#include <hip/hip_runtime.h>

#include "cell/mod.hpp"
#include "kernels/flash_attention_device.hpp"
#include "kernels/fused_two_gemms_device.hpp"
#include "kernels/gemm_device.hpp"
#include "types/mod.hpp"

using namespace tilefusion;
using namespace tilefusion::cell;
using namespace tilefusion::cell::copy;
namespace tl = tile_layout;

#define TT_API extern "C" __attribute__((visibility("default")))

static int launch_status() {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  return (int)hipDeviceSynchronize();
}

// ---- 1. global -> LDS -> global round trip (test_g2s_load.cu:19-45,144-268) ------------------
template <typename Element, typename WarpLayout, typename Layout, bool kSwizzled, int kBytes>
__global__ void k_g2s_roundtrip(const Element* in, Element* out) {
  extern __shared__ __attribute__((aligned(16))) unsigned char buf[];
  using Global = GlobalTile<Element, Layout>;
  using Shared = SharedTile<Element, Layout, kSwizzled, kBytes>;
  Global g_in(in), g_out(out);
  Shared s(reinterpret_cast<Element*>(buf));
  GlobalToSharedLoader<Shared, WarpLayout> load;
  SharedToGlobalStorer<Shared, WarpLayout> store;
  load(g_in, s);
  __copy_async();
  __syncthreads();
  store(s, g_out);
}
template <typename Element, typename WarpLayout, typename Layout, bool kSwizzled, int kBytes>
static int run_g2s(const void* in, void* out) {
  hipLaunchKernelGGL((k_g2s_roundtrip<Element, WarpLayout, Layout, kSwizzled, kBytes>), dim3(1),
                     dim3(tl::get_numel<WarpLayout> * WARP_SIZE), Layout::kNumel * sizeof(Element), 0,
                     static_cast<const Element*>(in), static_cast<Element*>(out));
  return launch_status();
}
TT_API int tt_g2s_roundtrip(int variant, const void* in, void* out) {
  switch (variant) {
    case 0: return run_g2s<__half, tl::RowMajor<1, 1>, tl::RowMajor<16, 64>, false, 128>(in, out);
    case 1: return run_g2s<__half, tl::RowMajor<1, 1>, tl::RowMajor<64, 64>, true, 128>(in, out);
    case 2: return run_g2s<__half, tl::RowMajor<2, 2>, tl::RowMajor<128, 128>, true, 128>(in, out);
    case 3: return run_g2s<__half, tl::RowMajor<2, 2>, tl::RowMajor<128, 128>, true, 64>(in, out);
    case 4: return run_g2s<__half, tl::RowMajor<4, 2>, tl::RowMajor<128, 256>, true, 64>(in, out);
    case 5: return run_g2s<__half, tl::RowMajor<2, 1>, tl::ColMajor<64, 64>, true, 128>(in, out);
    case 6: return run_g2s<__half, tl::RowMajor<2, 2>, tl::ColMajor<128, 64>, true, 64>(in, out);
    case 7: return run_g2s<float, tl::RowMajor<2, 2>, tl::RowMajor<64, 64>, true, 128>(in, out);
    case 8: return run_g2s<float, tl::RowMajor<1, 1>, tl::ColMajor<32, 32>, true, 64>(in, out);
    case 9: return run_g2s<__half, tl::RowMajor<1, 4>, tl::RowMajor<32, 256>, false, 128>(in, out);
    default: return -1;
  }
}
TT_API void tt_g2s_shape(int variant, int* rows, int* cols, int* elem_bytes, int* col_major) {
  static const int t[10][4] = {{16, 64, 2, 0}, {64, 64, 2, 0}, {128, 128, 2, 0}, {128, 128, 2, 0}, {128, 256, 2, 0},
                               {64, 64, 2, 1}, {128, 64, 2, 1}, {64, 64, 4, 0}, {32, 32, 4, 1}, {32, 256, 2, 0}};
  *rows = t[variant][0]; *cols = t[variant][1]; *elem_bytes = t[variant][2]; *col_major = t[variant][3];
}

// ---- 2. swizzled and plain LDS tiles give identical register fragments, and an accumulator
//         tile survives register -> LDS -> global (test_swizzled_copy.cu:27-94, test_s2r_copy.cu) --
template <typename WarpLayout, int kRows, int kCols, int kChunk, int kBytes, bool kWide>
__global__ void k_swizzled_fragments(const __half* a_in, const __half* b_in, int* mismatches) {
  // kWide: 16 x 32 operand base tiles (8 elements per lane), else the square 16 x 16 ones (4)
  constexpr int kDepth = kWide ? 32 : 16, kPerLane = kWide ? 8 : 4;
  using BaseA = std::conditional_t<kWide, RegTile<__half, tl::RowMajor<1, 8>>, BaseTileRowMajor<__half>>;
  using BaseB = std::conditional_t<kWide, RegTile<__half, tl::ColMajor<8, 1>>, BaseTileColMajor<__half>>;
  extern __shared__ __attribute__((aligned(16))) unsigned char buf[];
  __half* base = reinterpret_cast<__half*>(buf);
  using GlobalA = GlobalTile<__half, tl::RowMajor<kRows, kCols>>;
  using GlobalB = GlobalTile<__half, tl::ColMajor<kCols, kRows>>;
  using SA0 = SharedTile<__half, tl::RowMajor<kRows, kCols>, false, kBytes>;
  using SA1 = SharedTile<__half, tl::RowMajor<kRows, kCols>, true, kBytes>;
  using SB0 = SharedTile<__half, tl::ColMajor<kCols, kRows>, false, kBytes>;
  using SB1 = SharedTile<__half, tl::ColMajor<kCols, kRows>, true, kBytes>;
  SA0 sa0(base);
  SA1 sa1(base + kRows * kCols);
  SB0 sb0(base + 2 * kRows * kCols);
  SB1 sb1(base + 3 * kRows * kCols);
  GlobalA ga(a_in);
  GlobalB gb(b_in);
  { GlobalToSharedLoader<SA0, WarpLayout> l; l(ga, sa0); }
  { GlobalToSharedLoader<SA1, WarpLayout> l; l(ga, sa1); }
  { GlobalToSharedLoader<SB0, WarpLayout> l; l(gb, sb0); }
  { GlobalToSharedLoader<SB1, WarpLayout> l; l(gb, sb1); }
  __copy_async();
  __syncthreads();
  constexpr int kWR = tl::num_rows<WarpLayout>, kWC = tl::num_cols<WarpLayout>;
  using RegA = RegTile<BaseA, tl::RowMajor<kRows / kWR / 16, kChunk / kDepth>>;
  using RegB = RegTile<BaseB, tl::ColMajor<kChunk / kDepth, kRows / kWC / 16>>;
  using IterA0 = STileIterator<SA0, TileShape<kRows, kChunk>>;
  using IterA1 = STileIterator<SA1, TileShape<kRows, kChunk>>;
  using IterB0 = STileIterator<SB0, TileShape<kChunk, kRows>>;
  using IterB1 = STileIterator<SB1, TileShape<kChunk, kRows>>;
  IterA0 ia0(base);
  IterA1 ia1(base + kRows * kCols);
  IterB0 ib0(base + 2 * kRows * kCols);
  IterB1 ib1(base + 3 * kRows * kCols);
  SharedToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont> la;
  SharedToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont> lb;
  int bad = 0;
  for (int k = 0; k < IterA0::sc1; ++k) {
    RegA ra0, ra1;
    RegB rb0, rb1;
    la(ia0(k), ra0);
    la(ia1(k), ra1);
    lb(ib0(k), rb0);
    lb(ib1(k), rb1);
    const __half* p0 = ra0.data()[0].data();
    const __half* p1 = ra1.data()[0].data();
    for (int e = 0; e < RegA::kNumel * kPerLane; ++e) bad += (__half2float(p0[e]) != __half2float(p1[e]));
    const __half* q0 = rb0.data()[0].data();
    const __half* q1 = rb1.data()[0].data();
    for (int e = 0; e < RegB::kNumel * kPerLane; ++e) bad += (__half2float(q0[e]) != __half2float(q1[e]));
    // and the fragment really is the documented block of the source: element 0 of base tile (0,0)
    const int lane = threadIdx.x % WARP_SIZE;
    const int wr = warp::warp_row_id<WarpLayout>();
    const float want = __half2float(a_in[(wr * (kRows / kWR) + lane % 16) * kCols + k * kChunk + kPerLane * (lane / 16)]);
    bad += (__half2float(p0[0]) != want);
    // same for B (a column-major [kCols, kRows] matrix: element (r, c) at c * kCols + r)
    const int wc = warp::warp_col_id<WarpLayout>();
    const float want_b = __half2float(b_in[(wc * (kRows / kWC) + lane % 16) * kCols + k * kChunk + kPerLane * (lane / 16)]);
    bad += (__half2float(q0[0]) != want_b);
  }
  if (bad) atomicAdd(mismatches, bad);
}
template <bool kWide>
static int run_swizzled_fragments(int shape, const __half* pa, const __half* pb, int* mismatches) {
  switch (shape) {
    case 0:
      hipLaunchKernelGGL((k_swizzled_fragments<tl::RowMajor<1, 1>, 64, 64, 32, 128, kWide>), dim3(1), dim3(64), 4 * 64 * 64 * 2, 0, pa, pb, mismatches);
      break;
    case 1:
      hipLaunchKernelGGL((k_swizzled_fragments<tl::RowMajor<2, 2>, 128, 128, 64, 128, kWide>), dim3(1), dim3(256), 4 * 128 * 128 * 2, 0, pa, pb, mismatches);
      break;
    case 2:
      hipLaunchKernelGGL((k_swizzled_fragments<tl::RowMajor<2, 2>, 64, 128, 32, 64, kWide>), dim3(1), dim3(256), 4 * 64 * 128 * 2, 0, pa, pb, mismatches);
      break;
    case 3:
      hipLaunchKernelGGL((k_swizzled_fragments<tl::RowMajor<4, 1>, 64, 64, 64, 64, kWide>), dim3(1), dim3(256), 4 * 64 * 64 * 2, 0, pa, pb, mismatches);
      break;
    default: return -1;
  }
  return launch_status();
}
// variants 0-3: wide operand tiles, 4-7: the same shapes with square base tiles
TT_API int tt_swizzled_fragments(int variant, const void* a, const void* b, int* mismatches) {
  const __half* pa = static_cast<const __half*>(a);
  const __half* pb = static_cast<const __half*>(b);
  return variant < 4 ? run_swizzled_fragments<true>(variant, pa, pb, mismatches)
                     : run_swizzled_fragments<false>(variant - 4, pa, pb, mismatches);
}

template <typename WarpLayout, int kRows, int kCols, bool kColTiles>
__global__ void k_acc_roundtrip(const float* in, float* out_direct, float* out_via_lds, __half* out_half) {
  extern __shared__ __attribute__((aligned(16))) unsigned char buf[];
  constexpr int kWR = tl::num_rows<WarpLayout>, kWC = tl::num_cols<WarpLayout>;
  using Global = GlobalTile<float, tl::RowMajor<kRows, kCols>>;
  using GlobalH = GlobalTile<__half, tl::RowMajor<kRows, kCols>>;
  using Reg = RegTile<std::conditional_t<kColTiles, BaseTileColMajor<float>, BaseTileRowMajor<float>>,
                      tl::RowMajor<kRows / kWR / 16, kCols / kWC / 16>>;
  using RegH = RegTile<std::conditional_t<kColTiles, BaseTileColMajor<__half>, BaseTileRowMajor<__half>>,
                       tl::RowMajor<kRows / kWR / 16, kCols / kWC / 16>>;
  using Shared = SharedTile<float, tl::RowMajor<kRows, kCols>, true, 128>;
  Global g_in(in), g_direct(out_direct), g_lds(out_via_lds);
  GlobalH g_half(out_half);
  Shared s(reinterpret_cast<float*>(buf));
  Reg r;
  GlobalToRegLoader<Reg, WarpLayout, WarpReuse::kCont> g2r;
  g2r(g_in, r);
  RegToGlobalStorer<Global, Reg, WarpLayout> r2g;
  r2g(r, g_direct);
  RegToSharedStorer<Reg, WarpLayout> r2s;
  r2s(r, s);
  __syncthreads();
  SharedToGlobalStorer<Shared, WarpLayout> s2g;
  s2g(s, g_lds);
  RegH rh;
  compute::RegTileConvert<Reg, RegH> cast;
  cast(r, rh);
  RegToGlobalStorer<GlobalH, RegH, WarpLayout> r2gh;
  r2gh(rh, g_half);
}
TT_API int tt_acc_roundtrip(int variant, const void* in, void* out_direct, void* out_lds, void* out_half) {
  const float* pi = static_cast<const float*>(in);
  float* po = static_cast<float*>(out_direct);
  float* pl = static_cast<float*>(out_lds);
  __half* ph = static_cast<__half*>(out_half);
  switch (variant) {
    case 0:
      hipLaunchKernelGGL((k_acc_roundtrip<tl::RowMajor<1, 1>, 32, 64, false>), dim3(1), dim3(64), 32 * 64 * 4, 0, pi, po, pl, ph);
      break;
    case 1:
      hipLaunchKernelGGL((k_acc_roundtrip<tl::RowMajor<2, 2>, 128, 64, false>), dim3(1), dim3(256), 128 * 64 * 4, 0, pi, po, pl, ph);
      break;
    // the same shapes held as column-major base tiles (a lane owns part of a column)
    case 2:
      hipLaunchKernelGGL((k_acc_roundtrip<tl::RowMajor<1, 1>, 32, 64, true>), dim3(1), dim3(64), 32 * 64 * 4, 0, pi, po, pl, ph);
      break;
    case 3:
      hipLaunchKernelGGL((k_acc_roundtrip<tl::RowMajor<2, 2>, 128, 64, true>), dim3(1), dim3(256), 128 * 64 * 4, 0, pi, po, pl, ph);
      break;
    default: return -1;
  }
  return launch_status();
}

// ---- 3. the README example: GEMM with global -> register loaders only (README.md:56-112,
//         examples/101_gemm/01_gemm_global_reg/gemm.hpp:62-95); the tile counts are the reference's
//         formulas over the square BaseTileShape (gemm.hpp:19-56 there), the accumulator is the
//         BaseTileRowMajor<float> tile the README declares ----
namespace readme {
using InType = __half;
using AccType = float;
using WarpLayout = tl::RowMajor<2, 2>;
constexpr int kM = 128, kN = 64, kK = 256, kTK = 32;
using BaseShape = BaseTileShape<InType>;
constexpr int kWarpPerRow = tl::num_rows<WarpLayout>, kWarpPerCol = tl::num_cols<WarpLayout>;
using GlobalA = GlobalTile<InType, tl::RowMajor<kM, kK>>;
using IteratorA = TileIterator<GlobalA, TileShape<kM, kTK>>;
using RegA = RegTile<BaseTileRowMajor<InType>, tl::RowMajor<kM / kWarpPerRow / BaseShape::kRows, kTK / BaseShape::kCols>>;
using ALoader = GlobalToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont>;
using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kN>>;
using IteratorB = TileIterator<GlobalB, TileShape<kTK, kN>>;
using RegB = RegTile<BaseTileColMajor<InType>, tl::ColMajor<kTK / BaseShape::kRows, kN / kWarpPerCol / BaseShape::kCols>>;
using BLoader = GlobalToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont>;
using GlobalC = GlobalTile<AccType, tl::RowMajor<kM, kN>>;
using RegC = RegTile<BaseTileRowMajor<AccType>, tl::RowMajor<kM / kWarpPerRow / BaseShape::kRows, kN / kWarpPerCol / BaseShape::kCols>>;
using CStorer = RegToGlobalStorer<GlobalC, RegC, WarpLayout>;

__global__ void simple_gemm(const InType* dA, const InType* dB, AccType* dC) {
  IteratorA gAs(dA);
  RegA rA;
  ALoader loader_a;
  IteratorB gBs(dB);
  RegB rB;
  BLoader loader_b;
  RegC acc;
  GlobalC gC(dC);
  CStorer storer_c;
  for (int k = 0; k < IteratorA::sc1; ++k) {
    loader_a(gAs(k), rA);
    loader_b(gBs(k), rB);
    __syncthreads();
    compute::gemm(rA, rB, acc);
  }
  __syncthreads();
  storer_c(acc, gC);
}
}  // namespace readme
TT_API int tt_readme_gemm(const void* a, const void* b, void* c) {
  hipLaunchKernelGGL(readme::simple_gemm, dim3(1), dim3(tl::get_numel<readme::WarpLayout> * WARP_SIZE), 0, 0,
                     static_cast<const __half*>(a), static_cast<const __half*>(b), static_cast<float*>(c));
  return launch_status();
}

// ---- 3b. the same GEMM with the other MMA atoms: bf16 inputs, and fp16 inputs with an fp16
//          accumulator tile (include/cell/compute/gemm.hpp:63-150 in the reference) -------------
namespace atoms {
// kWide: wide 16 x 32 operand tiles; kColAcc: column-major accumulator base tiles; kTK = 48 walks
// an odd number of square base tiles per chunk (one 16x16x32 and one 16x16x16 instruction)
template <typename InType, typename AccType, bool kWide, bool kColAcc, int kTK>
__global__ void gemm_atom(const InType* dA, const InType* dB, AccType* dC) {
  using WarpLayout = tl::RowMajor<2, 2>;
  constexpr int kM = 128, kN = 64, kK = 192, kDepth = kWide ? 32 : 16;
  using BaseA = std::conditional_t<kWide, RegTile<InType, tl::RowMajor<1, 8>>, BaseTileRowMajor<InType>>;
  using BaseB = std::conditional_t<kWide, RegTile<InType, tl::ColMajor<8, 1>>, BaseTileColMajor<InType>>;
  using BaseC = std::conditional_t<kColAcc, BaseTileColMajor<AccType>, BaseTileRowMajor<AccType>>;
  using GlobalA = GlobalTile<InType, tl::RowMajor<kM, kK>>;
  using IteratorA = TileIterator<GlobalA, TileShape<kM, kTK>>;
  using RegA = RegTile<BaseA, tl::RowMajor<kM / 2 / 16, kTK / kDepth>>;
  using GlobalB = GlobalTile<InType, tl::ColMajor<kK, kN>>;
  using IteratorB = TileIterator<GlobalB, TileShape<kTK, kN>>;
  using RegB = RegTile<BaseB, tl::ColMajor<kTK / kDepth, kN / 2 / 16>>;
  using GlobalC = GlobalTile<AccType, tl::RowMajor<kM, kN>>;
  using RegC = RegTile<BaseC, tl::RowMajor<kM / 2 / 16, kN / 2 / 16>>;
  IteratorA gAs(dA);
  IteratorB gBs(dB);
  RegA rA;
  RegB rB;
  RegC acc;
  GlobalToRegLoader<RegA, WarpLayout, WarpReuse::kRowReuseCont> loader_a;
  GlobalToRegLoader<RegB, WarpLayout, WarpReuse::kColReuseCont> loader_b;
  for (int k = 0; k < IteratorA::sc1; ++k) {
    loader_a(gAs(k), rA);
    loader_b(gBs(k), rB);
    compute::gemm(rA, rB, acc);
  }
  GlobalC gC(dC);
  RegToGlobalStorer<GlobalC, RegC, WarpLayout> storer_c;
  storer_c(acc, gC);
}
// MmaAtom used directly on single base tiles: C[16,16] += A[16,16] * B[16,16] (one wavefront)
template <typename InType>
__global__ void single_atom(const InType* dA, const InType* dB, float* dC) {
  using Atom = compute::MmaAtom<InType, InType, float, compute::MMA_ATOM_16x16x16>;
  using WarpLayout = tl::RowMajor<1, 1>;
  using RegA = RegTile<typename Atom::BaseTileA, tl::RowMajor<1, 1>>;
  using RegB = RegTile<typename Atom::BaseTileB, tl::ColMajor<1, 1>>;
  using RegC = RegTile<typename Atom::BaseTileC, tl::RowMajor<1, 1>>;
  using GlobalA = GlobalTile<InType, tl::RowMajor<16, 16>>;
  using GlobalB = GlobalTile<InType, tl::ColMajor<16, 16>>;
  using GlobalC = GlobalTile<float, tl::RowMajor<16, 16>>;
  GlobalA gA(dA);
  GlobalB gB(dB);
  GlobalC gC(dC);
  RegA rA;
  RegB rB;
  RegC rC;
  GlobalToRegLoader<RegA, WarpLayout, WarpReuse::kCont> la;
  GlobalToRegLoader<RegB, WarpLayout, WarpReuse::kCont> lb;
  la(gA, rA);
  lb(gB, rB);
  Atom mma;
  mma(rA(0, 0), rB(0, 0), rC(0, 0));
  RegToGlobalStorer<GlobalC, RegC, WarpLayout> sc;
  sc(rC, gC);
}
}  // namespace atoms
// variant: 0 bf16 -> fp32, 1 fp16 -> fp16 accumulator, 2 fp16 -> fp32 with a column-major accumulator,
// 3 fp16 -> fp32 with an odd base-tile count per chunk, 4 bf16 odd count; +8: the same with wide
// operand tiles (variants 8, 9, 10).  A [128, 192], B [192, 64] column-major, C [128, 64].
TT_API int tt_atom_gemm(int variant, const void* a, const void* b, void* c) {
  const auto* ha = static_cast<const __half*>(a);
  const auto* hb = static_cast<const __half*>(b);
  const auto* ba = static_cast<const __bfloat16*>(a);
  const auto* bb = static_cast<const __bfloat16*>(b);
  const dim3 g(1), t(256);
  switch (variant) {
    case 0: hipLaunchKernelGGL((atoms::gemm_atom<__bfloat16, float, false, false, 32>), g, t, 0, 0, ba, bb, static_cast<float*>(c)); break;
    case 1: hipLaunchKernelGGL((atoms::gemm_atom<__half, __half, false, false, 32>), g, t, 0, 0, ha, hb, static_cast<__half*>(c)); break;
    case 2: hipLaunchKernelGGL((atoms::gemm_atom<__half, float, false, true, 32>), g, t, 0, 0, ha, hb, static_cast<float*>(c)); break;
    case 3: hipLaunchKernelGGL((atoms::gemm_atom<__half, float, false, false, 48>), g, t, 0, 0, ha, hb, static_cast<float*>(c)); break;
    case 4: hipLaunchKernelGGL((atoms::gemm_atom<__bfloat16, float, false, true, 48>), g, t, 0, 0, ba, bb, static_cast<float*>(c)); break;
    case 8: hipLaunchKernelGGL((atoms::gemm_atom<__bfloat16, float, true, false, 32>), g, t, 0, 0, ba, bb, static_cast<float*>(c)); break;
    case 9: hipLaunchKernelGGL((atoms::gemm_atom<__half, __half, true, false, 64>), g, t, 0, 0, ha, hb, static_cast<__half*>(c)); break;
    case 10: hipLaunchKernelGGL((atoms::gemm_atom<__half, float, true, true, 32>), g, t, 0, 0, ha, hb, static_cast<float*>(c)); break;
    default: return -1;
  }
  return launch_status();
}
// one MmaAtom on one base tile each: variant 0 fp16, 1 bf16
TT_API int tt_single_atom(int variant, const void* a, const void* b, void* c) {
  if (variant == 0)
    hipLaunchKernelGGL((atoms::single_atom<__half>), dim3(1), dim3(64), 0, 0, static_cast<const __half*>(a),
                       static_cast<const __half*>(b), static_cast<float*>(c));
  else if (variant == 1)
    hipLaunchKernelGGL((atoms::single_atom<__bfloat16>), dim3(1), dim3(64), 0, 0, static_cast<const __bfloat16*>(a),
                       static_cast<const __bfloat16*>(b), static_cast<float*>(c));
  else
    return -1;
  return launch_status();
}

// ---- 4. ke_gemm composed from the primitives (test_gemm.cu:172-215,316-375) ------------------
template <typename Traits, typename AccType>
__global__ __launch_bounds__(Traits::kThreads) void k_ke_gemm(const __half* a, const __half* b, AccType* c) {
  kernels::ke_gemm<__half, AccType, Traits>(a, b, c);
}
template <typename WarpLayout, typename AccType, int M, int N, int K, int TM, int TN, int TK, int RK, int Stages, int Bytes>
static int run_ke_gemm(const void* a, const void* b, void* c) {
  using Traits = kernels::KeGemmTraits<__half, AccType, WarpLayout, M, N, K, TM, TN, TK, RK, Stages, Bytes>;
  auto kern = k_ke_gemm<Traits, AccType>;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Traits::kSharedBytes) != hipSuccess) return -2;
  hipLaunchKernelGGL(kern, dim3(M / TM, N / TN), dim3(Traits::kThreads), Traits::kSharedBytes, 0,
                     static_cast<const __half*>(a), static_cast<const __half*>(b), static_cast<AccType*>(c));
  return launch_status();
}
TT_API int tt_ke_gemm(int variant, const void* a, const void* b, void* c) {
  switch (variant) {
    case 0: return run_ke_gemm<tl::RowMajor<1, 1>, float, 64, 64, 64, 64, 64, 64, 16, 1, 64>(a, b, c);
    case 1: return run_ke_gemm<tl::RowMajor<1, 1>, float, 128, 128, 128, 64, 64, 64, 16, 1, 64>(a, b, c);
    case 2: return run_ke_gemm<tl::RowMajor<2, 2>, float, 256, 256, 256, 128, 128, 64, 32, 2, 128>(a, b, c);
    case 3: return run_ke_gemm<tl::RowMajor<2, 2>, __half, 256, 128, 512, 64, 128, 128, 32, 2, 64>(a, b, c);
    case 4: return run_ke_gemm<tl::RowMajor<4, 1>, float, 128, 64, 256, 128, 64, 32, 32, 3, 64>(a, b, c);
    case 5: return run_ke_gemm<tl::RowMajor<2, 4>, float, 512, 512, 128, 128, 256, 64, 64, 2, 128>(a, b, c);
    default: return -1;
  }
}
TT_API void tt_ke_gemm_shape(int variant, int* m, int* n, int* k, int* c_is_half) {
  static const int t[6][4] = {{64, 64, 64, 0}, {128, 128, 128, 0}, {256, 256, 256, 0}, {256, 128, 512, 1}, {128, 64, 256, 0}, {512, 512, 128, 0}};
  *m = t[variant][0]; *n = t[variant][1]; *k = t[variant][2]; *c_is_half = t[variant][3];
}

// ---- 5. reduce / broadcast / map / mask on an accumulator tile (print-only in the reference:
//         tests/cpp/cell/test_reduce.cu, test_broadcast.cu, test_flash_attn.cu) ------------------
template <typename WarpLayout, int kRows, int kCols, int kVecCols>
__global__ void k_softmax_pieces(const float* in, float* row_max, float* row_sum, float* out, int row_offset,
                                 int col_offset) {
  constexpr int kWR = tl::num_rows<WarpLayout>;
  static_assert(tl::num_cols<WarpLayout> == 1, "rows must not be split across wavefronts");
  using Global = GlobalTile<float, tl::RowMajor<kRows, kCols>>;
  using Reg = RegTile<BaseTileRowMajor<float>, tl::RowMajor<kRows / kWR / 16, kCols / 16>>;
  // one row per lane and base-tile row; kVecCols = 2 is how kernels written for the reference
  // declare the vector (every column then holds the same value)
  using Vec = RegTile<float, tl::RowMajor<Reg::kRows, kVecCols>>;
  Global g_in(in), g_out(out);
  Reg t;
  GlobalToRegLoader<Reg, WarpLayout, WarpReuse::kCont> g2r;
  g2r(g_in, t);
  ApplyMask<Reg, WarpLayout, BaseTileShape<float>, MaskMode::kCausal> mask;
  mask(t, row_offset, col_offset, -INFINITY);
  Vec vmax, vsum;
  compute::MaxReduce<Reg, tl::Layout::kRowMajor> rmax;
  rmax(t, vmax);
  compute::BroadcastSub<Vec, Reg, tl::Layout::kRowMajor> bsub;
  bsub(vmax, t);
  compute::RegTileExp<Reg> rexp;
  rexp(t, t);
  compute::SumReduce<Reg, tl::Layout::kRowMajor> rsum;
  rsum(t, vsum);
  compute::BroadcastDiv<Vec, Reg, tl::Layout::kRowMajor> bdiv;
  bdiv(vsum, t);
  compute::BroadcastScalarMul<Reg> smul;
  smul(t, 2.0f, t);
  RegToGlobalStorer<Global, Reg, WarpLayout> r2g;
  r2g(t, g_out);
  const int lane = threadIdx.x % WARP_SIZE;
  const int wrow = warp::warp_row_id<WarpLayout>() * (kRows / kWR);
  // every one of the four lanes that share a row must hold the result: lane group g writes rows with row % 4 == g
  for (int i = 0; i < Reg::kRows; ++i)
    if ((lane % 16) % 4 == lane / 16) {
      row_max[wrow + 16 * i + lane % 16] = vmax(i, kVecCols - 1);
      row_sum[wrow + 16 * i + lane % 16] = vsum(i, kVecCols - 1);
    }
}
TT_API int tt_softmax_pieces(int variant, const void* in, void* row_max, void* row_sum, void* out, int row_offset,
                             int col_offset) {
  const float* pi = static_cast<const float*>(in);
  float *pm = static_cast<float*>(row_max), *ps = static_cast<float*>(row_sum), *po = static_cast<float*>(out);
  switch (variant) {
    case 0:
      hipLaunchKernelGGL((k_softmax_pieces<tl::RowMajor<1, 1>, 16, 16, 1>), dim3(1), dim3(64), 0, 0, pi, pm, ps, po, row_offset, col_offset);
      break;
    case 1:
      hipLaunchKernelGGL((k_softmax_pieces<tl::RowMajor<1, 1>, 32, 64, 2>), dim3(1), dim3(64), 0, 0, pi, pm, ps, po, row_offset, col_offset);
      break;
    case 2:
      hipLaunchKernelGGL((k_softmax_pieces<tl::RowMajor<4, 1>, 128, 128, 1>), dim3(1), dim3(256), 0, 0, pi, pm, ps, po, row_offset, col_offset);
      break;
    default: return -1;
  }
  return launch_status();
}

// ---- 6. fused back-to-back GEMM composed from the primitives (tests/python/test_fused_two_gemms.py:
//         M, N, K, P = 256, 128, 64, 64 with 64-wide tiles) ------------------------------------------
template <typename Traits>
__global__ __launch_bounds__(Traits::kThreads) void k_ke_fused(const __half* a, const __half* b, const __half* c, __half* d) {
  kernels::ke_fused_two_gemms<__half, float, Traits>(a, b, c, d);
}
template <typename WarpLayout, int B, int M, int N, int K, int P, int TM, int TN, int TK, int TP>
static int run_ke_fused(const void* a, const void* b, const void* c, void* d) {
  using Traits = kernels::FusedTwoGemmsTraits<__half, float, WarpLayout, M, N, K, P, TM, TN, TK, TP>;
  auto kern = k_ke_fused<Traits>;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Traits::kSharedBytes) != hipSuccess) return -2;
  hipLaunchKernelGGL(kern, dim3(M / TM, P / TP, B), dim3(Traits::kThreads), Traits::kSharedBytes, 0,
                     static_cast<const __half*>(a), static_cast<const __half*>(b), static_cast<const __half*>(c),
                     static_cast<__half*>(d));
  return launch_status();
}
static const int kFusedShapes[4][5] = {{1, 256, 128, 64, 64}, {1, 1024, 256, 128, 128}, {3, 128, 64, 32, 32}, {2, 512, 128, 128, 256}};
TT_API int tt_ke_fused(int variant, const void* a, const void* b, const void* c, void* d) {
  switch (variant) {
    case 0: return run_ke_fused<tl::RowMajor<2, 1>, 1, 256, 128, 64, 64, 64, 64, 64, 64>(a, b, c, d);
    case 1: return run_ke_fused<tl::RowMajor<4, 1>, 1, 1024, 256, 128, 128, 64, 128, 128, 128>(a, b, c, d);
    case 2: return run_ke_fused<tl::RowMajor<1, 1>, 3, 128, 64, 32, 32, 16, 32, 32, 16>(a, b, c, d);
    case 3: return run_ke_fused<tl::RowMajor<4, 1>, 2, 512, 128, 128, 256, 128, 64, 32, 64>(a, b, c, d);
    default: return -1;
  }
}
TT_API void tt_ke_fused_shape(int variant, int* batch, int* m, int* n, int* k, int* p) {
  const int* t = kFusedShapes[variant];
  *batch = t[0]; *m = t[1]; *n = t[2]; *k = t[3]; *p = t[4];
}

// ---- 7. flash attention composed from the primitives (tests/python/test_flash_attn.py:
//         (64,128,128,128) plain and (128,128,128,128) causal, tiles (64,128,128,128), 4 wavefronts) ---
template <typename Traits>
__global__ __launch_bounds__(Traits::kThreads) void k_ke_flash(const __half* q, const __half* k, const __half* v, __half* o) {
  kernels::ke_flash_attention<__half, float, __half, Traits>(q, k, v, o);
}
template <typename WarpLayout, int B, int M, int N, int K, int P, int TM, int TN, int TK, int TP, bool kCausal>
static int run_ke_flash(const void* q, const void* k, const void* v, void* o) {
  // softmax scale 1/sqrt(K): K is 128, 64 or 96 in the variants below
  constexpr double kScale = K == 128 ? 0.08838834764831845 : K == 64 ? 0.125 : 0.10206207261596575;
  using Traits = kernels::FlashAttentionTraits<__half, float, __half, TileShape<M, N, K, P>, TileShape<TM, TN, TK, TP>,
                                               WarpLayout, kScale, kCausal>;
  auto kern = k_ke_flash<Traits>;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Traits::kSharedBytes) != hipSuccess) return -2;
  hipLaunchKernelGGL(kern, dim3(M / TM, P / TP, B), dim3(Traits::kThreads), Traits::kSharedBytes, 0,
                     static_cast<const __half*>(q), static_cast<const __half*>(k), static_cast<const __half*>(v),
                     static_cast<__half*>(o));
  return launch_status();
}
static const int kFlashShapes[7][6] = {{1, 64, 128, 128, 128, 0},  {1, 128, 128, 128, 128, 1}, {2, 256, 512, 128, 128, 0},
                                       {2, 512, 512, 64, 64, 1},   {1, 128, 256, 64, 128, 0},  {3, 256, 256, 128, 64, 1},
                                       {2, 64, 128, 96, 64, 1}};
TT_API int tt_ke_flash(int variant, const void* q, const void* k, const void* v, void* o) {
  switch (variant) {
    case 0: return run_ke_flash<tl::RowMajor<4, 1>, 1, 64, 128, 128, 128, 64, 128, 128, 128, false>(q, k, v, o);
    case 1: return run_ke_flash<tl::RowMajor<4, 1>, 1, 128, 128, 128, 128, 64, 128, 128, 128, true>(q, k, v, o);
    case 2: return run_ke_flash<tl::RowMajor<4, 1>, 2, 256, 512, 128, 128, 64, 64, 128, 128, false>(q, k, v, o);
    case 3: return run_ke_flash<tl::RowMajor<4, 1>, 2, 512, 512, 64, 64, 128, 64, 64, 64, true>(q, k, v, o);
    case 4: return run_ke_flash<tl::RowMajor<2, 1>, 1, 128, 256, 64, 128, 32, 128, 32, 64, false>(q, k, v, o);
    case 5: return run_ke_flash<tl::RowMajor<1, 1>, 3, 256, 256, 128, 64, 16, 32, 64, 32, true>(q, k, v, o);
    // head dimension 96 walked in three 32-deep chunks (Q reloaded per key tile)
    case 6: return run_ke_flash<tl::RowMajor<2, 1>, 2, 64, 128, 96, 64, 32, 64, 32, 64, true>(q, k, v, o);
    default: return -1;
  }
}
TT_API void tt_ke_flash_shape(int variant, int* batch, int* m, int* n, int* k, int* p, int* causal) {
  const int* t = kFlashShapes[variant];
  *batch = t[0]; *m = t[1]; *n = t[2]; *k = t[3]; *p = t[4]; *causal = t[5];
}

// ---- 8. the pipelined GEMMs: Pipeline global -> LDS with asynchronous copies (level 1) plus a
//         register-level Pipeline (level 2); tests/python/test_gemm.py:75-135 cases and more ----
template <typename Traits, typename AccType, int kLevel>
__global__ __launch_bounds__(Traits::kThreads) void k_ke_gemm_pipe(const __half* a, const __half* b, AccType* c) {
  if constexpr (kLevel == 1) kernels::ke_gemm_level1_pipeline<__half, AccType, Traits>(a, b, c);
  else kernels::ke_gemm_level2_pipeline<__half, AccType, Traits>(a, b, c);
}
template <typename WarpLayout, typename AccType, int kLevel, int M, int N, int K, int TM, int TN, int TK, int RK,
          int Stages, int Bytes>
static int run_ke_gemm_pipe(const void* a, const void* b, void* c) {
  using Traits = kernels::KeGemmTraits<__half, AccType, WarpLayout, M, N, K, TM, TN, TK, RK, Stages, Bytes>;
  auto kern = k_ke_gemm_pipe<Traits, AccType, kLevel>;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                          Traits::kPipelineSharedBytes) != hipSuccess)
    return -2;
  hipLaunchKernelGGL(kern, dim3(M / TM, N / TN), dim3(Traits::kThreads), Traits::kPipelineSharedBytes, 0,
                     static_cast<const __half*>(a), static_cast<const __half*>(b), static_cast<AccType*>(c));
  return launch_status();
}
static const int kPipeShapes[9][4] = {{128, 128, 128, 0}, {256, 256, 256, 0}, {256, 256, 256, 0}, {512, 512, 512, 0},
                                      {256, 256, 512, 0}, {128, 128, 256, 0}, {256, 256, 512, 1}, {128, 128, 384, 0},
                                      {512, 256, 1024, 0}};
TT_API int tt_ke_gemm_pipe(int variant, const void* a, const void* b, void* c) {
  switch (variant) {
    // the reference's own cases 1-4 (64 x 64 x 64 tiles; level 1 with 2 slots, level 2 with 3)
    case 0: return run_ke_gemm_pipe<tl::RowMajor<2, 2>, float, 1, 128, 128, 128, 64, 64, 64, 32, 2, 64>(a, b, c);
    case 1: return run_ke_gemm_pipe<tl::RowMajor<2, 2>, float, 1, 256, 256, 256, 64, 64, 64, 32, 2, 64>(a, b, c);
    case 2: return run_ke_gemm_pipe<tl::RowMajor<2, 2>, float, 2, 256, 256, 256, 64, 64, 64, 32, 3, 64>(a, b, c);
    case 3: return run_ke_gemm_pipe<tl::RowMajor<2, 2>, float, 2, 512, 512, 512, 64, 64, 64, 32, 3, 64>(a, b, c);
    // level 1 with three slots (two chunks in flight), 128-byte swizzle
    case 4: return run_ke_gemm_pipe<tl::RowMajor<2, 2>, float, 1, 256, 256, 512, 128, 128, 64, 32, 3, 128>(a, b, c);
    // level 2 with two slots and ONE register step per chunk
    case 5: return run_ke_gemm_pipe<tl::RowMajor<2, 2>, float, 2, 128, 128, 256, 64, 64, 32, 32, 2, 64>(a, b, c);
    // level 2 with four slots, fp16 output
    case 6: return run_ke_gemm_pipe<tl::RowMajor<2, 2>, __half, 2, 256, 256, 512, 128, 128, 64, 32, 4, 128>(a, b, c);
    // level 2 with an odd number (3) of register steps per chunk: the register ring changes parity
    case 7: return run_ke_gemm_pipe<tl::RowMajor<1, 2>, float, 2, 128, 128, 384, 64, 64, 96, 32, 3, 64>(a, b, c);
    // level 2, 8 wavefronts, 16 chunks
    case 8: return run_ke_gemm_pipe<tl::RowMajor<2, 4>, float, 2, 512, 256, 1024, 128, 256, 64, 32, 3, 128>(a, b, c);
    default: return -1;
  }
}
TT_API void tt_ke_gemm_pipe_shape(int variant, int* m, int* n, int* k, int* c_is_half) {
  const int* t = kPipeShapes[variant];
  *m = t[0]; *n = t[1]; *k = t[2]; *c_is_half = t[3];
}

// ---- 9. Pipeline on its own: a [kRows, kCols] tile goes chunk by chunk through a ring of
//         kStages LDS slots (asynchronous copies, kStages - 1 chunks in flight, wait_group<N> with
//         the loader's exact load count) and is reassembled in a second LDS area ------------------
template <int kStages, int kRows, int kCols, int kChunkCols, typename WarpLayout>
__global__ void k_pipeline_roundtrip(const __half* in, __half* out, int* errors) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char buf[];
  using Global = GlobalTile<__half, tl::RowMajor<kRows, kCols>>;
  using GIter = GTileIterator<Global, TileShape<kRows, kChunkCols>>;
  using Shared = SharedTile<__half, tl::RowMajor<kRows, kChunkCols>, true, 128>;
  using Loader = GlobalToSharedLoader<Shared, WarpLayout>;
  using Pipe = Pipeline<__half, Global, Shared, GIter, Loader, kStages, GIter::sc1>;
  static_assert(Pipe::Iterations == GIter::sc1);
  constexpr int kChunks = GIter::sc1, kAhead = kStages - 1, kLoads = Loader::kLoadsPerLane;
  constexpr int kThreads = tl::get_numel<WarpLayout> * WARP_SIZE;
  __half* ring = reinterpret_cast<__half*>(buf);
  __half* whole = ring + kStages * Shared::kNumel;   // [kRows, kCols], plain row-major
  Pipe pipe(in, ring);
  int bad = 0;
#pragma unroll
  for (int i = 0; i < kAhead && i < kChunks; ++i) {
    pipe.commit();
    commit_copy_group();
  }
  for (int k = 0; k < kChunks; ++k) {
    if (k + kAhead <= kChunks) wait_group<kAhead - 1, kLoads>();
    else wait_group<0>();
    sync_threads_keep_copies();
    if (k + kAhead < kChunks) {
      pipe.commit();
      commit_copy_group();
    }
    const __half* slot = pipe.get_dst_ptr_by_index(k);
    bad += slot != ring + (k % kStages) * Shared::kNumel;
    bad += pipe.get_dst_tile_by_index(k).data() != slot;
    if (k + kAhead < kChunks && kStages >= 2) {
      // the chunk just committed is the newest one: get_cur_dst is its slot, get_prev_dst the
      // slot of the chunk before it
      bad += pipe.get_cur_dst() != ring + ((k + kAhead) % kStages) * Shared::kNumel;
      bad += pipe.get_prev_dst() != ring + ((k + kAhead - 1) % kStages) * Shared::kNumel;
    }
    Shared chunk(const_cast<__half*>(slot));
    for (int e = threadIdx.x; e < kRows * kChunkCols; e += kThreads) {
      const int r = e / kChunkCols, c = e % kChunkCols;
      whole[r * kCols + k * kChunkCols + c] = chunk(r, c);   // logical access: undoes the swizzle
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < kRows * kCols; e += kThreads) out[e] = whole[e];
  if (bad) atomicAdd(errors, bad);
}
template <int kStages, int kRows, int kCols, int kChunkCols, typename WarpLayout>
static int run_pipeline_roundtrip(const void* in, void* out, int* errors) {
  auto kern = k_pipeline_roundtrip<kStages, kRows, kCols, kChunkCols, WarpLayout>;
  const int lds = (kStages * kRows * kChunkCols + kRows * kCols) * 2;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -2;
  hipLaunchKernelGGL(kern, dim3(1), dim3(tl::get_numel<WarpLayout> * WARP_SIZE), lds, 0, static_cast<const __half*>(in),
                     static_cast<__half*>(out), errors);
  return launch_status();
}
TT_API int tt_pipeline_roundtrip(int variant, const void* in, void* out, int* errors) {
  switch (variant) {
    case 0: return run_pipeline_roundtrip<2, 64, 256, 64, tl::RowMajor<2, 2>>(in, out, errors);
    case 1: return run_pipeline_roundtrip<3, 64, 256, 64, tl::RowMajor<2, 2>>(in, out, errors);
    case 2: return run_pipeline_roundtrip<3, 64, 512, 64, tl::RowMajor<1, 1>>(in, out, errors);
    case 3: return run_pipeline_roundtrip<4, 32, 512, 64, tl::RowMajor<2, 1>>(in, out, errors);
    default: return -1;
  }
}
TT_API void tt_pipeline_shape(int variant, int* rows, int* cols) {
  static const int t[4][2] = {{64, 256}, {64, 256}, {64, 512}, {32, 512}};
  *rows = t[variant][0]; *cols = t[variant][1];
}

// ---- 10. a strided sub-tile as the loader's destination (the register-staged path), next to an
//          asynchronous load of the other half of the same LDS tile --------------------------------
__global__ void k_g2s_subtile(const __half* in, __half* out) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char buf[];
  using WarpLayout = tl::RowMajor<2, 2>;
  using Global = GlobalTile<__half, tl::RowMajor<64, 128>>;
  using GIter = GTileIterator<Global, TileShape<64, 64>>;
  using Shared = SharedTile<__half, tl::RowMajor<64, 128>, true, 128>;
  using SIter = STileIterator<Shared, TileShape<64, 64>>;
  using Sub = typename SIter::NewTile;
  static_assert(!GlobalToSharedLoader<Sub, WarpLayout>::kDirectCapable, "a strided sub-tile cannot be filled LDS-direct");
  static_assert(GlobalToSharedLoader<Shared, WarpLayout>::kDirectCapable, "a whole contiguous tile can");
  __half* lds = reinterpret_cast<__half*>(buf);
  for (int e = threadIdx.x; e < 64 * 128; e += 256) lds[e] = __float2half(-1.f);
  __syncthreads();
  Global g(in);
  GIter gi(in);
  Shared s(lds);
  SIter si(lds);
  GlobalToSharedLoader<Sub, WarpLayout> load_sub;
  auto right = si(1);
  load_sub(gi(1), right);           // right half only
  __copy_async();
  __syncthreads();
  SharedToGlobalStorer<Shared, WarpLayout> store;
  Global go(out);
  store(s, go);
}
TT_API int tt_g2s_subtile(const void* in, void* out) {
  hipLaunchKernelGGL(k_g2s_subtile, dim3(1), dim3(256), 64 * 128 * 2, 0, static_cast<const __half*>(in),
                     static_cast<__half*>(out));
  return launch_status();
}

// ---- 11. where a wavefront's share of a tile starts and how many base tiles it walks over:
//          warp::GlobalOffsetHelper / SharedOffsetHelper / ExecCounter for the three WarpReuse
//          modes (include/cell/copy/warp.hpp:158-300) -------------------------------------------
template <typename WarpLayout, WarpReuse kMode, typename Tile, typename BaseShape>
__global__ void k_warp_helpers(long long* out) {
  using Exec = warp::ExecCounter<BaseShape, Tile, WarpLayout, kMode>;
  const int wid = threadIdx.x / WARP_SIZE;
  if (threadIdx.x % WARP_SIZE == 0) {
    out[wid * 6 + 0] = warp::warp_row_id<WarpLayout>();
    out[wid * 6 + 1] = warp::warp_col_id<WarpLayout>();
    out[wid * 6 + 2] = warp::GlobalOffsetHelper<WarpLayout, kMode>{}.template get_warp_offset<Tile>();
    out[wid * 6 + 3] = warp::SharedOffsetHelper<WarpLayout, BaseShape, Tile, kMode>{}.get_warp_offset();
    out[wid * 6 + 4] = Exec::row_exec_count();
    out[wid * 6 + 5] = Exec::col_exec_count();
  }
}
struct Base16x16 { static constexpr int kRows = 16, kCols = 16; };
struct Base16x32 { static constexpr int kRows = 16, kCols = 32; };
struct Base32x16 { static constexpr int kRows = 32, kCols = 16; };
template <typename WarpLayout, typename Tile, typename BaseShape>
static int run_warp_helpers(int mode, long long* out) {
  const dim3 block(tl::get_numel<WarpLayout> * WARP_SIZE);
  if (mode == 0) hipLaunchKernelGGL((k_warp_helpers<WarpLayout, WarpReuse::kCont, Tile, BaseShape>), dim3(1), block, 0, 0, out);
  else if (mode == 1) hipLaunchKernelGGL((k_warp_helpers<WarpLayout, WarpReuse::kRowReuseCont, Tile, BaseShape>), dim3(1), block, 0, 0, out);
  else hipLaunchKernelGGL((k_warp_helpers<WarpLayout, WarpReuse::kColReuseCont, Tile, BaseShape>), dim3(1), block, 0, 0, out);
  return launch_status();
}
// layout 0: RowMajor<2,2> wavefronts, row-major [128, 256] tile with row stride 512
// layout 1: RowMajor<4,1> wavefronts, row-major [128, 64] tile
// layout 2: ColMajor<2,2> wavefronts, column-major [128, 64] tile with column stride 256
TT_API int tt_warp_helpers(int layout, int mode, long long* out) {
  switch (layout) {
    case 0: return run_warp_helpers<tl::RowMajor<2, 2>, GlobalTile<__half, tl::RowMajor<128, 256, 512>>, Base16x32>(mode, out);
    case 1: return run_warp_helpers<tl::RowMajor<4, 1>, GlobalTile<__half, tl::RowMajor<128, 64>>, Base16x32>(mode, out);
    case 2: return run_warp_helpers<tl::ColMajor<2, 2>, GlobalTile<__half, tl::ColMajor<128, 64, 256>>, Base32x16>(mode, out);
    // layout 3: as layout 0 with square 16 x 16 base tiles
    case 3: return run_warp_helpers<tl::RowMajor<2, 2>, GlobalTile<__half, tl::RowMajor<128, 256, 512>>, Base16x16>(mode, out);
    default: return -1;
  }
}

// ---- 12. STileIterator2 over plain, block and block-swizzled layouts: the six layouts of
//          tests/cpp/types/test_stile_iterator.cu:48-236 (print-only there) -----------------------
template <typename Shared, typename SIter>
__global__ void k_stile_iterator2(float* out_xy, float* out_rows, float* out_cols, float* out_single) {
  extern __shared__ __attribute__((aligned(16))) unsigned char buf[];
  using DType = typename Shared::DType;
  DType* lds = reinterpret_cast<DType*>(buf);
  for (int i = 0; i < Shared::kNumel; ++i) lds[i] = static_cast<DType>((float)i);
  Shared tile(lds);
  SIter it(&tile);
  constexpr int cr = SIter::kChunkRows, cc = SIter::kChunkCols;
  for (int x = 0; x < SIter::sc0; ++x)
    for (int y = 0; y < SIter::sc1; ++y) {
      auto sub = it(x, y);
      auto row_strip = it(x, _);
      auto col_strip = it(_, y);
      auto sub_r = row_strip(y);
      auto sub_c = col_strip(x);
      for (int r = 0; r < cr; ++r)
        for (int c = 0; c < cc; ++c) {
          const int o = ((x * SIter::sc1 + y) * cr + r) * cc + c;
          out_xy[o] = to_float(sub(r, c));
          out_rows[o] = to_float(sub_r(r, c));
          out_cols[o] = to_float(sub_c(r, c));
          if constexpr (SIter::sc0 == 1 || SIter::sc1 == 1) out_single[o] = to_float(it(SIter::sc0 == 1 ? y : x)(r, c));
        }
    }
  // to_tile gives the parent back
  auto parent = it.to_tile();
  if (parent.data() != tile.data()) out_xy[0] = -1.f;
}
template <typename Layout, int kChunkRows, int kChunkCols>
static int run_stile_iterator2(float* a, float* b, float* c, float* d) {
  using Shared = SharedTile<__half, Layout>;
  using SIter = STileIterator2<Shared, TileShape<kChunkRows, kChunkCols>>;
  hipLaunchKernelGGL((k_stile_iterator2<Shared, SIter>), dim3(1), dim3(1), Shared::kNumel * 2, 0, a, b, c, d);
  return launch_status();
}
TT_API int tt_stile_iterator2(int variant, float* out_xy, float* out_rows, float* out_cols, float* out_single) {
  switch (variant) {
    case 0: return run_stile_iterator2<tl::RowMajor<4, 24>, 4, 8>(out_xy, out_rows, out_cols, out_single);
    case 1: return run_stile_iterator2<tl::ColMajor<24, 4>, 8, 4>(out_xy, out_rows, out_cols, out_single);
    case 2: return run_stile_iterator2<tl::BlockRowMajor<tl::RowMajor<4, 16>, tl::RowMajor<2, 4>>, 4, 8>(out_xy, out_rows, out_cols, out_single);
    case 3: return run_stile_iterator2<tl::BlockColMajor<tl::ColMajor<16, 4>, tl::ColMajor<4, 2>>, 8, 4>(out_xy, out_rows, out_cols, out_single);
    case 4: return run_stile_iterator2<tl::BlockRowMajor<tl::RowMajor<8, 16>, SwizzledLayout<tl::RowMajor<2, 4>, Swizzle<1, 0, 2>>>, 8, 4>(out_xy, out_rows, out_cols, out_single);
    case 5: return run_stile_iterator2<tl::BlockColMajor<tl::ColMajor<32, 8>, SwizzledLayout<tl::ColMajor<4, 4>, Swizzle<2, 0, 2>>>, 8, 8>(out_xy, out_rows, out_cols, out_single);
    // a genuinely two-dimensional chunking (the reference leaves (x, y) unimplemented)
    case 6: return run_stile_iterator2<tl::BlockRowMajor<tl::RowMajor<8, 16>, tl::RowMajor<2, 4>>, 4, 8>(out_xy, out_rows, out_cols, out_single);
    case 7: return run_stile_iterator2<tl::RowMajor<8, 16>, 2, 4>(out_xy, out_rows, out_cols, out_single);
    default: return -1;
  }
}

// ---- 13. register-to-register copies, fixed-width vector moves and the remaining functors
//          (include/cell/copy/register.hpp:10-41, vectorize.hpp:14-59, math_functor.hpp) ----------
__global__ void k_reg_copy(const float* in, float* out_tile, float* out_base) {
  using WarpLayout = tl::RowMajor<1, 1>;
  using Global = GlobalTile<float, tl::RowMajor<32, 64>>;
  using Reg = RegTile<BaseTileRowMajor<float>, tl::RowMajor<2, 4>>;
  Global g(in), go(out_tile), gb(out_base);
  Reg r, copy, only_one;
  GlobalToRegLoader<Reg, WarpLayout, WarpReuse::kCont> g2r;
  g2r(g, r);
  RegTileCopy<Reg> tile_copy;
  tile_copy(r, copy);
  BaseTileCopy<typename Reg::DType> base_copy;
  base_copy(r(1, 2), only_one(1, 2));   // one base tile; the rest stays zero
  RegToGlobalStorer<Global, Reg, WarpLayout> r2g;
  r2g(copy, go);
  r2g(only_one, gb);
}
TT_API int tt_reg_copy(const void* in, void* out_tile, void* out_base) {
  hipLaunchKernelGGL(k_reg_copy, dim3(1), dim3(64), 0, 0, static_cast<const float*>(in), static_cast<float*>(out_tile),
                     static_cast<float*>(out_base));
  return launch_status();
}
__global__ void k_vectorize(const __half* hin, __half* hout, const float* fin, float* fout) {
  const int t = threadIdx.x;
  Vectorize<__half, 2> h2;   // 32 bits
  Vectorize<__half, 4> h4;   // 64 bits
  Vectorize<__half, 8> h8;   // 128 bits
  Vectorize<float, 2> f2;
  Vectorize<float, 4> f4;
  static_assert(Vectorize<__half, 8>::vectorize_bits == 128 && Vectorize<float, 2>::vectorize_bits == 64 &&
                Vectorize<__half, 2>::vectorize_nums == 2);
  h2(hin + 2 * t, hout + 2 * t);                      // elements [0, 128)
  h4(hin + 128 + 4 * t, hout + 128 + 4 * t);          // [128, 384)
  h8(hin + 384 + 8 * t, hout + 384 + 8 * t);          // [384, 896)
  f2(fin + 2 * t, fout + 2 * t);                      // [0, 128)
  f4.copy(fin + 128 + 4 * t, fout + 128 + 4 * t);     // [128, 384)
}
TT_API int tt_vectorize(const void* hin, void* hout, const void* fin, void* fout) {
  hipLaunchKernelGGL(k_vectorize, dim3(1), dim3(64), 0, 0, static_cast<const __half*>(hin), static_cast<__half*>(hout),
                     static_cast<const float*>(fin), static_cast<float*>(fout));
  return launch_status();
}
// out_add = x + rowvec (BroadcastAdd), out_log = log(relu(x) + 1), out_min = min(x, y),
// out_div = x / (|y| + 1), out_max = max(x, y), out_mul = rowvec * x (BroadcastMul), out_sub = x - y
__global__ void k_functors(const float* xin, const float* yin, float* out_add, float* out_log, float* out_min,
                           float* out_div, float* out_max, float* out_mul, float* out_sub) {
  using WarpLayout = tl::RowMajor<2, 1>;
  using Global = GlobalTile<float, tl::RowMajor<64, 32>>;
  using Reg = RegTile<BaseTileRowMajor<float>, tl::RowMajor<2, 2>>;
  using Vec = RegTile<float, tl::RowMajor<Reg::kRows, 1>>;
  Global gx(xin), gy(yin);
  Reg x, y, t, one;
  GlobalToRegLoader<Reg, WarpLayout, WarpReuse::kCont> g2r;
  g2r(gx, x);
  g2r(gy, y);
  RegToGlobalStorer<Global, Reg, WarpLayout> r2g;
  // the row vector: row sums of x
  Vec v;
  compute::SumReduce<Reg, tl::Layout::kRowMajor> rsum;
  rsum(x, v);
  { copy_tile(x, t); compute::BroadcastAdd<Vec, Reg, tl::Layout::kRowMajor> f; f(v, t); Global g(out_add); r2g(t, g); }
  { copy_tile(x, t); compute::BroadcastMul<Vec, Reg, tl::Layout::kRowMajor> f; f(v, t); Global g(out_mul); r2g(t, g); }
  {
    compute::RegTileRelu<Reg> relu; relu(x, t);
    compute::BroadcastScalar<Reg, compute::Add<float>> add1; add1(t, 1.0f, t);
    compute::RegTileLog<Reg> lg; lg(t, t);
    Global g(out_log); r2g(t, g);
  }
  { compute::RegTileMin<Reg> f; f(x, y, t); Global g(out_min); r2g(t, g); }
  { compute::RegTileMax<Reg> f; f(x, y, t); Global g(out_max); r2g(t, g); }
  { compute::RegTileSub<Reg> f; f(x, y, t); Global g(out_sub); r2g(t, g); }
  {
    compute::RegTileMul<Reg> sq; sq(y, y, one);                                   // y^2
    compute::BroadcastScalar<Reg, compute::Add<float>> add1; add1(one, 1.0f, one);  // y^2 + 1
    compute::RegTileDiv<Reg> f; f(x, one, t);
    Global g(out_div); r2g(t, g);
  }
}
TT_API int tt_functors(const void* x, const void* y, void* o_add, void* o_log, void* o_min, void* o_div, void* o_max,
                       void* o_mul, void* o_sub) {
  hipLaunchKernelGGL(k_functors, dim3(1), dim3(128), 0, 0, static_cast<const float*>(x), static_cast<const float*>(y),
                     static_cast<float*>(o_add), static_cast<float*>(o_log), static_cast<float*>(o_min),
                     static_cast<float*>(o_div), static_cast<float*>(o_max), static_cast<float*>(o_mul),
                     static_cast<float*>(o_sub));
  return launch_status();
}
