// Compile-time and host-run checks of the tile types: the integer known answers of the
// reference's tests/cpp/types/test_{layout,swizzle,gtile_iterator,warp_base_tile_shape}.cu,
// restated for the headers under tilefusion_amd/include.  Builds to a host executable that
// prints "ok" (no GPU needed).
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "types/mod.hpp"

using namespace tilefusion;
namespace tl = tile_layout;

#define CHECK(cond)                                                     \
  do {                                                                  \
    if (!(cond)) {                                                      \
      printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);          \
      exit(1);                                                          \
    }                                                                   \
  } while (0)

// ---- test_layout.cu:12-38 ------------------------------------------------------------------
using L1 = tl::RowMajor<4, 7>;
static_assert(tl::num_rows<L1> == 4 && tl::num_cols<L1> == 7 && tl::get_numel<L1> == 28);
static_assert(tl::row_stride<L1> == 7 && tl::col_stride<L1> == 1 && tl::layout_type<L1> == tl::Layout::kRowMajor);
using L2 = tl::ColMajor<4, 7>;
static_assert(tl::row_stride<L2> == 1 && tl::col_stride<L2> == 4 && tl::layout_type<L2> == tl::Layout::kColMajor);
static_assert(tl::is_contiguous<L1>::value && !tl::is_contiguous<tl::RowMajor<4, 7, 9>>::value);

// ---- test_layout.cu:40-120 -----------------------------------------------------------------
using BR = tl::BlockRowMajor<tl::RowMajor<14, 9>, tl::RowMajor<2, 3>>;
static_assert(BR::kTileRows == 7 && BR::kTileCols == 3 && BR::kRowStride == 18 && BR::kColStride == 6);
static_assert(BR{}(2, 0) == 18 && BR{}(2, 1) == 19 && BR{}(4, 3) == 42 && BR{}(4, 4) == 43);
using BC = tl::BlockColMajor<tl::ColMajor<14, 9>, tl::ColMajor<2, 3>>;
static_assert(BC::kRowStride == 6 && BC::kColStride == 42 && BC::kType == tl::Layout::kColMajor);
static_assert(BC{}(6, 0) == 18 && BC{}(7, 0) == 19 && BC{}(0, 3) == 42 && BC{}(1, 3) == 43);
using BM1 = tl::BlockMixed<tl::RowMajor<14, 9>, tl::ColMajor<2, 3>>;
static_assert(BM1{}(2, 0) == 18 && BM1{}(3, 0) == 19 && BM1{}(4, 3) == 42 && BM1{}(5, 3) == 43);
using BM2 = tl::BlockMixed<tl::ColMajor<14, 9>, tl::RowMajor<2, 3>>;
static_assert(BM2{}(6, 0) == 18 && BM2{}(6, 1) == 19 && BM2{}(0, 3) == 42 && BM2{}(0, 4) == 43);

// ---- test_swizzle.cu:19-64 -----------------------------------------------------------------
constexpr int swizzle_ref(int x, int y, int m, int s) { return (x << (m + s)) | ((x ^ (y >> m)) << m) | (y & ((1 << m) - 1)); }
static_assert(Swizzle<3, 3, 3>{}(0) == swizzle_ref(0, 0, 3, 3));
static_assert(Swizzle<3, 3, 3>{}(1 * 64 + 0) == swizzle_ref(1, 0, 3, 3));
static_assert(Swizzle<3, 3, 3>{}(1 * 64 + 4) == swizzle_ref(1, 4, 3, 3));
static_assert(Swizzle<3, 3, 3>{}(2 * 64 + 0) == swizzle_ref(2, 0, 3, 3));
static_assert(Swizzle<3, 3, 3>{}(2 * 64 + 4) == swizzle_ref(2, 4, 3, 3));

// ---- test_warp_base_tile_shape.cu:10-188 (32 lanes: the reference's answers; 64: ours) -------
template <typename T, int R, int C, tl::Layout K, int W, int er, int ec, int tr, int tc>
constexpr bool wbt() {
  using X = WarpBaseTileShape<T, TileShape<R, C>, K, W>;
  return X::kRows == er && X::kCols == ec && X::WarpThreadLayout::kRows == tr && X::WarpThreadLayout::kCols == tc;
}
constexpr auto RM = tl::Layout::kRowMajor, CM = tl::Layout::kColMajor;
static_assert(wbt<__half, 128, 8, RM, 32, 32, 8, 32, 1>() && wbt<__half, 64, 16, RM, 32, 16, 16, 16, 2>());
static_assert(wbt<__half, 16, 32, RM, 32, 8, 32, 8, 4>() && wbt<__half, 128, 128, RM, 32, 4, 64, 4, 8>());
static_assert(wbt<__half, 8, 128, CM, 32, 8, 32, 1, 32>() && wbt<__half, 16, 64, CM, 32, 16, 16, 2, 16>());
static_assert(wbt<__half, 32, 16, CM, 32, 32, 8, 4, 8>() && wbt<__half, 128, 128, CM, 32, 64, 4, 8, 4>());
static_assert(wbt<float, 128, 4, RM, 32, 32, 4, 32, 1>() && wbt<float, 64, 8, RM, 32, 16, 8, 16, 2>());
static_assert(wbt<float, 16, 16, RM, 32, 8, 16, 8, 4>() && wbt<float, 128, 128, RM, 32, 4, 32, 4, 8>());
static_assert(wbt<float, 4, 128, CM, 32, 4, 32, 1, 32>() && wbt<float, 8, 64, CM, 32, 8, 16, 2, 16>());
static_assert(wbt<float, 16, 32, CM, 32, 16, 8, 4, 8>() && wbt<float, 128, 128, CM, 32, 32, 4, 8, 4>());
static_assert(wbt<__half, 128, 128, RM, 64, 8, 64, 8, 8>() && wbt<__half, 128, 128, CM, 64, 64, 8, 8, 8>());
static_assert(wbt<float, 128, 128, RM, 64, 8, 32, 8, 8>() && wbt<__half, 64, 16, RM, 64, 32, 16, 32, 2>());

// ---- base tiles ------------------------------------------------------------------------------
// square base tiles for every type (include/types/base.hpp:62-68), 4 elements per lane on 64 lanes
static_assert(BaseTileShape<__half>::kRows == 16 && BaseTileShape<__half>::kCols == 16 && BaseTileShape<float>::kRows == 16 &&
              BaseTileShape<float>::kCols == 16 && BaseTileShape<__bfloat16>::kNumel == 256);
static_assert(BaseTileRowMajor<__half>::kNumel == 4 && BaseTileColMajor<__half>::kNumel == 4 && BaseTileRowMajor<float>::kNumel == 4 &&
              BaseTileRowMajor<float>::kNumel * WARP_SIZE == BaseTileShape<float>::kNumel);
static_assert(BaseTileTraits<BaseTileRowMajor<float>>::kIsRowMajor && !BaseTileTraits<BaseTileColMajor<__half>>::kIsRowMajor &&
              BaseTileTraits<BaseTileRowMajor<__half>>::kRows == 16 && BaseTileTraits<BaseTileRowMajor<__half>>::kCols == 16);
static_assert(WideBaseTileShape<__half>::kCols == 32 && WideBaseTileRowMajor<__half>::kNumel == 8 &&
              BaseTileTraits<WideBaseTileRowMajor<__half>>::kCols == 32 && BaseTileTraits<WideBaseTileColMajor<__half>>::kRows == 32 &&
              BaseTileTraits<WideBaseTileColMajor<__half>>::kCols == 16);
static_assert(dim_size<0, TileShape<128, 32>> == 128 && dim_size<1, TileShape<128, 32>> == 32 && get_numel<TileShape<2, 3, 4>> == 24);

int main() {
  // ---- test_swizzle.cu:66-105: swizzled block layouts equal the CuTe closed form -------------
  {
    using Lay = tl::BlockRowMajor<tl::RowMajor<16, 64>, SwizzledLayout<tl::RowMajor<8, 64>, Swizzle<3, 3, 3>>>;
    Lay lay;
    for (int i = 0; i < 16; ++i)
      for (int j = 0; j < 64; ++j) {
        const int idx = i * 64 + j;
        CHECK(lay(i, j) == (idx ^ (((idx >> 6) & 7) << 3)));
      }
    using LayC = tl::BlockColMajor<tl::ColMajor<64, 16>, SwizzledLayout<tl::ColMajor<64, 8>, Swizzle<3, 3, 3>>>;
    LayC layc;
    for (int i = 0; i < 64; ++i)
      for (int j = 0; j < 16; ++j) {
        const int idx = j * 64 + i;
        CHECK(layc(i, j) == (idx ^ (((idx >> 6) & 7) << 3)));
      }
  }
  // ---- test_gtile_iterator.cu:146-158 --------------------------------------------------------
  {
    std::vector<float> data(36);
    for (int i = 0; i < 36; ++i) data[i] = float(i);
    using Tile = GlobalTile<float, tl::RowMajor<4, 9>>;
    using Iter = GTileIterator<Tile, TileShape<2, 3>>;
    static_assert(Iter::sc0 == 2 && Iter::sc1 == 3);
    Iter iter(data.data());
    for (int i = 0; i < Iter::sc0; ++i)
      for (int j = 0; j < Iter::sc1; ++j) {
        auto tile = iter(i, j);
        const int start = i * 2 * 9 + j * 3;
        for (int m = 0; m < 2; ++m)
          for (int n = 0; n < 3; ++n) CHECK(int(tile(m, n)) == start + m * 9 + n);
      }
    using TileC = GlobalTile<float, tl::ColMajor<4, 9>>;
    using IterC = TileIterator<TileC, TileShape<2, 3>>;
    IterC iterc(data.data());
    for (int i = 0; i < IterC::sc0; ++i)
      for (int j = 0; j < IterC::sc1; ++j) {
        auto tile = iterc(i, j);
        const int start = i * 2 + j * 3 * 4;
        for (int m = 0; m < 2; ++m)
          for (int n = 0; n < 3; ++n) CHECK(int(tile(m, n)) == start + m + n * 4);
      }
    // slices: (x, _) is a 1 x sc1 iterator, (_, y) a sc0 x 1 iterator
    auto row1 = iter(1, _);
    static_assert(decltype(row1)::sc0 == 1 && decltype(row1)::sc1 == 3);
    CHECK(int(row1(2)(0, 0)) == 2 * 9 + 6);
    auto col2 = iter(_, 2);
    static_assert(decltype(col2)::sc0 == 2 && decltype(col2)::sc1 == 1);
    CHECK(int(col2(1)(1, 2)) == 3 * 9 + 8);
    // chunk offsets are 64-bit: a row-major tile with 2^31 elements does not wrap
    using Big = GlobalTile<__half, tl::RowMajor<32768, 65536>>;
    using BigIter = GTileIterator<Big, TileShape<512, 65536>>;
    static_assert(BigIter::chunk_offset(63, 0) == ptrdiff_t(63) * 512 * 65536);
  }
  printf("ok\n");
  return 0;
}
