// Workgroup-cooperative global <-> LDS tile movers (counterpart of
// include/cell/copy/global_to_shared.hpp:364-497).
//
// The tile is walked in 16-byte vectors along its contiguous dimension; consecutive lanes take
// consecutive vectors, so a wavefront reads whole 128-byte lines (8 lanes per line of fp16) and
// every lane issues global_load_dwordx4 / ds_write_b128.  The LDS side goes through
// SharedTile::fetch_physical_offset, i.e. the destination may be swizzled.  All
// |WarpLayout| x 64 threads of the workgroup take part; the caller synchronises afterwards
// (__copy_async() + __syncthreads()), like with the reference's cp.async version.
#pragma once

#include "cell/copy/copy_atom.hpp"
#include "cell/copy/warp.hpp"
#include "types/global.hpp"
#include "types/shared.hpp"

namespace tilefusion::cell::copy {
namespace tl = tile_layout;

namespace detail {
template <typename Tile, typename WarpLayout>
struct CoopVectorWalk {
  using DType = typename Tile::DType;
  static constexpr int kVec = 16 / sizeof(DType);  // elements per 16-byte vector
  static constexpr bool kRowMajor = Tile::kType == tl::Layout::kRowMajor;
  static constexpr int kContig = kRowMajor ? Tile::kCols : Tile::kRows;   // contiguous extent
  static constexpr int kLines = kRowMajor ? Tile::kRows : Tile::kCols;    // strided extent
  static_assert(kContig % kVec == 0, "the contiguous dimension must be a whole number of 16-byte vectors");
  static constexpr int kVecPerLine = kContig / kVec;
  static constexpr int kVectors = kVecPerLine * kLines;
  static constexpr int kThreads = tl::get_numel<WarpLayout> * WARP_SIZE;
  // logical (row, col) of the first element of vector v
  DEVICE static void coord(int v, int& r, int& c) {
    const int line = v / kVecPerLine, pos = (v % kVecPerLine) * kVec;
    r = kRowMajor ? line : pos;
    c = kRowMajor ? pos : line;
  }
};
}  // namespace detail

template <typename Shared_, typename WarpLayout_>
struct GlobalToSharedLoader {
  using Shared = Shared_;
  using WarpLayout = WarpLayout_;
  using DType = typename Shared::DType;

  template <typename Global>
  DEVICE void operator()(const Global& src, Shared& dst) {
    static_assert(Global::kRows == Shared::kRows && Global::kCols == Shared::kCols && Global::kType == Shared::kType,
                  "source and destination tiles must have the same shape and orientation");
    using Walk = detail::CoopVectorWalk<Shared, WarpLayout>;
    const DType* g = src.data();
    DType* s = dst.mutable_data();
#pragma unroll
    for (int v = threadIdx.x; v < Walk::kVectors; v += Walk::kThreads) {
      int r, c;
      Walk::coord(v, r, c);
      atom::ld_global_st_shared<16>(s + dst.fetch_physical_offset(r * Shared::kRowStride + c * Shared::kColStride),
                                    g + ptrdiff_t(r) * Global::kRowStride + ptrdiff_t(c) * Global::kColStride);
    }
  }
};

template <typename Shared_, typename WarpLayout_>
struct SharedToGlobalStorer {
  using Shared = Shared_;
  using WarpLayout = WarpLayout_;
  using DType = typename Shared::DType;

  template <typename Global>
  DEVICE void operator()(const Shared& src, Global& dst) {
    static_assert(Global::kRows == Shared::kRows && Global::kCols == Shared::kCols && Global::kType == Shared::kType,
                  "source and destination tiles must have the same shape and orientation");
    using Walk = detail::CoopVectorWalk<Shared, WarpLayout>;
    const DType* s = src.data();
    DType* g = dst.mutable_data();
#pragma unroll
    for (int v = threadIdx.x; v < Walk::kVectors; v += Walk::kThreads) {
      int r, c;
      Walk::coord(v, r, c);
      atom::ld_shared_st_global<16>(g + ptrdiff_t(r) * Global::kRowStride + ptrdiff_t(c) * Global::kColStride,
                                    s + src.fetch_physical_offset(r * Shared::kRowStride + c * Shared::kColStride));
    }
  }
};

}  // namespace tilefusion::cell::copy
