// Workgroup-cooperative global <-> LDS tile movers (counterpart of
// include/cell/copy/global_to_shared.hpp:364-497).
//
// The tile is walked in 16-byte vectors along its contiguous dimension; consecutive lanes take
// consecutive vectors, so a wavefront touches whole 128-byte lines.  All |WarpLayout| x 64
// threads of the workgroup take part.
//
// GlobalToSharedLoader is ASYNCHRONOUS whenever the destination allows it, like the reference's
// cp.async loader: the copy is issued as LDS-direct loads (global_load_lds_dwordx4, no register
// staging) and has landed only after wait_group<N>() and a barrier (__copy_async() +
// __syncthreads() in the simplest case).  An LDS-direct load writes lane l of a wavefront at
// base + 16 * l, i.e. one instruction fills 1 KiB of CONSECUTIVE LDS; the loader therefore
// walks the PHYSICAL vectors of the destination and applies the swizzle on the global side (the
// XOR swizzle is its own inverse: the logical vector that belongs in physical slot p is
// swizzle(p)).  That needs a destination that is contiguous in LDS, starts at its own base
// pointer and holds a whole number of 1 KiB blocks; any other destination (a strided sub-tile,
// a tile smaller than 1 KiB) is filled through registers (global_load_dwordx4 + ds_write_b128,
// through SharedTile::fetch_physical_offset), which the same wait_group<0>() + barrier
// completes.  kLoadsPerLane is the number of vector-memory loads each wavefront issues per
// call - the figure wait_group<N, kLoadsPerGroup>() takes.
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
  using Walk = detail::CoopVectorWalk<Shared, WarpLayout>;

  // the destination is one contiguous block of LDS made of whole 1 KiB wavefront blocks
  static constexpr int kStrided = Walk::kRowMajor ? Shared::kRowStride : Shared::kColStride;
  static constexpr int kUnit = Walk::kRowMajor ? Shared::kColStride : Shared::kRowStride;
  static constexpr bool kDirectCapable =
      kStrided == Walk::kContig && kUnit == 1 && Walk::kVectors % WARP_SIZE == 0;
  static constexpr int kWaveBlocks = Walk::kVectors / WARP_SIZE;               // 1 KiB blocks in the tile
  static constexpr int kWaves = Walk::kThreads / WARP_SIZE;
  // loads per wavefront and call (wavefronts that get one block less still issue at least
  // kLoadsPerLane of them when the blocks divide evenly, which is what wait_group needs)
  static constexpr int kLoadsPerLane =
      kDirectCapable ? kWaveBlocks / kWaves : (Walk::kVectors + Walk::kThreads - 1) / Walk::kThreads;

  template <typename Global>
  DEVICE void operator()(const Global& src, Shared& dst) {
    static_assert(Global::kRows == Shared::kRows && Global::kCols == Shared::kCols && Global::kType == Shared::kType,
                  "source and destination tiles must have the same shape and orientation");
    const DType* g = src.data();
    DType* s = dst.mutable_data();
    if constexpr (kDirectCapable) {
      if (dst.get_offset() == 0) {   // uniform: a view that starts at its own base pointer
        const int wave = threadIdx.x / WARP_SIZE, lane = threadIdx.x % WARP_SIZE;
        const unsigned lds_base = atom::lds_byte_address(s);
#pragma unroll
        for (int b = 0; b < (kWaveBlocks + kWaves - 1) / kWaves; ++b) {
          const int block = b * kWaves + wave;                 // 1 KiB block of this wavefront
          if (kWaveBlocks % kWaves != 0 && block >= kWaveBlocks) break;
          const int phys = (block * WARP_SIZE + lane) * Walk::kVec;          // element offset in LDS
          const int logical = dst.fetch_physical_offset(phys);               // the swizzle is an involution
          const int line = logical / kStrided, pos = logical % kStrided;
          const int r = Walk::kRowMajor ? line : pos, c = Walk::kRowMajor ? pos : line;
          atom::ld_global_direct_to_shared_16B(
              lds_base + block * (WARP_SIZE * 16),
              g + ptrdiff_t(r) * Global::kRowStride + ptrdiff_t(c) * Global::kColStride);
        }
        return;
      }
    }
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
