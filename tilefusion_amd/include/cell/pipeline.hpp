// Circular-buffer copy pipeline (counterpart of include/cell/pipeline.hpp:48-134).
//
// NUM_STAGES destination tiles form a ring; commit() copies the next chunk of the source
// iterator into the next ring slot with the `Copy` functor.  Two uses, as in the reference:
//   * global -> LDS (Copy = GlobalToSharedLoader): the copy is asynchronous, so commit() only
//     ISSUES it; the chunk is there after wait_group<N>() + a barrier;
//   * LDS -> registers (Copy = SharedToRegLoader): an ordinary load the compiler tracks, used
//     to fetch the fragments of step n+1 while step n multiplies.
// Typical schedule with one chunk in flight:
//
//   pipe.commit(); commit_copy_group();
//   for (i = 0; i < Pipeline::Iterations - 1; ++i) {
//     wait_group<0>(); __syncthreads();
//     pipe.commit(); commit_copy_group();     // chunk i + 1
//     compute(pipe.get_prev_dst());           // chunk i
//   }
//   wait_group<0>(); __syncthreads();
//   compute(pipe.get_cur_dst());
#pragma once

#include <type_traits>

#include "types/mod.hpp"
#include "util/debug.hpp"

namespace tilefusion::cell {

template <typename Element, typename SrcTile, typename DstTile, typename TileIterator, typename Copy,
          int NUM_STAGES, int Iterations_ = TileIterator::sc1 - NUM_STAGES + 1>
struct Pipeline {
  static_assert(NUM_STAGES >= 1, "a pipeline has at least one stage");
  static constexpr int Iterations = Iterations_;
  static constexpr int kNumStages = NUM_STAGES;

  // ring of NUM_STAGES tiles laid out back to back from dst_ptr
  DEVICE Pipeline(const Element* src_ptr, Element* dst_ptr)
      : next_chunk_(0), committed_(0), ring_base_(dst_ptr), contiguous_(true), src_tile_(src_ptr), tile_iter_(src_ptr) {}
  // ring of caller-provided tiles (register tiles, or LDS tiles placed elsewhere)
  DEVICE Pipeline(SrcTile src_tile, DstTile dst_tiles[])
      : next_chunk_(0), committed_(0), ring_base_(nullptr), contiguous_(false), src_tile_(src_tile), tile_iter_(src_tile.data()) {
#pragma unroll
    for (int i = 0; i < NUM_STAGES; ++i) stages_[i] = dst_tiles[i];
  }

  // Restart the chunk walk on another source tile; the ring position carries on.
  DEVICE void reset_src_tile(const Element* src_ptr) {
    src_tile_ = SrcTile(src_ptr);
    tile_iter_ = TileIterator(src_ptr);
    next_chunk_ = 0;
  }

  // Copies (or, for an asynchronous Copy, starts copying) the next chunk into the next slot.
  DEVICE void commit() {
    auto chunk = tile_iter_(next_chunk_);
    // The slot is picked by a chain of compile-time indices so that a ring of REGISTER tiles is
    // never indexed dynamically (which would push it out to scratch memory).
    const int slot = committed_ % NUM_STAGES;
    if constexpr (kPointerRing) {
      if (contiguous_) {   // slots laid out back to back: address arithmetic, no table lookup
        DstTile dst(ring_base_ + slot * DstTile::kNumel);
        copy_(chunk, dst);
        ++next_chunk_;
        ++committed_;
        return;
      }
    }
    select_and_copy<0>(slot, chunk);
    ++next_chunk_;
    ++committed_;
  }

  // The same with the ring slot named at compile time.  A ring of REGISTER tiles must be used
  // this way when the slot is not a compile-time constant after unrolling: registers cannot be
  // indexed at run time, and a run-time choice between them ends up in scratch memory.
  template <int kSlot>
  DEVICE void commit_to() {
    static_assert(kSlot >= 0 && kSlot < NUM_STAGES, "no such ring slot");
    if constexpr (kPointerRing) {
      if (contiguous_) {
        DstTile dst(ring_base_ + kSlot * DstTile::kNumel);
        copy_(tile_iter_(next_chunk_), dst);
        ++next_chunk_;
        ++committed_;
        return;
      }
    }
    copy_(tile_iter_(next_chunk_), stages_[kSlot]);
    ++next_chunk_;
    ++committed_;
  }
  template <int kSlot>
  DEVICE const DstTile& get_dst_tile() const {
    static_assert(kSlot >= 0 && kSlot < NUM_STAGES, "no such ring slot");
    static_assert(!kPointerRing, "for rings of register tiles; memory rings have get_dst_tile_by_index");
    return stages_[kSlot];
  }

  DEVICE int committed() const { return committed_; }
  DEVICE const Element* get_dst_ptr_by_index(int index) const {
    if constexpr (kPointerRing) {
      if (contiguous_) return ring_base_ + (index % NUM_STAGES) * DstTile::kNumel;
    }
    return stages_[index % NUM_STAGES].data();
  }
  // (by value: a slot of a back-to-back ring is made on the fly from its address)
  DEVICE DstTile get_dst_tile_by_index(int index) const {
    if constexpr (kPointerRing) {
      if (contiguous_) return DstTile(ring_base_ + (index % NUM_STAGES) * DstTile::kNumel);
    }
    return stages_[index % NUM_STAGES];
  }
  DEVICE const Element* get_prev_dst() const { return get_dst_ptr_by_index(committed_ - 2); }
  DEVICE const Element* get_cur_dst() const { return get_dst_ptr_by_index(committed_ - 1); }

  // Calls f(tile) with ring slot `index` picked through compile-time indices: the way to USE a
  // ring of register tiles whose slot number is only known at run time.
  template <typename F>
  DEVICE void with_dst_tile(int index, F&& f) const {
    visit<0>(index % NUM_STAGES, f);
  }

  DEVICE void dump_dst_tile_value(int index) const {
    if (thread0()) {
      printf("data[%d]:\n", index);
      get_dst_tile_by_index(index).dump_value();
    }
  }

 private:
  template <int kSlot, typename Chunk>
  DEVICE void select_and_copy(int slot, const Chunk& chunk) {
    if constexpr (kSlot + 1 == NUM_STAGES) {
      copy_(chunk, stages_[kSlot]);
    } else {
      if (slot == kSlot) copy_(chunk, stages_[kSlot]);
      else select_and_copy<kSlot + 1>(slot, chunk);
    }
  }

  template <int kSlot, typename F>
  DEVICE void visit(int slot, F& f) const {
    if constexpr (kSlot + 1 == NUM_STAGES) {
      f(stages_[kSlot]);
    } else {
      if (slot == kSlot) f(stages_[kSlot]);
      else visit<kSlot + 1>(slot, f);
    }
  }

  // a ring of tiles that are views of memory (LDS) can be addressed by pointer arithmetic
  static constexpr bool kPointerRing = std::is_constructible_v<DstTile, Element*>;

  int next_chunk_;
  int committed_;
  Element* ring_base_;   // first slot when the slots lie back to back in memory
  bool contiguous_;      // ... which is known at compile time once the constructor is inlined
  SrcTile src_tile_;
  DstTile stages_[NUM_STAGES];
  TileIterator tile_iter_;
  Copy copy_;
};

}  // namespace tilefusion::cell
