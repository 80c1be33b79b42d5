// Circular-buffer copy pipeline (counterpart of include/cell/pipeline.hpp:48-134): NUM_STAGES
// destination tiles; commit() copies the next chunk of the source iterator into the next stage.
#pragma once

#include "types/mod.hpp"

namespace tilefusion::cell {

template <typename Element, typename SrcTile, typename DstTile, typename TileIterator, typename Copy,
          int NUM_STAGES, int Iterations_ = TileIterator::sc1 - NUM_STAGES + 1>
struct Pipeline {
  static constexpr int Iterations = Iterations_;

  DEVICE Pipeline(const Element* src_ptr, Element* dst_ptr)
      : next_chunk_(0), committed_(0), src_tile_(src_ptr), tile_iter_(src_ptr) {
#pragma unroll
    for (int i = 0; i < NUM_STAGES; ++i) stages_[i] = DstTile(dst_ptr + i * DstTile::kNumel);
  }
  DEVICE Pipeline(SrcTile src_tile, DstTile dst_tiles[])
      : next_chunk_(0), committed_(0), src_tile_(src_tile), tile_iter_(src_tile.data()) {
#pragma unroll
    for (int i = 0; i < NUM_STAGES; ++i) stages_[i] = dst_tiles[i];
  }

  DEVICE void reset_src_tile(const Element* src_ptr) {
    src_tile_ = SrcTile(src_ptr);
    tile_iter_ = TileIterator(src_ptr);
    next_chunk_ = 0;
  }

  DEVICE void commit() {
    auto chunk = tile_iter_(next_chunk_++);
    copy_(chunk, stages_[committed_++ % NUM_STAGES]);
  }

  DEVICE const Element* get_dst_ptr_by_index(int index) const { return stages_[index % NUM_STAGES].data(); }
  DEVICE const DstTile& get_dst_tile_by_index(int index) const { return stages_[index % NUM_STAGES]; }
  DEVICE const Element* get_prev_dst() const { return stages_[(committed_ - 2) % NUM_STAGES].data(); }
  DEVICE const Element* get_cur_dst() const { return stages_[(committed_ - 1) % NUM_STAGES].data(); }

 private:
  int next_chunk_;
  int committed_;
  SrcTile src_tile_;
  DstTile stages_[NUM_STAGES];
  TileIterator tile_iter_;
  Copy copy_;
};

}  // namespace tilefusion::cell
