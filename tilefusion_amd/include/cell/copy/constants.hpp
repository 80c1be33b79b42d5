// How the wavefronts of a workgroup share a tile (counterpart of
// include/cell/copy/constants.hpp:7-14).
#pragma once

namespace tilefusion::cell::copy {
enum class WarpReuse {
  kCont = 0,          // wavefront (i, j) owns block (i, j) of the tile
  kRowReuseCont = 1,  // the wavefronts of row i all work on row block i, over all columns
  kColReuseCont = 2   // the wavefronts of column j all work on column block j, over all rows
};
}  // namespace tilefusion::cell::copy
