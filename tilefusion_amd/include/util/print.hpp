// Device-side tile dumps for debugging (counterpart of include/util/print.hpp:13-158).
#pragma once

#include <cstdio>

#include "types/base.hpp"

namespace tilefusion::util {

template <typename DType, typename Layout>
DEVICE void print_tile(const DType* data, const Layout& layout) {
  for (int i = 0; i < Layout::kRows; ++i) {
    for (int j = 0; j < Layout::kCols; ++j) printf("%.3f, ", to_float(data[layout(i, j)]));
    printf("\n");
  }
}

}  // namespace tilefusion::util
