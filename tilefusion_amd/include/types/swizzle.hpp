// XOR swizzles for LDS tiles (counterpart of include/types/swizzle.hpp:16-214).
//
// Swizzle<B, M, S> permutes a 1-D index of 2^(B+S+M) elements: the S "chunk" bits (above the
// M low bits that stay together - one 16-byte vector) are XORed with the B row bits above
// them.  Rows that sit a multiple of the bank period apart then use different banks.
#pragma once

#include "types/layout.hpp"

namespace tilefusion {
namespace tl = tile_layout;

template <int kB, int kM, int kS>
struct Swizzle {
  static constexpr int Bbits = kB, Mbits = kM, Sbits = kS;
  HOST_DEVICE constexpr int operator()(int idx) const {
    const int chunk = (idx >> Mbits) & ((1 << Sbits) - 1);
    const int row = idx >> (Mbits + Sbits);
    return (row << (Mbits + Sbits)) | ((row ^ chunk) << Mbits) | (idx & ((1 << Mbits) - 1));
  }
};

template <typename Layout, typename Swizzle, tl::Layout kType = Layout::kType>
struct SwizzledLayout;

// 2^B rows of 2^(S+M) contiguous elements
template <typename Layout_, typename Swizzle_>
struct SwizzledLayout<Layout_, Swizzle_, tl::Layout::kRowMajor> {
  using Layout = Layout_;
  using Swizzle = Swizzle_;
  static constexpr int Bbits = Swizzle::Bbits, Mbits = Swizzle::Mbits, Sbits = Swizzle::Sbits;
  static_assert(Layout::kRows == (1 << Bbits) && Layout::kCols == (1 << (Mbits + Sbits)),
                "a row-major swizzled layout is 2^B rows of 2^(S+M) columns");
  static constexpr int kRows = Layout::kRows, kCols = Layout::kCols, kNumel = Layout::kNumel;
  static constexpr tl::Layout kType = Layout::kType;

  HOST_DEVICE constexpr int operator()(int x, int y) const {
    const int sw = Swizzle{}((x << (Mbits + Sbits)) | y);
    return Layout{}(sw >> (Mbits + Sbits), sw & ((1 << (Mbits + Sbits)) - 1));
  }
};

// 2^B columns of 2^(S+M) contiguous elements
template <typename Layout_, typename Swizzle_>
struct SwizzledLayout<Layout_, Swizzle_, tl::Layout::kColMajor> {
  using Layout = Layout_;
  using Swizzle = Swizzle_;
  static constexpr int Bbits = Swizzle::Bbits, Mbits = Swizzle::Mbits, Sbits = Swizzle::Sbits;
  static_assert(Layout::kRows == (1 << (Mbits + Sbits)) && Layout::kCols == (1 << Bbits),
                "a column-major swizzled layout is 2^B columns of 2^(S+M) rows");
  static constexpr int kRows = Layout::kRows, kCols = Layout::kCols, kNumel = Layout::kNumel;
  static constexpr tl::Layout kType = Layout::kType;

  HOST_DEVICE constexpr int operator()(int x, int y) const {
    const int sw = Swizzle{}((y << (Mbits + Sbits)) | x);
    return Layout{}(sw & ((1 << (Mbits + Sbits)) - 1), sw >> (Mbits + Sbits));
  }
};

template <typename Layout_, typename Swizzle_, tl::Layout kType_>
HOST std::ostream& operator<<(std::ostream& out, const SwizzledLayout<Layout_, Swizzle_, kType_>&) {
  return out << "SwizzledLayout { " << Layout_{} << ", Swizzle<" << Swizzle_::Bbits << ", " << Swizzle_::Mbits
             << ", " << Swizzle_::Sbits << "> }";
}

// The block of a SharedTile inside which the swizzle acts, for 128-byte and 64-byte rows.
template <typename Element, int kBytes>
  requires BaseType<Element>
struct SwizzleBaseTileShape {
  static_assert(kBytes == 128 || kBytes == 64, "swizzle blocks have 128- or 64-byte rows");
  using DType = Element;
  static constexpr int M = sizeof(Element) == 2 ? 3 : 2;  // 16-byte vector
  static constexpr int S = kBytes == 128 ? 3 : 2;          // vectors per row
  static constexpr int B = S;                              // rows
  static constexpr int kRows = 1 << B;
  static constexpr int kCols = 1 << (M + S);
  static constexpr int kNumel = kRows * kCols;
};

}  // namespace tilefusion
