// scatter_nd for gfx950: data[indices[i, 0..k-1], ...] += updates[i, ...] for every index row i
// (duplicates accumulate), fp32 / fp16 / bf16.
//
// Counterpart of ke_scatter_nd and its host launcher (src/kernels/scatter_nd.cu:10-95).  What
// differs: one thread per (index row, slice element) so that a slice is read and written with
// consecutive lanes (the reference walks a slice serially in one thread); the strides travel
// as kernel arguments (the reference cudaMallocs them per call and never frees them); index
// rows that point outside `data` are skipped instead of written out of bounds.
#include <hip/hip_bf16.h>

#include "common.hpp"

namespace tfk {
namespace {

constexpr int kMaxRank = 8;
struct Strides {
  long long stride[kMaxRank];  // element stride of the first k dimensions of data
  long long dim[kMaxRank];     // their extents
};

TFK_DEVICE void atomic_add(float* p, float v) { atomicAdd(p, v); }

// 16-bit types: compare-and-swap on the aligned 32-bit word that holds the element
template <typename T>
TFK_DEVICE void atomic_add_16(T* p, T v) {
  const size_t addr = reinterpret_cast<size_t>(p);
  unsigned* word = reinterpret_cast<unsigned*>(addr & ~size_t(3));
  const bool high = addr & 2;
  unsigned old = *word, assumed;
  do {
    assumed = old;
    const unsigned short cur = high ? (assumed >> 16) : (assumed & 0xffffu);
    T x = __builtin_bit_cast(T, cur);
    x = (T)((float)x + (float)v);
    const unsigned short nxt = __builtin_bit_cast(unsigned short, x);
    const unsigned repl = high ? ((assumed & 0xffffu) | ((unsigned)nxt << 16)) : ((assumed & 0xffff0000u) | nxt);
    old = atomicCAS(word, assumed, repl);
  } while (old != assumed);
}
TFK_DEVICE void atomic_add(half_t* p, half_t v) { atomic_add_16(p, v); }
TFK_DEVICE void atomic_add(__bf16* p, __bf16 v) { atomic_add_16(p, v); }

template <typename T>
__global__ __launch_bounds__(256) void scatter_nd_kernel(const T* __restrict__ updates, T* __restrict__ data,
                                                         const long long* __restrict__ indices, Strides s,
                                                         long long n, int k, long long slice) {
  const long long total = n * slice;
  for (long long t = blockIdx.x * (long long)blockDim.x + threadIdx.x; t < total;
       t += (long long)gridDim.x * blockDim.x) {
    const long long row = t / slice, off = t - row * slice;
    long long base = 0;
    bool inside = true;
    for (int j = 0; j < k; ++j) {
      const long long ix = indices[row * k + j];
      inside &= ix >= 0 && ix < s.dim[j];
      base += ix * s.stride[j];
    }
    if (inside) atomic_add(data + base + off, updates[t]);
  }
}

template <typename T>
int launch(const void* updates, void* data, const long long* indices, const Strides& s, long long n, int k,
           long long slice, hipStream_t st) {
  const long long total = n * slice;
  const int grid = (int)std::min<long long>((total + 255) / 256, 256 * 32);
  hipLaunchKernelGGL(scatter_nd_kernel<T>, dim3(grid), dim3(256), 0, st, static_cast<const T*>(updates),
                     static_cast<T*>(data), indices, s, n, k, slice);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}

}  // namespace
}  // namespace tfk

extern "C" int tf_scatter_nd(const void* updates, void* data, const int64_t* indices, const int64_t* data_dims,
                             int rank, int64_t num_index_rows, int index_depth, int dtype, void* stream) {
  using namespace tfk;
  TFK_REQUIRE(updates && data && indices && data_dims, TF_ERR_INVALID_ARG, "tf_scatter_nd: null pointer");
  TFK_REQUIRE(rank >= 1 && rank <= kMaxRank, TF_ERR_INVALID_ARG, "tf_scatter_nd: rank %d outside 1..%d", rank,
              kMaxRank);
  TFK_REQUIRE(index_depth >= 1 && index_depth <= rank, TF_ERR_INVALID_ARG,
              "tf_scatter_nd: index depth %d outside 1..rank (%d)", index_depth, rank);
  TFK_REQUIRE(num_index_rows >= 0, TF_ERR_INVALID_ARG, "tf_scatter_nd: negative number of index rows");
  TFK_REQUIRE(dtype >= 0 && dtype <= 2, TF_ERR_UNSUPPORTED, "tf_scatter_nd: dtype %d (0 f32, 1 f16, 2 bf16)", dtype);
  Strides s{};
  long long stride = 1;
  for (int i = rank - 1; i >= 0; --i) {
    TFK_REQUIRE(data_dims[i] > 0, TF_ERR_INVALID_ARG, "tf_scatter_nd: data dimension %d is not positive", i);
    if (i < index_depth) {
      s.stride[i] = stride;
      s.dim[i] = data_dims[i];
    }
    stride *= data_dims[i];
  }
  long long slice = 1;
  for (int i = index_depth; i < rank; ++i) slice *= data_dims[i];
  if (num_index_rows == 0) return TF_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const long long* idx = reinterpret_cast<const long long*>(indices);
  if (dtype == 0) return launch<float>(updates, data, idx, s, num_index_rows, index_depth, slice, st);
  if (dtype == 1) return launch<half_t>(updates, data, idx, s, num_index_rows, index_depth, slice, st);
  return launch<__bf16>(updates, data, idx, s, num_index_rows, index_depth, slice, st);
}
