// Split-KV flash-decoding for gfx950: single-query attention per (batch x head) slice with the
// key/value range cut into `num_splits` chunks, followed by a log-sum-exp combine.
//
// No counterpart in the reference (it has no decoding kernel); the per-chunk algebra is the
// online softmax of include/kernels/flash_attention_device.cuh:257-301 with one query row.
// Both kernels are HBM-bound streaming kernels, MFMA is irrelevant (1 flop per byte):
//   * split kernel: grid (num_splits, batch_heads), 4 wavefronts.  One key row of 128 16-bit
//     elements is 256 bytes = 16 lanes x 16 bytes (head dimension 64: 8 lanes), so a wavefront
//     load instruction fetches 4 (8) whole rows fully coalesced; every group of 16 (8) lanes keeps
//     its own running (max, sum, o[D]) over the rows it sees and only the final merge of the 16
//     (32) groups of a workgroup goes through LDS.  The dot product is v_dot2 (fp16 or bf16) +
//     a DPP reduction inside the lane group;
//     two batches of 8 rows per group are in flight (32 KiB per wavefront), the next one
//     requested before the current one is consumed; the partials leave through streaming
//     stores (ordinary stores in the middle of the read stream cost 7% of its bandwidth);
//   * combine kernel: grid batch_heads, 128 threads, merges the fp32 partials.
// The kernels are templates of the element type (fp16 / bf16, the reference's 16-bit types,
// include/kernels/dispatch_macros.hpp:6-23) and of the head dimension (128 / 64).
// All offsets are 64-bit.
#include <mutex>
#include <type_traits>

#include "common.hpp"

namespace tfk {
namespace {

constexpr int kD = 128;   // head dimension of the benchmark configuration (and of the static entry point)
constexpr int kDecWaves = 4;
constexpr int kDecThreads = kDecWaves * kWaveSize;
constexpr int kBatchRows = 8;                // rows per lane group in one batch of loads (two batches in flight)

template <int CTRL>
TFK_DEVICE float dpp_f32(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
// Sum over a group of kLanes (16 or 8) adjacent lanes; every lane ends up with the total.
template <int kLanes>
TFK_DEVICE float group_sum(float x) {
  if constexpr (kLanes == 16) {
    x += dpp_f32<0x128>(x);  // row_ror:8
    x += dpp_f32<0x124>(x);  // row_ror:4
    x += dpp_f32<0x122>(x);  // row_ror:2
    x += dpp_f32<0x121>(x);  // row_ror:1
  } else {
    static_assert(kLanes == 8, "a key row is 16 or 8 lanes wide");
    x += dpp_f32<0x141>(x);  // row_half_mirror: lane i <-> 7 - i inside each half row
    x += dpp_f32<0xB1>(x);   // quad_perm [1, 0, 3, 2]
    x += dpp_f32<0x4E>(x);   // quad_perm [2, 3, 0, 1]
  }
  return x;
}

template <typename T>
struct Vec8 {
  using type = T __attribute__((ext_vector_type(8)));
};
template <typename T>
TFK_DEVICE float dot8(typename Vec8<T>::type k, typename Vec8<T>::type q) {
  float acc = 0.f;
#define TFK_DOT2(i)                                                                                         \
  if constexpr (std::is_same_v<T, bf16_t>)                                                                  \
    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(k, k, i, i + 1), __builtin_shufflevector(q, q, i, i + 1), acc, false); \
  else                                                                                                      \
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(k, k, i, i + 1), __builtin_shufflevector(q, q, i, i + 1), acc, false);
  TFK_DOT2(0) TFK_DOT2(2) TFK_DOT2(4) TFK_DOT2(6)
#undef TFK_DOT2
  return acc;
}

// workspace: o_part [batch_heads][num_splits][D] fp32, then ml_part [batch_heads][num_splits][2]
template <typename T, int D>
__global__ __launch_bounds__(kDecThreads) void flash_decode_split_kernel(
    const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
    float* __restrict__ o_part, float* __restrict__ ml_part, int64_t Lkv, int num_splits,
    int64_t chunk, float scale_log2) {
  using V8 = typename Vec8<T>::type;
  constexpr int kLanesPerRow = D / 8;                   // 16-byte vectors per row
  constexpr int kRowsPerWave = kWaveSize / kLanesPerRow;  // rows one wavefront load instruction covers
  constexpr int kRowsPerStep = kDecWaves * kRowsPerWave;  // ... and one workgroup load step
  constexpr int kGroups = kDecThreads / kLanesPerRow;
  __shared__ float s_o[kGroups][D];
  __shared__ float s_m[kGroups], s_l[kGroups];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lv = lane % kLanesPerRow, gw = lane / kLanesPerRow;   // vector of the row, row of the wavefront's load
  const int split = blockIdx.x;
  const int64_t bh = blockIdx.y;
  const int64_t row_begin = (int64_t)split * chunk;
  const int64_t row_end = min(row_begin + chunk, Lkv);

  const T* kbase = K + bh * Lkv * D + 8 * lv;
  const T* vbase = V + bh * Lkv * D + 8 * lv;
  const V8 q8 = *reinterpret_cast<const V8*>(Q + bh * D + 8 * lv);

  float m_run = -INFINITY, l_run = 0.f;
  float o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = 0.f;

  // Two register sets of kBatchRows rows per group: the loads of batch b+1 are issued before
  // batch b is consumed, so a wavefront always has loads on their way (a load-all / wait-all /
  // compute loop leaves the memory pipe of that wavefront empty while it computes).
  // `base` is workgroup-uniform.  A batch that lies inside the chunk is addressed as a scalar
  // base plus one per-lane 32-bit offset computed once (no per-load 64-bit arithmetic, no
  // clamps, no masks); only a batch that crosses the end of the chunk takes the clamped and
  // masked form.
  constexpr int64_t kBatchSpan = (int64_t)kBatchRows * kRowsPerStep;
  const int64_t lane_row = wave * kRowsPerWave + gw;
  const unsigned lane_off = (unsigned)(lane_row * D + 8 * lv) * 2u;   // bytes inside a batch
  const char* k_slice = reinterpret_cast<const char*>(K + bh * Lkv * D);
  const char* v_slice = reinterpret_cast<const char*>(V + bh * Lkv * D);
  auto load_batch = [&](V8* kd, V8* vd, int64_t base) __attribute__((always_inline)) {
    if (base + kBatchSpan <= row_end) {
      const char* kb = k_slice + base * (D * 2);
      const char* vb = v_slice + base * (D * 2);
#pragma unroll
      for (int u = 0; u < kBatchRows; ++u)
        kd[u] = __builtin_nontemporal_load(reinterpret_cast<const V8*>(kb + lane_off + u * (kRowsPerStep * D * 2)));
#pragma unroll
      for (int u = 0; u < kBatchRows; ++u)
        vd[u] = __builtin_nontemporal_load(reinterpret_cast<const V8*>(vb + lane_off + u * (kRowsPerStep * D * 2)));
    } else {
#pragma unroll
      for (int u = 0; u < kBatchRows; ++u) {
        const int64_t row = min(base + lane_row + (int64_t)u * kRowsPerStep, Lkv - 1);
        kd[u] = __builtin_nontemporal_load(reinterpret_cast<const V8*>(kbase + row * D));
      }
#pragma unroll
      for (int u = 0; u < kBatchRows; ++u) {
        const int64_t row = min(base + lane_row + (int64_t)u * kRowsPerStep, Lkv - 1);
        vd[u] = __builtin_nontemporal_load(reinterpret_cast<const V8*>(vbase + row * D));
      }
    }
    __builtin_amdgcn_sched_barrier(0);   // the requests leave before the other batch is consumed
  };
  auto consume = [&](const V8* kd, const V8* vd, int64_t base) __attribute__((always_inline)) {
    const bool full = base + kBatchSpan <= row_end;   // workgroup-uniform
    float s[kBatchRows];
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < kBatchRows; ++u) {
      const float d = group_sum<kLanesPerRow>(dot8<T>(kd[u], q8)) * scale_log2;
      s[u] = (full || base + lane_row + (int64_t)u * kRowsPerStep < row_end) ? d : -INFINITY;
      mx = fmaxf(mx, s[u]);
    }
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
    m_run = m_new;
    l_run *= alpha;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] *= alpha;
#pragma unroll
    for (int u = 0; u < kBatchRows; ++u) {
      const float p = __builtin_amdgcn_exp2f(s[u] - m_safe);
      l_run += p;
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] += p * (float)vd[u][i];
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  V8 k_a[kBatchRows], v_a[kBatchRows], k_b[kBatchRows], v_b[kBatchRows];
  if (row_begin < row_end) load_batch(k_a, v_a, row_begin);
  for (int64_t base = row_begin; base < row_end; base += 2 * kBatchSpan) {
    const bool more1 = base + kBatchSpan < row_end;
    if (more1) load_batch(k_b, v_b, base + kBatchSpan);
    consume(k_a, v_a, base);
    if (!more1) break;
    if (base + 2 * kBatchSpan < row_end) load_batch(k_a, v_a, base + 2 * kBatchSpan);
    consume(k_b, v_b, base + kBatchSpan);
  }

  // merge the lane groups of the workgroup
  const int grp = tid / kLanesPerRow;
#pragma unroll
  for (int i = 0; i < 8; ++i) s_o[grp][8 * lv + i] = o[i];
  if (lv == 0) {
    s_m[grp] = m_run;
    s_l[grp] = l_run;
  }
  __syncthreads();
  if (tid < D) {
    float big = -INFINITY;
#pragma unroll
    for (int g = 0; g < kGroups; ++g) big = fmaxf(big, s_m[g]);
    const float big_safe = (big == -INFINITY) ? 0.f : big;
    float acc = 0.f, l = 0.f;
#pragma unroll
    for (int g = 0; g < kGroups; ++g) {
      const float w = __builtin_amdgcn_exp2f(s_m[g] - big_safe);
      acc += w * s_o[g][tid];
      l += w * s_l[g];
    }
    const int64_t idx = bh * num_splits + split;
    // Streaming stores: an ordinary store of these few hundred bytes per workgroup, issued in
    // the middle of an 8 GiB read stream, costs 7% of the read bandwidth (6.6 against 7.15
    // TB/s in a plain two-stream read kernel with and without such a store; 7.05 with this one).
    __builtin_nontemporal_store(acc, o_part + idx * D + tid);
    if (tid == 0) {
      __builtin_nontemporal_store(big, ml_part + idx * 2);
      __builtin_nontemporal_store(l, ml_part + idx * 2 + 1);
    }
  }
}

template <typename T, int D>
__global__ __launch_bounds__(D) void flash_decode_combine_kernel(
    const float* __restrict__ o_part, const float* __restrict__ ml_part, T* __restrict__ O,
    int num_splits) {
  const int64_t bh = blockIdx.x;
  const int d = threadIdx.x;
  const float* ml = ml_part + bh * num_splits * 2;
  const float* op = o_part + bh * num_splits * D + d;
  float big = -INFINITY;
  for (int s = 0; s < num_splits; ++s) big = fmaxf(big, ml[2 * s]);
  float acc = 0.f, l = 0.f;
#pragma unroll 8
  for (int s = 0; s < num_splits; ++s) {
    const float w = __builtin_amdgcn_exp2f(ml[2 * s] - big);
    acc += w * op[(int64_t)s * D];
    l += w * ml[2 * s + 1];
  }
  O[bh * D + d] = (T)(acc / l);
}

}  // namespace
}  // namespace tfk

extern "C" size_t tf_flash_decode_workspace_bytes(int64_t batch_heads, int64_t D, int num_splits) {
  if (batch_heads <= 0 || D <= 0 || num_splits <= 0) return 0;
  return (size_t)batch_heads * (size_t)num_splits * (size_t)(D + 2) * sizeof(float);
}

namespace tfk {
namespace {

// Argument checks shared by both entry points.
int check_decode_args(const char* who, const void* Q, const void* K, const void* V, const void* O,
                      int64_t batch_heads, int64_t Lkv, int64_t D, int num_splits,
                      double softmax_scale) {
  TFK_REQUIRE(Q && K && V && O, TF_ERR_INVALID_ARG, "%s: null pointer", who);
  TFK_REQUIRE(batch_heads > 0 && Lkv > 0 && num_splits > 0, TF_ERR_INVALID_ARG,
              "%s: sizes must be positive", who);
  TFK_REQUIRE(batch_heads < 65536 && num_splits <= 65536, TF_ERR_INVALID_ARG,
              "%s: batch_heads / num_splits too large", who);
  TFK_REQUIRE(D == 128 || D == 64, TF_ERR_UNSUPPORTED, "%s: head dim must be 128 or 64 (got %lld)", who, (long long)D);
  TFK_REQUIRE(softmax_scale == softmax_scale && softmax_scale - softmax_scale == 0.0,
              TF_ERR_INVALID_ARG, "%s: softmax_scale must be finite", who);
  return TF_OK;
}

// Split kernel + combine kernel on `st`; `partials` holds o_part then ml_part.
template <typename T, int D>
int launch_decode_t(const void* Q, const void* K, const void* V, void* O, float* partials,
                    int64_t batch_heads, int64_t Lkv, int num_splits, double softmax_scale,
                    hipStream_t st) {
  float* o_part = partials;
  float* ml_part = o_part + (size_t)batch_heads * num_splits * D;
  const int64_t chunk = (Lkv + num_splits - 1) / num_splits;
  const float scale_log2 = (float)(softmax_scale * 1.4426950408889634);
  hipLaunchKernelGGL((flash_decode_split_kernel<T, D>), dim3(num_splits, (unsigned)batch_heads),
                     dim3(kDecThreads), 0, st, static_cast<const T*>(Q), static_cast<const T*>(K),
                     static_cast<const T*>(V), o_part, ml_part, Lkv, num_splits, chunk, scale_log2);
  TFK_HIP_TRY(hipGetLastError());
  hipLaunchKernelGGL((flash_decode_combine_kernel<T, D>), dim3((unsigned)batch_heads), dim3(D), 0, st,
                     o_part, ml_part, static_cast<T*>(O), num_splits);
  TFK_HIP_TRY(hipGetLastError());
  return TF_OK;
}
int launch_decode(const void* Q, const void* K, const void* V, void* O, float* partials, int dtype,
                  int64_t batch_heads, int64_t Lkv, int64_t D, int num_splits, double softmax_scale,
                  hipStream_t st) {
  if (dtype == TF_DTYPE_BF16) {
    if (D == 128) return launch_decode_t<bf16_t, 128>(Q, K, V, O, partials, batch_heads, Lkv, num_splits, softmax_scale, st);
    return launch_decode_t<bf16_t, 64>(Q, K, V, O, partials, batch_heads, Lkv, num_splits, softmax_scale, st);
  }
  if (D == 128) return launch_decode_t<half_t, 128>(Q, K, V, O, partials, batch_heads, Lkv, num_splits, softmax_scale, st);
  return launch_decode_t<half_t, 64>(Q, K, V, O, partials, batch_heads, Lkv, num_splits, softmax_scale, st);
}

int decode_with_workspace(const char* who, const void* Q, const void* K, const void* V, void* O, int dtype,
                          void* workspace, size_t workspace_bytes, int64_t batch_heads, int64_t Lkv, int64_t D,
                          int num_splits, double softmax_scale, void* stream) {
  TFK_REQUIRE(workspace, TF_ERR_INVALID_ARG, "%s: null pointer", who);
  if (int rc = check_decode_args(who, Q, K, V, O, batch_heads, Lkv, D, num_splits, softmax_scale)) return rc;
  const size_t need = tf_flash_decode_workspace_bytes(batch_heads, D, num_splits);
  TFK_REQUIRE(workspace_bytes >= need, TF_ERR_INVALID_ARG, "%s: workspace holds %zu bytes, %zu needed", who,
              workspace_bytes, need);
  TFK_REQUIRE(((uintptr_t)workspace & 15) == 0, TF_ERR_INVALID_ARG, "%s: workspace must be 16-byte aligned", who);
  return launch_decode(Q, K, V, O, static_cast<float*>(workspace), dtype, batch_heads, Lkv, D, num_splits,
                       softmax_scale, static_cast<hipStream_t>(stream));
}

}  // namespace
}  // namespace tfk

extern "C" int tf_flash_decode_f16(const void* Q, const void* K, const void* V, void* O,
                                   void* workspace, size_t workspace_bytes, int64_t batch_heads,
                                   int64_t Lkv, int64_t D, int num_splits, double softmax_scale,
                                   void* stream) {
  return tfk::decode_with_workspace("tf_flash_decode_f16", Q, K, V, O, TF_DTYPE_F16, workspace, workspace_bytes,
                                    batch_heads, Lkv, D, num_splits, softmax_scale, stream);
}

extern "C" int tf_flash_decode(const void* Q, const void* K, const void* V, void* O, int dtype,
                               void* workspace, size_t workspace_bytes, int64_t batch_heads,
                               int64_t Lkv, int64_t D, int num_splits, double softmax_scale,
                               void* stream) {
  using namespace tfk;
  TFK_REQUIRE(dtype == TF_DTYPE_F16 || dtype == TF_DTYPE_BF16, TF_ERR_UNSUPPORTED,
              "tf_flash_decode: dtype must be TF_DTYPE_F16 or TF_DTYPE_BF16");
  return decode_with_workspace("tf_flash_decode", Q, K, V, O, dtype, workspace, workspace_bytes, batch_heads, Lkv, D,
                               num_splits, softmax_scale, stream);
}

// ---- the same pair of kernels with the partials in a static device array -------------------
//
// For callers that cannot allocate device memory (code under HIP graph capture, tight serving
// loops, harnesses that forbid hipMalloc): no workspace argument, nothing allocated.  Every GPU
// the library runs on holds its own copy of `scratch` until the process ends.  The name
// `scratch` is only a host-side handle of the symbol, not a device address: the address on each
// device comes from hipGetSymbolAddress, once, with that device current, and only that pointer
// is ever handed to a kernel.
namespace tfk {
namespace {

constexpr size_t kScratchFloats = (size_t)TF_FLASH_DECODE_STATIC_MAX_PARTIALS * (kD + 2);
static __device__ __align__(256) float scratch[kScratchFloats];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (looked up on the first call per device).
int scratch_on_current_device(float** out) {
  int dev = -1;
  TFK_HIP_TRY(hipGetDevice(&dev));
  TFK_REQUIRE(dev >= 0 && dev < kMaxDevices, TF_ERR_UNSUPPORTED,
              "tf_flash_decode_static_f16: device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    TFK_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    TFK_REQUIRE(p != nullptr, TF_ERR_HIP, "tf_flash_decode_static_f16: null symbol address");
    g_scratch_ptr[dev] = static_cast<float*>(p);
  }
  *out = g_scratch_ptr[dev];
  return TF_OK;
}

}  // namespace
}  // namespace tfk

extern "C" size_t tf_flash_decode_static_max_partials(void) {
  return (size_t)TF_FLASH_DECODE_STATIC_MAX_PARTIALS;
}

extern "C" int tf_flash_decode_static_prepare(void) {
  float* unused = nullptr;
  return tfk::scratch_on_current_device(&unused);
}

extern "C" int tf_flash_decode_static_f16(const void* Q, const void* K, const void* V, void* O,
                                          int64_t batch_heads, int64_t Lkv, int64_t D,
                                          int num_splits, double softmax_scale, void* stream) {
  using namespace tfk;
  if (int rc = check_decode_args("tf_flash_decode_static_f16", Q, K, V, O, batch_heads, Lkv, D,
                                 num_splits, softmax_scale))
    return rc;
  TFK_REQUIRE(D == kD, TF_ERR_UNSUPPORTED, "tf_flash_decode_static_f16: head dim must be 128 (got %lld)", (long long)D);
  TFK_REQUIRE((uint64_t)batch_heads * (uint64_t)num_splits <= TF_FLASH_DECODE_STATIC_MAX_PARTIALS,
              TF_ERR_INVALID_ARG,
              "tf_flash_decode_static_f16: batch_heads * num_splits = %llu exceeds the static "
              "scratch array (%llu partials); use tf_flash_decode_f16 with a workspace",
              (unsigned long long)((uint64_t)batch_heads * (uint64_t)num_splits),
              (unsigned long long)TF_FLASH_DECODE_STATIC_MAX_PARTIALS);
  float* partials = nullptr;
  if (int rc = scratch_on_current_device(&partials)) return rc;
  // Nothing has to start at zero: the split kernel writes every (slice, split) partial the
  // combine kernel reads, so whatever an earlier call left in the array is never read.
  return launch_decode(Q, K, V, O, partials, TF_DTYPE_F16, batch_heads, Lkv, D, num_splits, softmax_scale,
                       static_cast<hipStream_t>(stream));
}
