// PyTorch operator bindings: registers torch.ops.tilefusion.{gemm, fused_two_gemms,
// flash_attention, flash_attention_fwd, flash_decode} for the CUDA dispatch key (HIP tensors
// are "cuda" tensors on PyTorch-ROCm) and forwards to the C ABI in tilefusion_c.h on the
// caller's current stream.
//
// Mirrors the reference's registry + binding (include/kernel_registry.hpp:20-88,
// include/kernels/kernel_list.hpp:11-30, src/torch_bind.cc:8-14): the first three schemas are
// byte-identical so existing callers of torch.ops.tilefusion.* keep working.  Differences:
// outputs may be fp16 for gemm, leading batch dimensions are accepted, dimensions are read
// from the right axes for non-square problems, launches go to the current stream instead of
// the null stream, and errors surface as c10::Error (RuntimeError) instead of exit().
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <functional>
#include <vector>

#include "tilefusion_c.h"

// The dtype switch of the reference (include/kernels/dispatch_macros.hpp:6-23).  This file is
// built by the host compiler without the device headers, so the element types are ATen's.
#define TILEFUSION_DISPATCH_HOST_TYPES
using __half = at::Half;
using __bfloat16 = at::BFloat16;
#include "kernels/dispatch_macros.hpp"

namespace tilefusion {

// Marks the host launchers the Python side binds (include/kernel_registry.hpp:20-24): C linkage and
// default visibility, so `gemm`, `fused_two_gemms`, `flash_attention` and `scatter_nd` are exported
// from libtilefusion.so under the names the reference's library exports them.
#define TILEFUSION_EXPORT extern "C" __attribute__((visibility("default")))

#define CHECK_CUDA(x) TORCH_CHECK((x).device().is_cuda(), #x " must be a CUDA tensor.")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous.")
#define CHECK_INPUT(x) \
  CHECK_CUDA(x);       \
  CHECK_CONTIGUOUS(x)
#define CHECK_HALF(x) TORCH_CHECK((x).scalar_type() == at::kHalf, #x " must be a float16 tensor.")
#define CHECK_SAME_TYPE(x, y) \
  TORCH_CHECK((x).scalar_type() == (y).scalar_type(), #x " and " #y " must have the same dtype.")

namespace {

void* current_stream() { return c10::hip::getCurrentHIPStream().stream(); }

void check_status(int status, const char* op) {
  TORCH_CHECK(status == TF_OK, "tilefusion::", op, " failed (status ", status, "): ", tf_last_error());
}

template <typename T>
struct DtypeCode;
template <>
struct DtypeCode<__half> { static constexpr int value = TF_DTYPE_F16; };
template <>
struct DtypeCode<__bfloat16> { static constexpr int value = TF_DTYPE_BF16; };
template <>
struct DtypeCode<float> { static constexpr int value = TF_DTYPE_F32; };

// fp16 or bf16 -> the C ABI's dtype code (fp32 operands are rejected by the caller)
int operand_dtype(const at::Tensor& t, const char* op) {
  int code = -1;
  TILEFUSION_DISPATCH_ALL_TYPES(t.scalar_type(), [&] { code = DtypeCode<scalar_t>::value; });
  TORCH_CHECK(code == TF_DTYPE_F16 || code == TF_DTYPE_BF16, "tilefusion::", op,
              ": operands must be float16 or bfloat16 tensors.");
  return code;
}

int64_t round_up(int64_t x, int64_t to) { return (x + to - 1) / to * to; }

int64_t leading_numel(const at::Tensor& t, int64_t keep) {
  int64_t n = 1;
  for (int64_t i = 0; i + keep < t.dim(); ++i) n *= t.size(i);
  return n;
}

}  // namespace

namespace kernels {

// gemm(A [M,K], B [N,K] (= column-major K x N), C [M,N] fp32 or fp16)
TILEFUSION_EXPORT void gemm(const at::Tensor& A, const at::Tensor& B, at::Tensor& C, int64_t tm, int64_t tn,
          int64_t tk, int64_t num_stages, int64_t pipeline_level) {
  CHECK_INPUT(A);
  CHECK_INPUT(B);
  CHECK_INPUT(C);
  const int dtype = operand_dtype(A, "gemm");
  CHECK_SAME_TYPE(A, B);
  TORCH_CHECK(C.scalar_type() == at::kFloat || C.scalar_type() == A.scalar_type(),
              "C must be a float32 tensor or have the dtype of A.");
  TORCH_CHECK(A.dim() == 2 && B.dim() == 2 && C.dim() == 2, "gemm expects 2-D tensors.");
  const int64_t m = A.size(0), k = A.size(1), n = B.size(0);
  TORCH_CHECK(B.size(1) == k, "B must be [N, K] (column-major K x N); got K = ", B.size(1),
              " vs ", k);
  TORCH_CHECK(C.size(0) == m && C.size(1) == n, "C must be [M, N].");
  check_status(tf_gemm(A.data_ptr(), B.data_ptr(), C.data_ptr(), dtype, C.scalar_type() == at::kFloat,
                       m, n, k, (int)tm, (int)tn, (int)tk, (int)num_stages, (int)pipeline_level,
                       current_stream()),
               "gemm");
}

// fused_two_gemms(A [.., M,K], B [.., N,K], C [.., P,N], D [.., M,P])
TILEFUSION_EXPORT void fused_two_gemms(const at::Tensor& A, const at::Tensor& B, const at::Tensor& C, at::Tensor& D,
                     int64_t tm, int64_t tn, int64_t tk, int64_t tp) {
  CHECK_INPUT(A);
  CHECK_INPUT(B);
  CHECK_INPUT(C);
  CHECK_INPUT(D);
  const int dtype = operand_dtype(A, "fused_two_gemms");
  CHECK_SAME_TYPE(A, B);
  CHECK_SAME_TYPE(A, C);
  CHECK_SAME_TYPE(A, D);
  TORCH_CHECK(A.dim() >= 2 && A.dim() == B.dim() && A.dim() == C.dim() && A.dim() == D.dim(),
              "fused_two_gemms expects tensors of equal rank >= 2.");
  const int64_t batch = leading_numel(A, 2);
  const int64_t m = A.size(-2), k = A.size(-1), n = B.size(-2), p = C.size(-2);
  TORCH_CHECK(B.size(-1) == k, "B must be [N, K].");
  TORCH_CHECK(C.size(-1) == n, "C must be [P, N].");
  TORCH_CHECK(D.size(-2) == m && D.size(-1) == p, "D must be [M, P].");
  TORCH_CHECK(leading_numel(B, 2) == batch && leading_numel(C, 2) == batch &&
                  leading_numel(D, 2) == batch,
              "batch dimensions must match.");
  // The kernels reduce 32 values of k (and of n, in the second product) per MFMA and write 16
  // columns per base tile.  Shapes the reference accepts with 16-wide base tiles (K or N = 48,
  // ...) are zero-padded here: zeros add nothing to either product.  A padded P goes through a
  // temporary D.
  const int64_t kp = round_up(k, 32), np = round_up(n, 32), pp = round_up(p, 16);
  const int64_t mp = m;
  if (kp == k && np == n && pp == p && mp == m) {
    // long-N problems are cut along N when the library is handed a workspace for the partial sums
    const size_t ws_bytes = tf_fused_two_gemms_workspace_bytes(dtype, batch, m, n, k, p);
    at::Tensor ws;
    if (ws_bytes > 0) ws = at::empty({(int64_t)ws_bytes}, A.options().dtype(at::kByte));
    check_status(tf_fused_two_gemms_ws(A.data_ptr(), B.data_ptr(), C.data_ptr(), D.data_ptr(), dtype, batch,
                                       m, n, k, p, (int)tm, (int)tn, (int)tk, (int)tp,
                                       ws_bytes > 0 ? ws.data_ptr() : nullptr, ws_bytes, current_stream()),
                 "fused_two_gemms");
    return;
  }
  // constant_pad_nd pads from the last dimension backwards: {last_lo, last_hi, prev_lo, prev_hi}
  at::Tensor Ap = at::constant_pad_nd(A, {0, kp - k, 0, mp - m}, 0).contiguous();
  at::Tensor Bp = at::constant_pad_nd(B, {0, kp - k, 0, np - n}, 0).contiguous();
  at::Tensor Cp = at::constant_pad_nd(C, {0, np - n, 0, pp - p}, 0).contiguous();
  const bool own_d = pp != p || mp != m;
  std::vector<int64_t> d_shape(D.sizes().begin(), D.sizes().end());
  d_shape[d_shape.size() - 2] = mp;
  d_shape[d_shape.size() - 1] = pp;
  at::Tensor Dp = own_d ? at::empty(d_shape, D.options()) : D;
  // the caller's tiles no longer divide the padded problem: whole-dimension tiles always do
  check_status(tf_fused_two_gemms(Ap.data_ptr(), Bp.data_ptr(), Cp.data_ptr(), Dp.data_ptr(), dtype, batch,
                                  mp, np, kp, pp, (int)(mp % tm == 0 ? tm : mp), (int)np, (int)kp, (int)pp,
                                  current_stream()),
               "fused_two_gemms");
  if (own_d) D.copy_(Dp.narrow(-2, 0, m).narrow(-1, 0, p));
}

namespace {
void attention_impl(const at::Tensor& Q, const at::Tensor& K, const at::Tensor& V, at::Tensor& O,
                    bool v_transposed, int64_t tq, int64_t tkv, int64_t thqk, int64_t thv,
                    double softmax_scale, bool causal, const char* op) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(O);
  const int dtype = operand_dtype(Q, op);
  CHECK_SAME_TYPE(Q, K);
  CHECK_SAME_TYPE(Q, V);
  CHECK_SAME_TYPE(Q, O);
  TORCH_CHECK(Q.dim() >= 2 && Q.dim() == K.dim() && Q.dim() == V.dim() && Q.dim() == O.dim(),
              op, " expects tensors of equal rank >= 2.");
  const int64_t batch = leading_numel(Q, 2);
  const int64_t lq = Q.size(-2), d = Q.size(-1), lkv = K.size(-2);
  const int64_t dv = v_transposed ? V.size(-2) : V.size(-1);
  const int64_t v_len = v_transposed ? V.size(-1) : V.size(-2);
  TORCH_CHECK(K.size(-1) == d, "K must be [Lkv, D].");
  TORCH_CHECK(v_len == lkv, "V does not match the key length.");
  TORCH_CHECK(O.size(-2) == lq && O.size(-1) == dv, "O must be [Lq, Dv].");
  TORCH_CHECK(leading_numel(K, 2) == batch && leading_numel(V, 2) == batch &&
                  leading_numel(O, 2) == batch,
              "batch dimensions must match.");
  // Head dimensions up to 128 without a tuned kernel are zero-padded to the next tuned size (64,
  // 96 or 128): zeros change neither the scores nor the kept output columns, and the tuned kernel
  // on the padded problem is well ahead of the header kernel compiled at run time on the exact
  // one, copies included.
  const bool tuned = d == dv && (d == 128 || d == 96 || d == 64);
  if (!tuned && d <= 128 && dv <= 128 && (!v_transposed || lkv % 8 == 0)) {
    const int64_t hmax = std::max(d, dv);
    const int64_t hp = hmax <= 64 ? 64 : hmax <= 96 ? 96 : 128;
    at::Tensor Qp = at::constant_pad_nd(Q, {0, hp - d}, 0).contiguous();
    at::Tensor Kp = at::constant_pad_nd(K, {0, hp - d}, 0).contiguous();
    at::Tensor Vp = (v_transposed ? at::constant_pad_nd(V, {0, 0, 0, hp - dv}, 0)
                                  : at::constant_pad_nd(V, {0, hp - dv}, 0)).contiguous();
    std::vector<int64_t> o_shape(O.sizes().begin(), O.sizes().end());
    o_shape[o_shape.size() - 1] = hp;
    at::Tensor Op = dv == hp ? O : at::empty(o_shape, O.options());
    check_status(tf_flash_attention_fwd(Qp.data_ptr(), Kp.data_ptr(), Vp.data_ptr(), Op.data_ptr(), dtype, batch,
                                        lq, lkv, hp, hp, v_transposed ? 1 : 0, (int)(lq % tq == 0 ? tq : lq),
                                        (int)(lkv % tkv == 0 ? tkv : lkv), (int)hp, (int)hp, softmax_scale,
                                        causal ? 1 : 0, current_stream()),
                 op);
    if (dv != hp) O.copy_(Op.narrow(-1, 0, dv));
    return;
  }
  const int status = tf_flash_attention_fwd(Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr(), dtype,
                                            batch, lq, lkv, d, dv, v_transposed ? 1 : 0, (int)tq,
                                            (int)tkv, (int)thqk, (int)thv, softmax_scale,
                                            causal ? 1 : 0, current_stream());
  if (status != TF_ERR_UNSUPPORTED) {
    check_status(status, op);
    return;
  }
  // No tuned kernel for these head dimensions / this dtype, and the run-time compiled kernel
  // wants a transposed V and whole MFMA base tiles: transpose V, zero-pad the head dimensions
  // (zeros change neither the scores nor the kept output columns) and the query rows (extra
  // rows are dropped).  The key length cannot be padded without changing the softmax.
  TORCH_CHECK(lkv % 32 == 0, "tilefusion::", op, ": head dims (", d, ", ", dv, ") with ",
              toString(Q.scalar_type()), " need a key length that is a multiple of 32 (got ", lkv, ").");
  const int64_t dp = round_up(d, 32), dvp = round_up(dv, 16), lqp = round_up(lq, 16);
  at::Tensor Qp = at::constant_pad_nd(Q, {0, dp - d, 0, lqp - lq}, 0).contiguous();
  at::Tensor Kp = at::constant_pad_nd(K, {0, dp - d}, 0).contiguous();
  at::Tensor Vt = v_transposed ? V : V.transpose(-1, -2);
  Vt = at::constant_pad_nd(Vt, {0, 0, 0, dvp - dv}, 0).contiguous();
  const bool own_o = dvp != dv || lqp != lq;
  std::vector<int64_t> o_shape(O.sizes().begin(), O.sizes().end());
  o_shape[o_shape.size() - 2] = lqp;
  o_shape[o_shape.size() - 1] = dvp;
  at::Tensor Op = own_o ? at::empty(o_shape, O.options()) : O;
  check_status(tf_flash_attention_fwd(Qp.data_ptr(), Kp.data_ptr(), Vt.data_ptr(), Op.data_ptr(), dtype, batch,
                                      lqp, lkv, dp, dvp, 1, (int)(lqp % tq == 0 ? tq : lqp),
                                      (int)(lkv % tkv == 0 ? tkv : lkv), (int)dp, (int)dvp, softmax_scale,
                                      causal ? 1 : 0, current_stream()),
               op);
  if (own_o) O.copy_(Op.narrow(-2, 0, lq).narrow(-1, 0, dv));
}
}  // namespace

// flash_attention(Q [.., Lq,D], K [.., Lkv,D], V [.., Dv,Lkv] (transposed, as the reference's
// Python wrapper passes it), O [.., Lq,Dv])
TILEFUSION_EXPORT void flash_attention(const at::Tensor& Q, const at::Tensor& K, const at::Tensor& V, at::Tensor& O,
                     int64_t tile_length_q, int64_t tile_length_kv, int64_t tile_hidden_qk,
                     int64_t tile_hidden_v, double softmax_scale, bool causal) {
  attention_impl(Q, K, V, O, true, tile_length_q, tile_length_kv, tile_hidden_qk, tile_hidden_v,
                 softmax_scale, causal, "flash_attention");
}

// flash_attention_fwd: same computation with V in its natural [.., Lkv, Dv] layout.
void flash_attention_fwd(const at::Tensor& Q, const at::Tensor& K, const at::Tensor& V,
                         at::Tensor& O, double softmax_scale, bool causal) {
  attention_impl(Q, K, V, O, false, 1, 1, 1, 1, softmax_scale, causal, "flash_attention_fwd");
}

// flash_decode(Q [.., D], K [.., Lkv, D], V [.., Lkv, D], O [.., D]); the fp32 split-KV
// partials live in a torch-allocated workspace.
void flash_decode(const at::Tensor& Q, const at::Tensor& K, const at::Tensor& V, at::Tensor& O,
                  int64_t num_splits, double softmax_scale) {
  CHECK_INPUT(Q);
  CHECK_INPUT(K);
  CHECK_INPUT(V);
  CHECK_INPUT(O);
  CHECK_SAME_TYPE(Q, K);
  CHECK_SAME_TYPE(Q, V);
  CHECK_SAME_TYPE(Q, O);
  const int dtype = operand_dtype(Q, "flash_decode");
  TORCH_CHECK(K.dim() >= 2 && V.dim() == K.dim(), "flash_decode: K and V must be [.., Lkv, D].");
  const int64_t d = K.size(-1), lkv = K.size(-2);
  const int64_t bh = leading_numel(K, 2);
  TORCH_CHECK(V.size(-1) == d && V.size(-2) == lkv && leading_numel(V, 2) == bh,
              "flash_decode: V must have the shape of K.");
  TORCH_CHECK(Q.numel() == bh * d && O.numel() == bh * d,
              "flash_decode: Q and O must hold one row of D per (batch, head).");
  TORCH_CHECK(num_splits > 0, "flash_decode: num_splits must be positive.");
  const size_t bytes = tf_flash_decode_workspace_bytes(bh, d, (int)num_splits);
  at::Tensor ws = at::empty({(int64_t)((bytes + 3) / 4)}, Q.options().dtype(at::kFloat));
  check_status(tf_flash_decode(Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr(), dtype,
                               ws.data_ptr(), bytes, bh, lkv, d, (int)num_splits, softmax_scale,
                               current_stream()),
               "flash_decode");
}

// scatter_nd(data [d0..dr-1], updates [n.., d_k..d_{r-1}], indices [n.., k] int64): data[idx] += updates.
// The reference's schema marks `updates` as the mutated tensor although its kernel writes
// `data` (src/kernels/scatter_nd.cu:86-92); the schema is kept, `data` is what changes.
TILEFUSION_EXPORT void scatter_nd(const at::Tensor& data, at::Tensor& updates, const at::Tensor& indices) {
  CHECK_INPUT(data);
  CHECK_INPUT(updates);
  CHECK_INPUT(indices);
  TORCH_CHECK(indices.scalar_type() == at::kLong, "indices must be an int64 tensor.");
  TORCH_CHECK(updates.scalar_type() == data.scalar_type(), "updates must have the dtype of data.");
  TORCH_CHECK(data.dim() >= 1 && data.dim() <= 8 && indices.dim() >= 1, "scatter_nd: data rank must be 1..8.");
  const int64_t k = indices.size(-1);
  TORCH_CHECK(k >= 1 && k <= data.dim(), "scatter_nd: the last dimension of indices (", k,
              ") must be within 1..rank of data (", data.dim(), ").");
  const int64_t n = indices.numel() / k;
  int64_t slice = 1;
  for (int64_t i = k; i < data.dim(); ++i) slice *= data.size(i);
  TORCH_CHECK(updates.numel() == n * slice, "scatter_nd: updates must hold ", n, " slices of ", slice,
              " elements; got ", updates.numel(), " elements.");
  int dtype = -1;
  if (data.scalar_type() == at::kFloat) dtype = 0;
  else if (data.scalar_type() == at::kHalf) dtype = 1;
  else if (data.scalar_type() == at::kBFloat16) dtype = 2;
  TORCH_CHECK(dtype >= 0, "scatter_nd: data must be float32, float16 or bfloat16.");
  std::vector<int64_t> dims(data.sizes().begin(), data.sizes().end());
  check_status(tf_scatter_nd(updates.data_ptr(), const_cast<at::Tensor&>(data).data_ptr(), indices.data_ptr<int64_t>(),
                             dims.data(), (int)dims.size(), n, (int)k, dtype, current_stream()),
               "scatter_nd");
}

}  // namespace kernels

// Self-registering op table: each REGISTER_OP adds (schema, installer) at load time, and the
// two TORCH_LIBRARY blocks below walk the table, like the reference's KernelRegistry.
class KernelRegistry {
 public:
  using Installer = std::function<void(torch::Library&)>;
  static KernelRegistry& instance() {
    static KernelRegistry r;
    return r;
  }
  template <typename Fn>
  bool add_kernel(const char* name, const char* schema, Fn fn) {
    schemas_.push_back(schema);
    installers_.push_back([name, fn](torch::Library& m) { m.impl(name, c10::DispatchKey::CUDA, fn); });
    return true;
  }
  void register_with_torch(torch::Library& m) const {
    for (const char* s : schemas_) m.def(s);
  }
  void register_implementations(torch::Library& m) const {
    for (const auto& f : installers_) f(m);
  }

 private:
  std::vector<const char*> schemas_;
  std::vector<Installer> installers_;
};

#define REGISTER_OP(name, schema, func) \
  static const bool name##_registered = KernelRegistry::instance().add_kernel(#name, schema, func)

REGISTER_OP(scatter_nd, "scatter_nd(Tensor data, Tensor(a!) updates, Tensor indices) -> ()", &kernels::scatter_nd);
REGISTER_OP(gemm,
            "gemm(Tensor A, Tensor B, Tensor(a!) C, int m, int n, int k, "
            "int num_stages, int pipeline_level) -> ()",
            &kernels::gemm);
REGISTER_OP(fused_two_gemms,
            "fused_two_gemms(Tensor A, Tensor B, Tensor C, Tensor(a!) D, "
            "int tm, int tn, int tk, int tp) ->()",
            &kernels::fused_two_gemms);
REGISTER_OP(flash_attention,
            "flash_attention(Tensor Q, Tensor K, Tensor V, Tensor(a!) O, "
            "int tile_length_q, int tile_length_kv, "
            "int tile_hidden_qk, int tile_hidden_v, "
            "float softmax_scale, bool causal) -> ()",
            &kernels::flash_attention);
REGISTER_OP(flash_attention_fwd,
            "flash_attention_fwd(Tensor Q, Tensor K, Tensor V, Tensor(a!) O, "
            "float softmax_scale, bool causal) -> ()",
            &kernels::flash_attention_fwd);
REGISTER_OP(flash_decode,
            "flash_decode(Tensor Q, Tensor K, Tensor V, Tensor(a!) O, "
            "int num_splits, float softmax_scale) -> ()",
            &kernels::flash_decode);

TORCH_LIBRARY(tilefusion, m) { KernelRegistry::instance().register_with_torch(m); }
TORCH_LIBRARY_IMPL(tilefusion, CUDA, m) { KernelRegistry::instance().register_implementations(m); }

}  // namespace tilefusion
