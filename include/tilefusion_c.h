/*
 * tilefusion_c.h - C ABI of the MI355X (gfx950) TileFusion hot path.
 *
 * Plain pointers and sizes only: every pointer is a device pointer owned by the caller,
 * every entry point enqueues on the HIP stream handed in (a hipStream_t passed as void*,
 * NULL = the null stream) and returns without synchronising.  Nothing is allocated on the
 * device.  Return value: TF_OK or an error code; tf_last_error() gives the thread-local
 * message of the last failing call.  No entry point ever calls exit().
 *
 * The reference exports its host launchers as `extern "C"` symbols that take
 * `torch::Tensor&` (include/kernels/ops.hpp:36-58), which is not a C ABI; the entry points
 * below are what a binding (src/torch_bind.cc:8-14) calls instead.
 */
#ifndef TILEFUSION_C_H_
#define TILEFUSION_C_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TF_API __attribute__((visibility("default")))

typedef enum {
  TF_OK = 0,
  TF_ERR_INVALID_ARG = 1, /* null pointer, non-positive size, tile that does not divide */
  TF_ERR_UNSUPPORTED = 2, /* legal in the reference but not compiled into this library  */
  TF_ERR_LDS = 3,         /* requested tile needs more than 160 KiB of LDS              */
  TF_ERR_HIP = 4          /* a HIP runtime call failed; message holds hipGetErrorString */
} tf_status_t;

/* Element types of the dtype-generic entry points (the codes tf_scatter_nd takes as well). */
typedef enum { TF_DTYPE_F32 = 0, TF_DTYPE_F16 = 1, TF_DTYPE_BF16 = 2 } tf_dtype_t;

/* C[M,N] = A[M,K] * B[K,N], fp16 inputs, fp32 accumulate.
 * A is row-major [M,K]; B is column-major K x N, i.e. a row-major [N,K] buffer; C is
 * row-major [M,N], fp32 when c_is_f16 == 0 (the reference op) or fp16 otherwise (the
 * reference benchmark variant).  tm/tn/tk/num_stages/pipeline_level are the reference's
 * tile-size and pipelining arguments: validated (tm | M, tn | N, tk | K, stages 1..3,
 * level 0..2) and otherwise treated as a hint - the library maps the call onto its own
 * MFMA tilings.  K must be a multiple of 8.
 * Replaces: tilefusion::kernels::gemm, src/kernels/gemm.cu:63-142
 * (schema include/kernels/kernel_list.hpp:15-18). */
TF_API int tf_gemm_f16(const void* A, const void* B, void* C, int c_is_f16, int64_t M,
                       int64_t N, int64_t K, int tm, int tn, int tk, int num_stages,
                       int pipeline_level, void* stream);

/* The same for fp16 or bf16 inputs (dtype = TF_DTYPE_F16 / TF_DTYPE_BF16, the reference's declared
 * type set, include/kernels/dispatch_macros.hpp:6-23 and include/cell/compute/gemm.hpp:107-150):
 * C is fp32 when c_is_f32 != 0, else of the input type.  fp16 is tf_gemm_f16.  bf16 runs the same
 * kernels with the bf16 MFMAs (any M, N; K a multiple of 8). */
TF_API int tf_gemm(const void* A, const void* B, void* C, int dtype, int c_is_f32, int64_t M,
                   int64_t N, int64_t K, int tm, int tn, int tk, int num_stages,
                   int pipeline_level, void* stream);

/* D[M,P] = (A[M,K] * B[K,N]) * C[N,P]; fp16 in/out, fp32 accumulate, A*B rounded to fp16
 * in registers and never written to memory.  A row-major [M,K]; B a row-major [N,K]
 * buffer; C a row-major [P,N] buffer; D row-major [M,P].  `batch` independent problems are
 * laid out back to back (A, D strided by M*K / M*P; B and C strided by N*K / P*N).
 * K and N must be multiples of 32, P a multiple of 16.
 * Replaces: tilefusion::kernels::fused_two_gemms, src/kernels/fused_two_gemms.cu:66-144
 * (schema include/kernels/kernel_list.hpp:20-23). */
TF_API int tf_fused_two_gemms_f16(const void* A, const void* B, const void* C, void* D,
                                  int64_t batch, int64_t M, int64_t N, int64_t K, int64_t P,
                                  int tm, int tn, int tk, int tp, void* stream);

/* The same for fp16 or bf16 (dtype as in tf_gemm): the same kernels with the bf16 MFMA, a bf16
 * intermediate and bf16 output. */
TF_API int tf_fused_two_gemms(const void* A, const void* B, const void* C, void* D, int dtype,
                              int64_t batch, int64_t M, int64_t N, int64_t K, int64_t P, int tm,
                              int tn, int tk, int tp, void* stream);

/* tf_fused_two_gemms with a caller-provided device workspace.  Long-N problems (K = P = 128, N
 * a multiple of 64, too few row blocks to fill the chip) are then cut along N wherever that is the
 * faster way: each workgroup takes a range of N for its rows, fp32 partial results go to the
 * workspace and a second kernel adds them up into D (fp16 and bf16).  tf_fused_two_gemms_workspace_bytes says how many bytes that takes
 * for a problem (0: it would not be cut); with a null or smaller workspace, and for every other
 * shape or type, tf_fused_two_gemms_ws is tf_fused_two_gemms.  The workspace must be 16-byte
 * aligned; its contents are scratch.  Results equal those of tf_fused_two_gemms up to the order of
 * the fp32 additions over N.
 * No counterpart in the reference, whose op has no workspace (src/kernels/fused_two_gemms.cu:66-144
 * launches M / tm x P / tp blocks that each walk all of N); the torch op of this library allocates
 * the workspace itself, so callers of the reference's Python / torch API get the cut for free. */
TF_API size_t tf_fused_two_gemms_workspace_bytes(int dtype, int64_t batch, int64_t M, int64_t N,
                                                 int64_t K, int64_t P);
TF_API int tf_fused_two_gemms_ws(const void* A, const void* B, const void* C, void* D, int dtype,
                                 int64_t batch, int64_t M, int64_t N, int64_t K, int64_t P, int tm,
                                 int tn, int tk, int tp, void* workspace, size_t workspace_bytes,
                                 void* stream);

/* O = softmax(scale * Q K^T (+ causal mask)) V for `batch` independent (batch x head)
 * slices laid out back to back.  fp16 in/out, fp32 scores, fp32 running max / sum.
 * Q [batch, Lq, D]; K [batch, Lkv, D]; V [batch, Lkv, Dv] when v_is_transposed == 0, or
 * [batch, Dv, Lkv] when 1 (what the reference op receives, python/ops/flash_attention.py:74);
 * O [batch, Lq, Dv].  Causal mask: key index > query index is masked
 * (include/cell/mask.hpp:75-82).  (D, Dv) = (128, 128), (96, 96) and (64, 64) run the tuned kernels: any Lq
 * and Lkv (a transposed V needs Lkv % 8 == 0 to keep its rows 16-byte aligned).  Other head
 * dimensions are compiled at run time from the header kernel with the caller's tile sizes, as
 * the reference does for every call (src/kernels/flash_attn.cu:16-55): that path needs a
 * transposed V, D % 32 == 0, Dv % 16 == 0, Lq % 16 == 0 and Lkv % 32 == 0, else
 * TF_ERR_UNSUPPORTED (the torch op pads and transposes so that it never fails).
 * The tuned kernels fold softmax_scale * log2(e) into an fp16 copy of Q: exact to the stated
 * tolerance whenever |Q| * softmax_scale * 1.4427 stays far below 65504 (saturates beyond).
 * Replaces: tilefusion::kernels::flash_attention, src/kernels/flash_attn.cu:58-152
 * (schema include/kernels/kernel_list.hpp:25-30). */
TF_API int tf_flash_attention_fwd_f16(const void* Q, const void* K, const void* V, void* O,
                                      int64_t batch, int64_t Lq, int64_t Lkv, int64_t D,
                                      int64_t Dv, int v_is_transposed, int tile_length_q,
                                      int tile_length_kv, int tile_hidden_qk, int tile_hidden_v,
                                      double softmax_scale, int causal, void* stream);

/* The same for fp16 or bf16 (dtype as in tf_gemm).  bf16 with (D, Dv) = (128, 128), (96, 96) or (64, 64) runs
 * the tuned kernels with the bf16 MFMA, bf16 softmax weights and bf16 output; other head dimensions
 * take the run-time compiled path as above. */
TF_API int tf_flash_attention_fwd(const void* Q, const void* K, const void* V, void* O, int dtype,
                                  int64_t batch, int64_t Lq, int64_t Lkv, int64_t D, int64_t Dv,
                                  int v_is_transposed, int tile_length_q, int tile_length_kv,
                                  int tile_hidden_qk, int tile_hidden_v, double softmax_scale,
                                  int causal, void* stream);

/* Single-query (decoding) attention with the KV range split into `num_splits` chunks:
 * kernel 1 writes per-split partial (o, max, sum) in fp32 into `workspace`, kernel 2 merges
 * them with a log-sum-exp weighted sum into O.
 * Q [batch_heads, D]; K, V [batch_heads, Lkv, D]; O [batch_heads, D]; D must be 128 or 64.
 * All offsets are 64-bit (K alone has 2^31 elements at the benchmark size).
 * No counterpart in the reference (it has no decoding kernel); built on the same online
 * softmax algebra as include/kernels/flash_attention_device.cuh:257-301. */
TF_API size_t tf_flash_decode_workspace_bytes(int64_t batch_heads, int64_t D, int num_splits);
TF_API int tf_flash_decode_f16(const void* Q, const void* K, const void* V, void* O,
                               void* workspace, size_t workspace_bytes, int64_t batch_heads,
                               int64_t Lkv, int64_t D, int num_splits, double softmax_scale,
                               void* stream);
/* The same for fp16 or bf16 (dtype as in tf_gemm; the 16-bit types of the reference's dispatch,
 * include/kernels/dispatch_macros.hpp:6-23): bf16 inputs, bf16 output, fp32 partials. */
TF_API int tf_flash_decode(const void* Q, const void* K, const void* V, void* O, int dtype,
                           void* workspace, size_t workspace_bytes, int64_t batch_heads,
                           int64_t Lkv, int64_t D, int num_splits, double softmax_scale,
                           void* stream);

/* tf_flash_decode_f16 without the workspace argument and without any allocation: the per-split
 * partials live in a static device array inside the library (TF_FLASH_DECODE_STATIC_MAX_PARTIALS
 * x (128 + 2) floats = 16.25 MiB, held by every GPU the library runs on until the process ends).
 * No counterpart in the reference.  It is for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The device that
 * owns `stream` must be current.  The first call on a device looks up the array's address there
 * (hipGetSymbolAddress, which may load the code object): make that first call - or
 * tf_flash_decode_static_prepare(), which does only the lookup for the current device - OUTSIDE any
 * stream capture; afterwards a call is two kernel launches and nothing else.  No call allocates or
 * frees.  The array is part of the library's code object: every process that loads the library
 * holds it on every GPU it uses, whether or not it calls this entry point.  batch_heads * num_splits above
 * TF_FLASH_DECODE_STATIC_MAX_PARTIALS is rejected with TF_ERR_INVALID_ARG; D must be 128.  Same kernels and
 * bit-identical results as tf_flash_decode_f16.  All calls on one GPU share the one array, so
 * calls that overlap on a GPU (different streams, or threads) race: serialise them. */
#define TF_FLASH_DECODE_STATIC_MAX_PARTIALS 32768 /* 512 (batch x head) slices x 64 splits */
TF_API size_t tf_flash_decode_static_max_partials(void);
TF_API int tf_flash_decode_static_prepare(void);
TF_API int tf_flash_decode_static_f16(const void* Q, const void* K, const void* V, void* O,
                                      int64_t batch_heads, int64_t Lkv, int64_t D, int num_splits,
                                      double softmax_scale, void* stream);

/* data[indices[i, 0..index_depth-1], ...] += updates[i, ...] for every index row i; duplicate
 * rows accumulate (atomic adds), rows that point outside `data` are skipped.  `data` has
 * `rank` dimensions data_dims (host array, row-major, contiguous); indices is a device
 * [num_index_rows, index_depth] int64 array; updates is [num_index_rows, prod(data_dims[
 * index_depth..])].  dtype: 0 fp32, 1 fp16, 2 bf16.  Nothing is allocated (the reference
 * cudaMallocs the strides on every call and leaks them).
 * Replaces: tilefusion::kernels::scatter_nd, src/kernels/scatter_nd.cu:36-95
 * (schema include/kernels/kernel_list.hpp:11-13). */
TF_API int tf_scatter_nd(const void* updates, void* data, const int64_t* indices,
                         const int64_t* data_dims, int rank, int64_t num_index_rows,
                         int index_depth, int dtype, void* stream);

/* Run-time compilation of kernels written against the tile headers (tilefusion_amd/include),
 * for shapes that are template parameters there.  tf_jit_compile builds `source` with
 * `hipcc --genco` for gfx950 (the tile headers are on the include path; include_paths and
 * compile_args are appended to the defaults), caches the code object on disk by content hash
 * and in the process by (hash, kernel_name), and returns the handle of the `extern "C"
 * __global__` function `kernel_name`.  tf_jit_launch enqueues it: kernel_args is the usual
 * array of pointers to the argument values.  A failed compile returns TF_ERR_HIP and leaves
 * the compiler's output in tf_last_error().
 * Replaces: tilefusion::jit::JitCompiler::compile_kernel / get_or_compile_kernel
 * (include/jit/compiler.hpp:21-81, src/jit/compiler.cc:123-225) and the cuLaunchKernel calls
 * of the host launchers (src/kernels/gemm.cu:136-141). */
TF_API int tf_jit_compile(const char* kernel_name, const char* source,
                          const char* const* include_paths, int num_include_paths,
                          const char* const* compile_args, int num_compile_args,
                          void** kernel_out);
TF_API int tf_jit_launch(void* kernel, unsigned grid_x, unsigned grid_y, unsigned grid_z,
                         unsigned block_x, unsigned block_y, unsigned block_z,
                         unsigned dynamic_lds_bytes, void* stream, void** kernel_args);
/* Drops the in-process kernel cache (JitCompiler::clear_cache, src/jit/compiler.cc:147-163). */
TF_API int tf_jit_clear_cache(void);
/* Directory of the on-disk code-object cache. */
TF_API const char* tf_jit_cache_dir(void);

/* Message of the last failing call on this thread ("" if none). */
TF_API const char* tf_last_error(void);
/* Library version string, e.g. "tilefusion-mi355x 0.1.0 (gfx950)". */
TF_API const char* tf_version(void);

#ifdef __cplusplus
}
#endif
#endif /* TILEFUSION_C_H_ */
