// Host launcher that instantiates the header attention kernel (kernels/flash_attention_device.hpp)
// at run time for head dimensions the ahead-of-time kernels of this library have no instance of.
//
// This is the reference's own launch path (src/kernels/flash_attn.cu:16-55,58-152; the same for
// its other ops, src/kernels/gemm.cu:21-59,63-142, src/kernels/fused_two_gemms.cu:35-63): the
// whole problem shape and the tile sizes become template arguments of a generated wrapper, which
// is compiled once per distinct argument set (JitCompiler caches it in the process and on disk)
// and launched on the caller's stream.  Here it is the fallback behind the tuned attention entry
// point; the GEMM and the fused op have ahead-of-time kernels for every shape and both element
// types (their run-time instantiations are reached through tf_jit_compile / tf_jit_launch).
#include <cmath>
#include <cstring>
#include <sstream>
#include <string>

#include "common.hpp"
#include "jit/compiler.hpp"
#include "jit_ops.hpp"

namespace tfk {
namespace {

using tilefusion::jit::JitCompiler;

const char* kPrelude =
    "#include \"kernels/flash_attention_device.hpp\"\n"
    "using namespace tilefusion;\n"
    "using namespace tilefusion::kernels;\n"
    "namespace tl = tile_layout;\n";

const char* type_name(int dtype) { return dtype == TF_DTYPE_BF16 ? "__bfloat16" : "__half"; }

// A double printed so that the compiler reads back exactly the same value (hex float).
std::string exact(double v) {
  char buf[64];
  snprintf(buf, sizeof(buf), "%a", v);
  return buf;
}
std::string bits_of(double v) {
  unsigned long long u;
  memcpy(&u, &v, sizeof(u));
  char buf[32];
  snprintf(buf, sizeof(buf), "%016llx", u);
  return buf;
}

int compile_and_launch(const std::string& name, const std::string& src, dim3 grid, unsigned threads,
                       unsigned lds, void** args, hipStream_t st) {
  TFK_REQUIRE(lds <= (unsigned)kMaxLdsBytes, TF_ERR_LDS,
              "%s: the requested tiles need %u bytes of LDS (a CU has 160 KiB)", name.c_str(), lds);
  hipFunction_t fn = JitCompiler::instance().get_or_compile_kernel(name, src);
  if (!fn) {
    set_error("%s: run-time compilation failed: %s", name.c_str(), JitCompiler::instance().last_log().c_str());
    return TF_ERR_HIP;
  }
  if (lds > 64 * 1024) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    (void)hipGetLastError();
  }
  TFK_HIP_TRY(hipModuleLaunchKernel(fn, grid.x, grid.y, grid.z, threads, 1, 1, lds, st, args, nullptr));
  return TF_OK;
}

// largest candidate that divides n (0 if none)
int pick_divisor(int64_t n, std::initializer_list<int> candidates) {
  for (int c : candidates)
    if (n % c == 0) return c;
  return 0;
}

// Replaces t by the largest multiple of `unit` below it that divides n and is at least `floor`;
// false when there is none.
bool shrink_tile(int& t, int64_t n, int unit, int floor) {
  for (int c = (t - 1) / unit * unit; c >= floor && c > 0; c -= unit)
    if (n % c == 0) {
      t = c;
      return true;
    }
  return false;
}

// LDS bytes of the header attention kernel: one Q, one K and one V tile of 2-byte elements.
unsigned attention_lds_bytes(int tq, int tkv, int thqk, int thv) {
  return (unsigned)(tq * thqk + thqk * tkv + tkv * thv) * 2u;
}

}  // namespace

bool jit_flash_attention_supports(int64_t Lq, int64_t Lkv, int64_t D, int64_t Dv, int v_is_transposed) {
  return v_is_transposed && D % 32 == 0 && Dv % 16 == 0 && Lq % 16 == 0 && Lkv % 32 == 0 && D <= 512 && Dv <= 512;
}

int jit_flash_attention(const void* Q, const void* K, const void* Vt, void* O, int dtype, int64_t batch,
                        int64_t Lq, int64_t Lkv, int64_t D, int64_t Dv, int tq, int tkv, int thqk, int thv,
                        double scale, int causal, hipStream_t st) {
  // The caller's tiles are used when they are whole MFMA base tiles (16 query rows per
  // wavefront, 32-deep reductions, 16 output columns); otherwise the nearest legal ones.
  if (tq % 16 != 0 || Lq % tq != 0 || tq > 128) tq = pick_divisor(Lq, {64, 32, 16});
  if (tkv % 32 != 0 || Lkv % tkv != 0 || tkv > 128) tkv = pick_divisor(Lkv, {64, 32});
  if (thqk % 32 != 0 || D % thqk != 0) thqk = (int)D;
  if (thv % 16 != 0 || Dv % thv != 0) thv = (int)Dv;
  TFK_REQUIRE(tq > 0 && tkv > 0, TF_ERR_UNSUPPORTED, "flash_attention: no legal tiling for Lq=%lld Lkv=%lld",
              (long long)Lq, (long long)Lkv);
  // Tiles that do not fit the CU's LDS are shrunk until they do.  The head-dimension chunks go
  // first (a shorter reduction chunk only re-fetches Q per key tile, a narrower output chunk
  // repeats Q K^T per chunk), each down to 128 before the sequence tiles go down to 64, then
  // everything to its smallest legal size.
  while (attention_lds_bytes(tq, tkv, thqk, thv) > (unsigned)kMaxLdsBytes) {
    if (thqk > 128 && shrink_tile(thqk, D, 32, 128)) continue;
    if (thv > 128 && shrink_tile(thv, Dv, 16, 128)) continue;
    if (tq > 64 && shrink_tile(tq, Lq, 16, 64)) continue;
    if (tkv > 64 && shrink_tile(tkv, Lkv, 32, 64)) continue;
    if (shrink_tile(thqk, D, 32, 32)) continue;
    if (shrink_tile(thv, Dv, 16, 16)) continue;
    if (shrink_tile(tq, Lq, 16, 16)) continue;
    if (shrink_tile(tkv, Lkv, 32, 32)) continue;
    break;  // smallest legal tiles: compile_and_launch reports the LDS need
  }
  // wavefronts stacked along the query rows: 16 rows each, at most 4
  int wr = tq / 16 > 4 ? 4 : tq / 16;
  while ((tq / wr) % 16 != 0) --wr;
  const char* T = type_name(dtype);
  std::ostringstream name, src;
  name << "tf_fa_" << (dtype == TF_DTYPE_BF16 ? "bf16_" : "f16_") << Lq << "_" << Lkv << "_" << D << "_" << Dv << "_"
       << tq << "_" << tkv << "_" << thqk << "_" << thv << "_" << (causal ? 1 : 0) << "_" << wr << "_" << bits_of(scale);
  src << kPrelude << "using Config = FlashAttentionTraits<" << T << ", float, " << T << ", TileShape<" << Lq << ", "
      << Lkv << ", " << D << ", " << Dv << ">, TileShape<" << tq << ", " << tkv << ", " << thqk << ", " << thv
      << ">, tl::RowMajor<" << wr << ", 1>, " << exact(scale) << ", " << (causal ? "true" : "false") << ">;\n"
      << "extern \"C\" __global__ __launch_bounds__(" << wr * 64 << ") void " << name.str() << "(const " << T
      << "* Q, const " << T << "* K, const " << T << "* V, " << T << "* O) {\n"
      << "  ke_flash_attention<" << T << ", float, " << T << ", Config>(Q, K, V, O);\n}\n";
  const unsigned lds = attention_lds_bytes(tq, tkv, thqk, thv);
  void* args[] = {&Q, &K, &Vt, &O};
  return compile_and_launch(name.str(), src.str(), dim3((unsigned)(Lq / tq), (unsigned)(Dv / thv), (unsigned)batch),
                            wr * 64, lds, args, st);
}

}  // namespace tfk
