// Run-time compiler for kernels written against the tile headers (counterpart of
// include/jit/compiler.hpp:21-81 and src/jit/compiler.cc:123-278).
//
// Same contract as the reference: source text + kernel name (an `extern "C" __global__`
// symbol) -> a launchable function handle, cached per process under a mutex.  What differs:
//   * the compiler is `hipcc --genco` (a gfx950 code object), loaded with hipModuleLoadData;
//   * the code object is also cached on disk, keyed by a hash of the source, the arguments,
//     the contents of the include directories and the compiler / library versions: the
//     reference writes randomly named files it never re-uses;
//   * failure returns nullptr and keeps the compiler's output in last_log() instead of
//     only logging it.
#pragma once

#include <hip/hip_runtime.h>

#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace tilefusion::jit {

class JitCompiler {
 public:
  static JitCompiler& instance();

  // Compiles (or re-loads from the disk cache) and returns the kernel, nullptr on failure.
  hipFunction_t compile_kernel(const std::string& kernel_name, const std::string& hip_source,
                               const std::vector<std::string>& include_paths = {},
                               const std::vector<std::string>& compile_args = {});

  // Returns the kernel from the in-process cache, compiling it on first use.
  hipFunction_t get_or_compile_kernel(const std::string& kernel_name, const std::string& hip_source,
                                      const std::vector<std::string>& include_paths = {},
                                      const std::vector<std::string>& compile_args = {});

  // Drops the in-process cache (loaded modules are unloaded); the disk cache stays.
  void clear_cache();

  // Compiler output of the last failing compile_kernel() on any thread.
  std::string last_log();

  // Directory of the on-disk cache ($TILEFUSION_CACHE_DIR, else ~/.cache/tilefusion_mi355x,
  // else /tmp/tilefusion_mi355x-<uid> if that is a private directory of this user, else a
  // fresh temporary directory of this process).
  static std::string cache_dir();

 private:
  JitCompiler() = default;
  ~JitCompiler() = default;
  JitCompiler(const JitCompiler&) = delete;
  JitCompiler& operator=(const JitCompiler&) = delete;

  // Path of the code object for this source, compiling it if the disk cache has none;
  // empty on failure.
  std::string compile_to_code_object(const std::string& key, const std::string& hip_source,
                                     const std::vector<std::string>& include_paths,
                                     const std::vector<std::string>& compile_args);
  hipFunction_t load_and_get_kernel(const std::string& key, const std::string& path,
                                    const std::string& kernel_name);

  std::unordered_map<std::string, hipModule_t> module_cache_;
  std::unordered_map<std::string, hipFunction_t> kernel_cache_;
  std::string last_log_;
  std::mutex mutex_;
};

}  // namespace tilefusion::jit
