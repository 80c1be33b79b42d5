// Run-time compiler: implementation of tilefusion::jit::JitCompiler and its C ABI.
// Counterpart of src/jit/compiler.cc:123-278 (popen(nvcc -ptx) -> cuModuleLoadData); here
// popen(hipcc --genco) -> hipModuleLoadData, with a content-addressed disk cache.
#include <dirent.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdio>
#include <cstdlib>
#include <ctime>
#include <algorithm>
#include <fstream>
#include <map>
#include <sstream>

#include "common.hpp"
#include "jit/compiler.hpp"
#include "jit/config.hpp"

namespace tilefusion::jit {
namespace {

// FNV-1a, 64 bit: names cache entries; collisions would need 2^32 distinct kernels.
std::string hash_hex(const std::string& s) {
  unsigned long long h = 1469598103934665603ull;
  for (unsigned char c : s) {
    h ^= c;
    h *= 1099511628211ull;
  }
  char buf[17];
  snprintf(buf, sizeof(buf), "%016llx", h);
  return buf;
}

// Digest of every regular file below `dir` (relative name + contents, names sorted): a header
// edited after a code object was cached must change the cache key.  Bounded in depth and file
// count so that a stray include path (say "/") cannot stall a compile; a walk that hits a bound
// reports it, and what was compiled against such a directory is not kept on disk.
constexpr int kMaxWalkDepth = 6;
constexpr size_t kMaxWalkFiles = 4096;

void collect_files(const std::string& dir, const std::string& rel, int depth, std::vector<std::string>& out,
                   bool& truncated) {
  if (depth > kMaxWalkDepth || out.size() >= kMaxWalkFiles) {
    truncated = true;
    return;
  }
  DIR* d = opendir((dir + "/" + rel).c_str());
  if (!d) return;
  std::vector<std::string> names;
  while (dirent* e = readdir(d)) {
    const std::string n = e->d_name;
    if (n != "." && n != "..") names.push_back(n);
  }
  closedir(d);
  std::sort(names.begin(), names.end());
  for (const auto& n : names) {
    const std::string r = rel.empty() ? n : rel + "/" + n;
    struct stat st;
    if (stat((dir + "/" + r).c_str(), &st) != 0) continue;
    if (S_ISDIR(st.st_mode)) {
      collect_files(dir, r, depth + 1, out, truncated);
    } else if (S_ISREG(st.st_mode)) {
      if (out.size() >= kMaxWalkFiles) {
        truncated = true;
        return;
      }
      out.push_back(r);
    }
  }
}

struct DirectoryDigest {
  std::string hex;
  bool complete;  // false: some file below the directory is not covered by `hex`
};

DirectoryDigest directory_digest(const std::string& dir) {
  std::vector<std::string> files;
  bool truncated = false;
  collect_files(dir, "", 0, files, truncated);
  std::string material;
  for (const auto& r : files) {
    std::ifstream f(dir + "/" + r, std::ios::binary);
    std::stringstream ss;
    ss << f.rdbuf();
    material += r + "\n" + hash_hex(ss.str()) + "\n";
  }
  return {hash_hex(material), !truncated};
}

// Differs between processes (and between runs that re-use a pid): keys that carry it never match
// a file another process left in the cache directory.
std::string process_nonce() {
  static const std::string nonce = [] {
    struct timespec ts;
    clock_gettime(CLOCK_REALTIME, &ts);
    std::ostringstream m;
    m << (long)getpid() << ':' << (long long)ts.tv_sec << ':' << ts.tv_nsec;
    return hash_hex(m.str());
  }();
  return nonce;
}

// The fall-back cache directory of a process without a usable home or per-user directory lives
// as long as the process: its files and the directory itself are removed at exit.
std::string g_fresh_dir;
void remove_fresh_dir() {
  if (g_fresh_dir.empty()) return;
  if (DIR* d = opendir(g_fresh_dir.c_str())) {
    while (dirent* e = readdir(d)) {
      const std::string n = e->d_name;
      if (n != "." && n != "..") remove((g_fresh_dir + "/" + n).c_str());
    }
    closedir(d);
  }
  rmdir(g_fresh_dir.c_str());
}

bool file_exists(const std::string& p) {
  struct stat st;
  return stat(p.c_str(), &st) == 0 && st.st_size > 0;
}

bool make_dirs(const std::string& dir) {
  std::string cur;
  for (size_t i = 0; i <= dir.size(); ++i) {
    if (i == dir.size() || dir[i] == '/') {
      if (!cur.empty() && mkdir(cur.c_str(), 0755) != 0 && errno != EEXIST) return false;
    }
    if (i < dir.size()) cur += dir[i];
  }
  return true;
}

// Single-quote for the shell; the arguments come from the caller, not from tensors.
std::string quoted(const std::string& s) {
  std::string out = "'";
  for (char c : s) out += (c == '\'') ? std::string("'\\''") : std::string(1, c);
  return out + "'";
}

std::string hipcc_path() {
  if (const char* p = getenv("TILEFUSION_HIPCC")) return p;
  return "/opt/rocm/bin/hipcc";
}

// What identifies the toolchain and this library in a cache key: the compiler's path, size and
// modification time (a ROCm update replaces the file) and the library version.
std::string toolchain_digest() {
  const std::string cc = hipcc_path();
  struct stat st;
  std::ostringstream m;
  m << cc << '\n' << tf_version() << '\n';
  char resolved[4096];
  const char* real = realpath(cc.c_str(), resolved);
  if (real && stat(real, &st) == 0) m << real << '\n' << (long long)st.st_size << '\n' << (long long)st.st_mtime;
  return hash_hex(m.str());
}

// A private directory: created with mode 0700, owned by this user, not writable by anyone else.
bool private_dir_ok(const std::string& dir) {
  if (mkdir(dir.c_str(), 0700) != 0 && errno != EEXIST) return false;
  struct stat st;
  if (lstat(dir.c_str(), &st) != 0 || !S_ISDIR(st.st_mode)) return false;
  return st.st_uid == geteuid() && (st.st_mode & (S_IWGRP | S_IWOTH)) == 0;
}

}  // namespace

JitCompiler& JitCompiler::instance() {
  static JitCompiler compiler;
  return compiler;
}

std::string JitCompiler::cache_dir() {
  if (const char* p = getenv("TILEFUSION_CACHE_DIR")) return p;
  if (const char* home = getenv("HOME")) {
    const std::string dir = std::string(home) + "/.cache/tilefusion_mi355x";
    if (make_dirs(dir) && access(dir.c_str(), W_OK) == 0) return dir;
  }
  // No usable home directory: a per-user directory under /tmp, accepted only if it is ours and
  // nobody else can write into it (a code object found there is loaded and run); failing
  // that, a fresh directory that lives as long as the process and is never re-used.
  const std::string shared = "/tmp/tilefusion_mi355x-" + std::to_string((long)geteuid());
  if (private_dir_ok(shared)) return shared;
  static const std::string fresh = [] {
    char tmpl[] = "/tmp/tilefusion_mi355x-XXXXXX";
    const char* d = mkdtemp(tmpl);
    if (d) {
      g_fresh_dir = d;
      atexit(remove_fresh_dir);
    }
    return std::string(d ? d : "");
  }();
  return fresh;
}

std::string JitCompiler::last_log() {
  std::lock_guard<std::mutex> lock(mutex_);
  return last_log_;
}

std::string JitCompiler::compile_to_code_object(const std::string& key, const std::string& hip_source,
                                                const std::vector<std::string>& include_paths,
                                                const std::vector<std::string>& compile_args) {
  const std::string dir = cache_dir();
  if (dir.empty() || !make_dirs(dir)) {
    last_log_ = "cannot create cache directory " + dir;
    return "";
  }
  const std::string object = dir + "/" + key + ".hsaco";
  if (file_exists(object)) return object;

  // unique temporaries, renamed into place: concurrent processes may build the same key
  const std::string stem = dir + "/" + key + "." + std::to_string((long)getpid());
  const std::string src = stem + ".hip", tmp_obj = stem + ".hsaco.tmp", log = stem + ".log";
  {
    std::ofstream f(src);
    if (!f) {
      last_log_ = "cannot write " + src;
      return "";
    }
    // nvcc pre-includes its runtime header for every source; do the same for HIP
    f << "#include <hip/hip_runtime.h>\n" << hip_source;
  }
  std::ostringstream cmd;
  cmd << quoted(hipcc_path()) << " --genco -x hip";
  for (const auto& a : compile_args) cmd << ' ' << quoted(a);
  for (const auto& p : include_paths) cmd << " -I" << quoted(p);
  cmd << ' ' << quoted(src) << " -o " << quoted(tmp_obj) << " > " << quoted(log) << " 2>&1";
  const int rc = system(cmd.str().c_str());
  std::string out;
  {
    std::ifstream f(log);
    std::stringstream ss;
    ss << f.rdbuf();
    out = ss.str();
  }
  remove(log.c_str());
  if (rc != 0 || !file_exists(tmp_obj)) {
    // diagnostics first (the head of the output names the first error), the command last
    if (out.size() > 3000) out.resize(3000);
    last_log_ = "hipcc failed (exit " + std::to_string(rc) + "):\n" + out + "\ncommand: " + cmd.str();
    remove(tmp_obj.c_str());
    if (!getenv("TILEFUSION_JIT_KEEP")) remove(src.c_str());
    return "";
  }
  if (!getenv("TILEFUSION_JIT_KEEP")) remove(src.c_str());
  if (rename(tmp_obj.c_str(), object.c_str()) != 0) {
    last_log_ = "cannot move code object into " + object;
    return "";
  }
  return object;
}

hipFunction_t JitCompiler::load_and_get_kernel(const std::string& key, const std::string& path,
                                               const std::string& kernel_name) {
  hipModule_t module = nullptr;
  auto it = module_cache_.find(key);
  if (it != module_cache_.end()) {
    module = it->second;
  } else {
    std::ifstream f(path, std::ios::binary);
    std::stringstream ss;
    ss << f.rdbuf();
    const std::string image = ss.str();
    const hipError_t e = hipModuleLoadData(&module, image.data());
    if (e != hipSuccess) {
      last_log_ = std::string("hipModuleLoadData failed: ") + hipGetErrorString(e);
      return nullptr;
    }
    module_cache_[key] = module;
  }
  hipFunction_t fn = nullptr;
  const hipError_t e = hipModuleGetFunction(&fn, module, kernel_name.c_str());
  if (e != hipSuccess) {
    last_log_ = "kernel '" + kernel_name + "' not found in the compiled module: " + hipGetErrorString(e);
    return nullptr;
  }
  return fn;
}

hipFunction_t JitCompiler::compile_kernel(const std::string& kernel_name, const std::string& hip_source,
                                          const std::vector<std::string>& include_paths,
                                          const std::vector<std::string>& compile_args) {
  std::vector<std::string> includes = get_default_include_paths();
  includes.insert(includes.end(), include_paths.begin(), include_paths.end());
  std::vector<std::string> args = get_default_compile_args();
  args.insert(args.end(), compile_args.begin(), compile_args.end());
  std::lock_guard<std::mutex> lock(mutex_);
  // The key covers everything the code object depends on: the source, the arguments, the
  // CONTENTS of the include directories and the compiler and library versions.  A directory is
  // digested once per process, the first time a compile names it: a header edited while the
  // process runs is picked up by the next process, not by this one.  A directory too large to
  // digest whole makes the result uncacheable: the key then carries a per-process nonce and the
  // code object is deleted from the cache directory once it is loaded.
  static const std::string toolchain = toolchain_digest();
  static std::map<std::string, DirectoryDigest> dir_digests;
  std::string material = hip_source + "\n" + toolchain;
  bool cacheable = true;
  for (const auto& p : includes) {
    auto it = dir_digests.find(p);
    if (it == dir_digests.end()) it = dir_digests.emplace(p, directory_digest(p)).first;
    material += "\n-I" + p + "=" + it->second.hex;
    cacheable = cacheable && it->second.complete;
  }
  if (!cacheable) material += "\nnonce=" + process_nonce();
  for (const auto& a : args) material += "\n" + a;
  const std::string key = hash_hex(material);

  const std::string cache_key = key + ":" + kernel_name;
  auto it = kernel_cache_.find(cache_key);
  if (it != kernel_cache_.end()) return it->second;
  const std::string object = compile_to_code_object(key, hip_source, includes, args);
  if (object.empty()) return nullptr;
  hipFunction_t fn = load_and_get_kernel(key, object, kernel_name);
  if (!cacheable) remove(object.c_str());  // the module holds its own copy of the image
  if (fn) kernel_cache_[cache_key] = fn;
  return fn;
}

hipFunction_t JitCompiler::get_or_compile_kernel(const std::string& kernel_name, const std::string& hip_source,
                                                 const std::vector<std::string>& include_paths,
                                                 const std::vector<std::string>& compile_args) {
  return compile_kernel(kernel_name, hip_source, include_paths, compile_args);
}

void JitCompiler::clear_cache() {
  std::lock_guard<std::mutex> lock(mutex_);
  for (auto& kv : module_cache_) (void)hipModuleUnload(kv.second);
  module_cache_.clear();
  kernel_cache_.clear();
}

}  // namespace tilefusion::jit

// ---- C ABI --------------------------------------------------------------------------------
using tilefusion::jit::JitCompiler;

extern "C" int tf_jit_compile(const char* kernel_name, const char* source, const char* const* include_paths,
                              int num_include_paths, const char* const* compile_args, int num_compile_args,
                              void** kernel_out) {
  using namespace tfk;
  TFK_REQUIRE(kernel_name && source && kernel_out, TF_ERR_INVALID_ARG, "tf_jit_compile: null pointer");
  TFK_REQUIRE(num_include_paths >= 0 && num_compile_args >= 0 && (num_include_paths == 0 || include_paths) &&
                  (num_compile_args == 0 || compile_args),
              TF_ERR_INVALID_ARG, "tf_jit_compile: bad argument lists");
  std::vector<std::string> inc, args;
  for (int i = 0; i < num_include_paths; ++i) inc.emplace_back(include_paths[i]);
  for (int i = 0; i < num_compile_args; ++i) args.emplace_back(compile_args[i]);
  hipFunction_t fn = JitCompiler::instance().compile_kernel(kernel_name, source, inc, args);
  if (!fn) {
    set_error("tf_jit_compile: %s", JitCompiler::instance().last_log().c_str());
    return TF_ERR_HIP;
  }
  *kernel_out = reinterpret_cast<void*>(fn);
  return TF_OK;
}

extern "C" int tf_jit_launch(void* kernel, unsigned grid_x, unsigned grid_y, unsigned grid_z, unsigned block_x,
                             unsigned block_y, unsigned block_z, unsigned dynamic_lds_bytes, void* stream,
                             void** kernel_args) {
  using namespace tfk;
  TFK_REQUIRE(kernel, TF_ERR_INVALID_ARG, "tf_jit_launch: null kernel");
  TFK_REQUIRE(grid_x && grid_y && grid_z && block_x && block_y && block_z, TF_ERR_INVALID_ARG,
              "tf_jit_launch: empty grid or block");
  TFK_REQUIRE((unsigned long long)block_x * block_y * block_z <= 1024, TF_ERR_INVALID_ARG,
              "tf_jit_launch: more than 1024 threads per workgroup");
  TFK_REQUIRE(dynamic_lds_bytes <= (unsigned)kMaxLdsBytes, TF_ERR_LDS,
              "tf_jit_launch: %u bytes of dynamic LDS exceed the 160 KiB of a CU", dynamic_lds_bytes);
  hipFunction_t fn = reinterpret_cast<hipFunction_t>(kernel);
  if (dynamic_lds_bytes > 64 * 1024) {
    // opt-in for more than 64 KiB; a runtime that does not need it for module functions may
    // refuse the call, which is not an error here
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)dynamic_lds_bytes);
    (void)hipGetLastError();
  }
  TFK_HIP_TRY(hipModuleLaunchKernel(fn, grid_x, grid_y, grid_z, block_x, block_y, block_z, dynamic_lds_bytes,
                                    static_cast<hipStream_t>(stream), kernel_args, nullptr));
  return TF_OK;
}

extern "C" int tf_jit_clear_cache(void) {
  JitCompiler::instance().clear_cache();
  return TF_OK;
}

extern "C" const char* tf_jit_cache_dir(void) {
  static thread_local std::string dir;
  dir = JitCompiler::cache_dir();
  return dir.c_str();
}
