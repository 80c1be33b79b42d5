// Default include paths and compiler arguments of the run-time compiler (counterpart of
// include/jit/config.hpp:8-29).
#pragma once

#include <string>
#include <vector>

namespace tilefusion::jit {

// The directory that holds types/, cell/, kernels/ - found from this header's own location.
inline std::vector<std::string> get_default_include_paths() {
  const std::string current_file = __FILE__;
  const size_t pos = current_file.rfind("/jit/");
  if (pos == std::string::npos) return {};
  return {current_file.substr(0, pos)};
}

// hipcc arguments for a gfx950 code object.  The packed-fp32 feature is switched off like in
// every other build of this library.
inline std::vector<std::string> get_default_compile_args() {
  return {"-O3", "-std=c++20", "--offload-arch=gfx950", "-DNDEBUG", "-Xclang", "-target-feature",
          "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"};
}

}  // namespace tilefusion::jit
