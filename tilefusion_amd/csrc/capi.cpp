// Error reporting and version of the C ABI (declared in include/tilefusion_c.h).
#include <cstring>

#include "common.hpp"

namespace tfk {
namespace {
thread_local char g_last_error[4096] = "";  // room for a compiler diagnostic
}

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

int hip_fail(hipError_t e, const char* what) {
  set_error("HIP error '%s' from %s", hipGetErrorString(e), what);
  return TF_ERR_HIP;
}
}  // namespace tfk

extern "C" {
const char* tf_last_error(void) { return tfk::g_last_error; }
const char* tf_version(void) { return "tilefusion-mi355x 0.1.0 (gfx950)"; }
}
