// Build configuration of the tile-programming headers for CDNA4 (gfx950).
// Same macro names as the reference's include/config.hpp:6-18; a wavefront has 64 lanes.
#pragma once

#include <hip/hip_runtime.h>

#define HOST_DEVICE __forceinline__ __host__ __device__
#define DEVICE __forceinline__ __device__
#define HOST inline __host__

#define WARP_SIZE 64

namespace tilefusion {
inline constexpr int kWarpSize = WARP_SIZE;
inline constexpr int kLdsBytesPerWorkgroup = 160 * 1024;
}  // namespace tilefusion
