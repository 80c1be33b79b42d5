// 16-byte copy atoms (counterpart of include/cell/copy/copy_atom.hpp:18-149).  The reference's
// atoms wrap cp.async / vectorised ld+st; on CDNA4 a lane moves 16 bytes with
// global_load_dwordx4 + ds_write_b128 (through a register) or, for layouts where the 64 lanes
// of a wavefront land on 1 KiB of consecutive LDS, with the LDS-direct load that never
// touches a VGPR.
#pragma once

#include "config.hpp"

namespace tilefusion::cell::copy::atom {

// global -> LDS through a register; complete once the lane's vmcnt and lgkmcnt have drained
template <int kBytes>
DEVICE void ld_global_st_shared(void* shared_dst, const void* global_src) {
  static_assert(kBytes == 4 || kBytes == 8 || kBytes == 16, "copy atoms move 4, 8 or 16 bytes");
  if constexpr (kBytes == 16) {
    *static_cast<uint4*>(shared_dst) = *static_cast<const uint4*>(global_src);
  } else if constexpr (kBytes == 8) {
    *static_cast<uint2*>(shared_dst) = *static_cast<const uint2*>(global_src);
  } else {
    *static_cast<unsigned*>(shared_dst) = *static_cast<const unsigned*>(global_src);
  }
}

// LDS -> global through a register
template <int kBytes>
DEVICE void ld_shared_st_global(void* global_dst, const void* shared_src) {
  ld_global_st_shared<kBytes>(global_dst, shared_src);
}

// Wavefront-wide LDS-direct load (global_load_lds_dwordx4): lane l's 16 bytes land at
// lds_base + 16 * l, where lds_base is uniform over the wavefront and 16-byte aligned;
// `global_src` is per lane.  No register staging; completion is tracked by vmcnt.
DEVICE void ld_global_direct_to_shared_16B(void* lds_base, const void* global_src) {
  __builtin_amdgcn_global_load_lds(global_src, (__attribute__((address_space(3))) void*)lds_base, 16, 0, 0);
}

}  // namespace tilefusion::cell::copy::atom
