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

// Wavefront-wide asynchronous copy (global_load_lds_dwordx4): lane l's 16 bytes land at LDS byte
// address `lds_wave_base` + 16 * l, where lds_wave_base is uniform over the wavefront and
// `global_src` is per lane.  No register staging; completion is tracked by vmcnt only, and the
// compiler is deliberately not told that LDS is written (it would otherwise drain the counter in
// front of every LDS read): ordering against readers is the caller's wait_group<N>() + barrier,
// exactly the contract of the reference's cp.async atom (include/cell/copy/copy_atom.hpp:18-48).
DEVICE void ld_global_direct_to_shared_16B(unsigned lds_wave_base, const void* global_src) {
  // readfirstlane: the value is uniform by contract, this makes it a scalar register by type
  const unsigned base = __builtin_amdgcn_readfirstlane(lds_wave_base);
  // M0 (the LDS destination) is an INPUT of the statement: the compiler writes it and cannot use
  // the register for anything else between that write and the load; the s_nop is the wait state
  // an M0 write needs in front of an LDS-direct load
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(global_src), "{m0}"(base)
               : "memory");
}
// LDS byte address of a pointer into LDS (what M0 takes).
DEVICE unsigned lds_byte_address(const void* p) {
  return (unsigned)(size_t)((__attribute__((address_space(3))) const char*)p);
}

}  // namespace tilefusion::cell::copy::atom
