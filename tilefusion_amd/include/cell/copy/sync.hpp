// Fences for asynchronous global -> LDS copies (counterpart of include/cell/copy/sync.hpp:10-26,
// which wraps cp.async.commit_group / cp.async.wait_group).
//
// On CDNA4 an asynchronous copy is an LDS-direct load (global_load_lds_dwordx4): it is issued
// like any vector-memory load, writes LDS without passing through a register, and is tracked by
// the wavefront's vector-memory counter (vmcnt), which retires loads in issue order.  A "copy
// group" is therefore simply the loads a wavefront issued between two commit_copy_group()
// calls, and "at most N groups still in flight" becomes "at most N x (loads per group) loads
// still in flight":
//
//   wait_group<N, kLoadsPerGroup>()  ->  s_waitcnt vmcnt(N * kLoadsPerGroup) lgkmcnt(0)
//
// kLoadsPerGroup must not exceed the number of loads EVERY wavefront issues in each group (a
// smaller value only waits longer, never too little); the default of 1 is right for any group
// that contains at least one workgroup-wide loader call, and the loaders export the exact
// figure as kLoadsPerLane for callers that want the last group to stay fully in flight.
// lgkmcnt(0) covers the loaders that stage through registers (their ds_write is the last step).
// Vector-memory STORES issued while groups are in flight share the counter and may retire out
// of order with the loads: in such a loop use wait_group<0>().
#pragma once

#include "config.hpp"

namespace tilefusion::cell::copy {

// Closes the current copy group: everything issued so far belongs to it.  The group itself needs
// no hardware state (the counter is per load); the call pins the issue order for the compiler.
DEVICE void commit_copy_group() { asm volatile("" ::: "memory"); }

template <int N, int kLoadsPerGroup = 1>
DEVICE void wait_group() {
  static_assert(N >= 0 && kLoadsPerGroup >= 0, "N groups of kLoadsPerGroup loads each may stay in flight");
  constexpr int kPending = N * kLoadsPerGroup > 63 ? 63 : N * kLoadsPerGroup;   // vmcnt is a 6-bit counter
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kPending) : "memory");
}

DEVICE void __copy_async() {
  commit_copy_group();
  wait_group<0>();
}

// Workgroup barrier that leaves asynchronous copies in flight: it waits for this wavefront's
// LDS traffic only.  (__syncthreads() is a full fence and may drain the vector-memory counter,
// which would turn every multi-stage pipeline into a two-stage one.)
DEVICE void sync_threads_keep_copies() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

}  // namespace tilefusion::cell::copy
