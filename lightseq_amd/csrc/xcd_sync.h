// Synchronisation among the workgroups of ONE XCD inside a running kernel.
//
// An MI355X has 8 XCDs of 32 compute units, each XCD with its own L2.  A device-wide barrier
// inside a kernel has to make one XCD's stores visible to the others, which means writing its
// L2 back (tens of microseconds).  Workgroups of the same XCD share their L2: a store that has
// been acknowledged is in that L2, an atomic executes there, and a load that skips the compute
// unit's vector cache (sc1) reads from there.  So a barrier among them needs no cache
// maintenance at all: every workgroup waits for its own stores (s_waitcnt vmcnt(0)), adds one
// to a counter in the L2, and polls the counter; data that another compute unit wrote during
// the launch is then read with sc1 loads.  Measured: ~1 us per barrier of 32 workgroups.
//
// The protocol below is written against a memory policy `Mem` (load / add / or / pause) so that
// the same text runs on the GPU (policy over L2-scope HIP atomics, in the kernel's source file)
// and in a host model with one thread per workgroup (tests/xcd_sync_model.cpp), where the
// give-up path can be driven.
//
//  * Counters only grow: round r of a launch waits for base + expected * (r + 1), `base` being
//    what the counter held before the launch (the host keeps count), compared modulo 2^32.
//  * Every wait is bounded: after `spin_limit` polls the waiter sets kXcdErrTimeout in the
//    error word and returns false; every waiter also looks at the error word (on entry and
//    every 64 polls) and returns false once it is set.  A caller that gets false leaves the
//    kernel at once -- every wavefront of the workgroup, through a flag in LDS -- so a kernel
//    whose workgroups could not all become resident ends instead of spinning.
//  * Which workgroups form an XCD is read from the hardware (the XCC_ID register); the kernel
//    that uses the barrier has to make sure that every XCD holds exactly `expected` of its
//    workgroups -- too few and the waiters give up (kXcdErrTimeout), too many and a round
//    would complete early, so a workgroup that finds its place taken sets kXcdErrMapping.
#pragma once

#ifndef LSH_XCD_FN
#define LSH_XCD_FN inline
#endif

namespace lsh {

constexpr unsigned kXcdErrTimeout = 1u;  // a wait gave up
constexpr unsigned kXcdErrMapping = 2u;  // two workgroups took the same place of an XCD
constexpr int kXcdCount = 8;
constexpr int kXcdCounterStride = 32;  // unsigned words between two XCDs' counters (128 bytes)

// One thread of the workgroup: announce the arrival, then wait until `expected` workgroups have
// arrived at this round.  True: all arrived.  False: give up (error word set by someone).
template <typename Mem>
LSH_XCD_FN bool xcd_arrive_and_wait(unsigned* counter, unsigned target, unsigned* error,
                                    int spin_limit) {
  if (Mem::load(error) != 0u) return false;
  Mem::add(counter, 1u);
  for (int spin = 0; spin < spin_limit; ++spin) {
    if ((int)(Mem::load(counter) - target) >= 0) return true;
    if ((spin & 63) == 63 && Mem::load(error) != 0u) return false;
    Mem::pause();
  }
  Mem::fetch_or(error, kXcdErrTimeout);
  return false;
}

}  // namespace lsh
