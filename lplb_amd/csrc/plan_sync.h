// How the workgroups of the one-launch plan talk to each other through memory.
//
// Everything that crosses workgroups is written and read with agent-scope atomics.
// What that relies on, on gfx950 (MI355X: eight XCDs, each with its own L2 that is not
// coherent with the others'):
//   * an agent-scope atomic store or load carries the sc1 bit, which makes it write
//     through / miss in the issuing XCD's L2, so the value lives in memory where every
//     XCD sees it; an agent-scope atomic add is carried out by the atomic unit behind
//     the caches, so there is no cached copy that could go stale;
//   * s_waitcnt vmcnt(0) after such stores waits for their acknowledgement, i.e. until
//     they are visible device-wide; the counter that announces them is bumped only
//     after that wait and a workgroup barrier;
//   * everything a workgroup reads of another's is read with such loads, never with plain
//     loads behind an acquire fence: the fence (buffer_inv sc1) would invalidate this XCD's
//     L2, which holds the batch's indices at that point, once per workgroup;
//   * the compiler does not move memory operations across s_waitcnt / fences / atomics
//     of the same or wider scope.
// tests/test_host.py compiles these helpers on their own and checks that the sc1 forms
// and the invalidate are really what the compiler emits, so a toolchain change that
// lowers them differently fails a test instead of silently breaking the exchange.
// (Checked with ROCm 7.2.0, clang 20.)
#pragma once
#include <hip/hip_runtime.h>

#ifndef LPLB_POLL_PAUSE
#define LPLB_POLL_PAUSE __builtin_amdgcn_s_sleep(2)
#endif

namespace lplb {

__device__ inline int agent_load(const int *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline unsigned long long agent_load(const unsigned long long *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void agent_store(int *p, int v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void agent_store(unsigned long long *p, unsigned long long v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline int agent_add(int *p, int v) {
  return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void agent_add(unsigned long long *p, unsigned long long v) {
  __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// All earlier stores and atomics of this wave have been acknowledged.
__device__ inline void stores_have_landed() { __builtin_amdgcn_s_waitcnt(0); }

// Counting arrivals.  Updates of one 64-byte line queue up behind each other in memory
// (measured: about 14 ns each, whether or not they hit the same word; 35 ns for one word),
// so a counter that hundreds of workgroups bump would itself take microseconds.  The count
// is kept in kArrivalStripes words instead, 256 bytes apart (workgroup i bumps word
// i % kArrivalStripes), and a waiting wave reads them with one load instruction, one word
// per lane.  Loads of one line queue up as well, so the stripes exist in up to
// kArrivalCopies copies, 4 KiB apart: an arriving workgroup bumps its word in every copy
// (lanes 0..copies-1 of one wave, one instruction), a waiting workgroup polls copy
// (its id % copies).
constexpr int kArrivalStripes = 16, kArrivalStripeInts = 64, kArrivalCopies = 8;
constexpr int kArrivalCopyInts = kArrivalStripes * kArrivalStripeInts;
// Called by a whole wave.
__device__ inline void announce_arrival(int *stripes, int copies, int id) {
  const int lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  if (lane < copies)
    agent_add(stripes + lane * kArrivalCopyInts + (id % kArrivalStripes) * kArrivalStripeInts, 1);
}
// All 64 lanes of one wave poll the stripes until they add up to `target` or `max_polls`
// polls have passed.  Returns whether the target was reached (the same in every lane).
// What the arrived workgroups wrote before they announced themselves is in memory then;
// read it with agent_load.
__device__ inline bool wait_for_arrivals(int *stripes, int target, int max_polls) {
  const int lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  bool reached = false;
  for (int polls = 0; polls < max_polls && !reached; ++polls) {
    int v = lane < kArrivalStripes ? agent_load(stripes + lane * kArrivalStripeInts) : 0;
#pragma unroll
    for (int m = 1; m < kArrivalStripes; m <<= 1)
      v += __shfl_xor(v, m);
    reached = __builtin_amdgcn_readfirstlane(v) >= target;
    if (!reached)
      LPLB_POLL_PAUSE;
  }
  return reached;
}

} // namespace lplb
