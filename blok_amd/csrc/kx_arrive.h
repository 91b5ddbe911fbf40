// kx_arrive.h -- "the last one in finishes the job": how workgroups of one launch hand results to each other
// without anybody waiting.  Used by the q_b GEMV that completes a head's query (kx_dense.hip), the router GEMV
// whose last workgroup does top-k and bucketing (kx_dense.hip) and the routed down GEMV that combines a block
// of rows (kx_i4.hip).  No counterpart in the reference, which runs each of these steps as a launch of its own
// (src/kimi_exec.cu:812-877).
//
// Protocol.  Every group (a workgroup on the GPU, a thread in the host model of it) first writes its results,
// then one caller of the group -- after a barrier behind which all the group's writes lie -- counts the group
// in with kx_arrive_is_last().  The group that completes `target` arrivals gets true: it may now read what all
// the groups wrote, finish the job and put the counter back to zero with kx_arrive_reset() (the next use of
// the counter is ordered behind it by the launch boundary).  Nobody spins, so nothing can deadlock.
//
// Ordering, in the terms of the C++ / HSA memory model: the increment is a release operation at agent scope
// and the group that sees the last count reads the counter back with an acquire load at agent scope.
// Read-modify-writes continue each other's release sequences, so the value that load sees (the last increment's)
// belongs to the release sequence of every group's increment and the load synchronizes with all of them: every
// group's writes happen before the finisher's reads.  (An acquire load and not a stand-alone fence, because
// ThreadSanitizer, which checks the host model of this protocol, does not follow fences.)  Inside a group the barrier orders the other lanes' writes before the counting lane's release, and
// its acquire before their reads.  On gfx950 the release writes the XCD's L2 back and the acquire invalidates
// the finisher's L1 and the non-coherent lines of its L2, which is what makes data from the other seven XCDs
// visible; the kernels additionally store and load the handed-over data with agent-scope accesses.
//
// The same header compiles for the host (tests build a thread model of the protocol under ThreadSanitizer:
// with the ordering above it is race-free, with relaxed operations it is reported).
#pragma once

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define KX_ARRIVE_FN __host__ __device__ inline
#else
#define KX_ARRIVE_FN static inline
#endif
#if defined(__HIP_DEVICE_COMPILE__)
#define KX_ARRIVE_ADD(p, order) __hip_atomic_fetch_add((p), 1, (order), __HIP_MEMORY_SCOPE_AGENT)
#define KX_ARRIVE_LOAD_ACQUIRE(p) __hip_atomic_load((p), __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT)
#else
#define KX_ARRIVE_ADD(p, order) __atomic_fetch_add((p), 1, (order))
#define KX_ARRIVE_LOAD_ACQUIRE(p) __atomic_load_n((p), __ATOMIC_ACQUIRE)
#endif

#ifndef KX_ARRIVE_ORDER
#define KX_ARRIVE_ORDER __ATOMIC_RELEASE  // a test may build the model with __ATOMIC_RELAXED to see it reported
#endif

// One caller per group.  True for the group that completes `target` arrivals; it has then acquired what every
// group released before counting itself in.
KX_ARRIVE_FN bool kx_arrive_is_last(int *counter, int target) {
  const bool last = KX_ARRIVE_ADD(counter, KX_ARRIVE_ORDER) == target - 1;
  if (last && KX_ARRIVE_ORDER != __ATOMIC_RELAXED) (void)KX_ARRIVE_LOAD_ACQUIRE(counter);
  return last;
}
// By the finishing group, once it is done: the counter is zero again for the next launch.
KX_ARRIVE_FN void kx_arrive_reset(int *counter) { __atomic_store_n(counter, 0, __ATOMIC_RELAXED); }
