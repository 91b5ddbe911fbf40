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
// Ordering, two forms.
//
// (1) The model form (host build; device build with -DKX_ARRIVE_STRICT).  In the terms of the C++ / HSA memory
// model: the increment is a release operation at agent scope and the group that sees the last count reads the
// counter back with an acquire load at agent scope.  Read-modify-writes continue each other's release
// sequences, so the value that load sees (the last increment's) belongs to the release sequence of every
// group's increment and the load synchronizes with all of them: every group's writes happen before the
// finisher's reads.  (An acquire load and not a stand-alone fence, because ThreadSanitizer, which checks the host
// model of this protocol, does not follow fences.)  Inside a group the barrier orders the other lanes' writes
// before the counting lane's release, and its acquire before their reads.  On gfx950 a release at agent scope
// writes the XCD's whole L2 back and the acquire invalidates caches; with 512 workgroups arriving per launch that
// costs 12 % of a decode step (measured: 4.62 against 4.07 ms per step, the routed down launch 41 against 24 us).
//
// (2) The device form that ships (default).  It does not lean on the language's memory model -- all accesses are
// relaxed atomics, which the model does not order -- but on what the gfx950 instructions do:
//   a. the handed-over data are written with agent-scope atomic stores, i.e. `global_store ... sc1`: written
//      through to the agent's point of coherence, never left dirty in the writing XCD's L2;
//   b. every lane then executes `s_waitcnt 0` (kx_arrive_writes_done): it returns when each of the wave's stores
//      has been acknowledged by that point of coherence;
//   c. the workgroup barrier follows, so when the counting lane issues its increment, every store of the
//      workgroup has been acknowledged (a wave issues its instructions in order; the barrier's workgroup-scope
//      fence also keeps the compiler from moving the stores or the increment across it);
//   d. the increment is an agent-scope atomic, performed at the same point of coherence, where the increments of
//      all workgroups are totally ordered.  The workgroup that reads target - 1 therefore knows that every other
//      workgroup's increment was performed, and so issued, after that workgroup's stores were acknowledged;
//   e. it reads the data with agent-scope atomic loads (`global_load ... sc1`), which are served by the point of
//      coherence and not by a line that its own L1 or XCD L2 might still hold, and it issues them after the
//      increment's return value has arrived (the branch on it needs the value; loads are not speculated).
// The plain accesses on these paths (routing weights, the residual row that is read, modified and written, the
// counter reset) touch only data that an earlier launch wrote or that no other workgroup of this launch touches.
// The GPU tests hold every kernel that uses the protocol to the oracle's bits in both forms of launch (fused and
// separate), which would differ if a finisher ever read a stale value.
//
// The same header compiles for the host (tests build a thread model of the protocol under ThreadSanitizer: in
// form (1) it is race-free, with relaxed operations it is reported).
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

// Every lane of a group, after its last write and before the group's barrier.
KX_ARRIVE_FN void kx_arrive_writes_done() {
#if defined(__HIP_DEVICE_COMPILE__) && !defined(KX_ARRIVE_STRICT)
  __builtin_amdgcn_s_waitcnt(0);  // this wave's stores have been acknowledged by the memory they were written through to
#endif
}
// One caller per group.  True for the group that completes `target` arrivals; it has then acquired what every
// group released before counting itself in.
KX_ARRIVE_FN bool kx_arrive_is_last(int *counter, int target) {
#if defined(__HIP_DEVICE_COMPILE__) && !defined(KX_ARRIVE_STRICT)
  return KX_ARRIVE_ADD(counter, __ATOMIC_RELAXED) == target - 1;
#endif
  const bool last = KX_ARRIVE_ADD(counter, KX_ARRIVE_ORDER) == target - 1;
  if (last && KX_ARRIVE_ORDER != __ATOMIC_RELAXED) (void)KX_ARRIVE_LOAD_ACQUIRE(counter);
  return last;
}
// The data accesses of the hand-over: every value one group writes for the finisher goes through kx_arrive_store,
// every read of such a value by the finisher through kx_arrive_load (relaxed, agent scope: written through to / read
// from the device's point of coherence).  A plain store or load on these paths would break the argument above
// silently, so the accesses carry a name that can be searched for.
#if defined(__HIPCC__)
template <class T>
__device__ __forceinline__ void kx_arrive_store(T *p, T v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
template <class T>
__device__ __forceinline__ T kx_arrive_load(const T *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
#endif
// By the finishing group, once it is done: the counter is zero again for the next launch.
KX_ARRIVE_FN void kx_arrive_reset(int *counter) { __atomic_store_n(counter, 0, __ATOMIC_RELAXED); }
