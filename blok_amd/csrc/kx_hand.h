// kx_hand.h -- values handed between the workgroups of one resident launch as tagged words.
// A value travels as one 32-bit word, the launch's 16-bit tag above its 16 payload bits (a bf16 value; an fp32 value
// as two words).  The writer stores the word with a relaxed agent-scope store; a reader requests the words it needs
// with agent-scope loads and asks again until every word carries the tag.  A word is one atomic object: no counter,
// no barrier, no acknowledgement, nothing to order or to reset; the tag differs from launch to launch on the same
// array, so a stale word is never taken for a fresh one.  Readers wait for writers, so every workgroup of the launch
// must be resident at once (the launchers check what they can: workgroups against CUs and the kernel's footprint).
// The wait is bounded: after KX_HAND_SPIN_LIMIT polls a reader sets the error flag and goes on with whatever it
// has, so the grid always drains; the host reports the flag at its next synchronisation.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace kxh {

constexpr int KX_HAND_SPIN_LIMIT = 1 << 16;  // polls of a microsecond or so each

// A value handed to other workgroups of the launch travels as one 32-bit word, the launch's tag above the bf16
// bits: whoever reads the word with the right tag has the value, so there is no counter to arrive at, no store to
// wait for and nothing to order -- each word is one relaxed atomic object.
__device__ __forceinline__ void hand_store(uint32_t *p, uint32_t tag, uint16_t v) {
  __hip_atomic_store(p, (tag << 16) | v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Four consecutive words at agent scope (served by the point of coherence, not by a line an L2 may still hold) as one
// 16-byte request; hand_wait completes the requests of a wave and ties the registers to the wait, so that no use of
// them is scheduled before it.
// the compiler may not move a memory access across this point: loads are requested in the order they are written
__device__ __forceinline__ void issue_order() { asm volatile("" ::: "memory"); }
typedef unsigned int hand4 __attribute__((ext_vector_type(4)));  // a register quad, as inline asm takes it
__device__ __forceinline__ void hand_request4(const uint32_t *p, hand4 &v) {
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
}
__device__ __forceinline__ void hand_wait(hand4 &a) { asm volatile("s_waitcnt vmcnt(0)" : "+v"(a)::"memory"); }
__device__ __forceinline__ void hand_wait(hand4 &a, hand4 &b) { asm volatile("s_waitcnt vmcnt(0)" : "+v"(a), "+v"(b)::"memory"); }
__device__ __forceinline__ bool hand_tagged(const hand4 &v, uint32_t tag) {
  return (v.x >> 16) == tag && (v.y >> 16) == tag && (v.z >> 16) == tag && (v.w >> 16) == tag;
}
// the bf16 halves of four tagged words as two packed words
__device__ __forceinline__ uint2 hand_pack(const hand4 &v) { return make_uint2((v.x & 0xffffu) | (v.y << 16), (v.z & 0xffffu) | (v.w << 16)); }
// one more poll has failed: true when the reader should give up (the flag is set: too many polls, or an earlier
// launch gave up already), so that the grid always drains
__device__ __forceinline__ bool hand_give_up(int &polls, int *err) {
  if (++polls > KX_HAND_SPIN_LIMIT || (polls == 1 && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
    __hip_atomic_store(err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return true;
  }
  __builtin_amdgcn_s_sleep(2);
  return false;
}
// reads N (4 or 8) consecutive words, 16-byte aligned, until all carry the tag; returns their bf16 halves packed
template <int N>
__device__ __forceinline__ void hand_load(const uint32_t *p, uint32_t tag, int *err, uint32_t (&packed)[N / 2]) {
  static_assert(N == 4 || N == 8, "words per call");
  int polls = 0;
  hand4 v0, v1 = {0, 0, 0, 0};
  while (true) {
    hand_request4(p, v0);
    if (N == 8) hand_request4(p + 4, v1);
    if (N == 8) hand_wait(v0, v1);
    else hand_wait(v0);
    if ((hand_tagged(v0, tag) && (N == 4 || hand_tagged(v1, tag))) || hand_give_up(polls, err)) break;
  }
  const uint2 a = hand_pack(v0);
  packed[0] = a.x; packed[1] = a.y;
  if constexpr (N == 8) {
    const uint2 b = hand_pack(v1);
    packed[2] = b.x; packed[3] = b.y;
  }
}

}  // namespace kxh
