// kx_lds_copy.h -- global -> LDS copies issued behind the compiler's back, and the barrier and waits that go
// with them.  Shared by the matrix-core kernels (kx_mla.hip, kx_prefill.hip, kx_skinny.hip), which stage their
// operand tiles through LDS several tiles ahead.  No counterpart in the reference (its kernels load straight
// into registers, src/kimi_exec.cu:272-323).
//
// Why asm: a copy the compiler knows of is completed (s_waitcnt vmcnt(0)) in front of every LDS access it
// cannot tell from the copy's target and in front of every fenced barrier, which makes the tiles copied ahead
// land at once.  Issued from asm the copy is unknown to it; the kernel waits for a tile itself, by count, where
// it needs the tile (copies of a wave complete in order), and its barrier carries no fence.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// global_load_lds_dwordx4: lane i's 16 bytes at `src` land at LDS byte address lds_base + 16 i.  lds_base must
// be wave-uniform.  The instruction takes the LDS address from m0; m0 is put back, the compiler owns it.
__device__ __forceinline__ void kx_copy16_to_lds(const void *src, uint32_t lds_base) {
  uint32_t m0_saved;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0"
               : "=&s"(m0_saved)
               : "s"(lds_base), "v"(src)
               : "memory");
}
// waits until at most N of this wave's copies (and loads) are in flight
template <int N>
__device__ __forceinline__ void kx_wait_copies() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// workgroup barrier without a fence: the wave's LDS operations are complete, nothing else is waited for
__device__ __forceinline__ void kx_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
