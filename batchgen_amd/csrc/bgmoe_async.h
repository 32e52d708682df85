// Asynchronous global -> LDS loads (gfx950 global_load_lds_*) and the hand-placed waits that go with them.
//
// The loads are issued from inline asm, so the compiler does not count them in its own s_waitcnt
// bookkeeping: a kernel that uses them waits with wait_vm<N>() (vector-memory loads complete in issue
// order, so "at most N outstanding" means everything older than the N youngest has landed) and makes
// the data visible to the other waves with block_barrier().
#pragma once
#include "bgmoe_common.h"
#include "bgmoe_hostdev.h"

// 64 lanes x 16 bytes -> LDS [lds_base, lds_base + 1024); lds_base must be wave-uniform.  No
// instruction offset is used: the hardware would add it to the LDS address as well as to the
// global address.
// The global address is a wave-uniform base plus a 32-bit byte offset per lane.
// s_nop 4: the base may have just been written by a VALU instruction (v_readlane restoring a spilled SGPR, a
// v_readfirstlane), and a vector-memory instruction that reads an SGPR needs five wait states after a VALU write
// to it; the compiler does not look inside the asm to insert them.
__device__ __forceinline__ void async_load16(const uint8_t* base, uint32_t lane_off, uint32_t lds_base) {
  asm volatile("s_nop 4\n\ts_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(lds_base), "v"(lane_off), "s"(base) : "memory", "m0");
}
// 64 lanes x 4 bytes -> LDS [lds_base, lds_base + 256)
__device__ __forceinline__ void async_load4(const float* base, uint32_t lane_off, uint32_t lds_base) {
  asm volatile("s_nop 4\n\ts_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :: "s"(lds_base), "v"(lane_off), "s"(base) : "memory", "m0");
}
template <typename T>
__device__ __forceinline__ const T* uniform_ptr(const T* p) {   // tell the compiler a pointer is wave-uniform
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  // the builtin returns `int`: bgmoe_compose_u64 takes both halves as unsigned, so bit 31 of the low half cannot
  // sign-extend into the high half
  return reinterpret_cast<const T*>(bgmoe_compose_u64(__builtin_amdgcn_readfirstlane((uint32_t)v),
                                                      __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32))));
}
template <int N>
__device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }
__device__ __forceinline__ void block_barrier() { asm volatile("s_barrier" ::: "memory"); }
// Barrier for an exchange through LDS only: this wave's LDS writes are done (lgkmcnt(0)), then the barrier.  Unlike
// __syncthreads() it does not wait for vector-memory operations, so asynchronous global -> LDS loads that are in
// flight for LATER use stay in flight across it.
__device__ __forceinline__ void lds_exchange_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

