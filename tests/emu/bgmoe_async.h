// TEST INFRASTRUCTURE: the CPU emulator's version of csrc/bgmoe_async.h (same names, same contracts).  The emulation
// build stages the kernel sources next to THIS file instead of the library's header, whose bodies are gfx950 inline
// assembly.
//
// Two completion models for the asynchronous global -> LDS loads (emu_core.cc, chosen per launch by the tests):
//  * eager: the copy happens when the load is issued -- the earliest a load can land.  A ring slot that is refilled
//    before every wave has finished reading it shows up as wrong data.
//  * lazy: the copy happens only when a wait_vm<N>() of the issuing lane leaves it no other choice (all but the N
//    youngest loads of that lane complete, in issue order) or when the lane ends -- the latest a load can land under
//    the kernel's own waits, IF the kernel's wait counts count nothing but these loads.  A wait that is too lenient
//    shows up as stale data.  Kernels whose wait counts also count ordinary loads in between (the weight-streaming
//    kernels) need the counted form of this model: the staged gload_* helpers report every ordinary global load, which
//    then takes a place in the lane's queue although its value arrives at once.
#pragma once
#include "bgmoe_common.h"
#include "bgmoe_hostdev.h"

__device__ __forceinline__ void async_load16(const uint8_t* base, uint32_t lane_off, uint32_t lds_base) {
  emu::async_load(base, lane_off, lds_base, 16);
}
__device__ __forceinline__ void async_load4(const float* base, uint32_t lane_off, uint32_t lds_base) {
  emu::async_load(base, lane_off, lds_base, 4);
}
template <typename T>
__device__ __forceinline__ const T* uniform_ptr(const T* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  return reinterpret_cast<const T*>(bgmoe_compose_u64(__builtin_amdgcn_readfirstlane((uint32_t)v),
                                                      __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32))));
}
template <int N>
__device__ __forceinline__ void wait_vm() { emu::wait_vm(N); }
__device__ __forceinline__ void block_barrier() { emu::block_barrier(); }
__device__ __forceinline__ void lds_exchange_barrier() { emu::block_barrier(); }
