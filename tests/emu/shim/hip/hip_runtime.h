// TEST INFRASTRUCTURE: a stand-in for <hip/hip_runtime.h> that lets the library's kernel sources be compiled as plain
// C++ for x86-64 and run on the CPU by tests/emu/emu_core.cc -- one fiber per GPU lane, wave-wide operations
// (matrix instructions, shuffles, ballots, readfirstlane) and barriers as rendezvous points between the fibers.
// It exists to execute a kernel's control flow, index arithmetic, LDS protocol and launch code before a GPU has
// run it; it is not a product path, nothing in the package loads what is built from it, and it says nothing about
// speed or about the hardware's rounding inside a matrix instruction (sums are taken in fp32 in ascending K).
#pragma once
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <functional>

#define BGMOE_CPU_EMU 1

// ---- qualifiers -------------------------------------------------------------------------------------------------------
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
// every __shared__ object lands in one ELF section, which the emulator poisons at the start of each block and uses
// to tell LDS addresses from others
#define __shared__ static __attribute__((section("emu_lds")))
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))

// ---- basic types ------------------------------------------------------------------------------------------------------
struct dim3 {
  unsigned x, y, z;
  constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct uint2 { unsigned x, y; };
struct uint4 { unsigned x, y, z, w; };
struct int2 { int x, y; };
struct int4 { int x, y, z, w; };
struct float2 { float x, y; };
struct float4 { float x, y, z, w; };
static inline uint2 make_uint2(unsigned x, unsigned y) { return uint2{x, y}; }
static inline uint4 make_uint4(unsigned x, unsigned y, unsigned z, unsigned w) { return uint4{x, y, z, w}; }
static inline float2 make_float2(float x, float y) { return float2{x, y}; }
static inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }

typedef struct emu_stream_t* hipStream_t;
typedef int hipError_t;
enum { hipSuccess = 0, hipErrorInvalidValue = 1 };
enum { hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
enum { hipDeviceAttributeMultiprocessorCount = 63 };
enum { hipMemcpyDeviceToHost = 2, hipMemcpyHostToDevice = 1 };
struct hipDeviceProp_t { int multiProcessorCount; char gcnArchName[64]; };

// ---- the emulator's interface (tests/emu/emu_core.cc) -----------------------------------------------------------------
namespace emu {
struct Lane {
  dim3 tid, bid, bdim, gdim;
  unsigned lane, wave;
};
Lane& lane();                                   // the fiber that is running
constexpr int kCus = 16;                        // the emulated device: 16 compute units (two per XCD)
void launch(dim3 grid, dim3 block, size_t dynamic_lds, const std::function<void()>& body);
uint8_t* dynamic_lds();
void block_barrier();
void wave_sync();                               // rendezvous of the wave's lanes (lanes are NOT in lockstep here)
uint32_t shfl32(uint32_t v, int src_lane);      // value of lane src_lane (mod 64); own value when that lane is absent
uint64_t ballot(bool pred);
uint32_t readfirstlane32(uint32_t v);
uint32_t readlane32(uint32_t v, int lane);
// v_mov_dpp: quad_perm (ctrl < 0x100), row_mirror 0x140, row_half_mirror 0x141, row_bcast15 0x142, row_bcast31 0x143
uint32_t update_dpp32(uint32_t old, uint32_t src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl);
// matrix instructions: every lane passes its operand registers, gets its result registers
void mfma_16x16x128_f8(const int32_t* a8, const int32_t* b8, const float* c4, float* d4);
void mfma_32x32x64_f8(const int32_t* a8, const int32_t* b8, const float* c16, float* d16);
void mfma_16x16x32_bf16(const uint16_t* a8, const uint16_t* b8, const float* c4, float* d4);
// asynchronous global -> LDS loads (see bgmoe_async.h of this directory)
void async_load(const void* base, uint32_t lane_off, uint32_t lds_base, unsigned bytes, bool uniform_base = true);
void wait_vm(int n);
void count_vm_load();                           // an ordinary global load, for the counted lazy model
float e4m3_to_f32(uint8_t b);
uint8_t f32_to_e4m3(float f);
}  // namespace emu

#define threadIdx (emu::lane().tid)
#define blockIdx (emu::lane().bid)
#define blockDim (emu::lane().bdim)
#define gridDim (emu::lane().gdim)

#define hipLaunchKernelGGL(kernel, grid, block, lds, stream, ...) \
  emu::launch((grid), (block), (size_t)(lds), [=]() { kernel(__VA_ARGS__); })

// events carry the host's clock (what an emulated kernel takes on the CPU, of no meaning for the GPU)
struct emu_event { double ms; };
typedef emu_event* hipEvent_t;
double emu_now_ms();
static inline hipError_t hipEventCreate(hipEvent_t* e) { *e = new emu_event{0.0}; return hipSuccess; }
static inline hipError_t hipEventRecord(hipEvent_t e, hipStream_t = nullptr) { e->ms = emu_now_ms(); return hipSuccess; }
static inline hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
static inline hipError_t hipEventElapsedTime(float* ms, hipEvent_t a, hipEvent_t b) { *ms = (float)(b->ms - a->ms); return hipSuccess; }
static inline hipError_t hipDeviceSynchronize() { return hipSuccess; }
static inline hipError_t hipMemcpy(void* dst, const void* src, size_t n, int) { memcpy(dst, src, n); return hipSuccess; }
static inline unsigned long long wall_clock64() { return (unsigned long long)(emu_now_ms() * 1e5); }
static inline hipError_t hipGetLastError() { return hipSuccess; }
static inline const char* hipGetErrorString(hipError_t) { return "emulated"; }
static inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
static inline hipError_t hipDeviceGetAttribute(int* v, int, int) { *v = emu::kCus; return hipSuccess; }
static inline hipError_t hipGetDeviceProperties(hipDeviceProp_t* p, int) {
  p->multiProcessorCount = emu::kCus;
  strcpy(p->gcnArchName, "gfx950-emulated");
  return hipSuccess;
}
static inline hipError_t hipFuncSetAttribute(const void*, int, int) { return hipSuccess; }
template <typename K>
static inline hipError_t hipOccupancyMaxActiveBlocksPerMultiprocessor(int* n, K, int, size_t) { *n = 2; return hipSuccess; }
#define HIP_SYMBOL(x) (&(x))
template <typename T>
static inline hipError_t hipGetSymbolAddress(void** p, T* sym) { *p = (void*)sym; return hipSuccess; }

// ---- device functions -------------------------------------------------------------------------------------------------
using std::max;
using std::min;
static inline unsigned min(unsigned a, int b) { return a < (unsigned)b ? a : (unsigned)b; }
static inline unsigned min(int a, unsigned b) { return (unsigned)a < b ? (unsigned)a : b; }
static inline int64_t min(int64_t a, int b) { return a < b ? a : (int64_t)b; }
static inline int64_t min(int a, int64_t b) { return a < b ? (int64_t)a : b; }
static inline int64_t max(int64_t a, int b) { return a > b ? a : (int64_t)b; }
static inline int64_t max(int a, int64_t b) { return a > b ? (int64_t)a : b; }

static inline float __uint_as_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline float __int_as_float(int u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t __float_as_uint(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline int __float_as_int(float f) { int u; memcpy(&u, &f, 4); return u; }
#define __expf(x) expf(x)
static inline float __fdividef(float a, float b) { return a / b; }
static inline int __popcll(unsigned long long v) { return __builtin_popcountll(v); }
static inline int __popc(unsigned v) { return __builtin_popcount(v); }
static inline int __ffsll(long long v) { return __builtin_ffsll(v); }
static inline int __ffs(int v) { return __builtin_ffs(v); }
static inline int __clz(int v) { return v ? __builtin_clz((unsigned)v) : 32; }
static inline void __syncthreads() { emu::block_barrier(); }
static inline void __threadfence() {}
static inline void __threadfence_block() {}

// lane values of 4 or 8 bytes travel as one or two 32-bit words
template <typename T>
static inline T emu_shfl_any(T v, int src) {
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "lane values of 4 or 8 bytes only");
  uint32_t w[2] = {0, 0};
  memcpy(w, &v, sizeof(T));
  w[0] = emu::shfl32(w[0], src);
  if (sizeof(T) == 8) w[1] = emu::shfl32(w[1], src);
  T t;
  memcpy(&t, w, sizeof(T));
  return t;
}
template <typename T>
static inline T __shfl(T v, int src, int = 64) { return emu_shfl_any(v, src); }
template <typename T>
static inline T __shfl_xor(T v, int mask, int = 64) { return emu_shfl_any(v, (int)(emu::lane().lane ^ (unsigned)mask)); }
template <typename T>
static inline T __shfl_up(T v, unsigned delta, int = 64) {
  const int src = (int)emu::lane().lane - (int)delta;
  const T got = emu_shfl_any(v, src < 0 ? (int)emu::lane().lane : src);
  return src < 0 ? v : got;
}
template <typename T>
static inline T __shfl_down(T v, unsigned delta, int = 64) {
  const int src = (int)emu::lane().lane + (int)delta;
  const T got = emu_shfl_any(v, src > 63 ? (int)emu::lane().lane : src);
  return src > 63 ? v : got;
}
template <typename T>
static inline T emu_from32(uint32_t u) { T t; static_assert(sizeof(T) == 4, "32-bit lane values only"); memcpy(&t, &u, 4); return t; }
template <typename T>
static inline uint32_t emu_to32(T t) { uint32_t u; static_assert(sizeof(T) == 4, "32-bit lane values only"); memcpy(&u, &t, 4); return u; }
static inline unsigned long long __ballot(int pred) { return emu::ballot(pred != 0); }
static inline int __any(int pred) { return emu::ballot(pred != 0) != 0; }
static inline int __all(int pred) { return emu::ballot(pred == 0) == 0; }

template <typename T>
static inline T atomicAdd(T* p, T v) { const T old = *p; *p = old + v; return old; }
template <typename T>
static inline T atomicExch(T* p, T v) { const T old = *p; *p = v; return old; }
template <typename T>
static inline T atomicOr(T* p, T v) { const T old = *p; *p = old | v; return old; }
template <typename T>
static inline T atomicMax(T* p, T v) { const T old = *p; *p = old > v ? old : v; return old; }

// ---- AMDGCN builtins ----------------------------------------------------------------------------------------------------
template <typename T>
static inline T emu_readfirstlane(T v) { return emu_from32<T>(emu::readfirstlane32(emu_to32(v))); }
template <typename T>
static inline T emu_readlane(T v, int l) { return emu_from32<T>(emu::readlane32(emu_to32(v), l)); }
#define __builtin_amdgcn_readfirstlane(v) emu_readfirstlane(v)
#define __builtin_amdgcn_readlane(v, l) emu_readlane((v), (l))
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_update_dpp(old, src, ctrl, rows, banks, bc) \
  ((int)emu::update_dpp32((uint32_t)(old), (uint32_t)(src), (ctrl), (rows), (banks), (bc)))
#define __builtin_amdgcn_fence(...) ((void)0)
#define __builtin_amdgcn_wave_barrier() emu::wave_sync()
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __builtin_amdgcn_rcp(x) (1.0 / (x))
#define __builtin_amdgcn_exp2f(x) exp2f(x)

typedef float emu_floatx4 __attribute__((ext_vector_type(4)));
typedef float emu_floatx16 __attribute__((ext_vector_type(16)));
typedef int emu_intx8 __attribute__((ext_vector_type(8)));
typedef __bf16 emu_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 emu_bf16x2 __attribute__((ext_vector_type(2)));

static inline emu_floatx4 emu_mfma_16x16x128(emu_intx8 a, emu_intx8 b, emu_floatx4 c, int = 0, int = 0, int = 0, int = 0,
                                             int = 0, int = 0) {
  int32_t av[8], bv[8];
  float cv[4], dv[4];
  memcpy(av, &a, 32); memcpy(bv, &b, 32); memcpy(cv, &c, 16);
  emu::mfma_16x16x128_f8(av, bv, cv, dv);
  emu_floatx4 d;
  memcpy(&d, dv, 16);
  return d;
}
static inline emu_floatx16 emu_mfma_32x32x64(emu_intx8 a, emu_intx8 b, emu_floatx16 c, int = 0, int = 0, int = 0, int = 0,
                                             int = 0, int = 0) {
  int32_t av[8], bv[8];
  float cv[16], dv[16];
  memcpy(av, &a, 32); memcpy(bv, &b, 32); memcpy(cv, &c, 64);
  emu::mfma_32x32x64_f8(av, bv, cv, dv);
  emu_floatx16 d;
  memcpy(&d, dv, 64);
  return d;
}
static inline emu_floatx4 emu_mfma_bf16(emu_bf16x8 a, emu_bf16x8 b, emu_floatx4 c, int = 0, int = 0, int = 0) {
  uint16_t av[8], bv[8];
  float cv[4], dv[4];
  memcpy(av, &a, 16); memcpy(bv, &b, 16); memcpy(cv, &c, 16);
  emu::mfma_16x16x32_bf16(av, bv, cv, dv);
  emu_floatx4 d;
  memcpy(&d, dv, 16);
  return d;
}
// (the format and scale arguments of the f8f6f4 forms are 0 everywhere in this library: e4m3 x e4m3, unit scales)
// (variadic: an operand written as a braced vector literal holds commas)
#define __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(...) emu_mfma_16x16x128(__VA_ARGS__)
#define __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(...) emu_mfma_32x32x64(__VA_ARGS__)
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(...) emu_mfma_bf16(__VA_ARGS__)

// byte `sel` of w holds two e2m1 values (low nibble first); each times `scale` (a power of two) is exact in bf16
static inline emu_bf16x2 emu_cvt_fp4(uint32_t w, float scale, int sel) {
  static const float kE2M1[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
  const uint32_t byte = (w >> (8 * sel)) & 0xffu;
  emu_bf16x2 r;
  for (int i = 0; i < 2; ++i) {
    const uint32_t nib = (byte >> (4 * i)) & 0xfu;
    const float v = (nib & 8u ? -1.0f : 1.0f) * kE2M1[nib & 7u] * scale;
    r[i] = (__bf16)v;
  }
  return r;
}
#define __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, sel) emu_cvt_fp4((w), (scale), (sel))
static inline int emu_cvt_pk_fp8(float a, float b, int old, bool hi) {
  const uint32_t pair = (uint32_t)emu::f32_to_e4m3(a) | ((uint32_t)emu::f32_to_e4m3(b) << 8);
  const uint32_t o = (uint32_t)old;
  return (int)(hi ? ((o & 0x0000ffffu) | (pair << 16)) : ((o & 0xffff0000u) | pair));
}
#define __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, hi) emu_cvt_pk_fp8((a), (b), (old), (hi))
