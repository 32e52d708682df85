// Shared device helpers for the gfx950 MoE kernels (wave64, OCP fp8).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/bgmoe.h"

#define BGMOE_WAVE 64

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef int intx8 __attribute__((ext_vector_type(8)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef short shortx8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// ---- error plumbing (host) ---------------------------------------------------
void bgmoe_set_error(const char* fmt, ...);
int bgmoe_check_launch(const char* what);

#define BGMOE_REQUIRE(cond, ...)            \
  do {                                      \
    if (!(cond)) {                          \
      bgmoe_set_error(__VA_ARGS__);         \
      return BGMOE_ERR_ARG;                 \
    }                                       \
  } while (0)

// ---- internal entry points shared between translation units ----------------------
int bgmoe_internal_dispatch_index(const int32_t* ids, int64_t nk, int expert_start, int e_local, int mtp,
                                  int row_align, int32_t* counts, int32_t* counters, int32_t* cu,
                                  int32_t* pos, int extra_count, int64_t extra_start, void* ws,
                                  size_t ws_bytes, hipStream_t st);
int bgmoe_internal_scatter_quant(const uint16_t* x, const int32_t* topk_pos, int n, int k, int h, uint8_t* y,
                                 float* scale, int64_t srow, int64_t skb, int extra_rows, int64_t extra_start,
                                 hipStream_t st);

// ---- optional per-launch timing (off by default; see bgmoe_prof_enable) -----------
enum BgmoeKernelId {
  BGMOE_K_ROUTER = 0, BGMOE_K_PERM_HIST, BGMOE_K_PERM_SCAN, BGMOE_K_PERM_RANK, BGMOE_K_GATHER_ROWS,
  BGMOE_K_ACT_QUANT, BGMOE_K_COMBINE, BGMOE_K_COMPACT,
  BGMOE_K_S1_SKINNY16, BGMOE_K_S1_SKINNY64, BGMOE_K_S1_TILED,
  BGMOE_K_GEMM_SKINNY16, BGMOE_K_GEMM_SKINNY64, BGMOE_K_GEMM_TILED,
  BGMOE_K_MXFP4_S1, BGMOE_K_MXFP4_GEMM, BGMOE_K_BF16_GEMM,
  BGMOE_K_COUNT
};
extern bool g_bgmoe_prof_on;
void bgmoe_prof_mark(int id, hipStream_t st, bool begin);
struct BgmoeProf {
  int id; hipStream_t st;
  BgmoeProf(int id_, hipStream_t st_) : id(id_), st(st_) { if (g_bgmoe_prof_on) bgmoe_prof_mark(id, st, true); }
  ~BgmoeProf() { if (g_bgmoe_prof_on) bgmoe_prof_mark(id, st, false); }
};

static inline hipStream_t bgmoe_stream(bgmoe_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// ---- bf16 <-> fp32 -----------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// round-to-nearest-even; NaN stays NaN (quiet)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

__device__ __forceinline__ float bf16_round_f32(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

// ---- fp8 e4m3fn (OCP on gfx950), RNE; inputs already clamped to +-448 ---------
__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d) {
  int v = 0;
  v = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, v, false);
  v = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, v, true);
  return (uint32_t)v;
}

// clamp as fmaxf(fminf(q, 448), -448): a NaN q becomes +448, as in the reference quantiser
__device__ __forceinline__ float clamp448(float q) { return fmaxf(fminf(q, 448.0f), -448.0f); }

// scale of one 128-block from its amax: fmaxf(amax, 1e-12f) * (1.0f / 448.0f)
__device__ __forceinline__ float quant_scale_from_amax(float amax) {
  constexpr float kInv448 = 1.0f / 448.0f;
  return fmaxf(amax, 1e-12f) * kInv448;
}

// ---- wave helpers ---------------------------------------------------------------
__device__ __forceinline__ int lane_id() { return threadIdx.x & (BGMOE_WAVE - 1); }

template <int WIDTH>
__device__ __forceinline__ float wave_max_xor(float v) {
#pragma unroll
  for (int off = WIDTH / 2; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, BGMOE_WAVE));
  return v;
}

__device__ __forceinline__ float silu_f32(float g) { return g / (1.0f + __expf(-g)); }
