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
int bgmoe_internal_dispatch_scatter_quant(const int32_t* ids, int n, int k, int h, int expert_start, int e_local, int mtp,
                                          int row_align, int32_t* counts, int32_t* counters, int32_t* cu, int32_t* pos,
                                          int extra_count, int64_t extra_start, const uint16_t* x, uint8_t* y,
                                          float* scale, int64_t srow, int64_t skb, hipStream_t st);
int bgmoe_internal_scatter_quant(const uint16_t* x, const int32_t* topk_pos, int n, int k, int h, uint8_t* y,
                                 float* scale, int64_t srow, int64_t skb, int extra_rows, int64_t extra_start,
                                 hipStream_t st);

int bgmoe_internal_scatter_fp8(const uint8_t* xq, const float* xs, int64_t xs_row, int64_t xs_kb,
                               const int32_t* topk_pos, int n, int k, int h, uint8_t* y, float* scale,
                               int64_t srow, int64_t skb, int extra_rows, int64_t extra_start, hipStream_t st);

// ---- optional per-launch timing (off by default; see bgmoe_prof_enable) -----------
enum BgmoeKernelId {
  BGMOE_K_ROUTER = 0, BGMOE_K_PERM_HIST, BGMOE_K_PERM_SCAN, BGMOE_K_PERM_RANK, BGMOE_K_GATHER_ROWS,
  BGMOE_K_ACT_QUANT, BGMOE_K_COMBINE, BGMOE_K_COMPACT,
  BGMOE_K_S1_SKINNY16, BGMOE_K_S1_SKINNY64, BGMOE_K_S1_TILED,
  BGMOE_K_GEMM_SKINNY16, BGMOE_K_GEMM_SKINNY64, BGMOE_K_GEMM_TILED,
  BGMOE_K_MXFP4_S1, BGMOE_K_MXFP4_GEMM, BGMOE_K_BF16_GEMM, BGMOE_K_ROUTER_GEMM, BGMOE_K_ROUTER_GEMM_REDUCE,
  BGMOE_K_NORM_QUANT, BGMOE_K_SITU, BGMOE_K_DENSE_GEMM,
  BGMOE_K_COUNT
};
extern bool g_bgmoe_prof_on;
void bgmoe_prof_mark(int id, hipStream_t st, bool begin);
struct BgmoeProf {
  int id; hipStream_t st;
  BgmoeProf(int id_, hipStream_t st_) : id(id_), st(st_) { if (g_bgmoe_prof_on) bgmoe_prof_mark(id, st, true); }
  ~BgmoeProf() { if (g_bgmoe_prof_on) bgmoe_prof_mark(id, st, false); }
};

// fused stage 1 when w1 != nullptr; row_bound = host-side upper bound on live rows (0 = m)
int bgmoe_internal_init_fp8_skinny();
int bgmoe_internal_init_fp8_tiled();
int bgmoe_internal_init_mxfp4();
int bgmoe_internal_init_router_gemm();
int bgmoe_internal_init_permute();
int bgmoe_internal_fp8_gemm(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* w0, const bgmoe_fp8_weight* w1,
                            const int32_t* seqlens, const int32_t* cu, int groups, int64_t m, int n, int k,
                            uint16_t* out, uint8_t* out_q, float* out_s, int64_t os_row, int64_t os_nb,
                            int64_t row_bound, int64_t group_bound, void* streamk_ws, size_t streamk_ws_bytes,
                            hipStream_t st);
int bgmoe_internal_init_fp8_streamk();
// balanced (stream-K) form of the weight-streaming kernel; BGMOE_ERR_WORKSPACE without a message = does not apply
int bgmoe_internal_fp8_streamk(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* w0, const bgmoe_fp8_weight* w1,
                               const int32_t* seqlens, const int32_t* cu, int groups, int n, int k, uint16_t* out,
                               uint8_t* out_q, float* out_s, int64_t os_row, int64_t os_nb, int hi, int64_t row_bound,
                               void* ws, size_t ws_bytes, hipStream_t st);

// router-GEMM logits as [*nplanes_out][n][e] fp32 planes for a consumer that adds them in plane order
int bgmoe_internal_router_gemm_planes(const uint16_t* hidden, const uint16_t* weight, int n, int h, int e,
                                      float* planes, size_t planes_bytes, int* nplanes_out, hipStream_t st);

static inline hipStream_t bgmoe_stream(bgmoe_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// ---- bf16 <-> fp32 -----------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// round-to-nearest-even with the hardware convert (v_cvt_pk_bf16_f32: two values per instruction); NaN stays
// a quiet NaN
typedef __bf16 bgmoe_bf16x2 __attribute__((ext_vector_type(2)));
typedef float bgmoe_floatx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
  const bgmoe_floatx2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bgmoe_bf16x2));
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return pack2_bf16(f, 0.0f) & 0xffffu; }

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

// x / s for many x and one s, bit for bit the IEEE quotient at a third of its instructions: with r = RN(1/s),
// q0 = RN(x*r) is within one ulp of x/s, e = x - q0*s is exact in an fma, and RN(q0 + e*r) is the correctly
// rounded quotient (Markstein's division step).  Valid while nothing over- or underflows: callers use it for
// s in (1e-30, 1e30) and |x/s| of order 448 at most (s comes from the block's amax), and take the IEEE
// division otherwise.  An exact quotient (e == 0, which includes x = +-0) is returned as it is, so a zero keeps
// its sign; quotients below 2^-126 may differ from the IEEE denormal in the last place and round to the same
// signed zero in e4m3.  bgmoe_selfcheck_scale_division compares the two on the device.
__device__ __forceinline__ bool scale_div_ok(float s) { return s > 1e-30f && s < 1e30f; }
__device__ __forceinline__ float div_by_scale(float x, float s, float r) {
  const float q0 = x * r;
  const float e = __builtin_fmaf(-q0, s, x);
  return e == 0.0f ? q0 : __builtin_fmaf(e, r, q0);
}
// q[i] = clamp(x[i] / s, +-448) for the N values of a lane that share the scale s
template <int N>
__device__ __forceinline__ void quant_div_clamp(const float (&x)[N], float s, float (&q)[N]) {
  if (scale_div_ok(s)) {
    const float r = 1.0f / s;
#pragma unroll
    for (int i = 0; i < N; ++i) q[i] = fmaxf(fminf(div_by_scale(x[i], s, r), 448.0f), -448.0f);
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) q[i] = fmaxf(fminf(x[i] / s, 448.0f), -448.0f);
  }
}

// scale of one 128-block from its amax: fmaxf(amax, 1e-12f) * (1.0f / 448.0f)
__device__ __forceinline__ float quant_scale_from_amax(float amax) {
  constexpr float kInv448 = 1.0f / 448.0f;
  return fmaxf(amax, 1e-12f) * kInv448;
}

// ---- explicit global-address-space loads --------------------------------------------
// A pointer that was itself loaded from memory (a per-group pointer table) is a generic ("flat")
// pointer to the compiler; flat loads count against both memory counters and force full waits.
// These helpers assert the global address space so that the loads are global_load_* and
// s_waitcnt vmcnt(N) can leave younger loads in flight.
#define BGMOE_GLOBAL __attribute__((address_space(1)))
__device__ __forceinline__ intx4 gload_x4(const void* p) {
  return *reinterpret_cast<const BGMOE_GLOBAL intx4*>((uintptr_t)p);
}
__device__ __forceinline__ intx4 gload_x4_stream(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const BGMOE_GLOBAL intx4*>((uintptr_t)p));
}
__device__ __forceinline__ float gload_f32(const float* p) {
  return *reinterpret_cast<const BGMOE_GLOBAL float*>((uintptr_t)p);
}
__device__ __forceinline__ uint32_t gload_u32(const void* p) {
  return *reinterpret_cast<const BGMOE_GLOBAL uint32_t*>((uintptr_t)p);
}
// The same for stores: a store through a generic pointer is a flat store, and while one is pending the compiler
// turns every wait for a load into a full wait (flat operations may complete out of order), which drains a
// software pipeline that runs into the next work item's loads.
typedef unsigned int bgmoe_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void gstore_x2(void* p, uint2 v) {
  *reinterpret_cast<BGMOE_GLOBAL bgmoe_u32x2*>((uintptr_t)p) = bgmoe_u32x2{v.x, v.y};
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
// same with the hardware reciprocal (1 ulp) instead of the correctly rounded division: for GEMM epilogues that
// evaluate it 64 times per lane, where the accumulation order already moves the last bits
__device__ __forceinline__ float silu_rcp_f32(float g) { return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)); }

// exp(t) for |t| <= 100, correctly rounded to fp32 but for about one input in 2^23: 2^k * P(r) in fp64 with the
// degree-11 Taylor polynomial on |r| <= ln2/2 (truncation 2^-47), rounded once.
__device__ __forceinline__ float exp_cr_f32(float t32) {
  const double t = (double)t32;
  const double k = __builtin_rint(t * 1.4426950408889634074);
  double r = __builtin_fma(-k, 6.93147180369123816490e-01, t);
  r = __builtin_fma(-k, 1.90821492927058770002e-10, r);
  double p = 1.0 / 39916800.0;
  p = __builtin_fma(p, r, 1.0 / 3628800.0);
  p = __builtin_fma(p, r, 1.0 / 362880.0);
  p = __builtin_fma(p, r, 1.0 / 40320.0);
  p = __builtin_fma(p, r, 1.0 / 5040.0);
  p = __builtin_fma(p, r, 1.0 / 720.0);
  p = __builtin_fma(p, r, 1.0 / 120.0);
  p = __builtin_fma(p, r, 1.0 / 24.0);
  p = __builtin_fma(p, r, 1.0 / 6.0);
  p = __builtin_fma(p, r, 0.5);
  p = __builtin_fma(p, r, 1.0);
  p = __builtin_fma(p, r, 1.0);
  return (float)__builtin_ldexp(p, (int)k);
}
// PyTorch's fp32 SiLU: x / (1 + exp(-x)) as three fp32 operations (exp, add, IEEE division).  Beyond |x| = 100
// exp(-x) is 0 or overflows to +inf in fp32 either way.
__device__ __forceinline__ float silu_exact_f32(float g) {
  const float e = g > 100.0f ? 0.0f : (g < -100.0f ? __builtin_huge_valf() : exp_cr_f32(-g));
  return g / (1.0f + e);
}

// bf16(silu_exact_f32(g)) at a third of the cost on almost every input.  The short evaluation (hardware exp2
// with the argument's rounding error carried separately, hardware reciprocal) stays within 4 fp32 ulps of the
// true SiLU and silu_exact_f32 within 2; if the short result lies more than 16 ulps from the nearest bf16
// rounding boundary both round to the same bf16.  `decided` = false asks the caller for the exact
// evaluation (about 1 input in 2000, and every |g| > 80 or non-finite g).  Returns the fp32 value to round.
__device__ __forceinline__ float silu_short_f32(float g, bool* decided) {
  const float x = -g;
  const float t_hi = x * 1.44269502162933349609375f;                         // log2(e) rounded to fp32
  const float t_lo = __builtin_fmaf(x, 1.44269502162933349609375f, -t_hi) + x * 1.925963033500011e-08f;
  const float e = __builtin_amdgcn_exp2f(t_hi) * __builtin_fmaf(t_lo, 0.693147182464599609375f, 1.0f);
  const float s = g * __builtin_amdgcn_rcpf(1.0f + e);
  const uint32_t low = __float_as_uint(s) & 0xffffu;
  *decided = fabsf(g) <= 80.0f && (low < 0x8000u - 16u || low > 0x8000u + 16u);
  return s;
}

// SiTU-and-multiply (Kimi-K3): beta * tanh(g / beta) * sigmoid(g), times u or, with a linear beta,
// lbeta * tanh(u / lbeta).  fp32 throughout, the library tanhf / expf and an IEEE division; the divisions by
// beta are multiplications by the rounded reciprocal, as in the reference kernels
// (batchgen_kernels/src/moe/marlin_grouped_gemm.cu:243-256, kimi_linear/situ_triton.py:41-45).
__device__ __forceinline__ float situ_gate_f32(float g, float beta, float inv_beta) {
  return beta * tanhf(g * inv_beta) * (1.0f / (1.0f + expf(-g)));
}
__device__ __forceinline__ float situ_linear_f32(float u, float lbeta, float inv_lbeta) {
  return lbeta * tanhf(u * inv_lbeta);
}
