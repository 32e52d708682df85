// Sigmoid + bias-corrected top-k routers for gfx950: ONE wave64 per token.
// A token's experts live in registers (expert id = i*64 + lane, VPL values per
// lane); every arg-max round is a lane-local scan plus a 6-step DPP reduction
// with the rule "larger value wins, equal values go to the lower expert id",
// which gives a unique winner whatever the reduction tree.
#include <math.h>

#include "bgmoe_common.h"

namespace {

constexpr float kNegInf = -__builtin_huge_valf();

// correctly rounded fp32 sigmoid: evaluate in fp64, round once
__device__ __forceinline__ float sigmoid_precise(float x) {
  return (float)(1.0 / (1.0 + exp(-(double)x)));
}

// The same value, 3x cheaper on the usual inputs.  A short fp64 evaluation -- exp(-x) = 2^k * P(r) with the
// degree-11 Taylor polynomial on |r| <= ln2/2 (truncation 2^-47), 1/(1+e) by the hardware reciprocal and two
// Newton steps -- gives y within 2^-46 of the true sigmoid.  If y(1 - 2^-43) and y(1 + 2^-43) round to the
// same float, that float is the correctly rounded result (rounding is monotonic and the true value, like the
// library evaluation above, lies between the two); otherwise, about once in 10^4 inputs, and for |x| > 80
// (results near the denormal range) or NaN, the library evaluation decides.  bgmoe_selfcheck_sigmoid
// compares the two paths bit for bit over any range of float bit patterns.
__device__ __forceinline__ bool sigmoid_short(float x, float* out) {
  if (!(fabsf(x) <= 80.0f)) return false;
  const double t = -(double)x;
  const double k = __builtin_rint(t * 1.4426950408889634074);
  double r = __builtin_fma(-k, 6.93147180369123816490e-01, t);      // ln2 split so that k*hi is exact
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
  const double d = 1.0 + __builtin_ldexp(p, (int)k);
  double y = __builtin_amdgcn_rcp(d);
  y = __builtin_fma(y, __builtin_fma(-d, y, 1.0), y);
  y = __builtin_fma(y, __builtin_fma(-d, y, 1.0), y);
  const float lo = (float)(y * (1.0 - 0x1p-43)), hi = (float)(y * (1.0 + 0x1p-43));
  *out = lo;
  return lo == hi;
}
__device__ __forceinline__ float sigmoid_cr(float x) {
  float v;
  return sigmoid_short(x, &v) ? v : sigmoid_precise(x);
}

// Data-parallel-primitive lane exchanges inside a row of 16 lanes (a VALU modifier, no LDS round trip):
// quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror.  Applied in this order with an
// order-independent merge, all 16 lanes of a row end up with the row's result.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140;
constexpr int kDppBcast15 = 0x142, kDppBcast31 = 0x143;

// branch-free on purpose: three compares, two mask operations, two selects (a short-circuit `if` turns into
// exec-mask juggling that costs more than the reduction itself)
__device__ __forceinline__ void argmax_merge(float& v, int& idx, float ov, int oi) {
  const bool gt = ov > v;
  const bool eq = ov == v;
  const bool lower = oi < idx;
  const bool take = gt | (eq & lower);
  v = take ? ov : v;
  idx = take ? oi : idx;
}

// "larger value wins, equal values go to the lower index": a total order, so any reduction network gives
// the same winner.  Rows of 16 lanes reduce with DPP butterflies (every lane of a row then holds the row's
// result); row_bcast15 folds rows 0/2 into rows 1/3, row_bcast31 folds row 1 into row 3, and lane 63 holds
// the wave's winner.  Rows left out by a row mask receive their own value, for which the merge is a no-op.
template <int CTRL, int ROWS>
__device__ __forceinline__ int dpp_rows_i32(int v) {
  return __builtin_amdgcn_update_dpp(v, v, CTRL, ROWS, 0xf, false);
}
__device__ __forceinline__ void wave_argmax(float& v, int& idx) {
  argmax_merge(v, idx, dpp_f32<kDppXor1>(v), dpp_i32<kDppXor1>(idx));
  argmax_merge(v, idx, dpp_f32<kDppXor2>(v), dpp_i32<kDppXor2>(idx));
  argmax_merge(v, idx, dpp_f32<kDppHalfMirror>(v), dpp_i32<kDppHalfMirror>(idx));
  argmax_merge(v, idx, dpp_f32<kDppMirror>(v), dpp_i32<kDppMirror>(idx));
  argmax_merge(v, idx, __int_as_float(dpp_rows_i32<kDppBcast15, 0xa>(__float_as_int(v))),
               dpp_rows_i32<kDppBcast15, 0xa>(idx));
  argmax_merge(v, idx, __int_as_float(dpp_rows_i32<kDppBcast31, 0xc>(__float_as_int(v))),
               dpp_rows_i32<kDppBcast31, 0xc>(idx));
  v = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
  idx = __builtin_amdgcn_readlane(idx, 63);
}

// two largest values (with multiplicity) of the union of two (m1 >= m2) pairs
__device__ __forceinline__ void top2_merge(float& m1, float& m2, float o1, float o2) {
  const float lo = fminf(m1, o1);
  m1 = fmaxf(m1, o1);
  m2 = fmaxf(lo, fmaxf(m2, o2));
}

struct RouterArgs {
  const float* in;        // scores or logits, row stride `stride`
  int64_t stride;
  int nsplit;             // > 0: `in` holds nsplit partial planes, plane_stride apart; the logit is their
  int64_t plane_stride;   //      sum in plane order starting from 0.0f (the router GEMM's split-K output)
  const float* bias;
  int n, e, top_k;
  float rsf;
  int apply_sigmoid;
  // grouped
  int n_group, topk_group;
  // outputs
  int32_t* ids32;
  int64_t* ids64;
  float* w;
  // padding
  const int32_t* num_valid;
  const int64_t* rank_counts;
  int rows_per_rank;
  // latent epilogue
  uint16_t* latent_out;
  int latent_offset, latent_size;
};

// GROUPED: moe_fused_gate semantics (floor -1e9, w = raw * (rsf / (sum + 1e-20)))
// else    : gate_sigmoid_topk semantics (floor -FLT_MAX, w = raw * (1/(sum+1e-20)) * rsf)
template <int VPL, bool GROUPED>
__global__ __launch_bounds__(256) void router_kernel(RouterArgs a) {
  extern __shared__ float s_lds[];   // GROUPED: [4][e] biased scores
  const int wave = threadIdx.x >> 6;
  const int lane = lane_id();
  const int token = blockIdx.x * 4 + wave;
  if (token >= a.n) return;          // whole wave; no block-level barrier is used below

  if constexpr (!GROUPED) {
    bool pad = false;
    if (a.num_valid) {
      pad = token >= *a.num_valid;
    } else if (a.rank_counts) {
      const int r = token / a.rows_per_rank;
      pad = (int64_t)(token - r * a.rows_per_rank) >= a.rank_counts[r];
    }
    if (pad) {
      if (lane < a.top_k) {
        if (a.ids64) a.ids64[(int64_t)token * a.top_k + lane] = -1;
        else a.ids32[(int64_t)token * a.top_k + lane] = -1;
        a.w[(int64_t)token * a.top_k + lane] = 0.0f;
      }
      if (a.latent_out)
        for (int i = lane; i < a.latent_size; i += BGMOE_WAVE)
          a.latent_out[(int64_t)token * a.latent_size + i] = 0;
      return;
    }
  }

  const float* row = a.in + (int64_t)token * a.stride;
  float raw[VPL], key[VPL];
  const float floor_v = GROUPED ? -1e9f : -3.402823466e+38f;
  float xin[VPL];
  if (a.nsplit > 0) {
    // split-K planes: logit = (((0 + p_0) + p_1) + ...); the VPL loads of a plane are in flight together
#pragma unroll
    for (int i = 0; i < VPL; ++i) xin[i] = 0.0f;
    constexpr int kBatch = VPL <= 4 ? 4 : 2;   // planes requested together
    for (int sp = 0; sp < a.nsplit; sp += kBatch) {
      float part[kBatch][VPL];
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        const float* prow = row + min(sp + b, a.nsplit - 1) * a.plane_stride;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
          const int ex = i * BGMOE_WAVE + lane;
          part[b][i] = ex < a.e ? prow[ex] : 0.0f;
        }
      }
#pragma unroll
      for (int b = 0; b < kBatch; ++b)
        if (sp + b < a.nsplit) {
#pragma unroll
          for (int i = 0; i < VPL; ++i) xin[i] += part[b][i];
        }
    }
  } else {
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int ex = i * BGMOE_WAVE + lane;
      xin[i] = ex < a.e ? row[ex] : 0.0f;
    }
  }
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int ex = i * BGMOE_WAVE + lane;
    if (ex < a.e) {
      raw[i] = a.apply_sigmoid ? sigmoid_cr(xin[i]) : xin[i];
      const float s = raw[i] + a.bias[ex];
      key[i] = s > floor_v ? s : kNegInf;     // NaN and <= floor are never candidates
    } else {
      raw[i] = 0.0f;
      key[i] = kNegInf;
    }
  }

  if constexpr (!GROUPED) {
    if (a.latent_out) {
      const float* lat = row + a.latent_offset;
      for (int i = lane; i < a.latent_size; i += BGMOE_WAVE)
        a.latent_out[(int64_t)token * a.latent_size + i] = (uint16_t)f32_to_bf16_bits(lat[i]);
    }
  }

  if constexpr (GROUPED) {
    // group score = sum of the group's two largest biased scores (strict '>' scan from -1e9, i.e. the two
    // largest values with multiplicity, -1e9 standing in for missing ones)
    const int epg = a.e / a.n_group;
    float gscore = kNegInf;
    if ((epg & (epg - 1)) == 0 && epg <= BGMOE_WAVE) {
      // a group is an aligned run of epg lanes of one register slot: top-2 butterfly in registers
      float gs[VPL];
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        float m1 = key[i] == kNegInf ? -1e9f : key[i], m2 = -1e9f;
        if (epg >= 2) top2_merge(m1, m2, dpp_f32<kDppXor1>(m1), dpp_f32<kDppXor1>(m2));
        if (epg >= 4) top2_merge(m1, m2, dpp_f32<kDppXor2>(m1), dpp_f32<kDppXor2>(m2));
        if (epg >= 8) top2_merge(m1, m2, dpp_f32<kDppHalfMirror>(m1), dpp_f32<kDppHalfMirror>(m2));
        if (epg >= 16) top2_merge(m1, m2, dpp_f32<kDppMirror>(m1), dpp_f32<kDppMirror>(m2));
        if (epg >= 32) top2_merge(m1, m2, __shfl_xor(m1, 16, BGMOE_WAVE), __shfl_xor(m2, 16, BGMOE_WAVE));
        if (epg >= 64) top2_merge(m1, m2, __shfl_xor(m1, 32, BGMOE_WAVE), __shfl_xor(m2, 32, BGMOE_WAVE));
        gs[i] = m1 + m2;
      }
      // lane g < n_group collects group g's score from its first expert g*epg = slot (g*epg)/64, lane (g*epg)%64
      const int ex0 = lane < a.n_group ? lane * epg : 0;
      float g = -1e9f;
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const float t = __shfl(gs[i], ex0 & (BGMOE_WAVE - 1), BGMOE_WAVE);
        if ((ex0 >> 6) == i) g = t;
      }
      if (lane < a.n_group) gscore = g > -1e9f ? g : kNegInf;
    } else if (epg % BGMOE_WAVE == 0) {
      // a group is a run of epg/64 whole register slots: per-lane top-2 over the run, then a wave butterfly
      const int spg = epg >> 6;
      float m1 = -1e9f, m2 = -1e9f;
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        if (i * BGMOE_WAVE < a.e) {
          top2_merge(m1, m2, key[i] == kNegInf ? -1e9f : key[i], -1e9f);
          if ((i + 1) % spg == 0) {
            top2_merge(m1, m2, dpp_f32<kDppXor1>(m1), dpp_f32<kDppXor1>(m2));
            top2_merge(m1, m2, dpp_f32<kDppXor2>(m1), dpp_f32<kDppXor2>(m2));
            top2_merge(m1, m2, dpp_f32<kDppHalfMirror>(m1), dpp_f32<kDppHalfMirror>(m2));
            top2_merge(m1, m2, dpp_f32<kDppMirror>(m1), dpp_f32<kDppMirror>(m2));
            top2_merge(m1, m2, __shfl_xor(m1, 16, BGMOE_WAVE), __shfl_xor(m2, 16, BGMOE_WAVE));
            top2_merge(m1, m2, __shfl_xor(m1, 32, BGMOE_WAVE), __shfl_xor(m2, 32, BGMOE_WAVE));
            const float g = m1 + m2;
            if (lane == i / spg) gscore = g > -1e9f ? g : kNegInf;
            m1 = m2 = -1e9f;
          }
        }
      }
    } else {
      float* s = s_lds + wave * a.e;
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int ex = i * BGMOE_WAVE + lane;
        if (ex < a.e) s[ex] = key[i] == kNegInf ? -1e9f : key[i];
      }
      // the slice is private to this wave: order its LDS writes before the reads below
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      if (lane < a.n_group) {
        float m1 = -1e9f, m2 = -1e9f;
        for (int i = 0; i < epg; ++i) {
          const float v = s[lane * epg + i];
          if (v > m1) { m2 = m1; m1 = v; }
          else if (v > m2) { m2 = v; }
        }
        const float g = m1 + m2;
        gscore = g > -1e9f ? g : kNegInf;
      }
    }
    unsigned long long gmask = 0ull;
    for (int r = 0; r < a.topk_group; ++r) {
      float v = gscore;
      int idx = v == kNegInf ? 0x7fffffff : lane;
      wave_argmax(v, idx);
      if (v != kNegInf) {
        gmask |= 1ull << idx;
        if (lane == idx) gscore = kNegInf;
      }
    }
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int ex = i * BGMOE_WAVE + lane;
      const int g = ex < a.e ? ex / epg : 0;
      if (!((gmask >> g) & 1ull)) key[i] = kNegInf;
    }
  }

  float total = 0.0f;
  int my_id = -1;
  float my_raw = 0.0f;
  for (int r = 0; r < a.top_k; ++r) {
    float v = kNegInf;
    int idx = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      if (key[i] > v) {                       // ascending ids per lane: strict '>' keeps the lowest
        v = key[i];
        idx = i * BGMOE_WAVE + lane;
      }
    }
    wave_argmax(v, idx);
    float rv = 0.0f;
    int id = -1;
    if (v != kNegInf) {
      id = idx;
      const int owner = idx & (BGMOE_WAVE - 1);
      const int slot = idx >> 6;
      float mine = 0.0f;
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        if (i == slot) {
          mine = raw[i];
          if (lane == owner) key[i] = kNegInf;
        }
      }
      rv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mine), owner));   // owner is wave-uniform
    }
    total = total + rv;                        // route order, from 0.0f
    if (lane == r) {
      my_id = id;
      my_raw = rv;
    }
  }

  if (lane < a.top_k) {
    float wv;
    if constexpr (GROUPED) {
      const float scale = a.rsf / (total + 1e-20f);
      wv = my_raw * scale;
    } else {
      const float inv = 1.0f / (total + 1e-20f);
      wv = my_raw * inv;
      wv = wv * a.rsf;
    }
    const int64_t o = (int64_t)token * a.top_k + lane;
    if (a.ids64) a.ids64[o] = my_id;
    else a.ids32[o] = my_id;
    a.w[o] = wv;
  }
}

template <bool GROUPED>
int launch_router(const RouterArgs& a, hipStream_t st) {
  if (a.n == 0) return BGMOE_OK;
  const dim3 grid((a.n + 3) / 4), block(256);
  const size_t lds = GROUPED ? (size_t)4 * a.e * sizeof(float) : 0;
  const int vpl = (a.e + 63) / 64;
  BgmoeProf prof(BGMOE_K_ROUTER, st);
#define BGMOE_ROUTER_CASE(V)                                                              \
  hipLaunchKernelGGL((router_kernel<V, GROUPED>), grid, block, lds, st, a)
  if (vpl <= 1) BGMOE_ROUTER_CASE(1);
  else if (vpl <= 2) BGMOE_ROUTER_CASE(2);
  else if (vpl <= 4) BGMOE_ROUTER_CASE(4);
  else if (vpl <= 8) BGMOE_ROUTER_CASE(8);
  else BGMOE_ROUTER_CASE(16);
#undef BGMOE_ROUTER_CASE
  return bgmoe_check_launch("router");
}

int check_fused_gate(int n, int e, int n_group, int topk_group, int top_k) {
  BGMOE_REQUIRE(n >= 0, "fused_gate: n < 0");
  BGMOE_REQUIRE(e >= 1 && e <= 1024, "fused_gate: n_routed_experts=%d outside [1,1024]", e);
  BGMOE_REQUIRE(n_group >= 1 && n_group <= 64, "fused_gate: n_group=%d outside [1,64]", n_group);
  BGMOE_REQUIRE(e % n_group == 0, "fused_gate: n_routed_experts (%d) must be divisible by n_group (%d)",
                e, n_group);
  BGMOE_REQUIRE(topk_group >= 1 && topk_group <= n_group, "fused_gate: topk_group=%d outside [1,%d]",
                topk_group, n_group);
  BGMOE_REQUIRE(top_k >= 1 && top_k <= 32 && top_k <= e, "fused_gate: unsupported top_k=%d", top_k);
  return BGMOE_OK;
}

int check_gate_sigmoid_topk(int n, int e, int k, const int32_t* num_valid_tokens,
                            const int64_t* rank_token_counts, int rows_per_rank) {
  BGMOE_REQUIRE(n >= 0, "gate_sigmoid_topk: n < 0");
  BGMOE_REQUIRE(e >= 1 && e <= 1024, "gate_sigmoid_topk: E=%d exceeds MAX_EXPERTS=1024", e);
  BGMOE_REQUIRE(k == 2 || k == 4 || k == 8 || k == 16, "gate_sigmoid_topk: Unsupported k=%d. Supported: 2, 4, 8, 16", k);
  BGMOE_REQUIRE(e >= k, "gate_sigmoid_topk: E=%d must be at least k=%d", e, k);
  BGMOE_REQUIRE(!(num_valid_tokens && rank_token_counts),
                "gate_sigmoid_topk: num_valid_tokens and rank_token_counts are mutually exclusive");
  BGMOE_REQUIRE(!rank_token_counts || rows_per_rank > 0, "gate_sigmoid_topk: rows_per_rank must be positive");
  return BGMOE_OK;
}

}  // namespace

extern "C" int bgmoe_fused_gate(const float* scores, const float* bias, int n, int e, int n_group,
                                int topk_group, int top_k, float routed_scaling_factor,
                                int apply_sigmoid, int32_t* topk_ids, float* topk_weights,
                                bgmoe_stream_t stream) {
  if (int rc = check_fused_gate(n, e, n_group, topk_group, top_k)) return rc;
  if (n == 0) return BGMOE_OK;
  BGMOE_REQUIRE(scores && bias && topk_ids && topk_weights, "fused_gate: null pointer");
  RouterArgs a{};
  a.in = scores; a.stride = e; a.bias = bias; a.n = n; a.e = e; a.top_k = top_k;
  a.rsf = routed_scaling_factor; a.apply_sigmoid = apply_sigmoid;
  a.n_group = n_group; a.topk_group = topk_group; a.ids32 = topk_ids; a.w = topk_weights;
  return launch_router<true>(a, bgmoe_stream(stream));
}

extern "C" int bgmoe_gate_sigmoid_topk(const float* logits, int64_t logits_stride, const float* bias,
                                       int n, int e, int k, float routed_scaling_factor,
                                       void* topk_ids, int ids_are_int64, float* topk_weights,
                                       const int32_t* num_valid_tokens,
                                       const int64_t* rank_token_counts, int rows_per_rank,
                                       uint16_t* latent_out, int latent_offset, int latent_size,
                                       bgmoe_stream_t stream) {
  if (int rc = check_gate_sigmoid_topk(n, e, k, num_valid_tokens, rank_token_counts, rows_per_rank)) return rc;
  BGMOE_REQUIRE(logits_stride >= e, "gate_sigmoid_topk: row stride %lld < E=%d", (long long)logits_stride, e);
  if (latent_out) {
    BGMOE_REQUIRE(latent_offset >= e, "gate_sigmoid_topk: latent_offset=%d must start at or after the %d router columns", latent_offset, e);
    BGMOE_REQUIRE((int64_t)latent_offset + latent_size <= logits_stride,
                  "gate_sigmoid_topk: latent columns exceed the row stride");
  }
  if (n == 0) return BGMOE_OK;
  BGMOE_REQUIRE(logits && bias && topk_ids && topk_weights, "gate_sigmoid_topk: null pointer");
  RouterArgs a{};
  a.in = logits; a.stride = logits_stride; a.bias = bias; a.n = n; a.e = e; a.top_k = k;
  a.rsf = routed_scaling_factor; a.apply_sigmoid = 1;
  if (ids_are_int64) a.ids64 = (int64_t*)topk_ids; else a.ids32 = (int32_t*)topk_ids;
  a.w = topk_weights; a.num_valid = num_valid_tokens; a.rank_counts = rank_token_counts;
  a.rows_per_rank = rows_per_rank; a.latent_out = latent_out; a.latent_offset = latent_offset;
  a.latent_size = latent_size;
  return launch_router<false>(a, bgmoe_stream(stream));
}

// hidden -> logits -> routes without the logits round trip: the GEMM leaves its split-K planes in the
// workspace and the router kernel adds them, in plane order, while it loads a token's row.
extern "C" int bgmoe_router_gemm_gate(const uint16_t* hidden, const uint16_t* weight, const float* bias,
                                      int n, int h, int e, int n_group, int topk_group, int top_k,
                                      float routed_scaling_factor, int32_t* topk_ids, float* topk_weights,
                                      const int64_t* rank_token_counts, int rows_per_rank, void* workspace,
                                      size_t workspace_bytes, bgmoe_stream_t stream) {
  const bool grouped = n_group > 0;
  if (grouped) {
    if (int rc = check_fused_gate(n, e, n_group, topk_group, top_k)) return rc;
    BGMOE_REQUIRE(!rank_token_counts, "router_gemm_gate: the grouped router has no padding rows");
  } else {
    if (int rc = check_gate_sigmoid_topk(n, e, top_k, nullptr, rank_token_counts, rows_per_rank)) return rc;
  }
  if (n == 0) return BGMOE_OK;
  BGMOE_REQUIRE(hidden && weight && bias && topk_ids && topk_weights, "router_gemm_gate: null pointer");
  hipStream_t st = bgmoe_stream(stream);
  int nseg = 0;
  if (int rc = bgmoe_internal_router_gemm_planes(hidden, weight, n, h, e, static_cast<float*>(workspace),
                                                 workspace_bytes, &nseg, st))
    return rc;
  RouterArgs a{};
  a.in = static_cast<const float*>(workspace); a.stride = e; a.nsplit = nseg; a.plane_stride = (int64_t)n * e;
  a.bias = bias; a.n = n; a.e = e; a.top_k = top_k; a.rsf = routed_scaling_factor; a.apply_sigmoid = 1;
  a.ids32 = topk_ids; a.w = topk_weights;
  if (grouped) {
    a.n_group = n_group; a.topk_group = topk_group;
    return launch_router<true>(a, st);
  }
  a.rank_counts = rank_token_counts; a.rows_per_rank = rows_per_rank;
  return launch_router<false>(a, st);
}

namespace {
__global__ __launch_bounds__(256) void sigmoid_selfcheck_kernel(uint32_t first_bits, uint64_t count,
                                                                unsigned long long* mismatches,
                                                                unsigned long long* fallbacks) {
  unsigned long long bad = 0, slow = 0;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (uint64_t)gridDim.x * blockDim.x) {
    const float x = __uint_as_float(first_bits + (uint32_t)i);
    const float a = sigmoid_cr(x), b = sigmoid_precise(x);
    bad += __float_as_uint(a) != __float_as_uint(b) && !(a != a && b != b);
    float v;
    slow += fabsf(x) <= 80.0f && !sigmoid_short(x, &v);   // inputs in range that the short evaluation hands on
  }
  for (int off = 32; off > 0; off >>= 1) {
    bad += __shfl_xor(bad, off, BGMOE_WAVE);
    slow += __shfl_xor(slow, off, BGMOE_WAVE);
  }
  if (lane_id() == 0) {
    if (bad) atomicAdd(mismatches, bad);
    if (slow && fallbacks) atomicAdd(fallbacks, slow);
  }
}
}  // namespace

extern "C" int bgmoe_selfcheck_sigmoid(uint32_t first_bits, uint64_t count, uint64_t* mismatches, uint64_t* fallbacks,
                                       bgmoe_stream_t stream) {
  BGMOE_REQUIRE(mismatches != nullptr, "selfcheck_sigmoid: null counter");
  BGMOE_REQUIRE(count <= (1ull << 32), "selfcheck_sigmoid: at most 2^32 bit patterns");
  if (count == 0) return BGMOE_OK;
  uint64_t blocks = (count + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL(sigmoid_selfcheck_kernel, dim3((unsigned)blocks), dim3(256), 0, bgmoe_stream(stream), first_bits,
                     count, reinterpret_cast<unsigned long long*>(mismatches),
                     reinterpret_cast<unsigned long long*>(fallbacks));
  return bgmoe_check_launch("selfcheck_sigmoid");
}
