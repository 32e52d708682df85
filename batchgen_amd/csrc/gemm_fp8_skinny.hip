// Block-scaled FP8 grouped GEMM for FEW rows per group (decode): a
// weight-streaming kernel bound by HBM bandwidth.
//
// Work split: block = (group, 128 gate + 128 up output columns) for the fused
// stage 1, (group, 256 output columns) for a single GEMM; 4 waves, each owning
// four 16-row weight tiles over the whole K.  Every weight byte is read from
// HBM exactly once, straight into registers (no LDS: no other wave needs it),
// with 16-byte loads and a multi-stage register prefetch so that each wave
// keeps 16-24 KB of loads in flight.
//
// MFMA: v_mfma_f32_16x16x128_f8f6f4 with the WEIGHT tile as the A operand
// (16 output features x 128 K) and the TOKEN tile as B (128 K x 16 tokens):
// one instruction is exactly one 128-K scale block, so its 16x16 fp32 result
// is promoted with acc += part * (x_scale[token,kb] * w_scale[nblk,kb]).
// Lane l supplies row (l % 16) and the 32 K-bytes {16q..16q+15, 64+16q..64+16q+15},
// q = l / 16, for both operands: the same K permutation on both sides leaves
// the dot product unchanged and makes each load instruction cover 64
// contiguous bytes per row.  D: lane l holds token (l % 16), features
// 4*(l / 16) + 0..3.
//
// Algorithmic bytes per group: n*k weight bytes (+ n*k/16384*4 scale bytes)
// per matrix; activations (rows*k) are re-read per block from L2.
#include "bgmoe_common.h"

namespace {

struct SkinnyArgs {
  bgmoe_fp8_act a;
  bgmoe_fp8_weight w0, w1;
  const int32_t* seqlens;
  const int32_t* cu;
  int groups, n, k;
  uint16_t* out;
  uint8_t* out_q;
  float* out_s;
  int64_t os_row, os_nb;
  int lo, hi;                 // this launch serves groups with lo < count <= hi
};

template <int TT, int NSC>
struct Stage {
  intx8 A[4];
  intx8 B[TT];
  float xs[TT];
  float ws[NSC];
};

__device__ __forceinline__ intx8 load32(const uint8_t* p) {
  const intx4 lo = *reinterpret_cast<const intx4*>(p);
  const intx4 hi = *reinterpret_cast<const intx4*>(p + 64);
  intx8 r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

__device__ __forceinline__ intx8 load32_stream(const uint8_t* p) {
  const intx4 lo = __builtin_nontemporal_load(reinterpret_cast<const intx4*>(p));
  const intx4 hi = __builtin_nontemporal_load(reinterpret_cast<const intx4*>(p + 64));
  intx8 r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

template <int TT, int NSTAGE, bool FUSED>
__global__ __launch_bounds__(256) void fp8_skinny_kernel(SkinnyArgs g) {
  constexpr int NT = 4;                  // weight tiles per wave
  constexpr int NSC = FUSED ? 2 : 1;     // weight-scale streams per wave
  __shared__ float s_amax[4][TT][16];

  const int grp = blockIdx.y;
  const int cnt = g.seqlens[grp];
  if (cnt <= g.lo || cnt > g.hi) return;          // whole block
  const int64_t row0 = g.cu[grp];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int r16 = lane & 15;
  const int kq = lane >> 4;
  const int K = g.k;
  const int KB = K >> 7;
  const int n0 = blockIdx.x * (FUSED ? 128 : 256);

  const uint8_t* wb[2];
  const float* wsb[2];
  wb[0] = g.w0.w_ptrs ? g.w0.w_ptrs[grp] : g.w0.w + (int64_t)grp * g.w0.w_group_stride;
  wsb[0] = g.w0.scale_ptrs ? g.w0.scale_ptrs[grp] : g.w0.scale + (int64_t)grp * g.w0.scale_group_stride;
  if constexpr (FUSED) {
    wb[1] = g.w1.w_ptrs ? g.w1.w_ptrs[grp] : g.w1.w + (int64_t)grp * g.w1.w_group_stride;
    wsb[1] = g.w1.scale_ptrs ? g.w1.scale_ptrs[grp] : g.w1.scale + (int64_t)grp * g.w1.scale_group_stride;
  }

  const uint8_t* wp[NT];
  bool tv[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int nrow = FUSED ? n0 + 32 * wave + 16 * (t & 1) : n0 + 64 * wave + 16 * t;
    tv[t] = nrow < g.n;
    wp[t] = wb[FUSED ? (t >> 1) : 0] + (int64_t)(nrow + r16) * K + 16 * kq;
  }
  const float* wsp[NSC];
  if constexpr (FUSED) {
    wsp[0] = wsb[0] + (int64_t)(n0 >> 7) * g.w0.scale_nb_stride;
    wsp[1] = wsb[1] + (int64_t)(n0 >> 7) * g.w1.scale_nb_stride;
  } else {
    const int nb = min(n0 + 64 * wave, g.n - 1) >> 7;
    wsp[0] = wsb[0] + (int64_t)nb * g.w0.scale_nb_stride;
  }

  for (int t0 = 0; t0 < cnt; t0 += 16 * TT) {
    const uint8_t* xp[TT];
    const float* xsp[TT];
    bool xv[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      const int tok = t0 + 16 * tt + r16;
      xv[tt] = tok < cnt;
      const int64_t r = row0 + (xv[tt] ? tok : 0);
      xp[tt] = g.a.x + r * K + 16 * kq;
      xsp[tt] = g.a.scale + r * g.a.scale_row_stride;
    }

    floatx4 acc[TT][NT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[tt][t] = floatx4{0.f, 0.f, 0.f, 0.f};

    Stage<TT, NSC> st[NSTAGE];
    auto load_stage = [&](Stage<TT, NSC>& s, int kb) {
      const int ko = kb << 7;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        if (tv[t]) s.A[t] = load32_stream(wp[t] + ko);
        else s.A[t] = intx8{0, 0, 0, 0, 0, 0, 0, 0};
      }
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        if (xv[tt]) {
          s.B[tt] = load32(xp[tt] + ko);
          s.xs[tt] = xsp[tt][(int64_t)kb * g.a.scale_kb_stride];
        } else {
          s.B[tt] = intx8{0, 0, 0, 0, 0, 0, 0, 0};
          s.xs[tt] = 0.0f;
        }
      }
#pragma unroll
      for (int i = 0; i < NSC; ++i) s.ws[i] = wsp[i][kb];
    };

#pragma unroll
    for (int s = 0; s < NSTAGE - 1; ++s)
      if (s < KB) load_stage(st[s], s);

    for (int kb0 = 0; kb0 < KB; kb0 += NSTAGE) {
#pragma unroll
      for (int s = 0; s < NSTAGE; ++s) {
        const int kb = kb0 + s;
        if (kb < KB) {
          if (kb + NSTAGE - 1 < KB) load_stage(st[(s + NSTAGE - 1) % NSTAGE], kb + NSTAGE - 1);
          const Stage<TT, NSC>& c = st[s];
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
              const floatx4 p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                  c.A[t], c.B[tt], floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
              const float sc = c.xs[tt] * c.ws[FUSED ? (t >> 1) : 0];
#pragma unroll
              for (int i = 0; i < 4; ++i) acc[tt][t][i] = fmaf(p[i], sc, acc[tt][t][i]);
            }
          }
        }
      }
    }

    // ---- epilogue -------------------------------------------------------------
    if constexpr (FUSED) {
      float hv[TT][2][4];
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        float am = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            hv[tt][j][i] = bf16_round_f32(silu_f32(acc[tt][j][i]) * acc[tt][j + 2][i]);
            am = fmaxf(am, fabsf(hv[tt][j][i]));
          }
        const int tok = t0 + 16 * tt + r16;
        if (g.out != nullptr && xv[tt]) {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            uint2 o;
            o.x = f32_to_bf16_bits(hv[tt][j][0]) | (f32_to_bf16_bits(hv[tt][j][1]) << 16);
            o.y = f32_to_bf16_bits(hv[tt][j][2]) | (f32_to_bf16_bits(hv[tt][j][3]) << 16);
            *reinterpret_cast<uint2*>(g.out + (row0 + tok) * g.n + n0 + 32 * wave + 16 * j + 4 * kq) = o;
          }
        }
        if (g.out_q != nullptr) {
          am = fmaxf(am, __shfl_xor(am, 16, BGMOE_WAVE));
          am = fmaxf(am, __shfl_xor(am, 32, BGMOE_WAVE));
          if (kq == 0) s_amax[wave][tt][r16] = am;
        }
      }
      if (g.out_q != nullptr) {
        __syncthreads();
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          const float am = fmaxf(fmaxf(s_amax[0][tt][r16], s_amax[1][tt][r16]),
                                 fmaxf(s_amax[2][tt][r16], s_amax[3][tt][r16]));
          const float sc = quant_scale_from_amax(am);
          const int tok = t0 + 16 * tt + r16;
          if (xv[tt]) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const uint32_t q = pack4_e4m3(clamp448(hv[tt][j][0] / sc), clamp448(hv[tt][j][1] / sc),
                                            clamp448(hv[tt][j][2] / sc), clamp448(hv[tt][j][3] / sc));
              *reinterpret_cast<uint32_t*>(g.out_q + (row0 + tok) * g.n + n0 + 32 * wave + 16 * j + 4 * kq) = q;
            }
            if (wave == 0 && kq == 0)
              g.out_s[(row0 + tok) * g.os_row + (int64_t)(n0 >> 7) * g.os_nb] = sc;
          }
        }
        __syncthreads();   // s_amax is reused by the next pass
      }
    } else {
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        const int tok = t0 + 16 * tt + r16;
        if (!xv[tt]) continue;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          if (!tv[t]) continue;
          uint2 o;
          o.x = f32_to_bf16_bits(acc[tt][t][0]) | (f32_to_bf16_bits(acc[tt][t][1]) << 16);
          o.y = f32_to_bf16_bits(acc[tt][t][2]) | (f32_to_bf16_bits(acc[tt][t][3]) << 16);
          *reinterpret_cast<uint2*>(g.out + (row0 + tok) * g.n + n0 + 64 * wave + 16 * t + 4 * kq) = o;
        }
      }
    }
  }
}

int check_common(const char* what, const bgmoe_fp8_act* a, const bgmoe_fp8_weight* w, const int32_t* seqlens,
                 const int32_t* cu, int groups, int64_t m, int n, int k) {
  BGMOE_REQUIRE(a && w, "%s: null operand descriptor", what);
  BGMOE_REQUIRE(groups >= 0 && groups <= 1024, "%s: groups=%d outside [0,1024]", what, groups);
  BGMOE_REQUIRE(m >= 0, "%s: m < 0", what);
  BGMOE_REQUIRE(k > 0 && k % 128 == 0, "%s: K=%d must be a positive multiple of 128", what, k);
  BGMOE_REQUIRE(n > 0 && n % 128 == 0, "%s: N=%d must be a positive multiple of 128", what, n);
  if (groups == 0 || m == 0) return BGMOE_OK;
  BGMOE_REQUIRE(seqlens && cu, "%s: null seqlens / cu_seqlens", what);
  BGMOE_REQUIRE(a->x && a->scale, "%s: null activation", what);
  BGMOE_REQUIRE((uintptr_t)a->x % 16 == 0, "%s: activations must be 16-byte aligned", what);
  BGMOE_REQUIRE((w->w || w->w_ptrs) && (w->scale || w->scale_ptrs), "%s: null weight", what);
  BGMOE_REQUIRE(w->w_ptrs || ((uintptr_t)w->w % 16 == 0 && w->w_group_stride % 16 == 0),
                "%s: weights must be 16-byte aligned", what);
  BGMOE_REQUIRE(w->scale_ptrs || w->scale_nb_stride >= k / 128, "%s: weight scale row stride %lld < K/128",
                what, (long long)w->scale_nb_stride);
  return BGMOE_OK;
}

}  // namespace

// defined in gemm_fp8_tiled.hip: serves groups with more than `lo` rows
int bgmoe_launch_fp8_tiled(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* w0, const bgmoe_fp8_weight* w1,
                           const int32_t* seqlens, const int32_t* cu, int groups, int64_t m, int n, int k,
                           uint16_t* out, uint8_t* out_q, float* out_s, int64_t os_row, int64_t os_nb,
                           int lo, hipStream_t st);

static int launch_skinny(bool fused, SkinnyArgs& g, int64_t m, hipStream_t st) {
  const int ntile = fused ? 128 : 256;
  const dim3 grid((g.n + ntile - 1) / ntile, g.groups), block(256);
  // rows per group in (0,16], (16,64]; more rows go to the LDS-tiled kernel
  g.lo = 0; g.hi = 16;
  {
    BgmoeProf prof(fused ? BGMOE_K_S1_SKINNY16 : BGMOE_K_GEMM_SKINNY16, st);
    if (fused) hipLaunchKernelGGL((fp8_skinny_kernel<1, 3, true>), grid, block, 0, st, g);
    else hipLaunchKernelGGL((fp8_skinny_kernel<1, 3, false>), grid, block, 0, st, g);
  }
  if (m > 16) {
    g.lo = 16; g.hi = 64;
    BgmoeProf prof(fused ? BGMOE_K_S1_SKINNY64 : BGMOE_K_GEMM_SKINNY64, st);
    if (fused) hipLaunchKernelGGL((fp8_skinny_kernel<2, 3, true>), grid, block, 0, st, g);
    else hipLaunchKernelGGL((fp8_skinny_kernel<2, 3, false>), grid, block, 0, st, g);
  }
  int rc = bgmoe_check_launch("fp8 grouped gemm (skinny)");
  if (rc != BGMOE_OK || m <= 64) return rc;
  return bgmoe_launch_fp8_tiled(&g.a, &g.w0, fused ? &g.w1 : nullptr, g.seqlens, g.cu, g.groups, m, g.n,
                                g.k, g.out, g.out_q, g.out_s, g.os_row, g.os_nb, 64, st);
}

extern "C" int bgmoe_fp8_grouped_gemm(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* b,
                                      const int32_t* seqlens, const int32_t* cu_seqlens, int groups,
                                      int64_t m, int n, int k, uint16_t* out, bgmoe_stream_t stream) {
  int rc = check_common("fp8_grouped_gemm", a, b, seqlens, cu_seqlens, groups, m, n, k);
  if (rc != BGMOE_OK) return rc;
  if (groups == 0 || m == 0) return BGMOE_OK;
  BGMOE_REQUIRE(out && (uintptr_t)out % 8 == 0, "fp8_grouped_gemm: output must be non-null, 8-byte aligned");
  SkinnyArgs g{};
  g.a = *a; g.w0 = *b; g.seqlens = seqlens; g.cu = cu_seqlens; g.groups = groups; g.n = n; g.k = k;
  g.out = out;
  return launch_skinny(false, g, m, bgmoe_stream(stream));
}

extern "C" int bgmoe_fp8_fused_s1(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* gate,
                                  const bgmoe_fp8_weight* up, const int32_t* seqlens,
                                  const int32_t* cu_seqlens, int groups, int64_t m, int n, int k,
                                  uint16_t* out, uint8_t* out_q, float* out_scale,
                                  int64_t out_scale_row_stride, int64_t out_scale_nb_stride,
                                  bgmoe_stream_t stream) {
  int rc = check_common("fp8_fused_s1", a, gate, seqlens, cu_seqlens, groups, m, n, k);
  if (rc != BGMOE_OK) return rc;
  rc = check_common("fp8_fused_s1", a, up, seqlens, cu_seqlens, groups, m, n, k);
  if (rc != BGMOE_OK) return rc;
  if (groups == 0 || m == 0) return BGMOE_OK;
  BGMOE_REQUIRE(out || out_q, "fp8_fused_s1: no output given");
  BGMOE_REQUIRE(!out_q || out_scale, "fp8_fused_s1: out_q needs out_scale");
  BGMOE_REQUIRE((uintptr_t)out % 8 == 0 && (uintptr_t)out_q % 4 == 0, "fp8_fused_s1: misaligned output");
  SkinnyArgs g{};
  g.a = *a; g.w0 = *gate; g.w1 = *up; g.seqlens = seqlens; g.cu = cu_seqlens; g.groups = groups;
  g.n = n; g.k = k; g.out = out; g.out_q = out_q; g.out_s = out_scale;
  g.os_row = out_scale_row_stride; g.os_nb = out_scale_nb_stride;
  return launch_skinny(true, g, m, bgmoe_stream(stream));
}
