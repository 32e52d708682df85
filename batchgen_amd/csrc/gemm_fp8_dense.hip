// Block-scaled FP8 GEMM of ONE weight matrix against few rows (decode-time dense MLP / shared expert outside
// the grouped launch): out[m, n] = bf16( sum_kb (x[m, kb] . w[n, kb]) * xs[m, kb] * ws[n / 128, kb] ).
//
// A grouped launch has one work item per (group, 128 columns); with a single group that is N / 128 items, fewer
// than the chip has wave slots.  Here the K axis is the parallel one, in two forms.  This file holds the wave
// split and the entry points; the block split (K-slices over blocks, fp32 partial sums in a caller workspace,
// chosen for more rows) reuses the grouped kernel's work item and lives beside it.  Wave split: a block owns 16, 32 or 64 weight rows over
// the whole K, its 8 waves own one K-slice each (a contiguous run of 128-byte scale blocks), and the partial
// sums meet in LDS where they are added in wave order, so the result does not depend on timing.  N / 16 blocks
// of 8 waves keep the whole weight matrix in flight at once; each wave issues all loads of up to four K-blocks
// before the first MFMA.
//
// MFMA operands and K permutation as in the grouped kernels: weight tile = A (16 features x 128 K), token tile
// = B, lane l supplies row l % 16 and K-bytes {16q..16q+15, 64+16q..64+16q+15}, q = l / 16; D: lane l holds
// token l % 16, features 4q..4q+3.
//
// The accumulation order is a function of K alone (slice length ceil(K/128 / 8)), and the choice between the two
// forms a function of the row count, K and the weight layout, never of N: the gate and up halves of a stacked [gate; up] weight give exactly the bytes of two separate calls.
//
// Algorithmic bytes: n*k weight bytes once per 64-row chunk; the m*k token bytes are re-read per block from L2.
#include "bgmoe_common.h"

namespace {

constexpr int kWaves = 8;

struct DenseArgs {
  bgmoe_fp8_act a;
  const uint8_t* w;
  const float* ws;
  int64_t ws_nb_stride;
  int64_t m;
  int n, k;
  uint16_t* out;
};

__device__ __forceinline__ intx8 load32(const uint8_t* p, bool stream) {
  intx4 lo, hi;
  if (stream) {
    lo = gload_x4_stream(p);
    hi = gload_x4_stream(p + 64);
  } else {
    lo = gload_x4(p);
    hi = gload_x4(p + 64);
  }
  return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

// TT token tiles (16 rows each) x NTB weight tiles per block; UN K-blocks of loads in flight per wave.
template <int TT, int NTB, int UN>
__global__ __launch_bounds__(kWaves * 64) void fp8_dense_kernel(DenseArgs g) {
  __shared__ floatx4 s_part[kWaves][TT * NTB][64];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int r16 = lane & 15, kq = lane >> 4;
  const int K = g.k, KB = K >> 7;
  const int per = (KB + kWaves - 1) / kWaves;
  const int kb_lo = wave * per;
  const int kb_hi = min(KB, kb_lo + per);
  const int n0 = blockIdx.x * 16 * NTB;
  const int64_t m0 = (int64_t)blockIdx.y * 16 * TT;
  const int live = (int)min<int64_t>(g.m - m0, 16 * TT);            // >= 1
  const bool stream = gridDim.y == 1;                                // weights read once: keep them out of L2

  const uint8_t* wp[NTB];
  const float* wsp[NTB];
#pragma unroll
  for (int t = 0; t < NTB; ++t) {
    const int nr = min(n0 + 16 * t, g.n - 16);                       // a tile past N re-reads the last one
    wp[t] = g.w + (int64_t)(nr + r16) * K + 16 * kq;
    wsp[t] = g.ws + (int64_t)(nr >> 7) * g.ws_nb_stride;
  }
  const uint8_t* xp[TT];
  const float* xsp[TT];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
    const int64_t row = m0 + min(16 * tt + r16, live - 1);           // rows past the end re-read the last row
    xp[tt] = g.a.x + row * K + 16 * kq;
    xsp[tt] = g.a.scale + row * g.a.scale_row_stride;
  }

  floatx4 acc[TT][NTB];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt)
#pragma unroll
    for (int t = 0; t < NTB; ++t) acc[tt][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  for (int kb0 = kb_lo; kb0 < kb_hi; kb0 += UN) {
    intx8 A[UN][NTB], B[UN][TT];
    float ws[UN][NTB], xs[UN][TT];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int kb = min(kb0 + u, kb_hi - 1);
#pragma unroll
      for (int t = 0; t < NTB; ++t) {
        A[u][t] = load32(wp[t] + (kb << 7), stream);
        ws[u][t] = gload_f32(wsp[t] + kb);
      }
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        B[u][tt] = load32(xp[tt] + (kb << 7), false);
        xs[u][tt] = gload_f32(xsp[tt] + (int64_t)kb * g.a.scale_kb_stride);
      }
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      if (kb0 + u < kb_hi) {
#pragma unroll
        for (int tt = 0; tt < TT; ++tt)
#pragma unroll
          for (int t = 0; t < NTB; ++t) {
            const floatx4 p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                A[u][t], B[u][tt], floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
            const float sc = xs[u][tt] * ws[u][t];
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[tt][t][i] = fmaf(p[i], sc, acc[tt][t][i]);
          }
      }
    }
  }

#pragma unroll
  for (int tt = 0; tt < TT; ++tt)
#pragma unroll
    for (int t = 0; t < NTB; ++t) s_part[wave][tt * NTB + t][lane] = acc[tt][t];
  __syncthreads();
#pragma unroll
  for (int c = wave; c < TT * NTB; c += kWaves) {                    // a wave adds the 8 partials of a tile, in order
    const int tt = c / NTB, t = c % NTB;
    floatx4 sum = s_part[0][c][lane];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) {
      const floatx4 p = s_part[w][c][lane];
#pragma unroll
      for (int i = 0; i < 4; ++i) sum[i] += p[i];
    }
    const int tok = 16 * tt + r16;
    const int col = n0 + 16 * t + 4 * kq;
    if (tok < live && n0 + 16 * t < g.n) {
      uint2 o;
      o.x = pack2_bf16(sum[0], sum[1]);
      o.y = pack2_bf16(sum[2], sum[3]);
      *reinterpret_cast<uint2*>(g.out + (m0 + tok) * g.n + col) = o;
    }
  }
}

template <int TT, int NTB, int UN>
void launch_dense(const DenseArgs& g, hipStream_t st) {
  const unsigned bx = (unsigned)((g.n / 16 + NTB - 1) / NTB);
  const unsigned by = (unsigned)((g.m + 16 * TT - 1) / (16 * TT));
  hipLaunchKernelGGL((fp8_dense_kernel<TT, NTB, UN>), dim3(bx, by), dim3(kWaves * 64), 0, st, g);
}

}  // namespace

// defined in gemm_fp8_skinny.hip
int bgmoe_internal_fp8_dense_splitk(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* w, int64_t m, int n, int k,
                                    int per, float* workspace, uint16_t* out, hipStream_t st);

// K-blocks per slice of the split-K form for m rows, 0 = use the wave-split kernel above.  A function of m, k and
// the layout only, never of n, so that a stacked [gate; up] weight and its halves are added in the same order.
static int splitk_per(int64_t m, int k, int layout) {
  const int deep = k >= 16384 ? 16 : 8;                 // measured: longer slices once K is long enough to fill the chip
  if (layout != BGMOE_W_ROW_MAJOR || m > 64) return deep;
  if (m <= 16) return 0;
  if (k >= 16384) return 16;
  return m > 32 && k >= 4096 ? 8 : 0;
}

extern "C" int64_t bgmoe_fp8_dense_gemm_workspace(int64_t m, int n, int k, int layout) {
  if (m <= 0 || n <= 0 || k <= 0) return 0;
  const int per = splitk_per(m, k, layout);
  if (per <= 0) return 0;
  return ((k / 128 + per - 1) / per) * m * n * (int64_t)sizeof(float);
}

extern "C" int bgmoe_fp8_dense_gemm_partials(const bgmoe_fp8_act* a, const uint8_t* w, const float* w_scale,
                                             int64_t scale_nb_stride, int layout, int64_t m, int n, int k,
                                             void* workspace, int64_t workspace_bytes, int* slices,
                                             bgmoe_stream_t stream) {
  BGMOE_REQUIRE(a != nullptr && slices != nullptr, "fp8_dense_gemm_partials: null argument");
  BGMOE_REQUIRE(m > 0 && m <= 65535LL * 16, "fp8_dense_gemm_partials: m=%lld out of range", (long long)m);
  BGMOE_REQUIRE(k > 0 && k % 128 == 0 && n > 0 && n % 128 == 0,
                "fp8_dense_gemm_partials: K=%d and N=%d must be positive multiples of 128", k, n);
  BGMOE_REQUIRE(layout == BGMOE_W_ROW_MAJOR || layout == BGMOE_W_TILE_MAJOR,
                "fp8_dense_gemm_partials: unknown weight layout %d", layout);
  const int per = splitk_per(m, k, layout);
  BGMOE_REQUIRE(per > 0, "fp8_dense_gemm_partials: m=%lld k=%d is served without partial sums "
                "(bgmoe_fp8_dense_gemm_workspace is 0): call bgmoe_fp8_dense_gemm", (long long)m, k);
  const int64_t need = bgmoe_fp8_dense_gemm_workspace(m, n, k, layout);
  BGMOE_REQUIRE(a->x && a->scale && w && w_scale, "fp8_dense_gemm_partials: null pointer");
  BGMOE_REQUIRE(scale_nb_stride >= k / 128, "fp8_dense_gemm_partials: weight-scale row stride %lld < K/128 = %d",
                (long long)scale_nb_stride, k / 128);
  BGMOE_REQUIRE(((uintptr_t)a->x | (uintptr_t)w) % 16 == 0, "fp8_dense_gemm_partials: x and w must be 16-byte aligned");
  BGMOE_REQUIRE(workspace != nullptr && workspace_bytes >= need && (uintptr_t)workspace % 16 == 0,
                "fp8_dense_gemm_partials: needs a 16-byte aligned workspace of %lld bytes, got %lld", (long long)need,
                (long long)workspace_bytes);
  hipStream_t st = bgmoe_stream(stream);
  BgmoeProf prof(BGMOE_K_DENSE_GEMM, st);
  bgmoe_fp8_act act = *a;
  act.scale_group_stride = 0;
  bgmoe_fp8_weight wd{};
  wd.w = w; wd.scale = w_scale; wd.scale_nb_stride = scale_nb_stride; wd.layout = layout;
  *slices = (k / 128 + per - 1) / per;
  return bgmoe_internal_fp8_dense_splitk(&act, &wd, m, n, k, per, (float*)workspace, nullptr, st);
}

extern "C" int bgmoe_fp8_dense_gemm(const bgmoe_fp8_act* a, const uint8_t* w, const float* w_scale,
                                    int64_t scale_nb_stride, int layout, int64_t m, int n, int k, uint16_t* out,
                                    void* workspace, int64_t workspace_bytes, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(a != nullptr, "fp8_dense_gemm: null operand descriptor");
  BGMOE_REQUIRE(m >= 0 && m <= 65535LL * 16, "fp8_dense_gemm: m=%lld out of range", (long long)m);
  BGMOE_REQUIRE(k > 0 && k % 128 == 0, "fp8_dense_gemm: K=%d must be a positive multiple of 128", k);
  BGMOE_REQUIRE(n > 0 && n % 128 == 0, "fp8_dense_gemm: N=%d must be a positive multiple of 128", n);
  BGMOE_REQUIRE(layout == BGMOE_W_ROW_MAJOR || layout == BGMOE_W_TILE_MAJOR, "fp8_dense_gemm: unknown weight layout %d",
                layout);
  if (m == 0) return BGMOE_OK;
  BGMOE_REQUIRE(a->x && a->scale && w && w_scale && out, "fp8_dense_gemm: null pointer");
  BGMOE_REQUIRE(scale_nb_stride >= k / 128, "fp8_dense_gemm: weight-scale row stride %lld < K/128 = %d",
                (long long)scale_nb_stride, k / 128);
  BGMOE_REQUIRE(((uintptr_t)a->x | (uintptr_t)w) % 16 == 0 && (uintptr_t)out % 8 == 0,
                "fp8_dense_gemm: x and w must be 16-byte aligned, out 8-byte aligned");
  hipStream_t st = bgmoe_stream(stream);
  BgmoeProf prof(BGMOE_K_DENSE_GEMM, st);
  const int per = splitk_per(m, k, layout);
  if (per > 0) {
    const int64_t need = bgmoe_fp8_dense_gemm_workspace(m, n, k, layout);
    BGMOE_REQUIRE(workspace != nullptr && workspace_bytes >= need && (uintptr_t)workspace % 16 == 0,
                  "fp8_dense_gemm: m=%lld n=%d k=%d needs a 16-byte aligned workspace of %lld bytes "
                  "(bgmoe_fp8_dense_gemm_workspace), got %lld", (long long)m, n, k, (long long)need,
                  (long long)workspace_bytes);
    bgmoe_fp8_act act = *a;
    act.scale_group_stride = 0;
    bgmoe_fp8_weight wd{};
    wd.w = w; wd.scale = w_scale; wd.scale_nb_stride = scale_nb_stride; wd.layout = layout;
    return bgmoe_internal_fp8_dense_splitk(&act, &wd, m, n, k, per, (float*)workspace, out, st);
  }
  DenseArgs g{};
  g.a = *a; g.w = w; g.ws = w_scale; g.ws_nb_stride = scale_nb_stride; g.m = m; g.n = n; g.k = k; g.out = out;
  // weight tiles per block (measured): more of them re-use the token bytes a block fetches from L2, fewer of
  // them give more blocks; a handful of rows is all weight traffic and wants the blocks
  const int tiles = n / 16;
  const int ntb = m <= 4 ? (tiles >= 384 && tiles < 1024 ? 2 : 1) : tiles >= 1024 ? 4 : tiles >= 384 ? 2 : 1;
  const int tt = m <= 16 ? 1 : m <= 32 ? 2 : 4;
#define BGMOE_DENSE_CASE(TT_, NTB_, UN_) \
  if (tt == TT_ && ntb == NTB_) launch_dense<TT_, NTB_, UN_>(g, st);
  BGMOE_DENSE_CASE(1, 1, 4) BGMOE_DENSE_CASE(1, 2, 4) BGMOE_DENSE_CASE(1, 4, 4)
  BGMOE_DENSE_CASE(2, 1, 4) BGMOE_DENSE_CASE(2, 2, 4) BGMOE_DENSE_CASE(2, 4, 2)
  BGMOE_DENSE_CASE(4, 1, 2) BGMOE_DENSE_CASE(4, 2, 2) BGMOE_DENSE_CASE(4, 4, 2)
#undef BGMOE_DENSE_CASE
  return bgmoe_check_launch("fp8_dense_gemm");
}
