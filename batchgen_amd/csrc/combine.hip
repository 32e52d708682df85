// Top-k weighted combine (un-permute) for gfx950, with the shared expert's
// output optionally folded into the same pass.  Gather-bound: each thread owns
// 8 consecutive columns of one token and reads K rows with 16-byte loads.
// The bf16 and fp32 forms accumulate acc = fma(value, weight, acc), k ascending: the
// reference kernels' `acc += val * w[k]` (dispatch_scatter_3d.cu:386-392, 421-431) is one
// fused multiply-add per term under nvcc's default contraction.  The ordered form rounds
// every product and partial sum to bf16 separately.  Both are reproducible bit for bit
// on the CPU.
#include "bgmoe_common.h"

namespace {

constexpr int kMaxK = 32;
constexpr int kThreads = 128;     // x 8 columns = 1024 columns per block

__device__ __forceinline__ void unpack8(const uint4& r, float* v) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = bf16_bits_to_f32(w[i] & 0xffffu);
    v[2 * i + 1] = bf16_bits_to_f32(w[i] >> 16);
  }
}

__device__ __forceinline__ uint4 pack8(const float* v) {
  uint4 o;
  o.x = pack2_bf16(v[0], v[1]);
  o.y = pack2_bf16(v[2], v[3]);
  o.z = pack2_bf16(v[4], v[5]);
  o.w = pack2_bf16(v[6], v[7]);
  return o;
}

// MODE 0: bf16 out, 1: fp32 out, 2: bf16 ordered (per-step bf16 rounding)
template <int MODE, bool VEC>
__global__ __launch_bounds__(kThreads) void combine_kernel(
    const uint16_t* __restrict__ y, const int32_t* __restrict__ pos, const int32_t* __restrict__ ids,
    const float* __restrict__ w, int h, int k, void* __restrict__ out,
    const uint16_t* __restrict__ shared, int shared_mode) {
  __shared__ int32_t s_pos[kMaxK];
  __shared__ float s_w[kMaxK];
  const int token = blockIdx.y;
  if ((!VEC || MODE == 2) && threadIdx.x == 0) {
    const int64_t base = (int64_t)token * k;
    if constexpr (MODE == 2) {
      int32_t eid[kMaxK];
      // insertion sort by expert id; strict '>' keeps equal ids in slot order
      for (int j = 0; j < k; ++j) {
        const int32_t e = ids[base + j];
        int q = j;
        while (q > 0 && eid[q - 1] > e) {
          eid[q] = eid[q - 1];
          s_pos[q] = s_pos[q - 1];
          s_w[q] = s_w[q - 1];
          --q;
        }
        eid[q] = e;
        s_pos[q] = pos[base + j];
        s_w[q] = bf16_round_f32(w[base + j]);
      }
    } else {
      for (int j = 0; j < k; ++j) {
        s_pos[j] = pos[base + j];
        s_w[j] = w[base + j];
      }
    }
  }
  __syncthreads();

  const int c0 = (blockIdx.x * kThreads + threadIdx.x) * (VEC ? 8 : 1);
  if (c0 >= h) return;
  constexpr int W = VEC ? 8 : 1;
  float acc[W];
#pragma unroll
  for (int i = 0; i < W; ++i) acc[i] = 0.0f;
  if constexpr (VEC && MODE != 2) {
    // rows of up to 8 routes are requested together (a route that is not local costs nothing), then
    // accumulated in route order: the loads overlap, the arithmetic keeps its order
    const int64_t base = (int64_t)token * k;
    for (int j0 = 0; j0 < k; j0 += 8) {
      uint4 raw[8];
      float wj[8];
      bool on[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int j = j0 + u;
        const int p = j < k ? pos[base + j] : -1;        // wave-uniform: scalar loads
        on[u] = p >= 0;
        wj[u] = 0.0f;
        raw[u] = uint4{0u, 0u, 0u, 0u};
        if (on[u]) {
          wj[u] = w[base + j];
          raw[u] = *reinterpret_cast<const uint4*>(y + (int64_t)p * h + c0);
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (on[u]) {
          float v[8];
          unpack8(raw[u], v);
#pragma unroll
          for (int i = 0; i < W; ++i) acc[i] = __builtin_fmaf(v[i], wj[u], acc[i]);
        }
      }
    }
  } else {
    for (int j = 0; j < k; ++j) {
      const int p = s_pos[j];
      if (p < 0) continue;
      const float wj = s_w[j];
      float v[W];
      if constexpr (VEC) {
        unpack8(*reinterpret_cast<const uint4*>(y + (int64_t)p * h + c0), v);
      } else {
        v[0] = bf16_bits_to_f32(y[(int64_t)p * h + c0]);
      }
#pragma unroll
      for (int i = 0; i < W; ++i) {
        if constexpr (MODE == 2) acc[i] = bf16_round_f32(acc[i] + bf16_round_f32(v[i] * wj));
        else acc[i] = __builtin_fmaf(v[i], wj, acc[i]);
      }
    }
  }
  const int64_t o = (int64_t)token * h + c0;
  if constexpr (MODE == 1) {
    float* of = reinterpret_cast<float*>(out) + o;
#pragma unroll
    for (int i = 0; i < W; ++i) of[i] = acc[i];
  } else {
    if (MODE == 0 && shared != nullptr) {
      float sv[W];
      if constexpr (VEC) unpack8(*reinterpret_cast<const uint4*>(shared + o), sv);
      else sv[0] = bf16_bits_to_f32(shared[o]);
#pragma unroll
      for (int i = 0; i < W; ++i)
        acc[i] = (shared_mode == 0 ? bf16_round_f32(acc[i]) : acc[i]) + sv[i];
    }
    uint16_t* ob = reinterpret_cast<uint16_t*>(out) + o;
    if constexpr (VEC) *reinterpret_cast<uint4*>(ob) = pack8(acc);
    else ob[0] = (uint16_t)f32_to_bf16_bits(acc[0]);
  }
}

template <int MODE>
int launch(const uint16_t* y, const int32_t* pos, const int32_t* ids, const float* w, int n, int h,
           int k, void* out, const uint16_t* shared, int shared_mode, hipStream_t st) {
  if (n == 0 || h == 0) return BGMOE_OK;
  const bool vec = (h % 8 == 0) && ((uintptr_t)y % 16 == 0) && ((uintptr_t)out % 16 == 0) &&
                   ((uintptr_t)shared % 16 == 0);
  const int cols = kThreads * (vec ? 8 : 1);
  const dim3 grid((h + cols - 1) / cols, n), block(kThreads);
  BgmoeProf prof(BGMOE_K_COMBINE, st);
  if (vec)
    hipLaunchKernelGGL((combine_kernel<MODE, true>), grid, block, 0, st, y, pos, ids, w, h, k, out,
                       shared, shared_mode);
  else
    hipLaunchKernelGGL((combine_kernel<MODE, false>), grid, block, 0, st, y, pos, ids, w, h, k, out,
                       shared, shared_mode);
  return bgmoe_check_launch("reduce_weighted_scatter");
}

}  // namespace

extern "C" int bgmoe_reduce_weighted_scatter(const uint16_t* expert_out, const int32_t* topk_pos,
                                             const float* topk_weights, int n, int h, int k,
                                             uint16_t* out, int num_valid_tokens,
                                             const uint16_t* shared, int shared_mode,
                                             bgmoe_stream_t stream) {
  BGMOE_REQUIRE(n >= 0 && h >= 0, "reduce_weighted_scatter: negative size");
  BGMOE_REQUIRE(k >= 1 && k <= kMaxK, "reduce_weighted_scatter: Unsupported K=%d", k);
  BGMOE_REQUIRE(shared_mode == 0 || shared_mode == 1, "reduce_weighted_scatter: bad shared_mode");
  const int rows = (num_valid_tokens > 0 && num_valid_tokens < n) ? num_valid_tokens : n;
  if (rows == 0 || h == 0) return BGMOE_OK;
  BGMOE_REQUIRE(expert_out && topk_pos && topk_weights && out, "reduce_weighted_scatter: null pointer");
  return launch<0>(expert_out, topk_pos, nullptr, topk_weights, rows, h, k, out, shared, shared_mode,
                   bgmoe_stream(stream));
}

extern "C" int bgmoe_reduce_weighted_scatter_fp32(const uint16_t* expert_out, const int32_t* topk_pos,
                                                  const float* topk_weights, int n, int h, int k,
                                                  float* out, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(n > 0 && h > 0, "reduce_weighted_scatter_fp32: N and H must be positive");
  BGMOE_REQUIRE(k >= 1 && k <= kMaxK, "reduce_weighted_scatter_fp32: Unsupported K=%d", k);
  BGMOE_REQUIRE(expert_out && topk_pos && topk_weights && out, "reduce_weighted_scatter_fp32: null pointer");
  return launch<1>(expert_out, topk_pos, nullptr, topk_weights, n, h, k, out, nullptr, 0,
                   bgmoe_stream(stream));
}

extern "C" int bgmoe_reduce_weighted_scatter_bf16_ordered(const uint16_t* expert_out,
                                                          const int32_t* topk_pos,
                                                          const int32_t* topk_ids,
                                                          const float* topk_weights, int n, int h,
                                                          int k, uint16_t* out,
                                                          bgmoe_stream_t stream) {
  BGMOE_REQUIRE(n > 0 && h > 0, "reduce_weighted_scatter_bf16_ordered: N and H must be positive");
  BGMOE_REQUIRE(k >= 1 && k <= kMaxK, "reduce_weighted_scatter_bf16_ordered: unsupported K=%d", k);
  BGMOE_REQUIRE(h % 8 == 0, "ordered BF16 combine requires H %% 8 == 0, got H=%d", h);
  BGMOE_REQUIRE(expert_out && topk_pos && topk_ids && topk_weights && out,
                "reduce_weighted_scatter_bf16_ordered: null pointer");
  BGMOE_REQUIRE((uintptr_t)expert_out % 16 == 0 && (uintptr_t)out % 16 == 0,
                "reduce_weighted_scatter_bf16_ordered: data must be 16-byte aligned");
  return launch<2>(expert_out, topk_pos, topk_ids, topk_weights, n, h, k, out, nullptr, 0,
                   bgmoe_stream(stream));
}
