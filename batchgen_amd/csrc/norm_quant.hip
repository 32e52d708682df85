// Residual add + RMSNorm + per-token 128-block e4m3fn cast in one pass for gfx950: the producer that hands
// the MoE layer its FP8 activation without a second trip through HBM.
//
// One block per row, H/8 threads, thread t owning columns 8t..8t+7 (16-byte loads and stores; the row stays
// in registers between the sum of squares and the normalisation).  4 B read + 5 B written per element
// (+ 4 B per 128); about 40 VALU operations per element (bf16 unpack/round, the IEEE division), which at
// 16K rows costs as much time as the memory traffic.  (One wave per row -- no barriers, more rows in flight
// -- measured the same at 16K rows and 3x slower at 256 rows.)  The sum of squares follows a fixed tree -- an
// fma chain over a thread's 8 columns, a 32-lane butterfly (offsets 16..1), then the 32-lane sums through the
// same butterfly -- so the result is one function of the row, reproducible on the CPU bit for bit.  rsqrt is
// the correctly rounded one (through fp64) and the quantiser divides in IEEE fp32.
#include "bgmoe_common.h"

namespace {

struct NormQuantArgs {
  uint16_t* residual;          // [rows,h] bf16, updated in place; nullptr: plain RMSNorm of `hidden`
  const uint16_t* hidden;      // [rows,h] bf16
  const uint16_t* weight;      // [h] bf16
  uint16_t* normed;            // [rows,h] bf16
  uint8_t* q;                  // [rows,h] e4m3fn, may be nullptr (no cast)
  float* scale;                // (r,kb) at scale[r*srow + kb*skb]
  int64_t srow, skb;
  float eps;
  int h;
  const int32_t* norm_nv;      // rows >= *norm_nv: nothing is read or written for the norm
  const int32_t* quant_nv;     // rows >= *quant_nv: bytes 0, scales 1e-12
  const uint16_t* row_valid;   // [rows] bf16 predicate on `hidden`
};

// lane 0 (and 32) of the result = the 32-lane shuffle-down tree with offsets 16, 8, 4, 2, 1
__device__ __forceinline__ float half_wave_sum(float v) {
#pragma unroll
  for (int off = 16; off >= 1; off >>= 1) v = v + __shfl_xor(v, off, BGMOE_WAVE);
  return v;
}

__global__ __launch_bounds__(1024) void add_rmsnorm_fp8_quant_kernel(NormQuantArgs a) {
  __shared__ float s_warp[32];
  __shared__ float s_inv;
  const int64_t row = blockIdx.x;
  const int t = threadIdx.x;
  const int threads = a.h >> 3;
  const bool live = t < threads;           // the block is rounded up to whole waves
  const bool quant_skip = a.quant_nv && row >= *a.quant_nv;
  const bool norm_skip = a.norm_nv && row >= *a.norm_nv;
  const int64_t base = row * a.h + (int64_t)t * 8;

  if (quant_skip && a.q) {
    if (live) *reinterpret_cast<uint2*>(a.q + base) = make_uint2(0u, 0u);
    if (t < (a.h >> 7)) a.scale[row * a.srow + (int64_t)t * a.skb] = 1e-12f;
  }
  if (norm_skip) return;                   // whole block

  const bool row_valid = !a.row_valid || bf16_bits_to_f32(a.row_valid[row]) != 0.0f;
  float rounded[8];
  float sum_sq = 0.0f;
  if (live) {
    const uint4 hh = *reinterpret_cast<const uint4*>(a.hidden + base);
    const uint4 rr = a.residual ? *reinterpret_cast<const uint4*>(a.residual + base) : hh;
    const uint32_t rw[4] = {rr.x, rr.y, rr.z, rr.w};
    const uint32_t hw[4] = {hh.x, hh.y, hh.z, hh.w};
    float sum[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t rb = (i & 1) ? rw[i >> 1] >> 16 : rw[i >> 1] & 0xffffu;
      const uint32_t hb = (i & 1) ? hw[i >> 1] >> 16 : hw[i >> 1] & 0xffffu;
      const float hv = row_valid ? bf16_bits_to_f32(hb) : 0.0f;   // a predicate, never a factor
      sum[i] = a.residual ? bf16_bits_to_f32(rb) + hv : hv;
      sum_sq = __builtin_fmaf(sum[i], sum[i], sum_sq);
    }
    uint32_t ow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ow[i] = pack2_bf16(sum[2 * i], sum[2 * i + 1]);
      rounded[2 * i] = __uint_as_float(ow[i] << 16);
      rounded[2 * i + 1] = __uint_as_float(ow[i] & 0xffff0000u);
    }
    if (a.residual) *reinterpret_cast<uint4*>(a.residual + base) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
  }
  // the reference's tree: 32-lane sums (one per half wave), then those sums through the same tree
  const float wsum = half_wave_sum(sum_sq);
  if ((t & 31) == 0) s_warp[t >> 5] = wsum;
  __syncthreads();
  if (t < BGMOE_WAVE) {
    const int nwarps = (threads + 31) >> 5;
    const float v = half_wave_sum((t < nwarps) ? s_warp[t] : 0.0f);   // lanes 32..63 carry zeros
    if (t == 0) {
      const float ms = v / (float)a.h + a.eps;
      s_inv = (float)(1.0 / __builtin_sqrt((double)ms));
    }
  }
  __syncthreads();
  if (!live) return;
  const float inv = s_inv;

  const uint4 ww = *reinterpret_cast<const uint4*>(a.weight + (int64_t)t * 8);
  const uint32_t wv[4] = {ww.x, ww.y, ww.z, ww.w};
  float nv[8];
  uint32_t nw[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float w0 = bf16_bits_to_f32(wv[i] & 0xffffu), w1 = __uint_as_float(wv[i] & 0xffff0000u);
    const float v0 = rounded[2 * i] * inv, v1 = rounded[2 * i + 1] * inv;
    nw[i] = pack2_bf16(v0 * w0, v1 * w1);
    nv[2 * i] = __uint_as_float(nw[i] << 16);            // the cast sees what a reader of `normed` would see
    nv[2 * i + 1] = __uint_as_float(nw[i] & 0xffff0000u);
  }
  *reinterpret_cast<uint4*>(a.normed + base) = make_uint4(nw[0], nw[1], nw[2], nw[3]);
  if (quant_skip || !a.q) return;

  // 16 consecutive threads share a 128-block; the xor offsets 1..8 stay inside that group
  float amax = fabsf(nv[0]);
#pragma unroll
  for (int i = 1; i < 8; ++i) amax = fmaxf(amax, fabsf(nv[i]));
  amax = wave_max_xor<16>(amax);
  amax = fmaxf(amax, 1.52587890625e-05f);
  constexpr float kInv448 = static_cast<float>(1.0 / 448.0);
  const float sc = fmaxf(amax * kInv448, 1e-12f);
  float qv[8];
  quant_div_clamp(nv, sc, qv);
#pragma unroll
  for (int i = 0; i < 8; ++i) qv[i] = fabsf(qv[i]) < 1e30f ? qv[i] : 0.0f;
  *reinterpret_cast<uint2*>(a.q + base) =
      make_uint2(pack4_e4m3(qv[0], qv[1], qv[2], qv[3]), pack4_e4m3(qv[4], qv[5], qv[6], qv[7]));
  if ((t & 15) == 0) a.scale[row * a.srow + (int64_t)(t >> 4) * a.skb] = sc;
}

}  // namespace

extern "C" int bgmoe_add_rmsnorm_fp8_quant(uint16_t* residual, const uint16_t* hidden, const uint16_t* weight,
                                           int64_t rows, int h, float eps, uint16_t* normed_out,
                                           uint8_t* quant_out, float* quant_scale, int64_t scale_row_stride,
                                           int64_t scale_kb_stride, const int32_t* norm_num_valid_tokens,
                                           const int32_t* quant_num_valid_tokens,
                                           const uint16_t* row_valid_mask, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(rows >= 0 && rows <= 0x7fffffffLL, "add_rmsnorm_fp8_quant: bad row count %lld", (long long)rows);
  BGMOE_REQUIRE(h >= 128 && h <= 8192 && h % 128 == 0,
                "add_rmsnorm_fp8_quant: hidden size %d must be a multiple of 128 in [128, 8192]", h);
  BGMOE_REQUIRE(!norm_num_valid_tokens || !quant_out || norm_num_valid_tokens == quant_num_valid_tokens,
                "add_rmsnorm_fp8_quant: norm_num_valid_tokens requires quant_num_valid_tokens to be the same "
                "tensor (a row the norm skips has no defined value to quantise)");
  BGMOE_REQUIRE(!quant_out || quant_scale, "add_rmsnorm_fp8_quant: quant_out without quant_scale");
  if (rows == 0) return BGMOE_OK;
  BGMOE_REQUIRE(residual && hidden && weight && normed_out, "add_rmsnorm_fp8_quant: null pointer");
  BGMOE_REQUIRE(((uintptr_t)residual | (uintptr_t)hidden | (uintptr_t)weight | (uintptr_t)normed_out) % 16 == 0 &&
                    (uintptr_t)quant_out % 8 == 0,
                "add_rmsnorm_fp8_quant: operands must be 16-byte aligned");
  NormQuantArgs a{};
  a.residual = residual; a.hidden = hidden; a.weight = weight; a.normed = normed_out;
  a.q = quant_out; a.scale = quant_scale; a.srow = scale_row_stride; a.skb = scale_kb_stride;
  a.eps = eps; a.h = h; a.norm_nv = norm_num_valid_tokens; a.quant_nv = quant_num_valid_tokens;
  a.row_valid = row_valid_mask;
  hipStream_t st = bgmoe_stream(stream);
  const int threads = ((h / 8) + BGMOE_WAVE - 1) / BGMOE_WAVE * BGMOE_WAVE;
  BgmoeProf prof(BGMOE_K_NORM_QUANT, st);
  hipLaunchKernelGGL(add_rmsnorm_fp8_quant_kernel, dim3((unsigned)rows), dim3(threads), 0, st, a);
  return bgmoe_check_launch("add_rmsnorm_fp8_quant");
}

// Plain RMSNorm: the kernel above without a residual (the row itself is what gets normalised, and nothing is
// written back), so the sum of squares, the reciprocal square root and the rounding are the fused op's.
extern "C" int bgmoe_rmsnorm(const uint16_t* x, const uint16_t* weight, int64_t rows, int h, float eps,
                             uint16_t* out, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(rows >= 0 && rows <= 0x7fffffffLL, "rmsnorm: bad row count %lld", (long long)rows);
  BGMOE_REQUIRE(h >= 8 && h <= 8192 && h % 8 == 0, "rmsnorm: hidden size %d must be a multiple of 8 in [8, 8192]", h);
  if (rows == 0) return BGMOE_OK;
  BGMOE_REQUIRE(x && weight && out, "rmsnorm: null pointer");
  BGMOE_REQUIRE(((uintptr_t)x | (uintptr_t)weight | (uintptr_t)out) % 16 == 0, "rmsnorm: operands must be 16-byte aligned");
  NormQuantArgs a{};
  a.hidden = x; a.weight = weight; a.normed = out; a.eps = eps; a.h = h;
  hipStream_t st = bgmoe_stream(stream);
  const int threads = ((h / 8) + BGMOE_WAVE - 1) / BGMOE_WAVE * BGMOE_WAVE;
  BgmoeProf prof(BGMOE_K_NORM_QUANT, st);
  hipLaunchKernelGGL(add_rmsnorm_fp8_quant_kernel, dim3((unsigned)rows), dim3(threads), 0, st, a);
  return bgmoe_check_launch("rmsnorm");
}
