// SiTU-and-multiply for gfx950: [rows, 2d] bf16 (gate | up) -> [rows, d] bf16, the activation of the Kimi-K3
// shared expert and dense MLP.  6 bytes of traffic per output element and two tanh, one exp and one division
// of arithmetic: one thread per 8 output columns (16-byte loads and stores), rows x column chunks in a flat
// grid.  When d, a stride or a pointer is not a multiple of 8 elements the same kernel runs one column per
// thread.
#include "bgmoe_common.h"

namespace {

struct SituArgs {
  const uint16_t* x;
  uint16_t* out;
  int64_t rows, xs, os;
  int d;
  float beta, inv_beta, lbeta, inv_lbeta;
  int has_linear;
  int swiglu;              // bf16(bf16(silu(g)) * u) instead: PyTorch's F.silu(gate) * up on bf16 tensors
};

__device__ __forceinline__ float situ_one(const SituArgs& a, float g, float u) {
  if (a.swiglu) {
    bool decided;
    float sv = silu_short_f32(g, &decided);
    if (!decided) sv = silu_exact_f32(g);
    return bf16_round_f32(sv) * u;
  }
  const float lin = a.has_linear ? situ_linear_f32(u, a.lbeta, a.inv_lbeta) : u;
  return situ_gate_f32(g, a.beta, a.inv_beta) * lin;
}

template <int VEC>
__global__ __launch_bounds__(256) void situ_and_mul_kernel(SituArgs a) {
  const int per_row = (a.d + VEC - 1) / VEC;
  const int64_t total = a.rows * per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = i / per_row;
    const int c = (int)(i - row * per_row) * VEC;
    const uint16_t* gp = a.x + row * a.xs + c;
    uint16_t* op = a.out + row * a.os + c;
    if constexpr (VEC == 8) {
      const uint4 gv = *reinterpret_cast<const uint4*>(gp);
      const uint4 uv = *reinterpret_cast<const uint4*>(gp + a.d);
      const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
      uint32_t ow[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float lo = situ_one(a, __uint_as_float(gw[j] << 16), __uint_as_float(uw[j] << 16));
        const float hi = situ_one(a, __uint_as_float(gw[j] & 0xffff0000u), __uint_as_float(uw[j] & 0xffff0000u));
        ow[j] = pack2_bf16(lo, hi);
      }
      *reinterpret_cast<uint4*>(op) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    } else {
      *op = (uint16_t)f32_to_bf16_bits(situ_one(a, bf16_bits_to_f32(gp[0]), bf16_bits_to_f32(gp[a.d])));
    }
  }
}

}  // namespace

static int act_and_mul(const uint16_t* x, int64_t rows, int d, int64_t x_row_stride, float beta, float linear_beta,
                       int swiglu, uint16_t* out, int64_t out_row_stride, bgmoe_stream_t stream);

extern "C" int bgmoe_situ_and_mul(const uint16_t* x, int64_t rows, int d, int64_t x_row_stride, float beta,
                                  float linear_beta, uint16_t* out, int64_t out_row_stride,
                                  bgmoe_stream_t stream) {
  BGMOE_REQUIRE(beta > 0.0f, "situ_and_mul: beta must be positive, got %g", (double)beta);
  return act_and_mul(x, rows, d, x_row_stride, beta, linear_beta, 0, out, out_row_stride, stream);
}

extern "C" int bgmoe_silu_and_mul(const uint16_t* x, int64_t rows, int d, int64_t x_row_stride, uint16_t* out,
                                  int64_t out_row_stride, bgmoe_stream_t stream) {
  return act_and_mul(x, rows, d, x_row_stride, 1.0f, 0.0f, 1, out, out_row_stride, stream);
}

static int act_and_mul(const uint16_t* x, int64_t rows, int d, int64_t x_row_stride, float beta, float linear_beta,
                       int swiglu, uint16_t* out, int64_t out_row_stride, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(rows >= 0 && d >= 0, "situ_and_mul: bad sizes rows=%lld d=%d", (long long)rows, d);
  if (rows == 0 || d == 0) return BGMOE_OK;
  BGMOE_REQUIRE(x && out, "situ_and_mul: null pointer");
  BGMOE_REQUIRE(x_row_stride >= 2 * (int64_t)d && out_row_stride >= d, "situ_and_mul: row strides smaller than the rows");
  BGMOE_REQUIRE((const void*)x != (const void*)out, "situ_and_mul: out must not alias x");
  SituArgs a{};
  a.x = x; a.out = out; a.rows = rows; a.xs = x_row_stride; a.os = out_row_stride; a.d = d;
  a.beta = beta; a.inv_beta = 1.0f / beta; a.swiglu = swiglu;
  a.has_linear = linear_beta > 0.0f;
  a.lbeta = a.has_linear ? linear_beta : 1.0f;
  a.inv_lbeta = 1.0f / a.lbeta;
  const bool vec = d % 8 == 0 && x_row_stride % 8 == 0 && out_row_stride % 8 == 0 &&
                   ((uintptr_t)x | (uintptr_t)out) % 16 == 0;
  const int64_t work = rows * (vec ? d / 8 : d);
  int64_t blocks = (work + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipStream_t st = bgmoe_stream(stream);
  BgmoeProf prof(BGMOE_K_SITU, st);
  if (vec) hipLaunchKernelGGL(situ_and_mul_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(situ_and_mul_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, st, a);
  return bgmoe_check_launch("situ_and_mul");
}
