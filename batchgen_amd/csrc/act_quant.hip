// Per-row, per-128 e4m3fn activation quantisation for gfx950: one wave64 per
// row, 16-byte loads, wave-shuffle amax, IEEE division, hardware RNE convert.
//
// One kernel serves every entry point; they differ in which rows are live
// (plain / masked by count / ragged spans / gathered through topk_pos) and in
// where a row's scales go (strides).  HBM-bound: 2 B read + 1 B written per
// element (+4 B per 128).
#include "bgmoe_common.h"

namespace {

enum RowMode { kPlain = 0, kMasked = 1, kRagged = 2, kGather = 3 };

struct QuantArgs {
  const uint16_t* x;     // gate when up != nullptr
  const uint16_t* up;    // optional: value = bf16(silu(x) * up)
  uint8_t* y;            // may be nullptr (silu_mul only)
  float* scale;
  uint16_t* h_out;       // optional bf16 copy of the value that is quantised
  int64_t jobs;          // rows (or pairs in gather mode)
  int k;
  int64_t srow, skb;
  const int32_t* counts; // masked: tokens_per_expert
  int mtp;
  const int32_t* seqlens;
  const int32_t* cu;
  int e;
  int row_align;
  int64_t max_rows;
  const int32_t* topk_pos;
  int topk;
  int64_t pairs;         // gather: jobs [0,pairs) are (token,k) pairs, jobs [pairs, jobs) copy
  int64_t extra_start;   //         token (job - pairs) to row extra_start + (job - pairs)
  int split_steps;       // 16-byte path: one wave per (row, 512 columns) instead of one wave per row
  int form_a;            // plain rows: amax floored at 2^-16, scale = max(amax * (1/448), 1e-12)
  const int32_t* num_valid;  // plain rows, optional: rows at or past *num_valid get zero bytes and scale 1e-12
};

__device__ __forceinline__ float row_scale_from_amax(const QuantArgs& a, float amax, bool pad) {
  if (!a.form_a) return quant_scale_from_amax(amax);
  constexpr float kInv448 = 1.0f / 448.0f;
  return pad ? 1e-12f : fmaxf(fmaxf(amax, 1.52587890625e-05f) * kInv448, 1e-12f);
}

// state of a destination row: 0 = leave untouched, 1 = valid, 2 = alignment pad
__device__ __forceinline__ int ragged_row_state(const QuantArgs& a, int64_t row) {
  const int64_t first = a.cu[0];
  const int64_t last = a.cu[a.e];
  if (row < first || row >= last || row >= a.max_rows) return 0;
  int lo = 0, hi = a.e - 1;
  while (lo < hi) {                 // rightmost group whose start is <= row
    const int mid = (lo + hi + 1) >> 1;
    if ((int64_t)a.cu[mid] <= row) lo = mid; else hi = mid - 1;
  }
  const int64_t rel = row - a.cu[lo];
  const int64_t valid = a.seqlens[lo];
  const int64_t span = (valid + a.row_align - 1) / a.row_align * a.row_align;
  if (rel >= span) return 0;
  return rel < valid ? 1 : 2;
}

// VEC8: the wave quantises the 512-column pieces [s_lo, s_hi) of the row.
template <bool VEC8>
__device__ __forceinline__ void quant_row(const QuantArgs& a, int64_t src, int64_t dst, bool pad, int s_lo, int s_hi) {
  const int lane = lane_id();
  const int k = a.k;
  const uint16_t* xr = a.x + src * (int64_t)k;
  const uint16_t* ur = a.up ? a.up + src * (int64_t)k : nullptr;
  uint8_t* yr = a.y ? a.y + dst * (int64_t)k : nullptr;
  uint16_t* hr = a.h_out ? a.h_out + dst * (int64_t)k : nullptr;
  float* sr = a.scale ? a.scale + dst * a.srow : nullptr;

  if constexpr (VEC8) {
    // 64 lanes x 8 elements = 4 blocks of 128 per step; 16 lanes share a block
    for (int s = s_lo; s < s_hi; ++s) {
      const int c0 = s * 512 + lane * 8;
      const bool in = c0 < k;
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = 0.0f;
      if (in && !pad) {
        const uint4 raw = *reinterpret_cast<const uint4*>(xr + c0);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[2 * i] = bf16_bits_to_f32(w[i] & 0xffffu);
          v[2 * i + 1] = bf16_bits_to_f32(w[i] >> 16);
        }
        if (ur) {
          const uint4 rawu = *reinterpret_cast<const uint4*>(ur + c0);
          const uint32_t wu[4] = {rawu.x, rawu.y, rawu.z, rawu.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            v[2 * i] = bf16_round_f32(silu_f32(v[2 * i]) * bf16_bits_to_f32(wu[i] & 0xffffu));
            v[2 * i + 1] = bf16_round_f32(silu_f32(v[2 * i + 1]) * bf16_bits_to_f32(wu[i] >> 16));
          }
          if (hr) {
            uint4 o;
            o.x = pack2_bf16(v[0], v[1]);
            o.y = pack2_bf16(v[2], v[3]);
            o.z = pack2_bf16(v[4], v[5]);
            o.w = pack2_bf16(v[6], v[7]);
            *reinterpret_cast<uint4*>(hr + c0) = o;
          }
        }
      }
      if (yr == nullptr) continue;
      float amax = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
      amax = wave_max_xor<16>(amax);
      const float sc = row_scale_from_amax(a, amax, pad);
      if (in) {
        float q[8];
        quant_div_clamp(v, sc, q);
        uint2 o;
        o.x = pack4_e4m3(q[0], q[1], q[2], q[3]);
        o.y = pack4_e4m3(q[4], q[5], q[6], q[7]);
        *reinterpret_cast<uint2*>(yr + c0) = o;
        if ((lane & 15) == 0) sr[(int64_t)(c0 >> 7) * a.skb] = sc;
      }
    }
  } else {
    // any k: one 128-block per step, two columns per lane
    const int kb = (k + 127) / 128;
    for (int b = 0; b < kb; ++b) {
      const int c0 = b * 128 + lane * 2;
      float v[2] = {0.0f, 0.0f};
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (c0 + i < k && !pad) {
          float g = bf16_bits_to_f32(xr[c0 + i]);
          if (ur) {
            g = bf16_round_f32(silu_f32(g) * bf16_bits_to_f32(ur[c0 + i]));
            if (hr) hr[c0 + i] = (uint16_t)f32_to_bf16_bits(g);
          }
          v[i] = g;
        }
      }
      if (yr == nullptr) continue;
      float amax = fmaxf(fabsf(v[0]), fabsf(v[1]));
      amax = wave_max_xor<64>(amax);
      const float sc = row_scale_from_amax(a, amax, pad);
      float q2[2];
      quant_div_clamp(v, sc, q2);
      const uint32_t p = pack4_e4m3(q2[0], q2[1], 0.0f, 0.0f);
      if (c0 < k) yr[c0] = (uint8_t)(p & 0xff);
      if (c0 + 1 < k) yr[c0 + 1] = (uint8_t)((p >> 8) & 0xff);
      if (lane == 0) sr[(int64_t)b * a.skb] = sc;
    }
  }
}

template <int MODE, bool VEC8>
__global__ __launch_bounds__(256) void act_quant_kernel(QuantArgs a) {
  const int wave = threadIdx.x >> 6;
  const int64_t stride = (int64_t)gridDim.x * 4;
  // few rows (16-byte path): one wave per (row, 512 columns), so that they still spread over the chip and no wave
  // carries a chain of dependent reductions; many rows: one wave per row, which overlaps the pieces' loads
  const int pieces = (a.k + 511) / 512;
  const int steps = VEC8 && a.split_steps ? pieces : 1;
  for (int64_t wjob = (int64_t)blockIdx.x * 4 + wave; wjob < a.jobs * steps; wjob += stride) {
    const int64_t job = wjob / steps;
    const int step = (int)(wjob - job * steps);
    int64_t src = job, dst = job;
    bool pad = false;
    if constexpr (MODE == kPlain) {
      if (a.num_valid) pad = job >= (int64_t)*a.num_valid;
    } else if constexpr (MODE == kMasked) {
      const int e = (int)(job / a.mtp);
      const int t = (int)(job - (int64_t)e * a.mtp);
      if (t >= a.counts[e]) continue;
    } else if constexpr (MODE == kRagged) {
      const int st = ragged_row_state(a, job);
      if (st == 0) continue;
      pad = st == 2;
    } else if constexpr (MODE == kGather) {
      if (job < a.pairs) {
        const int p = a.topk_pos[job];
        if (p < 0) continue;
        src = job / a.topk;
        dst = p;
      } else {
        src = job - a.pairs;
        dst = a.extra_start + src;
      }
    }
    quant_row<VEC8>(a, src, dst, pad, steps > 1 ? step : 0, steps > 1 ? step + 1 : pieces);
  }
}

// Permute + quantise: a token row is quantised ONCE and its bytes and scales are written to every row it
// is routed to (topk_pos, negative = not local) and to its identity row (extra rows: the shared expert).
// One wave per (token, 512 columns): a single 16-byte load per lane, no loop-carried latency chain.
__global__ __launch_bounds__(256) void scatter_quant_kernel(QuantArgs a, int steps, int extra_rows) {
  const int wave = threadIdx.x >> 6;
  const int lane = lane_id();
  const int k = a.k;
  const int64_t njobs = a.jobs * steps;               // a.jobs = tokens here
  const int64_t stride = (int64_t)gridDim.x * 4;
  for (int64_t job = (int64_t)blockIdx.x * 4 + wave; job < njobs; job += stride) {
    const int64_t tok = job / steps;
    const int c0 = (int)(job - tok * steps) * 512 + lane * 8;
    const bool in = c0 < k;
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = 0.0f;
    if (in) {
      const uint4 raw = *reinterpret_cast<const uint4*>(a.x + tok * (int64_t)k + c0);
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[2 * i] = bf16_bits_to_f32(w[i] & 0xffffu);
        v[2 * i + 1] = bf16_bits_to_f32(w[i] >> 16);
      }
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
    amax = wave_max_xor<16>(amax);
    const float sc = quant_scale_from_amax(amax);
    uint2 o;
    {
      float q[8];
      quant_div_clamp(v, sc, q);
      o.x = pack4_e4m3(q[0], q[1], q[2], q[3]);
      o.y = pack4_e4m3(q[4], q[5], q[6], q[7]);
    }
    const bool lead = (lane & 15) == 0;
    // all destinations of the token in one load (lane j holds destination j), not one dependent load per
    // route; only the live ones (local routes, the identity row) are visited
    int mine = -1;
    if (lane < a.topk) mine = a.topk_pos[tok * a.topk + lane];
    else if (lane == a.topk && tok < extra_rows) mine = (int)(a.extra_start + tok);
    unsigned long long live = __ballot(mine >= 0);
    while (live) {
      const int j = __ffsll((long long)live) - 1;
      live &= live - 1;
      const int64_t dst = __builtin_amdgcn_readlane(mine, j);
      if (in) {
        *reinterpret_cast<uint2*>(a.y + dst * (int64_t)k + c0) = o;
        if (lead) a.scale[dst * a.srow + (int64_t)(c0 >> 7) * a.skb] = sc;
      }
    }
  }
}

// Permute rows that are ALREADY quantised (a producer upstream wrote the bytes and scales): a token's bytes
// and scales are copied to every row it is routed to and to its identity row.  One wave per (token, 1024
// bytes = 8 scale blocks); source scale (t,kb) at xs[t*xs_row + kb*xs_kb].
__global__ __launch_bounds__(256) void scatter_fp8_kernel(const uint8_t* xq, const float* xs, int64_t xs_row,
                                                          int64_t xs_kb, QuantArgs a, int steps, int extra_rows) {
  const int wave = threadIdx.x >> 6;
  const int lane = lane_id();
  const int k = a.k;
  const int64_t njobs = a.jobs * steps;               // a.jobs = tokens here
  const int64_t stride = (int64_t)gridDim.x * 4;
  for (int64_t job = (int64_t)blockIdx.x * 4 + wave; job < njobs; job += stride) {
    const int64_t tok = job / steps;
    const int step = (int)(job - tok * steps);
    const int c0 = step * 1024 + lane * 16;
    const bool in = c0 < k;
    const int kb = step * 8 + lane;                    // lanes 0..7 carry the step's scales
    const bool has_scale = lane < 8 && kb * 128 < k;
    uint4 bytes = make_uint4(0u, 0u, 0u, 0u);
    float sc = 0.0f;
    if (in) bytes = *reinterpret_cast<const uint4*>(xq + tok * (int64_t)k + c0);
    if (has_scale) sc = xs[tok * xs_row + (int64_t)kb * xs_kb];
    int mine = -1;
    if (lane < a.topk) mine = a.topk_pos[tok * a.topk + lane];
    else if (lane == a.topk && tok < extra_rows) mine = (int)(a.extra_start + tok);
    unsigned long long live = __ballot(mine >= 0);
    while (live) {
      const int j = __ffsll((long long)live) - 1;
      live &= live - 1;
      const int64_t dst = __builtin_amdgcn_readlane(mine, j);
      if (in) *reinterpret_cast<uint4*>(a.y + dst * (int64_t)k + c0) = bytes;
      if (has_scale) a.scale[dst * a.srow + (int64_t)kb * a.skb] = sc;
    }
  }
}

constexpr int64_t kSplitBelowRows = 4097;      // up to about two rows per wave slot of the chip (measured cross-over
                                               // between 4096 and 8192 fully live rows)

template <int MODE>
int launch(const QuantArgs& a_in, hipStream_t st) {
  QuantArgs a = a_in;
  if (a.jobs <= 0 || a.k <= 0) return BGMOE_OK;
  auto aligned = [](const void* p, size_t n) { return p == nullptr || ((uintptr_t)p % n) == 0; };
  const bool vec = (a.k % 8 == 0) && aligned(a.x, 16) && aligned(a.up, 16) && aligned(a.y, 8) &&
                   aligned(a.h_out, 16);
  a.split_steps = vec && a.jobs < kSplitBelowRows;
  int64_t blocks = (a.jobs * (a.split_steps ? (a.k + 511) / 512 : 1) + 3) / 4;
  if (blocks > 16384) blocks = 16384;
  BgmoeProf prof(BGMOE_K_ACT_QUANT, st);
  if (vec)
    hipLaunchKernelGGL((act_quant_kernel<MODE, true>), dim3((unsigned)blocks), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL((act_quant_kernel<MODE, false>), dim3((unsigned)blocks), dim3(256), 0, st, a);
  return bgmoe_check_launch("act_quant");
}

}  // namespace

extern "C" int bgmoe_act_quant_rows(const uint16_t* x, int64_t rows, int k, uint8_t* y, float* scale,
                                    int64_t scale_row_stride, int64_t scale_kb_stride,
                                    bgmoe_stream_t stream) {
  BGMOE_REQUIRE(rows >= 0 && k >= 0, "act_quant_rows: negative size");
  BGMOE_REQUIRE(rows == 0 || k == 0 || (x && y && scale), "act_quant_rows: null pointer");
  QuantArgs a{};
  a.x = x; a.y = y; a.scale = scale; a.jobs = rows; a.k = k;
  a.srow = scale_row_stride; a.skb = scale_kb_stride;
  return launch<kPlain>(a, bgmoe_stream(stream));
}

extern "C" int bgmoe_act_quant_rows_1d(const uint16_t* x, int64_t rows, int k, uint8_t* y, float* scale,
                                       int64_t scale_row_stride, int64_t scale_kb_stride,
                                       const int32_t* num_valid_tokens, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(rows >= 0 && k >= 0, "act_quant_rows_1d: negative size");
  BGMOE_REQUIRE(rows == 0 || k == 0 || (x && y && scale), "act_quant_rows_1d: null pointer");
  QuantArgs a{};
  a.x = x; a.y = y; a.scale = scale; a.jobs = rows; a.k = k;
  a.srow = scale_row_stride; a.skb = scale_kb_stride;
  a.form_a = 1; a.num_valid = num_valid_tokens;
  return launch<kPlain>(a, bgmoe_stream(stream));
}

extern "C" int bgmoe_act_quant_3d(const uint16_t* x, const int32_t* tokens_per_expert, int e, int mtp,
                                  int k, uint8_t* y, float* scale, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(e >= 0 && mtp >= 0 && k >= 0, "act_quant_3d: negative size");
  if ((int64_t)e * mtp == 0 || k == 0) return BGMOE_OK;
  BGMOE_REQUIRE(x && y && scale && tokens_per_expert, "act_quant_3d: null pointer");
  QuantArgs a{};
  a.x = x; a.y = y; a.scale = scale; a.jobs = (int64_t)e * mtp; a.k = k;
  a.skb = 1; a.srow = (k + 127) / 128; a.counts = tokens_per_expert; a.mtp = mtp;
  return launch<kMasked>(a, bgmoe_stream(stream));
}

extern "C" int bgmoe_act_quant_ragged(const uint16_t* x, const int32_t* seqlens,
                                      const int32_t* cu_seqlens, int e, int64_t max_rows, int k,
                                      uint8_t* y, float* scale_t, int row_align,
                                      bgmoe_stream_t stream) {
  BGMOE_REQUIRE(e > 0, "act_quant_ragged: need at least one group");
  BGMOE_REQUIRE(row_align > 0 && (row_align & (row_align - 1)) == 0,
                "act_quant_ragged: row_align must be a positive power of two, got %d", row_align);
  BGMOE_REQUIRE(max_rows >= 0 && k >= 0, "act_quant_ragged: negative size");
  if (max_rows == 0 || k == 0) return BGMOE_OK;
  BGMOE_REQUIRE(x && y && scale_t && seqlens && cu_seqlens, "act_quant_ragged: null pointer");
  QuantArgs a{};
  a.x = x; a.y = y; a.scale = scale_t; a.jobs = max_rows; a.k = k;
  a.srow = 1; a.skb = max_rows;
  a.seqlens = seqlens; a.cu = cu_seqlens; a.e = e; a.row_align = row_align; a.max_rows = max_rows;
  return launch<kRagged>(a, bgmoe_stream(stream));
}

extern "C" int bgmoe_silu_mul_3d(const uint16_t* gate, const uint16_t* up,
                                 const int32_t* tokens_per_expert, int e, int mtp, int k,
                                 uint16_t* out, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(e >= 0 && mtp >= 0 && k >= 0, "silu_mul_3d: negative size");
  if ((int64_t)e * mtp == 0 || k == 0) return BGMOE_OK;
  BGMOE_REQUIRE(gate && up && out && tokens_per_expert, "silu_mul_3d: null pointer");
  QuantArgs a{};
  a.x = gate; a.up = up; a.h_out = out; a.jobs = (int64_t)e * mtp; a.k = k;
  a.counts = tokens_per_expert; a.mtp = mtp;
  return launch<kMasked>(a, bgmoe_stream(stream));
}

extern "C" int bgmoe_fused_silu_quant_3d(const uint16_t* gate, const uint16_t* up,
                                         const int32_t* tokens_per_expert, int e, int mtp, int k,
                                         uint8_t* y, float* scale, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(e >= 0 && mtp >= 0 && k >= 0, "fused_silu_quant_3d: negative size");
  if ((int64_t)e * mtp == 0 || k == 0) return BGMOE_OK;
  BGMOE_REQUIRE(gate && up && y && scale && tokens_per_expert, "fused_silu_quant_3d: null pointer");
  QuantArgs a{};
  a.x = gate; a.up = up; a.y = y; a.scale = scale; a.jobs = (int64_t)e * mtp; a.k = k;
  a.skb = 1; a.srow = (k + 127) / 128; a.counts = tokens_per_expert; a.mtp = mtp;
  return launch<kMasked>(a, bgmoe_stream(stream));
}

namespace {
// Copies, per expert, the first `span` columns (the live rows rounded up to span_align) of its [kb, s] scale
// block into columns [e*s, e*s + span) of the [kb, e_count*s] matrix: 16-byte units, a fixed (experts x 8) grid
// whose work shrinks with the counts.  A count outside [0, s] copies nothing and raises *status.
constexpr int kRepackThreads = 256;
constexpr int kRepackSlices = 8;
__global__ __launch_bounds__(kRepackThreads) void scale_repack_kernel(const float* __restrict__ src,
                                                                      const int32_t* __restrict__ recv_count,
                                                                      float* __restrict__ dst, int experts, int kb,
                                                                      int s, int span_align, int32_t* status) {
  const int e = blockIdx.x;
  const int rc = recv_count[e];
  if (rc < 0 || rc > s) {
    if (status && blockIdx.y == 0 && threadIdx.x == 0) atomicOr(status, 1);
    return;
  }
  const int quads = (rc + span_align - 1) / span_align * (span_align / 4);
  const float4* from = reinterpret_cast<const float4*>(src + (int64_t)e * kb * s);
  float4* to = reinterpret_cast<float4*>(dst + (int64_t)e * s);
  const int64_t to_pitch = (int64_t)experts * s / 4;
  const int from_pitch = s / 4;
  const int total = kb * quads;
  for (int i = blockIdx.y * kRepackThreads + threadIdx.x; i < total; i += kRepackSlices * kRepackThreads) {
    const int row = i / quads;
    const int q = i - row * quads;
    to[row * to_pitch + q] = from[(int64_t)row * from_pitch + q];
  }
}
}  // namespace

extern "C" int bgmoe_deepep_ll_scale_repack(const float* recv_scales, const int32_t* recv_count, float* out,
                                            int experts, int kb, int s, int span_align, int32_t* status,
                                            bgmoe_stream_t stream) {
  BGMOE_REQUIRE(experts > 0 && kb > 0 && s > 0, "deepep_ll_scale_repack: recv_scales must be non-empty (E=%d KB=%d S=%d)",
                experts, kb, s);
  BGMOE_REQUIRE((int64_t)experts * kb * s <= 0x7fffffffLL, "deepep_ll_scale_repack: recv_scales too large for int32 indexing");
  BGMOE_REQUIRE(span_align > 0 && span_align % 4 == 0 && s % span_align == 0,
                "deepep_ll_scale_repack: span_align (%d) must be a positive multiple of 4 dividing the expert stride %d",
                span_align, s);
  BGMOE_REQUIRE(recv_scales && recv_count && out, "deepep_ll_scale_repack: null pointer");
  BGMOE_REQUIRE(((uintptr_t)recv_scales | (uintptr_t)out) % 16 == 0,
                "deepep_ll_scale_repack: recv_scales and out must be 16-byte aligned");
  const uintptr_t a = (uintptr_t)recv_scales, b = (uintptr_t)out, bytes = (uintptr_t)experts * kb * s * sizeof(float);
  BGMOE_REQUIRE(a + bytes <= b || b + bytes <= a, "deepep_ll_scale_repack: recv_scales and out must not overlap");
  hipLaunchKernelGGL(scale_repack_kernel, dim3((unsigned)experts, kRepackSlices), dim3(kRepackThreads), 0,
                     bgmoe_stream(stream), recv_scales, recv_count, out, experts, kb, s, span_align, status);
  return bgmoe_check_launch("deepep_ll_scale_repack");
}

int bgmoe_internal_scatter_quant(const uint16_t* x, const int32_t* topk_pos, int n, int k, int h, uint8_t* y,
                                 float* scale, int64_t srow, int64_t skb, int extra_rows, int64_t extra_start,
                                 hipStream_t st) {
  QuantArgs a{};
  a.x = x; a.y = y; a.scale = scale; a.pairs = (int64_t)n * k; a.jobs = a.pairs + extra_rows; a.k = h;
  a.srow = srow; a.skb = skb; a.topk_pos = topk_pos; a.topk = k; a.extra_start = extra_start;
  const bool vec = h % 8 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 8 == 0 && extra_rows <= n && k < 64;
  if (!vec) return launch<kGather>(a, st);          // odd shapes: one wave per destination row
  if (n <= 0 || h <= 0) return BGMOE_OK;
  a.jobs = n;
  const int steps = (h + 511) / 512;
  int64_t blocks = ((int64_t)n * steps + 3) / 4;
  if (blocks > 65536) blocks = 65536;
  BgmoeProf prof(BGMOE_K_ACT_QUANT, st);
  hipLaunchKernelGGL(scatter_quant_kernel, dim3((unsigned)blocks), dim3(256), 0, st, a, steps, extra_rows);
  return bgmoe_check_launch("scatter_quant");
}

extern "C" int bgmoe_scatter_quant(const uint16_t* x, const int32_t* topk_pos, int n, int k, int h,
                                   uint8_t* y, float* scale, int64_t scale_row_stride,
                                   int64_t scale_kb_stride, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(n >= 0 && k > 0 && h >= 0, "scatter_quant: bad size");
  if (n == 0 || h == 0) return BGMOE_OK;
  BGMOE_REQUIRE(x && y && scale && topk_pos, "scatter_quant: null pointer");
  return bgmoe_internal_scatter_quant(x, topk_pos, n, k, h, y, scale, scale_row_stride, scale_kb_stride, 0, 0,
                                      bgmoe_stream(stream));
}

int bgmoe_internal_scatter_fp8(const uint8_t* xq, const float* xs, int64_t xs_row, int64_t xs_kb,
                               const int32_t* topk_pos, int n, int k, int h, uint8_t* y, float* scale,
                               int64_t srow, int64_t skb, int extra_rows, int64_t extra_start, hipStream_t st) {
  BGMOE_REQUIRE(h % 16 == 0 && (uintptr_t)xq % 16 == 0 && (uintptr_t)y % 16 == 0,
                "scatter_fp8_rows: h must be a multiple of 16 and the byte buffers 16-byte aligned");
  BGMOE_REQUIRE(k < 64 && extra_rows <= n, "scatter_fp8_rows: top_k must be below 64");
  if (n <= 0 || h <= 0) return BGMOE_OK;
  QuantArgs a{};
  a.y = y; a.scale = scale; a.jobs = n; a.k = h; a.srow = srow; a.skb = skb;
  a.topk_pos = topk_pos; a.topk = k; a.extra_start = extra_start;
  const int steps = (h + 1023) / 1024;
  int64_t blocks = ((int64_t)n * steps + 3) / 4;
  if (blocks > 65536) blocks = 65536;
  BgmoeProf prof(BGMOE_K_ACT_QUANT, st);
  hipLaunchKernelGGL(scatter_fp8_kernel, dim3((unsigned)blocks), dim3(256), 0, st, xq, xs, xs_row, xs_kb, a, steps,
                     extra_rows);
  return bgmoe_check_launch("scatter_fp8_rows");
}

extern "C" int bgmoe_scatter_fp8_rows(const uint8_t* xq, const float* xs, int64_t xs_row_stride,
                                      int64_t xs_kb_stride, const int32_t* topk_pos, int n, int k, int h,
                                      uint8_t* y, float* scale, int64_t scale_row_stride,
                                      int64_t scale_kb_stride, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(n >= 0 && k > 0 && h >= 0, "scatter_fp8_rows: bad size");
  if (n == 0 || h == 0) return BGMOE_OK;
  BGMOE_REQUIRE(xq && xs && y && scale && topk_pos, "scatter_fp8_rows: null pointer");
  return bgmoe_internal_scatter_fp8(xq, xs, xs_row_stride, xs_kb_stride, topk_pos, n, k, h, y, scale,
                                    scale_row_stride, scale_kb_stride, 0, 0, bgmoe_stream(stream));
}

namespace {
struct GroupQuantArgs {
  const uint16_t* gate;
  const uint16_t* up;
  int64_t ise, iss;
  const int32_t* counts;
  const int32_t* starts;
  int groups;
  int64_t max_rows;
  int n, form, split_steps;
  uint8_t* out;
  int64_t ose, oss;
  float* scale;
  int64_t sse, sss, ssg;
  uint16_t* prod;
  const float* part;     // optional: gate | up as fp32 partial-sum planes [slices][rows][2n] instead of bf16 rows
  int slices;
  int64_t part_slice_stride;
};

// 8 columns per lane and pass, 16 lanes per 128-column quantisation group.  Few rows: one wave per (group, row,
// 512 columns); many rows: one wave per (group, row).
__global__ __launch_bounds__(256) void silu_mul_group_quant_kernel(GroupQuantArgs a) {
  const int lane = lane_id();
  const int steps = a.split_steps ? (a.n + 511) / 512 : 1;
  const int64_t jobs = (int64_t)a.groups * a.max_rows * steps;
  const int64_t stride = (int64_t)gridDim.x * 4;
  for (int64_t wjob = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); wjob < jobs; wjob += stride) {
    const int64_t job = wjob / steps;
    const int step = (int)(wjob - job * steps);
    const int e = (int)(job / a.max_rows);
    const int64_t r = job - (int64_t)e * a.max_rows;
    if (a.counts && r >= a.counts[e]) continue;
    const int64_t row = (a.starts ? (int64_t)a.starts[e] : 0) + r;
    const uint16_t* gp = a.gate + e * a.ise + row * a.iss;
    const uint16_t* upp = a.up + e * a.ise + row * a.iss;
    uint8_t* op = a.out + e * a.ose + row * a.oss;
    float* sp = a.scale + e * a.sse + row * a.sss;
    const int c_end = a.split_steps ? min(a.n, (step + 1) * 512) : a.n;
    for (int c0 = step * 512 + lane * 8; c0 < c_end; c0 += 512) {
      uint32_t gw[4], uw[4];
      if (a.part != nullptr) {
        // the GEMM's K-slices are added here, in slice order, and rounded to bf16 as the GEMM's own output would be
        const float* pg = a.part + row * (2 * (int64_t)a.n) + c0;
        floatx4 sg0 = *reinterpret_cast<const floatx4*>(pg), sg1 = *reinterpret_cast<const floatx4*>(pg + 4);
        floatx4 su0 = *reinterpret_cast<const floatx4*>(pg + a.n), su1 = *reinterpret_cast<const floatx4*>(pg + a.n + 4);
        for (int sl = 1; sl < a.slices; ++sl) {
          const float* ps = pg + sl * a.part_slice_stride;
          const floatx4 g0 = *reinterpret_cast<const floatx4*>(ps), g1 = *reinterpret_cast<const floatx4*>(ps + 4);
          const floatx4 u0 = *reinterpret_cast<const floatx4*>(ps + a.n), u1 = *reinterpret_cast<const floatx4*>(ps + a.n + 4);
#pragma unroll
          for (int j = 0; j < 4; ++j) { sg0[j] += g0[j]; sg1[j] += g1[j]; su0[j] += u0[j]; su1[j] += u1[j]; }
        }
        gw[0] = pack2_bf16(sg0[0], sg0[1]); gw[1] = pack2_bf16(sg0[2], sg0[3]);
        gw[2] = pack2_bf16(sg1[0], sg1[1]); gw[3] = pack2_bf16(sg1[2], sg1[3]);
        uw[0] = pack2_bf16(su0[0], su0[1]); uw[1] = pack2_bf16(su0[2], su0[3]);
        uw[2] = pack2_bf16(su1[0], su1[1]); uw[3] = pack2_bf16(su1[2], su1[3]);
      } else {
        const uint4 gv = *reinterpret_cast<const uint4*>(gp + c0);
        const uint4 uv = *reinterpret_cast<const uint4*>(upp + c0);
        gw[0] = gv.x; gw[1] = gv.y; gw[2] = gv.z; gw[3] = gv.w;
        uw[0] = uv.x; uw[1] = uv.y; uw[2] = uv.z; uw[3] = uv.w;
      }
      float p[8];
      uint32_t pw[4];
      float sv[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float gi = (i & 1) ? __uint_as_float(gw[i >> 1] & 0xffff0000u) : __uint_as_float(gw[i >> 1] << 16);
        bool decided;
        sv[i] = silu_short_f32(gi, &decided);
        if (__any(!decided)) {                 // rare: one exact evaluation for the lanes that need it
          if (!decided) sv[i] = silu_exact_f32(gi);
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t sw = pack2_bf16(sv[2 * j], sv[2 * j + 1]);
        pw[j] = pack2_bf16(__uint_as_float(sw << 16) * __uint_as_float(uw[j] << 16),
                           __uint_as_float(sw & 0xffff0000u) * __uint_as_float(uw[j] & 0xffff0000u));
        p[2 * j] = __uint_as_float(pw[j] << 16);
        p[2 * j + 1] = __uint_as_float(pw[j] & 0xffff0000u);
      }
      if (a.prod)
        *reinterpret_cast<uint4*>(a.prod + e * a.ose + row * a.oss + c0) = make_uint4(pw[0], pw[1], pw[2], pw[3]);
      float amax = fabsf(p[0]);
#pragma unroll
      for (int i = 1; i < 8; ++i) amax = fmaxf(amax, fabsf(p[i]));
      amax = wave_max_xor<16>(amax);
      float sc, q[8];
      if (a.form == 1) {
        sc = fmaxf(amax, 1e-10f) / 448.0f;
        quant_div_clamp(p, sc, q);
      } else {
        constexpr float kInv448 = static_cast<float>(1.0 / 448.0);
        sc = fmaxf(fmaxf(amax, 1.52587890625e-05f) * kInv448, 1e-12f);
        quant_div_clamp(p, sc, q);
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = fabsf(q[i]) < 1e30f ? q[i] : 0.0f;
      }
      *reinterpret_cast<uint2*>(op + c0) = make_uint2(pack4_e4m3(q[0], q[1], q[2], q[3]), pack4_e4m3(q[4], q[5], q[6], q[7]));
      if ((lane & 15) == 0) sp[(int64_t)(c0 >> 7) * a.ssg] = sc;
    }
  }
}
}  // namespace

extern "C" int bgmoe_silu_mul_group_quant(const uint16_t* gate, const uint16_t* up, int64_t in_stride_e,
                                          int64_t in_stride_s, const int32_t* counts, const int32_t* starts,
                                          int groups, int64_t max_rows, int n, int form, uint8_t* out,
                                          int64_t out_stride_e, int64_t out_stride_s, float* scale,
                                          int64_t scale_stride_e, int64_t scale_stride_s, int64_t scale_stride_g,
                                          uint16_t* prod_out, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(groups >= 0 && max_rows >= 0, "silu_mul_group_quant: negative size");
  BGMOE_REQUIRE(n > 0 && n % 128 == 0, "silu_mul_group_quant: width %d must be a positive multiple of the quant group 128", n);
  BGMOE_REQUIRE(form == 0 || form == 1, "silu_mul_group_quant: form must be 0 (1-D quantiser) or 1 (amax / 448)");
  if (groups == 0 || max_rows == 0) return BGMOE_OK;
  BGMOE_REQUIRE(gate && up && out && scale, "silu_mul_group_quant: null pointer");
  BGMOE_REQUIRE(((uintptr_t)gate | (uintptr_t)up | (uintptr_t)prod_out) % 16 == 0 && (uintptr_t)out % 8 == 0 &&
                    in_stride_e % 8 == 0 && in_stride_s % 8 == 0 && out_stride_e % 8 == 0 && out_stride_s % 8 == 0,
                "silu_mul_group_quant: rows must be 16-byte aligned (strides multiples of 8 elements)");
  BGMOE_REQUIRE(in_stride_s >= n && out_stride_s >= n, "silu_mul_group_quant: row strides smaller than the rows");
  GroupQuantArgs a{};
  a.gate = gate; a.up = up; a.ise = in_stride_e; a.iss = in_stride_s; a.counts = counts; a.starts = starts;
  a.groups = groups; a.max_rows = max_rows; a.n = n; a.form = form; a.out = out; a.ose = out_stride_e;
  a.oss = out_stride_s; a.scale = scale; a.sse = scale_stride_e; a.sss = scale_stride_s; a.ssg = scale_stride_g;
  a.prod = prod_out;
  a.split_steps = (int64_t)groups * max_rows < kSplitBelowRows;
  int64_t blocks = ((int64_t)groups * max_rows * (a.split_steps ? (n + 511) / 512 : 1) + 3) / 4;
  if (blocks > 16384) blocks = 16384;
  hipStream_t st = bgmoe_stream(stream);
  BgmoeProf prof(BGMOE_K_ACT_QUANT, st);
  hipLaunchKernelGGL(silu_mul_group_quant_kernel, dim3((unsigned)blocks), dim3(256), 0, st, a);
  return bgmoe_check_launch("silu_mul_group_quant");
}

extern "C" int bgmoe_silu_mul_group_quant_partials(const float* partials, int slices, int64_t slice_stride,
                                                   int64_t rows, int n, int form, uint8_t* out, int64_t out_stride_s,
                                                   float* scale, int64_t scale_stride_s, int64_t scale_stride_g,
                                                   bgmoe_stream_t stream) {
  BGMOE_REQUIRE(rows >= 0 && slices >= 1, "silu_mul_group_quant_partials: bad sizes rows=%lld slices=%d", (long long)rows,
                slices);
  BGMOE_REQUIRE(n > 0 && n % 128 == 0, "silu_mul_group_quant_partials: width %d must be a positive multiple of 128", n);
  BGMOE_REQUIRE(form == 0 || form == 1, "silu_mul_group_quant_partials: form must be 0 or 1");
  if (rows == 0) return BGMOE_OK;
  BGMOE_REQUIRE(partials && out && scale, "silu_mul_group_quant_partials: null pointer");
  BGMOE_REQUIRE((uintptr_t)partials % 16 == 0 && slice_stride % 4 == 0 && (uintptr_t)out % 8 == 0 && out_stride_s % 8 == 0 &&
                    out_stride_s >= n,
                "silu_mul_group_quant_partials: misaligned buffers or row stride smaller than the row");
  GroupQuantArgs a{};
  a.groups = 1; a.max_rows = rows; a.n = n; a.form = form; a.out = out; a.oss = out_stride_s;
  a.scale = scale; a.sss = scale_stride_s; a.ssg = scale_stride_g;
  a.part = partials; a.slices = slices; a.part_slice_stride = slice_stride;
  a.split_steps = rows < kSplitBelowRows;
  int64_t blocks = (rows * (a.split_steps ? (n + 511) / 512 : 1) + 3) / 4;
  if (blocks > 16384) blocks = 16384;
  hipStream_t st = bgmoe_stream(stream);
  BgmoeProf prof(BGMOE_K_ACT_QUANT, st);
  hipLaunchKernelGGL(silu_mul_group_quant_kernel, dim3((unsigned)blocks), dim3(256), 0, st, a);
  return bgmoe_check_launch("silu_mul_group_quant_partials");
}

namespace {
__device__ __forceinline__ uint32_t mix32(uint64_t v) {
  v ^= v >> 33; v *= 0xff51afd7ed558ccdULL; v ^= v >> 33; v *= 0xc4ceb9fe1a85ec53ULL; v ^= v >> 33;
  return (uint32_t)v;
}
// Pseudo-random (s, x) pairs from the quantisers' domain: s anywhere in (1e-30, 1e30), |x| <= 448.5 * s, x
// either a full fp32 value or rounded down to bf16 (what the quantisers are fed).  Counts the pairs whose
// short division differs from the IEEE one in the e4m3 byte, and in any bit of a normal-range quotient.
__global__ __launch_bounds__(256) void scale_division_selfcheck_kernel(uint64_t seed, uint64_t count,
                                                                       unsigned long long* byte_mismatches,
                                                                       unsigned long long* bit_mismatches) {
  unsigned long long bad_byte = 0, bad_bits = 0;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (uint64_t)gridDim.x * blockDim.x) {
    const uint32_t h0 = mix32(seed + 2 * i), h1 = mix32(seed + 2 * i + 1);
    const int ex = 28 + (int)(h0 >> 23) % 199;                               // biased exponent 28 .. 226
    const float s = __uint_as_float(((uint32_t)ex << 23) | (h0 & 0x7fffffu));
    if (!scale_div_ok(s)) continue;
    const float t = (float)(h1 >> 8) * (1.0f / 16777216.0f) * 448.5f;        // [0, 448.5)
    float x = t * s;
    if (h1 & 1u) x = __uint_as_float(__float_as_uint(x) & 0xffff0000u);      // a bf16 value
    if (h1 & 2u) x = -x;
    if ((h1 & 0xfcu) == 0) x = (h1 & 2u) ? -0.0f : 0.0f;                     // signed zeros now and then
    const float r = 1.0f / s;
    const float a = div_by_scale(x, s, r), b = x / s;
    const uint32_t pa = pack4_e4m3(clamp448(a), 0.0f, 0.0f, 0.0f) & 0xffu;
    const uint32_t pb = pack4_e4m3(clamp448(b), 0.0f, 0.0f, 0.0f) & 0xffu;
    bad_byte += pa != pb;
    bad_bits += fabsf(b) >= 1.17549435e-38f && __float_as_uint(a) != __float_as_uint(b);
  }
  for (int off = 32; off > 0; off >>= 1) {
    bad_byte += __shfl_xor(bad_byte, off, BGMOE_WAVE);
    bad_bits += __shfl_xor(bad_bits, off, BGMOE_WAVE);
  }
  if (lane_id() == 0) {
    if (bad_byte) atomicAdd(byte_mismatches, bad_byte);
    if (bad_bits) atomicAdd(bit_mismatches, bad_bits);
  }
}
}  // namespace

extern "C" int bgmoe_selfcheck_scale_division(uint64_t seed, uint64_t count, uint64_t* byte_mismatches,
                                              uint64_t* bit_mismatches, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(byte_mismatches && bit_mismatches, "selfcheck_scale_division: null counter");
  if (count == 0) return BGMOE_OK;
  uint64_t blocks = (count + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL(scale_division_selfcheck_kernel, dim3((unsigned)blocks), dim3(256), 0, bgmoe_stream(stream), seed,
                     count, reinterpret_cast<unsigned long long*>(byte_mismatches),
                     reinterpret_cast<unsigned long long*>(bit_mismatches));
  return bgmoe_check_launch("selfcheck_scale_division");
}
