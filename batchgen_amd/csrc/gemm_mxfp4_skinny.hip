// W4A16 grouped GEMM for MXFP4 weights (e2m1 values, one e8m0 scale per 32 along K) and bf16
// activations: a weight-streaming kernel bound by HBM bandwidth (decode).
//
// Same work split and scheduling as the FP8 weight-streaming kernel: item = (group, 64-token chunk,
// 128 gate + 128 up columns | 256 columns), 4 waves x four 16-row weight tiles, register prefetch,
// tokens shared through an LDS ring, persistent grid.
// Weights are dequantised IN REGISTERS: one lane's 16-byte load is one row's 32-value scale group;
// v_cvt_scalef32_pk_bf16_fp4 turns a byte (low nibble = even K) into two bf16 already multiplied by
// 2^(scale-127), exactly (a power-of-two times a 2-bit-mantissa value), so the MFMA consumes the
// same bf16 weights as "dequantise, then bf16 x bf16 -> fp32 GEMM".  MFMA: v_mfma_f32_16x16x32_bf16,
// weight tile as A, token tile as B; 4 MFMAs per 128-K block.  K permutation (same on both
// operands): in step s of a block, lane group q = lane/16 covers k = 32q + 8s .. 32q + 8s + 7.
//
// Layouts (bgmoe_mxfp4_weight.layout): ROW_MAJOR = checkpoint layout, packed [n, k/2] bytes and
// scales [n, k/32] bytes; TILE_MAJOR = per (16 rows, 128 K) tile 1024 packed bytes in lane order
// (lane l = q*16 + r holds row r, bytes 16q..16q+15 of the row's 64-byte segment) and 64 scale bytes
// [r][4] -- one contiguous 1 KiB load per wave and tile.
//
// Algorithmic bytes per group and matrix: n*k/2 + n*k/32.
#include <stdlib.h>

#include "bgmoe_common.h"
#include "bgmoe_sched.h"
#include "bgmoe_async.h"

namespace {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

struct Mx4Args {
  const uint16_t* x;            // [m, k] bf16; with row_pair: [tokens, k], row r of a group's range reads token
                                // row_pair[r] / pair_div
  const int32_t* row_pair;      // optional [m]: the (token, slot) pair placed in each live row (pair = token * top_k + slot)
  int pair_div;                 // top_k
  uint32_t last_token;          // tokens - 1: a row's token index is clamped to it (no entry of the map can make a lane
                                // read outside the token matrix)
  bgmoe_mxfp4_weight w0, w1;
  const int32_t* seqlens;
  const int32_t* cu;
  int groups, n, k;
  uint16_t* out;                // [m, n] bf16, row r of the activation buffer -> row r
  uint16_t* const* out_ptrs;    // or: per-group output base (row = token index inside the group)
  int lo, hi;
  int64_t row_bound;
  int activation;               // fused stage 1: BGMOE_ACT_SWIGLU or BGMOE_ACT_SITU
};

struct Mx4Stage {
  intx4 A[4];                   // packed fp4: one 32-value scale group per lane and tile
  uint32_t S[4];                // the row's four scale bytes of this 128-K block
};

__device__ __forceinline__ bf16x8 dequant8(uint32_t w, float scale) {
  const bf16x2_t v0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 0);
  const bf16x2_t v1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 1);
  const bf16x2_t v2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 2);
  const bf16x2_t v3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 3);
  return bf16x8{v0[0], v0[1], v1[0], v1[1], v2[0], v2[1], v3[0], v3[1]};
}

// One work item: up to 16*TT rows of one group x one n-tile, streamed over K.  Weights go from HBM
// straight into registers; the item's bf16 tokens (4x the bytes of the fp4 weights they meet) are shared by
// the four waves through an LDS ring filled by asynchronous global -> LDS loads.  A token tile is 16 rows x
// 256 bytes per K-block; a load covers 4 rows: lane p = (row p>>4, LDS chunk p&15) fetches the row's 16-byte
// chunk (p&15) ^ row, so that the MFMA operand reads (16 rows, same chunk) hit 16 different bank groups.
// KEEP: the group has more row chunks than this one, so its weights are loaded with the default cache
// policy (the next chunk finds them in L2); otherwise as a non-temporal stream.
template <int TT, int NSTAGE, bool FUSED, int LAYOUT, bool KEEP, int NT, bool MAPPED = false>
__device__ __forceinline__ void mxfp4_item(const Mx4Args& g, const BgmoeItem& it, const uint8_t* ring, uint32_t ring_lds) {
  constexpr int NH = NT / 2;                      // fused: gate tiles (= up tiles) per wave
  constexpr int NW = FUSED ? 16 * NH : 16 * NT;   // output columns per wave
  constexpr int kSlot = TT * 4096;
  const int grp = it.grp, cnt = it.cnt;
  const int64_t row0 = g.cu[grp];
  const int wave = threadIdx.x >> 6;
  const uint32_t wave_u = __builtin_amdgcn_readfirstlane((uint32_t)wave);
  const int lane = threadIdx.x & 63;
  const int r16 = lane & 15;
  const int kq = lane >> 4;
  const int K = g.k;
  const int KB = K >> 7;
  const int n0 = it.ntile * (4 * NW);

  const uint8_t* wb[2];
  const uint8_t* sb[2];
  wb[0] = g.w0.w_ptrs ? g.w0.w_ptrs[grp] : g.w0.w + (int64_t)grp * g.w0.w_group_stride;
  sb[0] = g.w0.scale_ptrs ? g.w0.scale_ptrs[grp] : g.w0.scale + (int64_t)grp * g.w0.scale_group_stride;
  if constexpr (FUSED) {
    wb[1] = g.w1.w_ptrs ? g.w1.w_ptrs[grp] : g.w1.w + (int64_t)grp * g.w1.w_group_stride;
    sb[1] = g.w1.scale_ptrs ? g.w1.scale_ptrs[grp] : g.w1.scale + (int64_t)grp * g.w1.scale_group_stride;
  }
  const uint8_t* wp[NT];
  const uint8_t* sp[NT];
  bool tv[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int nrow = FUSED ? n0 + NW * wave + 16 * (t % NH) : n0 + NW * wave + 16 * t;
    tv[t] = nrow < g.n;
    const int nr = min(nrow, g.n - 16);
    const int mi = FUSED ? (t / NH) : 0;
    if constexpr (LAYOUT == BGMOE_W_ROW_MAJOR) {
      wp[t] = wb[mi] + (int64_t)(nr + r16) * (K >> 1) + 16 * kq;
      sp[t] = sb[mi] + (int64_t)(nr + r16) * (K >> 5);
    } else {
      wp[t] = wb[mi] + (int64_t)(nr >> 4) * KB * 1024 + lane * 16;
      sp[t] = sb[mi] + (int64_t)(nr >> 4) * KB * 64 + r16 * 4;
    }
  }

  const int t0 = it.chunk * 16 * TT;
  const int live = cnt - t0;
  const int tiles = min(TT, (live + 15) >> 4);
  uint16_t* const obase = g.out_ptrs ? g.out_ptrs[grp] : g.out + row0 * g.n;

  // tokens: wave w loads quarter-tiles w*TT .. w*TT+TT-1 (4 rows x 256 bytes each)
  // With a row -> pair map the rows are read where the tokens lie (no gathered copy of them exists): the base is
  // the token matrix and a lane's offset is its row's token times the row pitch (the host checks that the whole
  // token matrix is addressable with 32-bit offsets).  Rows past the count repeat the last live row, as without.
  const uint8_t* tok_base = uniform_ptr(reinterpret_cast<const uint8_t*>(MAPPED ? g.x : g.x + (row0 + t0) * K));
  uint32_t tok_off[TT];
  bool tok_on[TT];
#pragma unroll
  for (int i = 0; i < TT; ++i) {
    const int qt = (int)wave_u * TT + i;                  // quarter-tile 0 .. 4*TT-1
    const int rt = 4 * (qt & 3) + (lane >> 4);            // row inside its tile
    const int row = min(16 * (qt >> 2) + rt, live - 1);
    uint32_t src = (uint32_t)row;
    if constexpr (MAPPED) src = min((uint32_t)g.row_pair[row0 + t0 + row] / (uint32_t)g.pair_div, g.last_token);
    tok_off[i] = src * (uint32_t)(2 * K) + (uint32_t)((((lane & 15) ^ rt) & 15) * 16);
    tok_on[i] = (qt >> 2) < tiles;
  }
  auto issue_tokens = [&](int kb, int slot) {
    const uint32_t sbs = ring_lds + (uint32_t)slot * kSlot;
#pragma unroll
    for (int i = 0; i < TT; ++i)
      if (tok_on[i]) async_load16(tok_base + (kb << 8), tok_off[i], sbs + (wave_u * TT + i) * 1024);
  };

  floatx4 acc[TT][NT];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[tt][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  Mx4Stage st[NSTAGE];
  auto load_stage = [&](Mx4Stage& s, int kb) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if constexpr (LAYOUT == BGMOE_W_ROW_MAJOR) {
        s.A[t] = KEEP ? gload_x4(wp[t] + (kb << 6)) : gload_x4_stream(wp[t] + (kb << 6));
        s.S[t] = gload_u32(sp[t] + (kb << 2));
      } else {
        s.A[t] = KEEP ? gload_x4(wp[t] + ((int64_t)kb << 10)) : gload_x4_stream(wp[t] + ((int64_t)kb << 10));
        s.S[t] = gload_u32(sp[t] + (kb << 6));
      }
    }
  };
  auto compute = [&](const Mx4Stage& c, int slot) {
    const uint8_t* b = ring + slot * kSlot + r16 * 256;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int boff = (((4 * kq + j) ^ r16) & 15) * 16;
      bf16x8 a[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const float sc = __uint_as_float(((c.S[t] >> (8 * kq)) & 0xffu) << 23);    // 2^(e8m0 - 127)
        a[t] = dequant8((uint32_t)c.A[t][j], sc);
      }
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        if (tt < tiles) {
          const bf16x8 bv = __builtin_bit_cast(bf16x8, *reinterpret_cast<const intx4*>(b + tt * 4096 + boff));
#pragma unroll
          for (int t = 0; t < NT; ++t) acc[tt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t], bv, acc[tt][t], 0, 0, 0);
        }
      }
    }
  };

  // Same pipeline as the FP8 streaming kernel: tokens are requested before the weights of the same
  // K-block, loads complete in issue order, so "at most the 2*NT weight loads of the youngest stage
  // outstanding" means the stage about to be computed has landed for this wave; the barrier extends
  // that to the other waves' token loads and frees the slot refilled next.
  // With more than three stages several younger stages are in flight at the wait: each of them has at least its
  // 2*NT weight loads outstanding (token loads of dead tiles are skipped, so they cannot be counted on), and so has
  // the stage about to be computed, whose weight loads follow its token loads: "at most 2*NT*(NSTAGE-1)
  // outstanding" is then what says that this stage's tokens have landed (its weights are the compiler's own loads
  // and waited for by the compiler).
  constexpr int kWaitLoads = NSTAGE <= 3 ? 2 * NT : 2 * NT * (NSTAGE - 1);
  static_assert(kWaitLoads <= 63, "s_waitcnt vmcnt holds six bits");
#pragma unroll
  for (int s = 0; s < NSTAGE - 1; ++s) {
    issue_tokens(min(s, KB - 1), s);
    load_stage(st[s], min(s, KB - 1));
  }
  const int kb_main = KB - KB % NSTAGE;
  for (int kb0 = 0; kb0 < kb_main; kb0 += NSTAGE) {
#pragma unroll
    for (int s = 0; s < NSTAGE; ++s) {
      wait_vm<kWaitLoads>();
      block_barrier();
      issue_tokens(min(kb0 + s + NSTAGE - 1, KB - 1), (s + NSTAGE - 1) % NSTAGE);
      load_stage(st[(s + NSTAGE - 1) % NSTAGE], min(kb0 + s + NSTAGE - 1, KB - 1));
      compute(st[s], s);
    }
  }
  wait_vm<0>();           // the tail needs everything; no asynchronous write may outlive the item
  block_barrier();
#pragma unroll
  for (int s = 0; s < NSTAGE - 1; ++s)
    if (kb_main + s < KB) compute(st[s], s);

#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
    const int tok = t0 + 16 * tt + r16;
    if (16 * tt + r16 >= live) continue;
    if constexpr (FUSED) {
#pragma unroll
      for (int j = 0; j < NH; ++j) {
        float h[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (g.activation == BGMOE_ACT_SITU) {
            // both branches are rounded to bf16 first (marlin_grouped_gemm.cu:1055-1069); beta 4, linear beta 25
            const float gg = bf16_round_f32(acc[tt][j][i]), uu = bf16_round_f32(acc[tt][j + NH][i]);
            h[i] = situ_gate_f32(gg, 4.0f, 0.25f) * situ_linear_f32(uu, 25.0f, 0.04f);
          } else {
            h[i] = silu_f32(acc[tt][j][i]) * acc[tt][j + NH][i];
          }
        }
        uint2 o;
        o.x = pack2_bf16(h[0], h[1]);
        o.y = pack2_bf16(h[2], h[3]);
        gstore_x2(obase + (int64_t)tok * g.n + n0 + NW * wave + 16 * j + 4 * kq, o);
      }
    } else {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        if (!tv[t]) continue;
        uint2 o;
        o.x = pack2_bf16(acc[tt][t][0], acc[tt][t][1]);
        o.y = pack2_bf16(acc[tt][t][2], acc[tt][t][3]);
        gstore_x2(obase + (int64_t)tok * g.n + n0 + NW * wave + 16 * t + 4 * kq, o);
      }
    }
  }
}

// Persistent grid: block b works on virtual blocks b, b + gridDim.x, ... until the item list ends.
// Item width is chosen per launch on the device: with 4 weight tiles per wave (128 fused / 256 plain output
// columns per item) when that already gives every resident block an item, else with 2 tiles per wave --
// fp4 weight stages are small, so with few items twice as many narrower ones keep more loads in flight.
// TALL > 0 (mixed item heights): groups with more than 16 * TT rows are cut into items of 16 * TALL rows with
// kMxTallStages prefetch stages, all others into items of 16 * TT rows with NSTAGE stages -- a small group gets the
// deep pipeline, a larger one is still streamed once per 16 * TALL rows.  Every output element is computed by the
// same chain of operations whatever the item height.
constexpr int kMxTallStages = 3;
template <int TT, int NSTAGE, bool FUSED, int LAYOUT, bool MAPPED, int NT, int TALL>
__device__ __forceinline__ void mxfp4_run_item(const Mx4Args& g, const BgmoeItem& it, const uint8_t* ring, uint32_t ring_lds) {
  if constexpr (TALL > 0) {
    if (it.rows != 16 * TT) {               // wave-uniform: a tall group's item
      if (it.cnt > 16 * TALL) mxfp4_item<TALL, kMxTallStages, FUSED, LAYOUT, true, NT, MAPPED>(g, it, ring, ring_lds);
      else mxfp4_item<TALL, kMxTallStages, FUSED, LAYOUT, false, NT, MAPPED>(g, it, ring, ring_lds);
      return;
    }
  }
  if (it.cnt > 16 * TT) mxfp4_item<TT, NSTAGE, FUSED, LAYOUT, true, NT, MAPPED>(g, it, ring, ring_lds);
  else mxfp4_item<TT, NSTAGE, FUSED, LAYOUT, false, NT, MAPPED>(g, it, ring, ring_lds);
}

template <int TT, int NSTAGE, bool FUSED, int LAYOUT, bool MAPPED = false, int TALL = 0>
__global__ __launch_bounds__(256) void mxfp4_skinny_kernel(Mx4Args g, unsigned vblocks, unsigned slots) {
  constexpr int kRingShort = NSTAGE * TT * 4096;
  constexpr int kRingTall = TALL > 0 ? kMxTallStages * TALL * 4096 : 0;
  __shared__ __align__(16) uint8_t s_ring[kRingShort > kRingTall ? kRingShort : kRingTall];
  const uint32_t ring_lds = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)s_ring);
  const int wide_cols = FUSED ? 128 : 256;
  const int ntiles_wide = (g.n + wide_cols - 1) / wide_cols;
  const BgmoeTall tall{TALL > 0 ? 16 * TT : 0, 16 * TALL};      // tall above one short item's rows
  const int chunks = bgmoe_total_chunks(g.seqlens, g.groups, g.lo, g.hi, 16 * TT, tall);
  const bool narrow = (int64_t)chunks * ((ntiles_wide + 7) & ~7) < (int64_t)slots;   // slots: blocks resident at once
  if (narrow) {
    const int ntiles = (g.n + wide_cols / 2 - 1) / (wide_cols / 2);
    for (unsigned vb = blockIdx.x; vb < vblocks; vb += gridDim.x) {
      const BgmoeItem it = bgmoe_decode_item(g.seqlens, g.groups, g.lo, g.hi, 16 * TT, ntiles, vb, tall);
      if (it.grp == BGMOE_ITEM_END) break;
      if (it.grp == BGMOE_ITEM_PAD) continue;
      if constexpr (TALL > 0) {
        mxfp4_run_item<TT, NSTAGE, FUSED, LAYOUT, MAPPED, 2, TALL>(g, it, s_ring, ring_lds);
      } else {
        if (it.cnt > 16 * TT) mxfp4_item<TT, NSTAGE, FUSED, LAYOUT, true, 2, MAPPED>(g, it, s_ring, ring_lds);
        else mxfp4_item<TT, NSTAGE, FUSED, LAYOUT, false, 2, MAPPED>(g, it, s_ring, ring_lds);
      }
      __syncthreads();                    // the token ring is reused by the next item
    }
  } else {
    for (unsigned vb = blockIdx.x; vb < vblocks; vb += gridDim.x) {
      const BgmoeItem it = bgmoe_decode_item(g.seqlens, g.groups, g.lo, g.hi, 16 * TT, ntiles_wide, vb, tall);
      if (it.grp == BGMOE_ITEM_END) break;
      if (it.grp == BGMOE_ITEM_PAD) continue;
      if constexpr (TALL > 0) {
        mxfp4_run_item<TT, NSTAGE, FUSED, LAYOUT, MAPPED, 4, TALL>(g, it, s_ring, ring_lds);
      } else {
        if (it.cnt > 16 * TT) mxfp4_item<TT, NSTAGE, FUSED, LAYOUT, true, 4, MAPPED>(g, it, s_ring, ring_lds);
        else mxfp4_item<TT, NSTAGE, FUSED, LAYOUT, false, 4, MAPPED>(g, it, s_ring, ring_lds);
      }
      __syncthreads();
    }
  }
}

// row-major -> tile-major for packed values (16-byte chunks) and scales (4-byte chunks)
__global__ __launch_bounds__(256) void mxfp4_repack_kernel(const uint8_t* __restrict__ w, const uint8_t* __restrict__ s,
                                                           uint8_t* __restrict__ wo, uint8_t* __restrict__ so,
                                                           int64_t chunks, int n, int k) {
  const int kb_n = k >> 7;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < chunks; c += stride) {
    const int lane = (int)(c & 63);
    const int64_t tile = c >> 6;                       // (group*n/16 + nt) * kb_n + kb
    const int kb = (int)(tile % kb_n);
    const int64_t nt_all = tile / kb_n;
    const int r = lane & 15, q = lane >> 4;
    const int64_t row = nt_all * 16 + r;
    *reinterpret_cast<uint4*>(wo + c * 16) = *reinterpret_cast<const uint4*>(w + row * (k >> 1) + kb * 64 + 16 * q);
    if (q == 0)
      *reinterpret_cast<uint32_t*>(so + (tile * 16 + r) * 4) = *reinterpret_cast<const uint32_t*>(s + row * (k >> 5) + kb * 4);
  }
}

int check_w(const char* what, const bgmoe_mxfp4_weight* w) {
  BGMOE_REQUIRE(w != nullptr, "%s: null weight descriptor", what);
  BGMOE_REQUIRE((w->w || w->w_ptrs) && (w->scale || w->scale_ptrs), "%s: null weight", what);
  BGMOE_REQUIRE(w->layout == BGMOE_W_ROW_MAJOR || w->layout == BGMOE_W_TILE_MAJOR, "%s: unknown weight layout %d", what, w->layout);
  BGMOE_REQUIRE(w->w_ptrs || ((uintptr_t)w->w % 16 == 0 && w->w_group_stride % 16 == 0), "%s: packed weights must be 16-byte aligned", what);
  BGMOE_REQUIRE(w->scale_ptrs || ((uintptr_t)w->scale % 4 == 0 && w->scale_group_stride % 4 == 0), "%s: scales must be 4-byte aligned", what);
  return BGMOE_OK;
}

// blocks resident on the whole device at once, a multiple of 8 (queried once per kernel)
template <int TT, int NS, bool FUSED, int LAYOUT, bool MAPPED = false, int TALL = 0>
unsigned mx_resident() {
  static unsigned resident = 0;
  if (resident == 0) {
    int per_cu = 0, dev = 0, cus = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, mxfp4_skinny_kernel<TT, NS, FUSED, LAYOUT, MAPPED, TALL>, 256, 0) != hipSuccess || per_cu < 1)
      per_cu = 1;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1)
      cus = 256;
    resident = (unsigned)(per_cu * cus) & ~7u;
    if (resident == 0) resident = 8;
  }
  return resident;
}

template <int TT, int NS, bool FUSED, int LAYOUT, bool MAPPED = false, int TALL = 0>
void launch_one(unsigned vblocks, const Mx4Args& g, hipStream_t st) {
  // Twice as many blocks as fit at once: with up to two rounds of items every block has one item and the
  // hardware hands the second round out as blocks finish, which evens out items of unequal length (a 64-row
  // item takes 1.7x a 16-row one); beyond that the blocks stride.  Measured: skewed counts 14% faster,
  // uniform ones 3% slower (the late blocks' start-up).
  const unsigned slots = mx_resident<TT, NS, FUSED, LAYOUT, MAPPED, TALL>();
  const dim3 grid(vblocks < 2 * slots ? vblocks : 2 * slots), block(256);
  hipLaunchKernelGGL((mxfp4_skinny_kernel<TT, NS, FUSED, LAYOUT, MAPPED, TALL>), grid, block, 0, st, g, vblocks,
                     vblocks < slots ? vblocks : slots);
}

constexpr int kMxTT = 4;           // 64-row items: every group is streamed once per 64 rows
// The opt-in variant: 32-row items with six prefetch stages.  fp4 weight stages are small (4 KB per wave and K-block
// against 8 KB of the FP8 kernel), so three stages keep 8 KB per wave in flight; the accumulators of the other 32 rows
// pay for three more stages (20 KB in flight per wave) at the same two blocks per CU and the same 48 KB token ring.
// bf16 token rows weigh four times their weights, so a 32-row item is also the better-balanced unit.
constexpr int kMxTT2 = 2, kMxNS2 = 6;
// Mixed item heights (variant 2): the 64-row items' 64 accumulators and the 32-row items' prefetch stages share one
// register budget, which leaves the 32-row items five stages at two blocks per CU.
constexpr int kMxNSMixed = 5;
// The default item height with one more stage (variant 3): 64-row items keep every group of up to 64 rows a single pass
// over its weights; the fourth stage costs 20 registers (171 + 64) and a 64 KB token ring, still two blocks per CU.
constexpr int kMxNSDeep = 4;
int g_mx_variant = 0;

template <int TT, int NS, int TALL = 0>
void launch_shape(bool fused, bool tm, unsigned vblocks, const Mx4Args& g, hipStream_t st) {
  if (fused && g.row_pair != nullptr) {                  // stage 1 reading its rows through the row -> pair map
    if (tm) launch_one<TT, NS, true, 1, true, TALL>(vblocks, g, st);
    else launch_one<TT, NS, true, 0, true, TALL>(vblocks, g, st);
  } else if (fused) {
    if (tm) launch_one<TT, NS, true, 1, false, TALL>(vblocks, g, st);
    else launch_one<TT, NS, true, 0, false, TALL>(vblocks, g, st);
  } else {
    if (tm) launch_one<TT, NS, false, 1, false, TALL>(vblocks, g, st);
    else launch_one<TT, NS, false, 0, false, TALL>(vblocks, g, st);
  }
}

int launch(bool fused, Mx4Args& g, int64_t m, hipStream_t st) {
  const int tt = g_mx_variant >= 1 ? kMxTT2 : kMxTT;      // (tall items only lower the item count: the same bound holds)
  const int ntile = fused ? 64 : 128;      // the narrow item width bounds the virtual block count of both widths
  const int64_t bound = g.row_bound > 0 && g.row_bound < m ? g.row_bound : m;
  const unsigned vblocks = bgmoe_item_grid((g.n + ntile - 1) / ntile, g.groups, bound, 0x7fffffff, 16 * tt);
  g.lo = 0; g.hi = 0x7fffffff;     // every group: more rows = more chunks (weights re-streamed)
  const bool tm = g.w0.layout == BGMOE_W_TILE_MAJOR;
  BgmoeProf prof(fused ? BGMOE_K_MXFP4_S1 : BGMOE_K_MXFP4_GEMM, st);
  if (g_mx_variant == 3) launch_shape<kMxTT, kMxNSDeep>(fused, tm, vblocks, g, st);
  else if (g_mx_variant == 2) launch_shape<kMxTT2, kMxNSMixed, kMxTT>(fused, tm, vblocks, g, st);
  else if (g_mx_variant == 1) launch_shape<kMxTT2, kMxNS2>(fused, tm, vblocks, g, st);
  else launch_shape<kMxTT, 3>(fused, tm, vblocks, g, st);
  return bgmoe_check_launch("mxfp4 grouped gemm");
}

int check_shape(const char* what, const uint16_t* x, const int32_t* seqlens, const int32_t* cu, int groups, int64_t m,
                int n, int k, const uint16_t* out, uint16_t* const* out_ptrs) {
  BGMOE_REQUIRE(groups >= 0 && groups <= 1024, "%s: groups=%d outside [0,1024]", what, groups);
  BGMOE_REQUIRE(m >= 0, "%s: m < 0", what);
  BGMOE_REQUIRE(k > 0 && k % 128 == 0, "%s: K=%d must be a positive multiple of 128", what, k);
  BGMOE_REQUIRE(n > 0 && n % 128 == 0, "%s: N=%d must be a positive multiple of 128", what, n);
  if (groups == 0 || m == 0) return BGMOE_OK;
  BGMOE_REQUIRE(x && seqlens && cu && (out || out_ptrs), "%s: null pointer", what);
  BGMOE_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)out % 8 == 0, "%s: misaligned activations / output", what);
  return BGMOE_OK;
}

}  // namespace

int bgmoe_internal_init_mxfp4() {
  mx_resident<kMxTT, 3, true, 1>();
  mx_resident<kMxTT, 3, true, 0>();
  mx_resident<kMxTT, 3, false, 1>();
  mx_resident<kMxTT, 3, false, 0>();
  mx_resident<kMxTT, 3, true, 1, true>();
  mx_resident<kMxTT, 3, true, 0, true>();
  mx_resident<kMxTT2, kMxNS2, true, 1>();
  mx_resident<kMxTT2, kMxNS2, true, 0>();
  mx_resident<kMxTT2, kMxNS2, false, 1>();
  mx_resident<kMxTT2, kMxNS2, false, 0>();
  mx_resident<kMxTT2, kMxNS2, true, 1, true>();
  mx_resident<kMxTT2, kMxNS2, true, 0, true>();
  mx_resident<kMxTT, kMxNSDeep, true, 1>();
  mx_resident<kMxTT, kMxNSDeep, true, 0>();
  mx_resident<kMxTT, kMxNSDeep, false, 1>();
  mx_resident<kMxTT, kMxNSDeep, false, 0>();
  mx_resident<kMxTT, kMxNSDeep, true, 1, true>();
  mx_resident<kMxTT, kMxNSDeep, true, 0, true>();
  mx_resident<kMxTT2, kMxNSMixed, true, 1, false, kMxTT>();
  mx_resident<kMxTT2, kMxNSMixed, true, 0, false, kMxTT>();
  mx_resident<kMxTT2, kMxNSMixed, false, 1, false, kMxTT>();
  mx_resident<kMxTT2, kMxNSMixed, false, 0, false, kMxTT>();
  mx_resident<kMxTT2, kMxNSMixed, true, 1, true, kMxTT>();
  mx_resident<kMxTT2, kMxNSMixed, true, 0, true, kMxTT>();
  return BGMOE_OK;
}

extern "C" int bgmoe_set_mxfp4_variant(int variant) {
  BGMOE_REQUIRE(variant >= 0 && variant <= 3, "set_mxfp4_variant: variant must be 0 (64-row items, three stages), 1 "
                "(32-row items, six stages), 2 (per group: 32-row items up to 32 rows, 64-row items above) or 3 (64-row "
                "items, four stages), got %d", variant);
  g_mx_variant = variant;
  return BGMOE_OK;
}

extern "C" int bgmoe_mxfp4_grouped_gemm(const uint16_t* x, const bgmoe_mxfp4_weight* w, const int32_t* seqlens,
                                        const int32_t* cu_seqlens, int groups, int64_t m, int n, int k,
                                        uint16_t* out, uint16_t* const* out_ptrs, int64_t row_bound,
                                        bgmoe_stream_t stream) {
  int rc = check_shape("mxfp4_grouped_gemm", x, seqlens, cu_seqlens, groups, m, n, k, out, out_ptrs);
  if (rc != BGMOE_OK) return rc;
  if (groups == 0 || m == 0) return BGMOE_OK;
  rc = check_w("mxfp4_grouped_gemm", w);
  if (rc != BGMOE_OK) return rc;
  Mx4Args g{};
  g.x = x; g.w0 = *w; g.seqlens = seqlens; g.cu = cu_seqlens; g.groups = groups; g.n = n; g.k = k; g.out = out;
  g.out_ptrs = out_ptrs; g.row_bound = row_bound;
  return launch(false, g, m, bgmoe_stream(stream));
}

extern "C" int bgmoe_mxfp4_fused_s1(const uint16_t* x, const bgmoe_mxfp4_weight* gate, const bgmoe_mxfp4_weight* up,
                                    const int32_t* seqlens, const int32_t* cu_seqlens, int groups, int64_t m, int n,
                                    int k, uint16_t* out, uint16_t* const* out_ptrs, int activation,
                                    int64_t row_bound, bgmoe_stream_t stream) {
  int rc = check_shape("mxfp4_fused_s1", x, seqlens, cu_seqlens, groups, m, n, k, out, out_ptrs);
  if (rc != BGMOE_OK) return rc;
  BGMOE_REQUIRE(activation == BGMOE_ACT_SWIGLU || activation == BGMOE_ACT_SITU,
                "mxfp4_fused_s1: activation must be BGMOE_ACT_SWIGLU (0) or BGMOE_ACT_SITU (1)");
  if (groups == 0 || m == 0) return BGMOE_OK;
  rc = check_w("mxfp4_fused_s1", gate);
  if (rc != BGMOE_OK) return rc;
  rc = check_w("mxfp4_fused_s1", up);
  if (rc != BGMOE_OK) return rc;
  BGMOE_REQUIRE(gate->layout == up->layout, "mxfp4_fused_s1: gate and up weights must use the same layout");
  Mx4Args g{};
  g.x = x; g.w0 = *gate; g.w1 = *up; g.seqlens = seqlens; g.cu = cu_seqlens; g.groups = groups; g.n = n; g.k = k;
  g.out = out; g.out_ptrs = out_ptrs; g.row_bound = row_bound; g.activation = activation;
  return launch(true, g, m, bgmoe_stream(stream));
}

extern "C" int bgmoe_mxfp4_fused_s1_gather(const uint16_t* x_tokens, int64_t n_tokens, const int32_t* row_pair, int top_k,
                                           const bgmoe_mxfp4_weight* gate, const bgmoe_mxfp4_weight* up,
                                           const int32_t* seqlens, const int32_t* cu_seqlens, int groups, int64_t m,
                                           int n, int k, uint16_t* out, uint16_t* const* out_ptrs, int activation,
                                           int64_t row_bound, bgmoe_stream_t stream) {
  int rc = check_shape("mxfp4_fused_s1_gather", x_tokens, seqlens, cu_seqlens, groups, m, n, k, out, out_ptrs);
  if (rc != BGMOE_OK) return rc;
  BGMOE_REQUIRE(activation == BGMOE_ACT_SWIGLU || activation == BGMOE_ACT_SITU,
                "mxfp4_fused_s1_gather: activation must be BGMOE_ACT_SWIGLU (0) or BGMOE_ACT_SITU (1)");
  BGMOE_REQUIRE(top_k > 0 && n_tokens >= 0, "mxfp4_fused_s1_gather: bad top_k=%d or n_tokens=%lld", top_k,
                (long long)n_tokens);
  // a lane addresses its token row with a 32-bit byte offset from the start of the token matrix
  BGMOE_REQUIRE(n_tokens * 2 * (int64_t)k <= 4294967296LL,
                "mxfp4_fused_s1_gather: token matrix of %lld x %d bf16 exceeds 4 GiB", (long long)n_tokens, k);
  if (groups == 0 || m == 0) return BGMOE_OK;
  BGMOE_REQUIRE(row_pair != nullptr && n_tokens > 0, "mxfp4_fused_s1_gather: null row_pair or no tokens");
  rc = check_w("mxfp4_fused_s1_gather", gate);
  if (rc != BGMOE_OK) return rc;
  rc = check_w("mxfp4_fused_s1_gather", up);
  if (rc != BGMOE_OK) return rc;
  BGMOE_REQUIRE(gate->layout == up->layout, "mxfp4_fused_s1_gather: gate and up weights must use the same layout");
  Mx4Args g{};
  g.x = x_tokens; g.row_pair = row_pair; g.pair_div = top_k; g.last_token = (uint32_t)(n_tokens - 1);
  g.w0 = *gate; g.w1 = *up; g.seqlens = seqlens; g.cu = cu_seqlens; g.groups = groups; g.n = n; g.k = k;
  g.out = out; g.out_ptrs = out_ptrs; g.row_bound = row_bound; g.activation = activation;
  return launch(true, g, m, bgmoe_stream(stream));
}

extern "C" int bgmoe_mxfp4_weight_repack(const uint8_t* w_packed, const uint8_t* scales, uint8_t* w_out,
                                         uint8_t* scales_out, int groups, int n, int k, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(groups >= 0 && n > 0 && k > 0, "mxfp4_weight_repack: bad sizes");
  BGMOE_REQUIRE(n % 16 == 0 && k % 128 == 0, "mxfp4_weight_repack: N=%d must be a multiple of 16 and K=%d of 128", n, k);
  if (groups == 0) return BGMOE_OK;
  BGMOE_REQUIRE(w_packed && scales && w_out && scales_out && w_packed != w_out && scales != scales_out,
                "mxfp4_weight_repack: needs distinct non-null buffers");
  BGMOE_REQUIRE((uintptr_t)w_packed % 16 == 0 && (uintptr_t)w_out % 16 == 0 && (uintptr_t)scales % 4 == 0 &&
                (uintptr_t)scales_out % 4 == 0, "mxfp4_weight_repack: misaligned buffers");
  const int64_t chunks = (int64_t)groups * n * (k >> 1) / 16;
  int64_t blocks = (chunks + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(mxfp4_repack_kernel, dim3((unsigned)blocks), dim3(256), 0, bgmoe_stream(stream), w_packed, scales,
                     w_out, scales_out, chunks, n, k);
  return bgmoe_check_launch("mxfp4_weight_repack");
}
