// Router GEMM for gfx950: logits[n,e] (fp32) = hidden[n,h] (bf16) x router_weight[e,h]^T (bf16).
//
// The value of one logit is a fixed function of its token row and its expert row -- whatever the
// number of tokens in the call, the tile the token falls in, or the launch shape picked for the size:
//   * K is cut into segments of 512 elements; a segment's partial sum is one chain of
//     v_mfma_f32_16x16x32_bf16 over its 64-element steps in ascending order (fp32 accumulation inside);
//   * the logit is (((0 + p_0) + p_1) + ...) over the segments in ascending order, in fp32.
// Two launch shapes compute exactly that: "whole" (a block walks every segment and folds as it goes; used
// when the token count alone fills the chip) and "split" (one block per segment writes its partial plane to
// the workspace; a reduce pass -- or the router kernel itself -- adds the planes in order).
//
// Operands go from global memory straight to MFMA registers: lane (r, q) of a 16-row tile reads the 32
// contiguous bytes [q*16, q*16+16) elements of row r in a 64-element step, so the four lanes of a row fetch
// one whole 128-byte line; tokens and experts use the same K permutation, which a dot product does not see.
// Experts are the MFMA's row operand, so a lane ends up with 4 consecutive experts of one token: 16-byte
// stores.
#include "bgmoe_async.h"
#include "bgmoe_tilemap.h"
#include "bgmoe_common.h"

namespace {

constexpr int kSeg = 512;        // K elements per segment
constexpr int kStep = 64;        // K elements per load step (two MFMAs)
constexpr int kStepsPerSeg = kSeg / kStep;

struct RouterGemmArgs {
  const uint16_t* x;             // [n,h] bf16
  const uint16_t* w;             // [e,h] bf16
  float* out;                    // whole: logits [n,e]; split: planes [nseg][n][e]
  uint16_t* out16;               // optional: the result rounded to bf16 [n,e] instead of `out` (a linear layer)
  const int64_t* rank_counts;    // whole only: rows past a rank's count get 0
  int bucket, world;
  int n, h, e, nseg;
  int ttiles, eblocks;           // split: token tiles and expert blocks of the launch (1-D grid decode)
};

template <int TM, int NE>
struct Stage {
  intx4 a[NE][2];                // NE expert tiles x two 16-byte halves of the lane's 32 bytes
  intx4 b[TM][2];                // TM token tiles
};

// four consecutive results of one row as bf16 (`left` = columns left in the row from the first of them)
__device__ __forceinline__ void store_bf16x4(uint16_t* dst, floatx4 v, int left, bool vec) {
  if (vec) {
    if (left > 0) {
      uint2 o;
      o.x = pack2_bf16(v[0], v[1]);
      o.y = pack2_bf16(v[2], v[3]);
      *reinterpret_cast<uint2*>(dst) = o;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < left) dst[i] = (uint16_t)f32_to_bf16_bits(v[i]);
  }
}

__device__ __forceinline__ bool row_is_padding(const RouterGemmArgs& a, int row) {
  if (!a.rank_counts) return false;
  const int rank = row / a.bucket;
  if (rank >= a.world) return true;
  return (int64_t)(row - rank * a.bucket) >= a.rank_counts[rank];
}

// A block is WAVES waves; a wave owns NE 16-expert tiles x TM 16-token tiles, the block WAVES*16*NE experts.
template <int TM, int NE, int DEPTH, bool SPLIT, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void router_gemm_kernel(RouterGemmArgs a) {
  const int wave = threadIdx.x >> 6;
  const int lane = lane_id();
  const int r = lane & 15, q = lane >> 4;
  // Split shape: a unit = (K segment, expert block); all token tiles of a unit run on ONE XCD (hardware
  // deals consecutive block ids round-robin over the 8 XCDs), so an XCD's L2 fetches only its units'
  // slices of the weights and of the tokens instead of every XCD fetching everything.
  int bx = blockIdx.x, by = blockIdx.y, seg_lo = 0;
  if constexpr (SPLIT) {
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    const int ul = j / a.ttiles;
    const int unit = ul * 8 + xcd;
    if (unit >= a.nseg * a.eblocks) return;
    bx = j - ul * a.ttiles;
    seg_lo = unit / a.eblocks;
    by = unit - seg_lo * a.eblocks;
  }
  const int t0 = bx * (16 * TM);
  const int e0 = (by * WAVES + wave) * (16 * NE);
  if (e0 >= a.e) return;         // whole wave; the kernel uses no block-level barrier

  // rows past the end are clamped for the loads and never stored
  const uint8_t* wp[NE];
  const uint8_t* xp[TM];
#pragma unroll
  for (int tn = 0; tn < NE; ++tn) {
    const int er = min(e0 + tn * 16 + r, a.e - 1);
    wp[tn] = reinterpret_cast<const uint8_t*>(a.w) + ((int64_t)er * a.h + q * 16) * 2;
  }
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int tr = min(t0 + tm * 16 + r, a.n - 1);
    xp[tm] = reinterpret_cast<const uint8_t*>(a.x) + ((int64_t)tr * a.h + q * 16) * 2;
  }

  const int seg_hi = SPLIT ? seg_lo + 1 : a.nseg;
  const int k_lo = seg_lo * kSeg;
  const int k_hi = min(seg_hi * kSeg, a.h);
  const int full = (k_hi - k_lo) / kStep;          // whole 64-element steps (uniform)
  const int tail = (k_hi - k_lo) - full * kStep;   // 0, or a multiple of 8 below 64

  floatx4 acc[TM][NE], tot[TM][NE];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < NE; ++tn) {
      acc[tm][tn] = floatx4{0.f, 0.f, 0.f, 0.f};
      tot[tm][tn] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

  auto load = [&](Stage<TM, NE>& s, int step) {
    const int64_t off = (int64_t)(k_lo + step * kStep) * 2;
#pragma unroll
    for (int tn = 0; tn < NE; ++tn) {
      s.a[tn][0] = gload_x4(wp[tn] + off);
      s.a[tn][1] = gload_x4(wp[tn] + off + 16);
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      s.b[tm][0] = gload_x4(xp[tm] + off);
      s.b[tm][1] = gload_x4(xp[tm] + off + 16);
    }
  };
  auto compute = [&](const Stage<TM, NE>& s) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < NE; ++tn)
          acc[tm][tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, s.a[tn][j]),
                                                                __builtin_bit_cast(bf16x8, s.b[tm][j]),
                                                                acc[tm][tn], 0, 0, 0);
  };
  auto fold = [&]() {            // end of a segment
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int tn = 0; tn < NE; ++tn) {
        tot[tm][tn] += acc[tm][tn];
        acc[tm][tn] = floatx4{0.f, 0.f, 0.f, 0.f};
      }
  };

  Stage<TM, NE> ring[DEPTH];
  if (SPLIT && full == kStepsPerSeg) {
    // a whole segment (all but possibly the last): every load is unconditional, so the compiler keeps
    // DEPTH steps in flight and waits for exactly the step it is about to use
    // (the scheduling barriers keep the compiler from sinking the prefetches down to their uses, which
    // it otherwise does to save registers -- and which leaves one step in flight instead of DEPTH)
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) load(ring[d], d);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int step = 0; step < kStepsPerSeg; ++step) {
      compute(ring[step % DEPTH]);
      if (step + DEPTH < kStepsPerSeg) load(ring[step % DEPTH], step + DEPTH);
      __builtin_amdgcn_sched_barrier(0);
    }
  } else {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (d < full) load(ring[d], d);
    __builtin_amdgcn_sched_barrier(0);
    int base = 0;
    if constexpr (!SPLIT) {
      // steady state, one segment per trip: every step and every prefetch is in range, so nothing is
      // conditional and the waits are exact; the guarded loop below finishes the last steps
      static_assert(kStepsPerSeg % DEPTH == 0, "ring slots must line up with segment starts");
      for (; base + kStepsPerSeg + DEPTH <= full; base += kStepsPerSeg) {
#pragma unroll
        for (int step = 0; step < kStepsPerSeg; ++step) {
          compute(ring[step % DEPTH]);
          load(ring[step % DEPTH], base + step + DEPTH);
          __builtin_amdgcn_sched_barrier(0);
        }
        fold();
      }
    }
    for (int s = base; s < full; s += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int step = s + d;
        if (step < full) {
          compute(ring[d]);
          if (step + DEPTH < full) load(ring[d], step + DEPTH);
          if constexpr (!SPLIT)
            if ((step & (kStepsPerSeg - 1)) == kStepsPerSeg - 1) fold();
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  if (tail) {
    // the last, partial step of the last segment: 16-byte pieces past the end of K count as zeros
    Stage<TM, NE> s;
    const int kbase = k_lo + full * kStep + q * 16;
    const int64_t off = (int64_t)(k_lo + full * kStep) * 2;
    const intx4 zero = intx4{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const bool live = kbase + j * 8 < k_hi;
#pragma unroll
      for (int tn = 0; tn < NE; ++tn) s.a[tn][j] = live ? gload_x4(wp[tn] + off + j * 16) : zero;
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) s.b[tm][j] = live ? gload_x4(xp[tm] + off + j * 16) : zero;
    }
    compute(s);
  }
  // a segment still open (the split shape's only segment, or a last one shorter than 512): fold it
  if (SPLIT || tail || (full & (kStepsPerSeg - 1)) != 0) fold();

  float* plane = a.out + (SPLIT ? (int64_t)seg_lo * a.n * a.e : 0);
  const bool vec = (a.e & 3) == 0;
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int token = t0 + tm * 16 + r;
    if (token >= a.n) continue;
    bool pad = false;
    if constexpr (!SPLIT) pad = row_is_padding(a, token);
#pragma unroll
    for (int tn = 0; tn < NE; ++tn) {
      const int ex = e0 + tn * 16 + q * 4;
      floatx4 v = pad ? floatx4{0.f, 0.f, 0.f, 0.f} : tot[tm][tn];
      if (!SPLIT && a.out16 != nullptr) {
        store_bf16x4(a.out16 + (int64_t)token * a.e + ex, v, a.e - ex, vec);
        continue;
      }
      float* dst = plane + (int64_t)token * a.e + ex;
      if (vec) {
        if (ex < a.e) *reinterpret_cast<floatx4*>(dst) = v;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (ex + i < a.e) dst[i] = v[i];
      }
    }
  }
}

// ---- many tokens: operands shared through LDS ------------------------------------------------------
// A CU sustains only ~35-60 GB/s of load requests, so with many tokens the time goes where the requested
// bytes go.  Four waves that each fetch their own 64 + 64 rows request twice what the block needs; here the
// block's 128 experts + 128 tokens of a 64-element K step (256 rows x 128 B = 32 KB) are fetched ONCE, by
// asynchronous global->LDS loads into a 4-slot ring, and every wave reads its share of the tile from LDS.
// A row's eight 16-byte pieces land XOR-swizzled by (row & 7) -- done by choosing which piece each lane
// fetches -- so that the 16-row operand reads hit all banks.  Lane (r, q) reads pieces 2q and 2q+1 of row
// r: the same K assignment, MFMA order and segment folds as the register kernel above, hence the same bits.
constexpr int kLdsStages = 4;
constexpr int kLdsStageBytes = 256 * 128;
constexpr int kLdsBytes = kLdsStages * kLdsStageBytes;

// 8 waves = 2 expert halves x 4 token quarters (wave tile 64 experts x 32 tokens): two waves per SIMD, which
// a single wave's MFMA issue rate needs (one wave alone issues a 16x16x32 MFMA every ~28 cycles, two
// interleaved reach ~20 per SIMD -- measured), and which lets one wave's LDS reads hide behind the other's
// MFMAs.
constexpr int kLdsWaves = 8;
constexpr int kLdsTM = 128 / (kLdsWaves / 2) / 16;      // 16-token tiles per wave

template <bool SPLIT>
__global__ __launch_bounds__(64 * kLdsWaves) void router_gemm_lds_kernel(RouterGemmArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  constexpr int TM = kLdsTM;
  const uint32_t smem_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem);
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int lane = lane_id();
  const int r16 = lane & 15, q = lane >> 4;
  // consecutive block ids go round-robin over the 8 XCDs: the expert blocks of one token tile stay on one
  // XCD (its L2 then serves the tile's second reader), token tiles are dealt over the XCDs
  // (split shape: a unit = (K segment, expert block) with all its token tiles on one XCD, as in the register
  // kernel)
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  int bx, by, seg = 0;
  if constexpr (SPLIT) {
    const int ul = j / a.ttiles;
    const int unit = ul * 8 + xcd;
    if (unit >= a.nseg * a.eblocks) return;
    bx = j - ul * a.ttiles;
    seg = unit / a.eblocks;
    by = unit - seg * a.eblocks;
  } else {
    const int tl = j / a.eblocks;
    by = j - tl * a.eblocks;
    bx = tl * 8 + xcd;
    if (bx >= a.ttiles) return;            // whole block, before any barrier
  }
  const int t0 = bx * 128, e0 = by * 128;
  const int we = wave & 1, wt = wave >> 1;  // this wave's expert half and token share of the block tile

  // loader: the first half of the waves fetches the 128 expert rows, the second half the 128 token rows;
  // one issue = 8 rows x 128 B, lane p -> row p>>3, LDS piece p&7 <- global piece (p&7) ^ (row&7)
  constexpr int kHalf = kLdsWaves / 2;
  constexpr int kIssues = 16 / kHalf;       // issues per wave and step
  const bool load_tokens = wave >= kHalf;
  const int lrow0 = (wave % kHalf) * (8 * kIssues);
  const uint8_t* src = load_tokens ? reinterpret_cast<const uint8_t*>(a.x) + (int64_t)t0 * a.h * 2
                                   : reinterpret_cast<const uint8_t*>(a.w) + (int64_t)e0 * a.h * 2;
  src = uniform_ptr(src);
  const int row_lim = (load_tokens ? a.n - t0 : a.e - e0) - 1;      // clamp: rows past the end re-read the last
  uint32_t loff[kIssues];
#pragma unroll
  for (int i = 0; i < kIssues; ++i) {
    const int row = lrow0 + i * 8 + (lane >> 3);
    const int piece = (lane & 7) ^ (row & 7);
    loff[i] = (uint32_t)min(row, row_lim) * (uint32_t)a.h * 2u + (uint32_t)piece * 16u;
  }
  const uint32_t ldst = smem_base + (load_tokens ? 16384u : 0u) + (uint32_t)lrow0 * 128u;
  auto issue = [&](int step) {
    const uint32_t d = ldst + (uint32_t)(step & (kLdsStages - 1)) * kLdsStageBytes;
    const uint8_t* p = src + (int64_t)step * (kStep * 2);
#pragma unroll
    for (int i = 0; i < kIssues; ++i) async_load16(p, loff[i], d + i * 1024);
  };

  floatx4 acc[TM][4], tot[TM][4];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < 4; ++tn) {
      acc[tm][tn] = floatx4{0.f, 0.f, 0.f, 0.f};
      tot[tm][tn] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
  // the host sends only h % 64 == 0 here; the split shape walks one segment's steps
  const int step0 = SPLIT ? seg * kStepsPerSeg : 0;
  const int nsteps = SPLIT ? min(kStepsPerSeg, a.h / kStep - step0) : a.h / kStep;
  src += (int64_t)step0 * (kStep * 2);
  const int rd_a = (we * 64 + r16) * 128, rd_b = 16384 + (wt * (16 * TM) + r16) * 128;
  const int sw = r16 & 7;

#pragma unroll
  for (int s = 0; s < kLdsStages - 1; ++s)
    if (s < nsteps) issue(s);
  for (int s = 0; s < nsteps; ++s) {
    // the step's loads have landed once at most the younger steps' loads are outstanding
    const int younger = min(kLdsStages - 2, nsteps - 1 - s);      // steps requested after this one
    if (younger >= 2) wait_vm<2 * kIssues>();
    else if (younger == 1) wait_vm<kIssues>();
    else wait_vm<0>();
    block_barrier();                       // everyone's loads of step s are in; everyone is done with step s-1
    if (s + kLdsStages - 1 < nsteps) issue(s + kLdsStages - 1);   // into the slot step s-1 just freed
    const uint8_t* sb = smem + (s & (kLdsStages - 1)) * kLdsStageBytes;
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      const int piece = ((2 * q + jj) ^ sw) * 16;
      intx4 av[4], bv[TM];
#pragma unroll
      for (int tn = 0; tn < 4; ++tn) av[tn] = *reinterpret_cast<const intx4*>(sb + rd_a + tn * 2048 + piece);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) bv[tm] = *reinterpret_cast<const intx4*>(sb + rd_b + tm * 2048 + piece);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < 4; ++tn)
          acc[tm][tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av[tn]),
                                                                __builtin_bit_cast(bf16x8, bv[tm]),
                                                                acc[tm][tn], 0, 0, 0);
    }
    if ((s & (kStepsPerSeg - 1)) == kStepsPerSeg - 1 || s == nsteps - 1) {   // end of a segment
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < 4; ++tn) {
          tot[tm][tn] += acc[tm][tn];
          acc[tm][tn] = floatx4{0.f, 0.f, 0.f, 0.f};
        }
    }
  }

  const bool vec = (a.e & 3) == 0;
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int token = t0 + wt * (16 * TM) + tm * 16 + r16;
    if (token >= a.n) continue;
    const bool pad = SPLIT ? false : row_is_padding(a, token);
#pragma unroll
    for (int tn = 0; tn < 4; ++tn) {
      const int ex = e0 + we * 64 + tn * 16 + q * 4;
      const floatx4 v = pad ? floatx4{0.f, 0.f, 0.f, 0.f} : tot[tm][tn];
      if (!SPLIT && a.out16 != nullptr) {
        store_bf16x4(a.out16 + (int64_t)token * a.e + ex, v, a.e - ex, vec);
        continue;
      }
      float* dst = a.out + (SPLIT ? (int64_t)seg * a.n * a.e : 0) + (int64_t)token * a.e + ex;
      if (vec) {
        if (ex < a.e) *reinterpret_cast<floatx4*>(dst) = v;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (ex + i < a.e) dst[i] = v[i];
      }
    }
  }
}

// The same kernel with a block tile of 128 tokens x 64 experts (whole K only): for shapes whose 128 x 128 tiles
// number fewer than the CUs (a 512-row linear layer onto 4096 columns: 128 tiles on 256 CUs), twice as many,
// narrower tiles put every CU to work.  A K step is 64 expert rows + 128 token rows = 24 KB; 8 waves = 8 token
// eighths, wave tile 64 experts x 16 tokens.  Every wave issues three loads per step: issue j = 3 * wave + i of the
// block's 24 covers rows 8j .. 8j+7 of the list [64 expert rows; 128 token rows].  Lane map, swizzle, K assignment,
// MFMA order and segment folds are the wide kernel's, hence the same bits.  Opt-in (bgmoe_set_router_gemm_plan).
constexpr int kLds64Experts = 64;
constexpr int kLds64Issues = (kLds64Experts + 128) / 8 / kLdsWaves;      // 3
static_assert(kLds64Issues * kLdsWaves * 8 == kLds64Experts + 128, "24 issues of 8 rows cover the step's 192 rows");
static_assert(kLds64Experts == (int)BGMOE_RG64_EXPERTS && kLds64Issues == 3, "the lane maps of bgmoe_tilemap.h assume this shape");

__global__ __launch_bounds__(64 * kLdsWaves) void router_gemm_lds64_kernel(RouterGemmArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  constexpr int EB = kLds64Experts;
  constexpr int kIssues = kLds64Issues;
  const uint32_t smem_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem);
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int lane = lane_id();
  const int r16 = lane & 15, q = lane >> 4;
  const int xcd = blockIdx.x & 7, j0 = blockIdx.x >> 3;
  const int tl = j0 / a.eblocks;
  const int by = j0 - tl * a.eblocks;
  const int bx = tl * 8 + xcd;
  if (bx >= a.ttiles) return;              // whole block, before any barrier
  const int t0 = bx * 128, e0 = by * EB;
  const int wt = wave;                      // this wave's 16 tokens of the block tile

  // loader: per issue a wave-uniform choice between the expert rows and the token rows
  const uint8_t* src_e = uniform_ptr(reinterpret_cast<const uint8_t*>(a.w) + (int64_t)e0 * a.h * 2);
  const uint8_t* src_t = uniform_ptr(reinterpret_cast<const uint8_t*>(a.x) + (int64_t)t0 * a.h * 2);
  const int lim_e = a.e - e0 - 1, lim_t = a.n - t0 - 1;                 // clamp: rows past the end re-read the last
  uint32_t loff[kIssues], ldst[kIssues];
  bool tok[kIssues];
#pragma unroll
  for (int i = 0; i < kIssues; ++i) {                                   // lane maps: bgmoe_tilemap.h
    tok[i] = bgmoe_rg64_issue_is_token((uint32_t)wave, (uint32_t)i);    // wave-uniform
    const int row = (int)bgmoe_rg64_lane_row((uint32_t)wave, (uint32_t)i, (uint32_t)lane);
    const uint32_t piece = bgmoe_rg64_lane_piece((uint32_t)row, (uint32_t)lane);
    loff[i] = (uint32_t)min(row, tok[i] ? lim_t : lim_e) * (uint32_t)a.h * 2u + piece * 16u;
    ldst[i] = smem_base + bgmoe_rg64_issue_lds((uint32_t)wave, (uint32_t)i);
  }
  auto issue = [&](int step) {
    const uint32_t d = (uint32_t)(step & (kLdsStages - 1)) * kLdsStageBytes;
    const int64_t ko = (int64_t)step * (kStep * 2);
#pragma unroll
    for (int i = 0; i < kIssues; ++i)
      async_load16(uniform_ptr((tok[i] ? src_t : src_e) + ko), loff[i],
                   __builtin_amdgcn_readfirstlane(ldst[i] + d));
  };

  floatx4 acc[4], tot[4];
#pragma unroll
  for (int tn = 0; tn < 4; ++tn) {
    acc[tn] = floatx4{0.f, 0.f, 0.f, 0.f};
    tot[tn] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  const int nsteps = a.h / kStep;            // the host sends only h % 64 == 0 here

#pragma unroll
  for (int s = 0; s < kLdsStages - 1; ++s)
    if (s < nsteps) issue(s);
  for (int s = 0; s < nsteps; ++s) {
    const int younger = min(kLdsStages - 2, nsteps - 1 - s);      // steps requested after this one
    if (younger >= 2) wait_vm<2 * kIssues>();
    else if (younger == 1) wait_vm<kIssues>();
    else wait_vm<0>();
    block_barrier();                       // everyone's loads of step s are in; everyone is done with step s-1
    if (s + kLdsStages - 1 < nsteps) issue(s + kLdsStages - 1);   // into the slot step s-1 just freed
    const uint8_t* sb = smem + (s & (kLdsStages - 1)) * kLdsStageBytes;
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      intx4 av[4];
#pragma unroll
      for (int tn = 0; tn < 4; ++tn)
        av[tn] = *reinterpret_cast<const intx4*>(sb + bgmoe_rg64_read_expert((uint32_t)tn, (uint32_t)lane, (uint32_t)jj));
      const intx4 bv = *reinterpret_cast<const intx4*>(sb + bgmoe_rg64_read_token((uint32_t)wt, (uint32_t)lane, (uint32_t)jj));
#pragma unroll
      for (int tn = 0; tn < 4; ++tn)
        acc[tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av[tn]),
                                                          __builtin_bit_cast(bf16x8, bv), acc[tn], 0, 0, 0);
    }
    if ((s & (kStepsPerSeg - 1)) == kStepsPerSeg - 1 || s == nsteps - 1) {   // end of a segment
#pragma unroll
      for (int tn = 0; tn < 4; ++tn) {
        tot[tn] += acc[tn];
        acc[tn] = floatx4{0.f, 0.f, 0.f, 0.f};
      }
    }
  }

  const bool vec = (a.e & 3) == 0;
  const int token = t0 + wt * 16 + r16;
  if (token >= a.n) return;
  const bool pad = row_is_padding(a, token);
#pragma unroll
  for (int tn = 0; tn < 4; ++tn) {
    const int ex = e0 + tn * 16 + q * 4;
    const floatx4 v = pad ? floatx4{0.f, 0.f, 0.f, 0.f} : tot[tn];
    if (a.out16 != nullptr) {
      store_bf16x4(a.out16 + (int64_t)token * a.e + ex, v, a.e - ex, vec);
      continue;
    }
    float* dst = a.out + (int64_t)token * a.e + ex;
    if (vec) {
      if (ex < a.e) *reinterpret_cast<floatx4*>(dst) = v;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (ex + i < a.e) dst[i] = v[i];
    }
  }
}

// logits = (((0 + p_0) + p_1) + ...) over the planes; rows past a rank's count get 0
__global__ __launch_bounds__(256) void router_gemm_reduce_kernel(RouterGemmArgs a, const float* planes) {
  const int64_t total = (int64_t)a.n * a.e;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int row = (int)(i / a.e);
  float v = 0.0f;
  if (!row_is_padding(a, row))
    for (int s = 0; s < a.nseg; ++s) v += planes[(int64_t)s * total + i];
  if (a.out16 != nullptr) a.out16[i] = (uint16_t)f32_to_bf16_bits(v);
  else a.out[i] = v;
}

int g_plan_tm = -1, g_plan_split = -1;
bool g_lds_ready = false;            // the LDS kernel's 128 KB opt-in succeeded on this process's device
bool g_lds64_ready = false;          // likewise for the 64-expert-block variant (opt-in)

struct Plan { int tm; int ne; int waves; bool split; bool lds; bool eb64; };

// Launch shape from the sizes alone (results do not depend on it).
// A CU sustains only ~35-60 GB/s of load requests whatever hits in cache, so what matters for few tokens
// is (a) every CU busy and (b) few requested bytes per CU: one-wave blocks with the largest wave tile
// (64 tokens x 64 experts: 128 rows requested per 4096 outputs), one K segment each.
Plan make_plan(int n, int h, int e) {
  const int nseg = (h + kSeg - 1) / kSeg;
  const int64_t ey4 = (e + 255) / 256;
  Plan p;
  p.ne = 4;
  p.waves = 4;
  p.eb64 = false;
  // Measured on MI355X (h = 7168): an LDS block needs ~0.6 us per K step whatever else runs, so the whole-K LDS
  // shape costs ~67 us per round of 256 tiles; one block per segment fills the chip from ~1K tokens on at the
  // price of the planes (write + reduce); below that the one-wave register blocks win.
  const bool planes_small = (int64_t)n * e * nseg <= (int64_t)16 << 20;      // <= 64 MiB of partial planes
  const bool lds_ok = h % kStep == 0 && g_lds_ready;
  const int64_t tiles128 = ((int64_t)(n + 127) / 128) * ((e + 127) / 128);
  p.lds = false;
  if (lds_ok && (tiles128 >= 96 || (nseg == 1 && tiles128 >= 16))) {
    p.split = false;
    p.lds = true;
    p.tm = 4;
  } else if (lds_ok && nseg > 1 && planes_small && tiles128 * nseg >= 128) {
    p.split = true;
    p.lds = true;
    p.tm = 4;
  } else if (nseg == 1 || !planes_small || ((int64_t)(n + 63) / 64) * ey4 >= 192) {
    p.split = false;
    p.tm = n > 2048 ? 4 : n > 512 ? 2 : 1;
  } else {
    p.split = true;
    p.waves = 1;
    p.tm = n > 32 ? 4 : n > 16 ? 2 : 1;
  }
  if (g_plan_tm == 1 || g_plan_tm == 2 || g_plan_tm == 4) p.tm = g_plan_tm;
  if (g_plan_split == 0) { p.split = false; p.waves = 4; p.lds = false; }
  if (g_plan_split == 3) { p.split = false; p.waves = 4; p.lds = h % kStep == 0 && g_lds_ready; }
  if (g_plan_split == 4) { p.split = true; p.waves = 4; p.lds = h % kStep == 0 && g_lds_ready; }
  if (g_plan_split == 1) { p.split = true; p.waves = 4; p.lds = false; }
  if (g_plan_split == 2) { p.split = true; p.waves = 1; p.lds = false; }
  if (g_plan_split == 5 && h % kStep == 0 && g_lds64_ready) { p.split = false; p.waves = 4; p.lds = true; p.eb64 = true; }
  return p;
}

template <bool SPLIT>
void launch_gemm(const RouterGemmArgs& a0, const Plan& p, hipStream_t st) {
  RouterGemmArgs a = a0;
  if (!SPLIT && p.lds && p.eb64) {
    a.ttiles = (a.n + 127) / 128;
    a.eblocks = (a.e + kLds64Experts - 1) / kLds64Experts;
    const unsigned blocks = (unsigned)(8 * ((a.ttiles + 7) / 8) * a.eblocks);
    hipLaunchKernelGGL(router_gemm_lds64_kernel, dim3(blocks), dim3(64 * kLdsWaves), kLdsBytes, st, a);
    return;
  }
  if (p.lds) {
    a.ttiles = (a.n + 127) / 128;
    a.eblocks = (a.e + 127) / 128;
    const unsigned blocks = SPLIT ? (unsigned)(8 * ((a.nseg * a.eblocks + 7) / 8) * a.ttiles)
                                  : (unsigned)(8 * ((a.ttiles + 7) / 8) * a.eblocks);
    hipLaunchKernelGGL(router_gemm_lds_kernel<SPLIT>, dim3(blocks), dim3(64 * kLdsWaves), kLdsBytes, st, a);
    return;
  }
  const dim3 block(64 * p.waves);
  a.ttiles = (a.n + 16 * p.tm - 1) / (16 * p.tm);
  a.eblocks = (a.e + 16 * p.ne * p.waves - 1) / (16 * p.ne * p.waves);
  dim3 grid(a.ttiles, a.eblocks, 1);
  if (SPLIT) grid = dim3((unsigned)(8 * ((a.nseg * a.eblocks + 7) / 8) * a.ttiles), 1, 1);
  if (p.waves == 1) {
    if (p.tm == 4) hipLaunchKernelGGL((router_gemm_kernel<4, 4, 4, SPLIT, 1>), grid, block, 0, st, a);
    else if (p.tm == 2) hipLaunchKernelGGL((router_gemm_kernel<2, 4, 4, SPLIT, 1>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((router_gemm_kernel<1, 4, 4, SPLIT, 1>), grid, block, 0, st, a);
  } else {
    if (p.tm == 4) hipLaunchKernelGGL((router_gemm_kernel<4, 4, 2, SPLIT, 4>), grid, block, 0, st, a);
    else if (p.tm == 2) hipLaunchKernelGGL((router_gemm_kernel<2, 4, 4, SPLIT, 4>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((router_gemm_kernel<1, 4, 4, SPLIT, 4>), grid, block, 0, st, a);
  }
}

int check_shapes(int n, int h, int e) {
  BGMOE_REQUIRE(n >= 0 && h >= 8 && e >= 1, "router_gemm: bad sizes n=%d h=%d e=%d", n, h, e);
  BGMOE_REQUIRE(h % 8 == 0, "router_gemm: hidden size %d must be a multiple of 8 (16-byte row pieces)", h);
  return BGMOE_OK;
}

}  // namespace

// one-time: the LDS kernel needs more than the default 64 KB of dynamic LDS
int bgmoe_internal_init_router_gemm() {
  static int state = 0;                // 0 = not tried, 1 = ready, -1 = failed (the register kernels serve)
  if (state == 0) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(router_gemm_lds_kernel<false>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e == hipSuccess)
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(router_gemm_lds_kernel<true>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    state = e == hipSuccess ? 1 : -1;
    if (e != hipSuccess) (void)hipGetLastError();
    g_lds_ready = state == 1;
    // the opt-in narrow variant on its own: a failure here leaves the kernels above as they are
    const hipError_t e64 = hipFuncSetAttribute(reinterpret_cast<const void*>(router_gemm_lds64_kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e64 != hipSuccess) (void)hipGetLastError();
    g_lds64_ready = e64 == hipSuccess;
  }
  return BGMOE_OK;
}

extern "C" int bgmoe_set_router_gemm_plan(int token_tiles, int split) {
  BGMOE_REQUIRE(token_tiles == -1 || token_tiles == 1 || token_tiles == 2 || token_tiles == 4,
                "set_router_gemm_plan: token_tiles must be -1, 1, 2 or 4");
  BGMOE_REQUIRE(split >= -1 && split <= 5, "set_router_gemm_plan: split must be -1 ... 5");
  g_plan_tm = token_tiles;
  g_plan_split = split;
  return BGMOE_OK;
}

extern "C" size_t bgmoe_router_gemm_workspace_bytes(int n, int h, int e) {
  if (n <= 0 || h <= 0 || e <= 0) return 0;
  bgmoe_internal_init_router_gemm();
  const Plan p = make_plan(n, h, e);
  const int nseg = (h + kSeg - 1) / kSeg;
  return (size_t)(p.split ? nseg : 1) * (size_t)n * (size_t)e * sizeof(float);
}

// For the fused router: the logits as planes to be added in order, [*nplanes_out][n][e] fp32 -- the split-K
// planes, or one plane of finished logits when the whole-K shape is the one for these sizes.
int bgmoe_internal_router_gemm_planes(const uint16_t* hidden, const uint16_t* weight, int n, int h, int e,
                                      float* planes, size_t planes_bytes, int* nplanes_out, hipStream_t st) {
  if (int rc = check_shapes(n, h, e)) return rc;
  bgmoe_internal_init_router_gemm();
  RouterGemmArgs a{};
  a.x = hidden; a.w = weight; a.out = planes; a.n = n; a.h = h; a.e = e;
  a.nseg = (h + kSeg - 1) / kSeg;
  const Plan p = make_plan(n, h, e);
  *nplanes_out = p.split ? a.nseg : 1;
  if (n == 0) return BGMOE_OK;
  if (planes_bytes < bgmoe_router_gemm_workspace_bytes(n, h, e) || !planes) {
    bgmoe_set_error("router_gemm: workspace of %zu bytes is smaller than the %zu needed", planes_bytes,
                    bgmoe_router_gemm_workspace_bytes(n, h, e));
    return BGMOE_ERR_WORKSPACE;
  }
  BgmoeProf prof(BGMOE_K_ROUTER_GEMM, st);
  if (p.split) launch_gemm<true>(a, p, st);
  else launch_gemm<false>(a, p, st);
  return bgmoe_check_launch("router_gemm");
}

static int router_gemm_run(const uint16_t* hidden, const uint16_t* weight, int n, int h, int e,
                           const int64_t* rank_token_counts, int bucket_size, int world_size, float* logits,
                           uint16_t* out16, void* workspace, size_t workspace_bytes, bgmoe_stream_t stream);

extern "C" int bgmoe_router_gemm(const uint16_t* hidden, const uint16_t* weight, int n, int h, int e,
                                 const int64_t* rank_token_counts, int bucket_size, int world_size,
                                 float* logits, void* workspace, size_t workspace_bytes,
                                 bgmoe_stream_t stream) {
  BGMOE_REQUIRE(n == 0 || logits, "router_gemm: null pointer");
  return router_gemm_run(hidden, weight, n, h, e, rank_token_counts, bucket_size, world_size, logits, nullptr, workspace,
                         workspace_bytes, stream);
}

extern "C" int bgmoe_bf16_linear(const uint16_t* x, const uint16_t* weight, int n, int h, int e, uint16_t* out,
                                 void* workspace, size_t workspace_bytes, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(n == 0 || out, "bf16_linear: null output");
  BGMOE_REQUIRE(e % 4 == 0 || (uintptr_t)out % 2 == 0, "bf16_linear: misaligned output");
  BGMOE_REQUIRE(e % 4 != 0 || (uintptr_t)out % 8 == 0, "bf16_linear: output must be 8-byte aligned");
  return router_gemm_run(x, weight, n, h, e, nullptr, 0, 0, nullptr, out, workspace, workspace_bytes, stream);
}

static int router_gemm_run(const uint16_t* hidden, const uint16_t* weight, int n, int h, int e,
                           const int64_t* rank_token_counts, int bucket_size, int world_size, float* logits,
                           uint16_t* out16, void* workspace, size_t workspace_bytes, bgmoe_stream_t stream) {
  if (int rc = check_shapes(n, h, e)) return rc;
  if (rank_token_counts) {
    BGMOE_REQUIRE(world_size > 0, "router_gemm: world_size must be positive when rank_token_counts is provided");
    BGMOE_REQUIRE(bucket_size > 0, "router_gemm: bucket_size must be positive when rank_token_counts is provided");
  }
  if (n == 0) return BGMOE_OK;
  BGMOE_REQUIRE(hidden && weight && (logits || out16), "router_gemm: null pointer");
  bgmoe_internal_init_router_gemm();
  hipStream_t st = bgmoe_stream(stream);
  RouterGemmArgs a{};
  a.x = hidden; a.w = weight; a.n = n; a.h = h; a.e = e; a.out16 = out16;
  a.rank_counts = rank_token_counts; a.bucket = bucket_size; a.world = world_size;
  a.nseg = (h + kSeg - 1) / kSeg;
  Plan p = make_plan(n, h, e);
  // without a workspace the whole-K shape is the only one possible (slower for few tokens, same bits)
  if (p.split && (!workspace || workspace_bytes < bgmoe_router_gemm_workspace_bytes(n, h, e))) {
    BGMOE_REQUIRE(g_plan_split < 1, "router_gemm: the split shape was forced but the workspace is too small");
    p.split = false;
    p.waves = 4;
  }
  if (!p.split) {
    a.out = logits;
    BgmoeProf prof(BGMOE_K_ROUTER_GEMM, st);
    launch_gemm<false>(a, p, st);
    return bgmoe_check_launch("router_gemm");
  }
  {
    RouterGemmArgs g = a;
    g.out = static_cast<float*>(workspace);
    g.out16 = nullptr;
    g.rank_counts = nullptr;
    BgmoeProf prof(BGMOE_K_ROUTER_GEMM, st);
    launch_gemm<true>(g, p, st);
    if (int rc = bgmoe_check_launch("router_gemm")) return rc;
  }
  a.out = logits;
  const int64_t total = (int64_t)n * e;
  BgmoeProf prof(BGMOE_K_ROUTER_GEMM_REDUCE, st);
  hipLaunchKernelGGL(router_gemm_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, a,
                     static_cast<const float*>(workspace));
  return bgmoe_check_launch("router_gemm_reduce");
}
