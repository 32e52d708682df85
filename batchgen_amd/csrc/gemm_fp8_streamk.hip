// Block-scaled FP8 grouped GEMM for FEW rows per group (decode), balanced form: the weight-streaming kernel
// of gemm_fp8_skinny.hip with the work cut into equal shares instead of whole items.
//
// Why: a decode launch has a few hundred items (group x row chunk x 128-column slab) of 0.25-1.8 MB each for
// 512 resident blocks, and one block streams only ~15 GB/s, so whole items leave CUs idle (320 equal items on 512
// slots take as long as 512) and every item pays a pipeline fill and drain.  Here all K-blocks of all items form
// one sequence, each weighted by the 2-KiB tiles it requests (weights + token tiles); block r owns the units whose
// start lies in [r*C/G, (r+1)*C/G) of the cumulative cost C.  A block's share usually covers the end of one item
// and the start of the next: the register prefetch ring and the token ring in LDS run on across the boundary (the
// load cursor is NSTAGE-1 units ahead of the compute cursor and switches items on its own), so a block issues
// loads without a gap from its first unit to its last.
//
// An item whose K-blocks are split over several blocks is finished by whichever of them arrives last: every
// part writes its fp32 partial sums to its own slot of the workspace, publishes them (device-scope fence +
// atomic counter) and the part that finds the counter complete adds all slots IN BLOCK ORDER and runs the
// epilogue.  No block waits for another.  The sum of an item is therefore (p_first + ... + p_last) with each
// part an ascending chain over its K-blocks: it depends on where the cuts fall, i.e. on the group sizes of the
// launch, but not on timing -- the same launch gives the same bits every time.  Counters are left at zero.
//
// Everything else (MFMA operand mapping, tile-major weight layout, async token ring, SwiGLU + requant epilogue)
// is the weight-streaming kernel's; see gemm_fp8_skinny.hip.
#include "bgmoe_common.h"
#include "bgmoe_async.h"
#include "bgmoe_hostdev.h"

namespace {

struct StreamKArgs {
  bgmoe_fp8_act a;
  bgmoe_fp8_weight w0, w1;
  const int32_t* seqlens;
  const int32_t* cu;
  int groups, n, k;
  uint16_t* out;
  uint8_t* out_q;
  float* out_s;
  int64_t os_row, os_nb;
  int hi;                     // serves groups with 0 < count <= hi
  floatx4* slots;             // 2 * gridDim.x partial-sum slots of TT*NT*256 floatx4
  int32_t* counters;          // gridDim.x counters, zero before and after every launch
  uint64_t* trace;            // optional (tuning): 4 timestamps per share (start, first unit, end of stream, end)
  int xcd_w[8];               // relative size of a share on XCD 0..7 (the XCDs do not stream equally fast)
  int32_t* error_flag;        // device word, bit 0 set by a share that found no unit (see bgmoe_debug_streamk_status)
};

// Share arithmetic (cumulative weights, share bounds, the unit search inside a group): bgmoe_hostdev.h, shared with
// the host-compiled checks that walk it over random launches on the CPU.
constexpr int kMaxGroups = 320;         // per-group tables live in LDS

// Cost of one K-block of an item, the measure in which shares are equal: its weight tiles (2 KiB each) count kCostW
// in a group's first row chunk, where they come from HBM, and kCostR in its later chunks, which run at the same time
// on the same XCD and find them in its L2; its token tiles (L2 as well) count kCostT each.
#ifndef BGMOE_SK_COST_W
#define BGMOE_SK_COST_W 4
#endif
#ifndef BGMOE_SK_COST_R
#define BGMOE_SK_COST_R 2
#endif
#ifndef BGMOE_SK_COST_T
#define BGMOE_SK_COST_T 2
#endif
constexpr int kCostW = BGMOE_SK_COST_W, kCostR = BGMOE_SK_COST_R, kCostT = BGMOE_SK_COST_T;
constexpr BgmoeSkCost kCost{kCostW, kCostR, kCostT};
// cost of one K-block of all row chunks of one slab of a group with c rows (tiles of 16 rows, chunks of TT tiles)
template <int TT, int WC>
__device__ __forceinline__ uint32_t group_cost_per_kb(int c) {
  return bgmoe_sk_group_cost_per_kb(BgmoeSkShape{TT, WC}, kCost, c);
}

// One prefetch stage of a wave: NT weight tiles as the two 16-byte halves a lane loads.
template <int NT>
struct Stage {
  intx4 lo[NT], hi[NT];
};

// Weight loads issued from inline asm, so that the compiler keeps no wait-count bookkeeping for them: with the
// stream running across item boundaries (epilogues, partial-sum stores and item look-ups between the loads and
// their uses) its own bookkeeping ends in s_waitcnt vmcnt(0) at the head of every step, which empties the
// prefetch ring.  The kernel waits by hand (wait_vm<N>, loads complete in issue order) and then passes the stage's
// registers through stage_landed(), an empty asm that the compiler must treat as their definition: nothing may read
// or copy them before.  The registers of a stage in flight must never be spilled or copied, so the kernel has to
// fit its register budget without spills (the build checks that).
// base is wave-uniform, off a per-lane byte offset; the second half of a tile lies 1024 bytes further on.
// s_nop 4: five wait states between a VALU write of the base's SGPRs (v_readlane restoring a spilled SGPR) and the
// vector-memory instruction that reads them; the compiler does not look inside the asm to insert them.
template <bool KEEP>
__device__ __forceinline__ void asm_load_tile(intx4& lo, intx4& hi, const uint8_t* base, uint32_t off) {
  if constexpr (KEEP) {
    asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %2, %3\n\tglobal_load_dwordx4 %1, %2, %3 offset:1024"
                 : "=&v"(lo), "=&v"(hi) : "v"(off), "s"(base) : "memory");
  } else {
    asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %2, %3 nt\n\tglobal_load_dwordx4 %1, %2, %3 offset:1024 nt"
                 : "=&v"(lo), "=&v"(hi) : "v"(off), "s"(base) : "memory");
  }
}
template <int NT>
__device__ __forceinline__ void stage_landed(Stage<NT>& s) {
#pragma unroll
  for (int t = 0; t < NT; ++t) asm volatile("" : "+v"(s.lo[t]), "+v"(s.hi[t]));
}
// Partial sums cross from one block to another, i.e. from one XCD's L2 to another's.  A device-scope fence would do
// (write back / invalidate the whole L2), but hundreds of blocks issuing whole-cache operations serialise on them
// (measured: +300 us per launch).  Instead the partial sums themselves are stored write-through and loaded past
// the caches (sc0 sc1), ordered by the wave's own wait for its stores before the block's counter is incremented.
// base is wave-uniform, off a per-lane byte offset (the s_nop: see asm_load_tile)
__device__ __forceinline__ void store_coherent(const floatx4* base, uint32_t off, floatx4 v) {
  asm volatile("s_nop 4\n\tglobal_store_dwordx4 %0, %1, %2 sc0 sc1" :: "v"(off), "v"(v), "s"(base) : "memory");
}
__device__ __forceinline__ void load_coherent(floatx4& v, const floatx4* base, uint32_t off) {
  asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2 sc0 sc1" : "=&v"(v) : "v"(off), "s"(base) : "memory");
}
// a value the compiler may not hoist, precompute or keep in many registers: redefined where it is used
__device__ __forceinline__ uint32_t opaque(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}

// LDS ring slot of one unit: TT 2-KiB token tile images, one token scale per row (64 per loading wave), and the
// unit's weight scales (lane j of the loading wave brings scale stream j & 1)
template <int TT>
struct TokSlot {
  static constexpr int kScaleWaves = (TT + 3) / 4;
  static constexpr int kWs = TT * 2048 + 256 * kScaleWaves;
  static constexpr int kBytes = kWs + 256;
};
// 64 lanes x 4 bytes from per-lane addresses -> LDS [lds_base, lds_base + 256)
__device__ __forceinline__ void async_load4_ptr(const float* lane_ptr, uint32_t lds_base) {
  asm volatile("s_nop 4\n\ts_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
               :: "s"(lds_base), "v"(lane_ptr) : "memory", "m0");
}

// One contiguous run of K-blocks [kb_lo, kb_hi) of one item; wave-uniform.
using Part = BgmoeSkPart;

__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ uint32_t uniu(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }

// The first unit (item, K-block) whose start cost is >= x, cut at x1 (exclusive).  false: no unit starts in [x, x1).
// s_gpre[g] = cost of all groups before g; all row chunks of a group but its last hold TT token tiles.
template <int TT, int WC>
__device__ __forceinline__ bool locate(const uint32_t* s_gpre, const int32_t* s_cnt, int groups, int ntiles, int KB,
                                       uint32_t x, uint32_t x1, Part& p) {
  const int lane = threadIdx.x & 63;
#pragma unroll 1
  for (int iter = 0; iter < 2; ++iter) {
    if (x >= x1) return false;
    int g = 0;
    for (int g0 = 0; g0 < groups; g0 += 64) {
      const int gi = g0 + lane;
      g += __popcll(__ballot(gi < groups && s_gpre[gi + 1] <= x));
    }
    g = uni(g);
    const int c = uni(s_cnt[g]);
    // inside a group: row chunk by row chunk, each chunk slab by slab.  Blocks that run at the same time then hold
    // the same slab of neighbouring chunks, so a group with several chunks fetches its weights from HBM once
    Part q;
    uint32_t next = 0;
    if (!bgmoe_sk_locate_in_group(BgmoeSkShape{TT, WC}, kCost, g, c, uniu(s_gpre[g]), ntiles, KB, x, x1, &q, &next)) {
      x = next;                           // x lies inside the item's last K-block: the next item's first unit
      continue;
    }
    p.grp = g;
    p.ntile = uni(q.ntile);
    p.chunk = uni(q.chunk);
    p.cnt = c;
    p.kb_lo = uni(q.kb_lo);
    p.kb_hi = uni(q.kb_hi);
    p.start = uniu(q.start);
    p.cpk = uni(q.cpk);
    return true;
  }
  return false;
}

template <int TT, int NSTAGE, bool FUSED, int NT>
__global__ __launch_bounds__(256, 2) void fp8_streamk_kernel(StreamKArgs g) {
  static_assert(TT % 2 == 0, "two half-tile loads per token tile, spread over four waves");
  static_assert(NT == 4 || (!FUSED && NT == 2), "stage 1 pairs two gate and two up tiles per wave");
  static_assert(NSTAGE >= 2, "one stage in flight at least");
  constexpr int NSC = FUSED ? 2 : 1;
  constexpr int WC = 4 * NT;               // weight tiles (2 KiB) per K-block of an item
  constexpr int LT = TT / 2;
  constexpr int kSlot = TokSlot<TT>::kBytes;
  constexpr int WCOLS = 16 * NT;
  constexpr int kItemCols = FUSED ? 128 : 64 * NT;
  constexpr int kSlotVec = TT * NT * 256;  // floatx4 per partial-sum slot
  __shared__ float s_amax[4][TT][16];
  __shared__ __align__(16) uint8_t s_ring[NSTAGE * kSlot];
  __shared__ uint32_t s_gpre[kMaxGroups + 1];
  __shared__ int32_t s_cnt[kMaxGroups];
  // per group: first row, weight and weight-scale base pointers.  The stream switches items without a memory
  // round trip (under load one costs several microseconds of an idle prefetch ring)
  __shared__ int32_t s_row0[kMaxGroups];
  __shared__ uint64_t s_wptr[kMaxGroups][NSC];
  __shared__ uint64_t s_sptr[kMaxGroups][NSC];
  // a cut first part's sums until the share's stream has ended (2 / 4 token tiles: what fits beside the ring with
  // two blocks per CU)
  constexpr int kSaveTiles = NT == 4 ? 2 : 4;
  __shared__ floatx4 s_save[kSaveTiles * NT * 256];
  __shared__ int s_flag[2];
  const uint32_t ring_lds = uniu((uint32_t)(uintptr_t)s_ring);
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const uint32_t wave_u = uniu((uint32_t)wave);
  const int lane = tid & 63;
  const int r16 = lane & 15;
  const int kq = lane >> 4;
  const int K = g.k;
  const int KB = K >> 7;
  const int ntiles = (g.n + kItemCols - 1) / kItemCols;
  const int groups = g.groups;

  const uint64_t t_begin = g.trace ? wall_clock64() : 0;
  // ---- cost table of the launch (every block builds the same one) ----
  if (tid < 64) {
    uint32_t base = 0;
    for (int g0 = 0; g0 < groups; g0 += 64) {
      const int gi = g0 + lane;
      int c = gi < groups ? g.seqlens[gi] : 0;
      if (c < 0 || c > g.hi) c = 0;
      uint32_t inc = (uint32_t)ntiles * (uint32_t)KB * group_cost_per_kb<TT, WC>(c);
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const uint32_t up = (uint32_t)__shfl_up((int)inc, off, BGMOE_WAVE);
        if (lane >= off) inc += up;
      }
      if (gi < groups) {
        s_gpre[gi + 1] = base + inc;
        s_cnt[gi] = c;
      }
      base += (uint32_t)__shfl((int)inc, 63, BGMOE_WAVE);
    }
    if (lane == 0) s_gpre[0] = 0;
  }
  for (int gi = tid; gi < groups; gi += 256) {
    s_row0[gi] = g.cu[gi];
    s_wptr[gi][0] = (uint64_t)(g.w0.w_ptrs ? g.w0.w_ptrs[gi] : g.w0.w + (int64_t)gi * g.w0.w_group_stride);
    s_sptr[gi][0] = (uint64_t)(g.w0.scale_ptrs ? g.w0.scale_ptrs[gi] : g.w0.scale + (int64_t)gi * g.w0.scale_group_stride);
    if constexpr (FUSED) {
      s_wptr[gi][1] = (uint64_t)(g.w1.w_ptrs ? g.w1.w_ptrs[gi] : g.w1.w + (int64_t)gi * g.w1.w_group_stride);
      s_sptr[gi][1] = (uint64_t)(g.w1.scale_ptrs ? g.w1.scale_ptrs[gi] : g.w1.scale + (int64_t)gi * g.w1.scale_group_stride);
    }
  }
  __syncthreads();
  const uint32_t C = uniu(s_gpre[groups]);
  if (C == 0) return;
  // every share is at least one unit's cost, so every share below G has a unit and an item cut over shares
  // b_first..b_last has exactly one part in each of them
  const uint32_t grid = gridDim.x;
  // (and at least kMinUnits of them: a launch too small for that uses fewer blocks rather than cut every item into
  // single K-blocks)
  constexpr uint32_t kMinUnits = 8;
  const uint32_t G = bgmoe_sk_num_shares(C, grid, bgmoe_sk_share_unit(BgmoeSkShape{TT, WC}, kCost), kMinUnits);
  // Blocks of one XCD (blockIdx % 8) own neighbouring shares: an item's parts and the tokens of a group stay in one
  // L2.  A share's size follows its XCD's weight.
  const uint32_t n8 = G >= 8 ? G >> 3 : 1;
  if ((blockIdx.x >> 3) >= n8) return;
  const uint32_t r = (blockIdx.x & 7u) * n8 + (blockIdx.x >> 3);
  if (r >= G) return;
  const uint32_t Wg = bgmoe_sk_cum_weight(g.xcd_w, n8, G);
  const uint32_t x0 = bgmoe_sk_bound(g.xcd_w, n8, Wg, C, r);           // cost at which this share begins ...
  const uint32_t x1 = bgmoe_sk_bound(g.xcd_w, n8, Wg, C, r + 1);       // ... and ends

  // ---- load cursor ----
  Part pl;
  if (!locate<TT, WC>(s_gpre, s_cnt, groups, ntiles, KB, x0, x1, pl)) {
    // A share without a unit: impossible while every share is at least one unit's cost (bgmoe_sk_weights_ok and
    // the choice of G guarantee it; the host-side checks walk the same arithmetic).  Items that span this share
    // would never complete, so say so instead of leaving stale rows silently.
    if (tid == 0 && g.error_flag != nullptr) atomicOr(g.error_flag, 1);
    return;
  }
  const uint8_t* l_wp[NT];
  const float* l_ws;                          // per lane: the scale stream this lane brings
  const uint8_t* l_tok;
  const float* l_xs;
  uint32_t l_tok_off[LT];
  bool l_tok_on[LT];
  uint32_t l_xs_off;
  bool l_keep, l_live = true;
  int kbl;
  const uint32_t lane16 = (uint32_t)lane * 16u;
  auto setup_load = [&]() __attribute__((always_inline)) {
    const int grp = pl.grp;
    const int n0 = pl.ntile * kItemCols;
    const uint8_t* wb0 = reinterpret_cast<const uint8_t*>(s_wptr[grp][0]);
    const float* wsb0 = reinterpret_cast<const float*>(s_sptr[grp][0]);
    const uint8_t* wb1 = wb0;
    const float* wsb1 = wsb0;
    if constexpr (FUSED) {
      wb1 = reinterpret_cast<const uint8_t*>(s_wptr[grp][1]);
      wsb1 = reinterpret_cast<const float*>(s_sptr[grp][1]);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int nrow = FUSED ? n0 + 32 * (int)wave_u + 16 * (t & 1) : n0 + WCOLS * (int)wave_u + 16 * t;
      const int nr = min(nrow, g.n - 16);        // a tile past N streams the last valid one; never stored
      l_wp[t] = uniform_ptr((FUSED && (t >> 1) ? wb1 : wb0) + (int64_t)(nr >> 4) * K * 16);
    }
    // weight scales of the item: stream 0 / 1 = gate / up (stage 1), or the item's first / second 128-column block
    if constexpr (FUSED) {
      l_ws = (lane & 1) ? wsb1 + (int64_t)(n0 >> 7) * g.w1.scale_nb_stride : wsb0 + (int64_t)(n0 >> 7) * g.w0.scale_nb_stride;
    } else {
      const int nb = min(n0 + 128 * (lane & 1), g.n - 1) >> 7;
      l_ws = wsb0 + (int64_t)nb * g.w0.scale_nb_stride;
    }
    const int64_t row0 = uni(s_row0[grp]);
    const int t0 = pl.chunk * 16 * TT;
    const int live = pl.cnt - t0;
    const int tiles = min(TT, (live + 15) >> 4);
    l_tok = uniform_ptr(g.a.x + (row0 + t0) * K);
#pragma unroll
    for (int i = 0; i < LT; ++i) {
      const int h = (int)wave_u * LT + i;
      const int row = min(8 * h + (lane >> 3), live - 1);
      l_tok_off[i] = (uint32_t)row * (uint32_t)K + (uint32_t)(((lane & 7) ^ (lane >> 3)) * 16);
      l_tok_on[i] = (h >> 1) < tiles;
    }
    l_xs = uniform_ptr(g.a.scale_group_stride
                           ? g.a.scale + grp * g.a.scale_group_stride + (int64_t)t0 * g.a.scale_row_stride
                           : g.a.scale + (row0 + t0) * g.a.scale_row_stride);
    l_xs_off = (uint32_t)min(64 * (int)wave_u + lane, live - 1) * (uint32_t)g.a.scale_row_stride * 4u;
    l_keep = pl.cnt > 16 * TT;                   // more row chunks stream the same weights: keep them cacheable
    kbl = pl.kb_lo;
  };
  setup_load();

  using St = Stage<NT>;
  St st[NSTAGE];
  // Loads of one unit: tokens and weight scales (both asynchronous, into ring slot `slot`), weights.  Nothing is
  // issued once the share is exhausted.
  auto issue = [&](St& s, int slot) __attribute__((always_inline)) {
    if (!l_live) return;
    const uint32_t sb = ring_lds + (uint32_t)slot * kSlot;
    // (the asm operands must be SGPRs: say once more that they are uniform, whatever registers the compiler kept
    // the cursor in)
    const uint8_t* tokp = uniform_ptr(l_tok + (kbl << 7));
#pragma unroll
    for (int i = 0; i < LT; ++i)
      if (l_tok_on[i]) async_load16(tokp, l_tok_off[i], uniu(sb + (wave_u * LT + i) * 1024));
    if (wave_u < (uint32_t)TokSlot<TT>::kScaleWaves)
      async_load4(uniform_ptr(l_xs + (int64_t)kbl * g.a.scale_kb_stride), l_xs_off, uniu(sb + TT * 2048 + wave_u * 256));
    if (wave_u == 3u) async_load4_ptr(l_ws + kbl, uniu(sb + TokSlot<TT>::kWs));
    const uint32_t off = ((uint32_t)kbl << 11) + lane16;
    if (l_keep) {
#pragma unroll
      for (int t = 0; t < NT; ++t) asm_load_tile<true>(s.lo[t], s.hi[t], uniform_ptr(l_wp[t]), off);
    } else {
#pragma unroll
      for (int t = 0; t < NT; ++t) asm_load_tile<false>(s.lo[t], s.hi[t], uniform_ptr(l_wp[t]), off);
    }
    // advance
    if (kbl + 1 < pl.kb_hi) {
      ++kbl;
    } else {
      Part nx;
      if (locate<TT, WC>(s_gpre, s_cnt, groups, ntiles, KB, pl.start + (uint32_t)pl.kb_hi * (uint32_t)pl.cpk, x1, nx)) {
        pl = nx;
        setup_load();
      } else {
        l_live = false;
      }
    }
  };

  // ---- compute cursor ----
  Part pc = pl;
  int kbc = pc.kb_lo;
  int c_tiles, c_live, c_t0, c_n0;
  int64_t c_row0;
  auto setup_compute = [&]() __attribute__((always_inline)) {
    c_row0 = uni(s_row0[pc.grp]);
    c_t0 = pc.chunk * 16 * TT;
    c_live = pc.cnt - c_t0;
    c_tiles = min(TT, (c_live + 15) >> 4);
    c_n0 = pc.ntile * kItemCols;
    kbc = pc.kb_lo;
  };
  setup_compute();
  if (g.trace && tid == 0) {
    g.trace[4 * r] = t_begin;
    g.trace[4 * r + 1] = wall_clock64();
  }

  floatx4 acc[TT][NT];
  auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[tt][t] = floatx4{0.f, 0.f, 0.f, 0.f};
  };
  zero_acc();

  const int sw_lo = r16 * 128 + ((kq ^ (r16 & 7)) * 16);
  auto compute = [&](const St& c, int slot) __attribute__((always_inline)) {
    const uint8_t* b = s_ring + slot * kSlot;
    const float* bxs = reinterpret_cast<const float*>(b + TT * 2048);
    const float* bws = reinterpret_cast<const float*>(b + TokSlot<TT>::kWs);
    float ws[NSC];
#pragma unroll
    for (int i = 0; i < NSC; ++i) ws[i] = bws[FUSED ? i : (WCOLS * wave >= 128 ? 1 : 0)];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      if (tt < c_tiles) {
        const intx4 lo = *reinterpret_cast<const intx4*>(b + tt * 2048 + sw_lo);
        const intx4 hi = *reinterpret_cast<const intx4*>(b + tt * 2048 + (sw_lo ^ 64));
        const intx8 B = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        const float xs = bxs[16 * tt + r16];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          const intx8 A = intx8{c.lo[t][0], c.lo[t][1], c.lo[t][2], c.lo[t][3],
                                c.hi[t][0], c.hi[t][1], c.hi[t][2], c.hi[t][3]};
          const floatx4 p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
              A, B, floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
          const float sc = xs * ws[FUSED ? (t >> 1) : 0];
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[tt][t][i] = fmaf(p[i], sc, acc[tt][t][i]);
        }
        // one token tile at a time: the scheduler would otherwise issue all TT*NT MFMAs first and keep their
        // results (4 registers each) alive together
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  auto epilogue = [&]() __attribute__((always_inline)) {
    bool xv[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) xv[tt] = 16 * tt + r16 < c_live;
    if constexpr (FUSED) {
      // the bf16-rounded products, kept as packed pairs across the amax exchange (half the registers)
      uint32_t pk[TT][2][2];
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        float am = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const uint32_t w = pack2_bf16(silu_f32(acc[tt][j][2 * i]) * acc[tt][j + 2][2 * i],
                                          silu_f32(acc[tt][j][2 * i + 1]) * acc[tt][j + 2][2 * i + 1]);
            pk[tt][j][i] = w;
            am = fmaxf(am, fmaxf(fabsf(bf16_bits_to_f32(w & 0xffffu)), fabsf(bf16_bits_to_f32(w >> 16))));
          }
        const int tok = c_t0 + 16 * tt + r16;
        if (g.out != nullptr && xv[tt]) {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            uint2 o;
            o.x = pk[tt][j][0];
            o.y = pk[tt][j][1];
            *reinterpret_cast<uint2*>(g.out + (c_row0 + tok) * g.n + c_n0 + 32 * wave + 16 * j + 4 * kq) = o;
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
          const int tok = c_t0 + 16 * tt + r16;
          if (xv[tt]) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const float hv[4] = {bf16_bits_to_f32(pk[tt][j][0] & 0xffffu), bf16_bits_to_f32(pk[tt][j][0] >> 16),
                                   bf16_bits_to_f32(pk[tt][j][1] & 0xffffu), bf16_bits_to_f32(pk[tt][j][1] >> 16)};
              float qv[4];
              quant_div_clamp(hv, sc, qv);
              const uint32_t q = pack4_e4m3(qv[0], qv[1], qv[2], qv[3]);
              *reinterpret_cast<uint32_t*>(g.out_q + (c_row0 + tok) * g.n + c_n0 + 32 * wave + 16 * j + 4 * kq) = q;
            }
            if (wave == 0 && kq == 0)
              g.out_s[(c_row0 + tok) * g.os_row + (int64_t)(c_n0 >> 7) * g.os_nb] = sc;
          }
        }
        __syncthreads();                       // s_amax is written again by the next item's epilogue
      }
    } else {
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        const int tok = c_t0 + 16 * tt + r16;
        if (!xv[tt]) continue;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          if (c_n0 + WCOLS * wave + 16 * t >= g.n) continue;
          uint2 o;
          o.x = pack2_bf16(acc[tt][t][0], acc[tt][t][1]);
          o.y = pack2_bf16(acc[tt][t][2], acc[tt][t][3]);
          *reinterpret_cast<uint2*>(g.out + (c_row0 + tok) * g.n + c_n0 + WCOLS * wave + 16 * t + 4 * kq) = o;
        }
      }
    }
  };

  // ---- items cut over several shares -------------------------------------------------------------------
  // A share has at most two cut parts: its first (the item began in an earlier share) and its last (the item goes
  // on in a later one).  Nothing that belongs to them may hold up the stream: vector-memory operations complete
  // in order, so a store of partial sums in mid-stream would have to land before any younger weight load could be
  // waited for -- a round trip of idle prefetch ring (measured: 15 us per launch).  So the first part's sums wait
  // in LDS and the last part's stay in registers until the share's stream has ended.  Then the block stores both
  // to their slots (write-through), waits, and adds 1 to each item's counter (at the index of the share the item
  // begins in).  The block whose increment completes an item's count adds the other parts' slots to its own sums
  // IN SHARE ORDER and runs the epilogue; it leaves the counter at zero.  Nobody waits for another block.
  auto first_block = [&](const Part& p) __attribute__((always_inline)) {
    return uniu(bgmoe_sk_share_of_cost(g.xcd_w, n8, Wg, C, p.start));
  };
  auto last_block = [&](const Part& p) __attribute__((always_inline)) {
    return uniu(bgmoe_sk_share_of_cost(g.xcd_w, n8, Wg, C, p.start + (uint32_t)(KB - 1) * (uint32_t)p.cpk));
  };
  Part cut_head = pc;
  bool has_head = false, has_tail = false, head_saved = false;
  int head_tiles = 0;
  const uint32_t lane_off16 = (uint32_t)tid * 16u;
  auto finish = [&]() __attribute__((always_inline)) {
    if (pc.kb_lo == 0 && pc.kb_hi == KB) {
      epilogue();
      zero_acc();
    } else if (pc.kb_lo > 0) {
      cut_head = pc;
      has_head = true;
      head_tiles = c_tiles;
      head_saved = c_tiles <= kSaveTiles;
      if (head_saved) {
#pragma unroll
        for (int tt = 0; tt < kSaveTiles; ++tt)
          if (tt < c_tiles) {
#pragma unroll
            for (int t = 0; t < NT; ++t) s_save[(tt * NT + t) * 256 + tid] = acc[tt][t];
          }
      } else {                                 // too many rows for the LDS copy: store now, at the price of the stall
        const floatx4* mine = uniform_ptr(g.slots + (size_t)(2 * r) * kSlotVec);
        const uint32_t lo = opaque(lane_off16);
#pragma unroll
        for (int tt = 0; tt < TT; ++tt)
          if (tt < c_tiles) {
#pragma unroll
            for (int t = 0; t < NT; ++t) store_coherent(mine, lo + (uint32_t)(tt * NT + t) * 4096u, acc[tt][t]);
          }
      }
      zero_acc();
    } else {
      has_tail = true;                         // the share ends here; the sums stay in registers
    }
  };
  // acc += one part's slot, two token tiles per round trip (registers: the loads' destinations must never spill)
  auto add_slot = [&](const floatx4* slot) __attribute__((always_inline)) {
    const floatx4* sl = uniform_ptr(slot);
    const uint32_t lo = opaque(lane_off16);
#pragma unroll
    for (int t0 = 0; t0 < TT; t0 += 2) {
      if (t0 < c_tiles) {
        floatx4 v[2][NT];
#pragma unroll
        for (int u = 0; u < 2; ++u)
          if (t0 + u < c_tiles) {
#pragma unroll
            for (int t = 0; t < NT; ++t) load_coherent(v[u][t], sl, lo + (uint32_t)((t0 + u) * NT + t) * 4096u);
          }
        wait_vm<0>();
#pragma unroll
        for (int u = 0; u < 2; ++u)
          if (t0 + u < c_tiles) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
              asm volatile("" : "+v"(v[u][t]));
#pragma unroll
              for (int i = 0; i < 4; ++i) acc[t0 + u][t][i] += v[u][t][i];
            }
          }
      }
    }
  };
  auto settle = [&]() __attribute__((always_inline)) {
    if (has_head && head_saved) {
      const floatx4* mine = uniform_ptr(g.slots + (size_t)(2 * r) * kSlotVec);
      const uint32_t lo = opaque(lane_off16);
#pragma unroll
      for (int tt = 0; tt < kSaveTiles; ++tt)
        if (tt < head_tiles) {
#pragma unroll
          for (int t = 0; t < NT; ++t)
            store_coherent(mine, lo + (uint32_t)(tt * NT + t) * 4096u, s_save[(tt * NT + t) * 256 + tid]);
        }
    }
    if (has_tail) {                            // pc is still the share's last part, its sums in acc
      const floatx4* mine = uniform_ptr(g.slots + (size_t)(2 * r + 1) * kSlotVec);
      const uint32_t lo = opaque(lane_off16);
#pragma unroll
      for (int tt = 0; tt < TT; ++tt)
        if (tt < c_tiles) {
#pragma unroll
          for (int t = 0; t < NT; ++t) store_coherent(mine, lo + (uint32_t)(tt * NT + t) * 4096u, acc[tt][t]);
        }
    }
    wait_vm<0>();                              // this wave's partial sums are in memory (and its LDS writes done) ...
    __syncthreads();                           // ... and so are the other waves'
    if (!has_head && !has_tail) return;
    const uint32_t head_bf = has_head ? first_block(cut_head) : 0;
    if (tid == 1 && has_head) s_flag[0] = atomicAdd(&g.counters[head_bf], 1);
    if (tid == 0 && has_tail) s_flag[1] = atomicAdd(&g.counters[r], 1);
    __syncthreads();
    if (has_tail) {
      const uint32_t bl = last_block(pc);
      if (uni(s_flag[1]) == (int)(bl - r)) {
        for (uint32_t b2 = r + 1; b2 <= bl; ++b2) add_slot(g.slots + (size_t)(2 * b2) * kSlotVec);
        if (tid == 0) atomicExch(&g.counters[r], 0);
        epilogue();
      }
    }
    if (has_head) {
      const uint32_t bl = last_block(cut_head);
      if (uni(s_flag[0]) == (int)(bl - head_bf)) {
        pc = cut_head;
        setup_compute();
        zero_acc();
        for (uint32_t b2 = head_bf; b2 <= bl; ++b2) {
          if (b2 == r && head_saved) {
#pragma unroll
            for (int tt = 0; tt < kSaveTiles; ++tt)
              if (tt < c_tiles) {
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                  const floatx4 v = s_save[(tt * NT + t) * 256 + tid];
#pragma unroll
                  for (int i = 0; i < 4; ++i) acc[tt][t][i] += v[i];
                }
              }
          } else {
            add_slot(g.slots + (size_t)(2 * b2 + (b2 > head_bf ? 0 : 1)) * kSlotVec);
          }
        }
        if (tid == 0) atomicExch(&g.counters[head_bf], 0);
        epilogue();
      }
    }
  };

  // ---- the stream: NSTAGE-1 units ahead, across item boundaries ----
  // Loads complete in issue order.  Before step s the units s .. s+NSTAGE-2 are in flight; unit s has landed once at
  // most the NSTAGE-2 younger units' weight loads are outstanding (their token loads, not counted, only make the
  // wait stricter).  Once the load cursor has run out fewer units are in flight than that count assumes, and the
  // wait is for everything.  The barrier extends the wait to the other waves' token loads and says that the ring
  // slot refilled next is no longer read.
#pragma unroll
  for (int s = 0; s < NSTAGE - 1; ++s) issue(st[s], s);
  for (;;) {
#pragma unroll
    for (int s = 0; s < NSTAGE; ++s) {
      if (l_live) wait_vm<(NSTAGE - 2) * 2 * NT>();
      else wait_vm<0>();
      block_barrier();
      stage_landed(st[s]);
      issue(st[(s + NSTAGE - 1) % NSTAGE], (s + NSTAGE - 1) % NSTAGE);
      compute(st[s], s);
      if (++kbc == pc.kb_hi) {
        finish();
        if (!locate<TT, WC>(s_gpre, s_cnt, groups, ntiles, KB, pc.start + (uint32_t)pc.kb_hi * (uint32_t)pc.cpk, x1, pc))
          goto done;
        setup_compute();
      }
    }
  }
done:
  if (g.trace && tid == 0) g.trace[4 * r + 2] = wall_clock64();
  settle();
  if (g.trace && tid == 0) g.trace[4 * r + 3] = wall_clock64();                                    // (its wait also covers the asynchronous LDS writes)
}

template <typename Kern>
unsigned resident(Kern kernel, unsigned* cache) {
  if (*cache == 0) {
    int per_cu = 0, dev = 0, cus = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, 0) != hipSuccess || per_cu < 1) per_cu = 1;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1)
      cus = 256;
    unsigned v = (unsigned)(per_cu * cus) & ~7u;
    if (v > 1024) v = 1024;
    if (v == 0) v = 8;
    *cache = v;
  }
  return *cache;
}

// launch shapes: stage 1 = 64-row chunks, 128 gate + 128 up columns; plain GEMM = 64-row chunks, kDownNT*64 columns
#ifndef BGMOE_SK_S1_NS
#define BGMOE_SK_S1_NS 2
#endif
#ifndef BGMOE_SK_S1_TT
#define BGMOE_SK_S1_TT 4
#endif
constexpr int kS1TT = BGMOE_SK_S1_TT, kS1NS = BGMOE_SK_S1_NS;
#ifndef BGMOE_SK_DOWN_NT
#define BGMOE_SK_DOWN_NT 2
#endif
#ifndef BGMOE_SK_DOWN_NS
#define BGMOE_SK_DOWN_NS 4
#endif
constexpr int kDownTT = 4, kDownNS = BGMOE_SK_DOWN_NS, kDownNT = BGMOE_SK_DOWN_NT;
unsigned g_res_s1 = 0, g_res_down = 0;

unsigned grid_s1() { return resident(fp8_streamk_kernel<kS1TT, kS1NS, true, 4>, &g_res_s1); }
unsigned grid_down() { return resident(fp8_streamk_kernel<kDownTT, kDownNS, false, kDownNT>, &g_res_down); }

constexpr size_t kCounterBytes = 4096;         // 1024 counters
uint64_t* g_trace = nullptr;
// Sticky status word of the balanced launches on this device (one copy per GPU, at its own address there).
__device__ int32_t g_sk_status_word;
constexpr int kMaxDevices = 16;
int32_t* g_sk_status_ptr[kMaxDevices] = {};
int32_t* status_ptr() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  if (g_sk_status_ptr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_sk_status_word)) != hipSuccess) return nullptr;
    g_sk_status_ptr[dev] = static_cast<int32_t*>(p);
  }
  return g_sk_status_ptr[dev];
}
// measured on MI355X: the odd XCDs stream about 9% slower than the even ones
int g_xcd_w[8] = {23, 21, 23, 21, 23, 21, 23, 21};

}  // namespace

// Tuning aid (no reference counterpart): with a device buffer of 4 * 1024 uint64 set, every share of the next
// balanced launches records the constant-rate clock at its start, before its first unit, at the end of its stream
// and at its end.  NULL switches it off.
extern "C" int bgmoe_debug_streamk_trace(uint64_t* device_buffer) {
  g_trace = device_buffer;
  return BGMOE_OK;
}

// Tuning knob (no reference counterpart): relative share sizes of the eight XCDs, each in [1, 64] and their sum at
// most 32 times the smallest: the share count is sized from the AVERAGE share, and a share far below the average
// could fall under the cost of one unit, own nothing, and leave the items that span it unfinished.
extern "C" int bgmoe_set_streamk_xcd_weights(const int* w) {
  BGMOE_REQUIRE(w != nullptr, "set_streamk_xcd_weights: null");
  int ww[8];
  for (int i = 0; i < 8; ++i) {
    BGMOE_REQUIRE(w[i] >= 1 && w[i] <= 64, "set_streamk_xcd_weights: weight %d outside [1,64]", w[i]);
    ww[i] = w[i];
  }
  BGMOE_REQUIRE(bgmoe_sk_weights_ok(ww), "set_streamk_xcd_weights: the weights' sum exceeds 32 times the smallest one "
                "(the lightest XCD's shares could fall below one unit of work)");
  for (int i = 0; i < 8; ++i) g_xcd_w[i] = w[i];
  return BGMOE_OK;
}

// Debug aid (no reference counterpart): reads the device's sticky status word of the balanced launches into
// *host_out and clears it; synchronises the device.  Bit 0: a share found no unit of work (its items' rows are
// stale).  The share arithmetic makes that impossible for accepted XCD weights; the word exists so that a
// violation would be seen rather than silently produce stale rows.
extern "C" int bgmoe_debug_streamk_status(int32_t* host_out) {
  BGMOE_REQUIRE(host_out != nullptr, "debug_streamk_status: null");
  int32_t* p = status_ptr();
  if (p == nullptr) {
    bgmoe_set_error("debug_streamk_status: cannot locate the status word");
    return BGMOE_ERR_HIP;
  }
  const int32_t zero = 0;
  if (hipMemcpy(host_out, p, sizeof(int32_t), hipMemcpyDeviceToHost) != hipSuccess ||
      hipMemcpy(p, &zero, sizeof(int32_t), hipMemcpyHostToDevice) != hipSuccess) {
    bgmoe_set_error("debug_streamk_status: copy failed");
    return BGMOE_ERR_HIP;
  }
  return BGMOE_OK;
}

int bgmoe_internal_init_fp8_streamk() {
  grid_s1();
  grid_down();
  (void)status_ptr();              // resolve this device's status word here, not inside a launch a caller may be capturing
  return BGMOE_OK;
}

extern "C" size_t bgmoe_fp8_streamk_workspace_bytes(void) {
  const size_t s1 = (size_t)2 * grid_s1() * (kS1TT * 4 * 256) * sizeof(floatx4);
  const size_t dn = (size_t)2 * grid_down() * (kDownTT * kDownNT * 256) * sizeof(floatx4);
  return kCounterBytes + (s1 > dn ? s1 : dn);
}

// BGMOE_OK: launched.  BGMOE_ERR_WORKSPACE (without an error message): this form does not apply, the caller
// takes the item-per-block kernel.
int bgmoe_internal_fp8_streamk(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* w0, const bgmoe_fp8_weight* w1,
                               const int32_t* seqlens, const int32_t* cu, int groups, int n, int k, uint16_t* out,
                               uint8_t* out_q, float* out_s, int64_t os_row, int64_t os_nb, int hi, int64_t row_bound,
                               void* ws, size_t ws_bytes, hipStream_t st) {
  const bool fused = w1 != nullptr;
  if (ws == nullptr || (uintptr_t)ws % 16 != 0 || ws_bytes < bgmoe_fp8_streamk_workspace_bytes()) return BGMOE_ERR_WORKSPACE;
  if (w0->layout != BGMOE_W_TILE_MAJOR || (fused && w1->layout != BGMOE_W_TILE_MAJOR)) return BGMOE_ERR_WORKSPACE;
  if (groups > kMaxGroups || cu == nullptr || hi <= 0) return BGMOE_ERR_WORKSPACE;
  const int tt = fused ? kS1TT : kDownTT, nt = fused ? 4 : kDownNT;
  const int item_cols = fused ? 128 : 64 * nt;
  const int64_t ntiles = (n + item_cols - 1) / item_cols;
  // the cumulative cost must fit 32 bits with room for the share arithmetic
  const int64_t chunks = groups + row_bound / (16 * tt), tiles = groups + row_bound / 16;
  if (ntiles * (k >> 7) * (chunks * 4 * nt * kCostW + tiles * kCostT) >= (int64_t)1 << 31) return BGMOE_ERR_WORKSPACE;
  StreamKArgs g{};
  g.a = *a; g.w0 = *w0; if (fused) g.w1 = *w1;
  g.seqlens = seqlens; g.cu = cu; g.groups = groups; g.n = n; g.k = k;
  g.out = out; g.out_q = out_q; g.out_s = out_s; g.os_row = os_row; g.os_nb = os_nb; g.hi = hi;
  g.trace = g_trace;
  g.error_flag = status_ptr();
  for (int i = 0; i < 8; ++i) g.xcd_w[i] = g_xcd_w[i];
  g.counters = reinterpret_cast<int32_t*>(ws);
  g.slots = reinterpret_cast<floatx4*>(reinterpret_cast<uint8_t*>(ws) + kCounterBytes);
  if (fused)
    hipLaunchKernelGGL((fp8_streamk_kernel<kS1TT, kS1NS, true, 4>), dim3(grid_s1()), dim3(256), 0, st, g);
  else
    hipLaunchKernelGGL((fp8_streamk_kernel<kDownTT, kDownNS, false, kDownNT>), dim3(grid_down()), dim3(256), 0, st, g);
  return bgmoe_check_launch("fp8 grouped gemm (stream-K)");
}
