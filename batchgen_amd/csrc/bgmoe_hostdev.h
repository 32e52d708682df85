// Index and address arithmetic that the kernels share with host-compiled checks.
//
// Everything here is plain C++ over fixed-width integers: hipcc compiles it for the device (and the host), g++
// compiles the same text into the host-side check library (csrc/hostcheck.cc), whose tests walk the arithmetic
// over random launches on the CPU.  A kernel that needs one of these computations calls the function here
// instead of writing it out again: what the CPU tests pin is then what the GPU runs.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define BGMOE_HD __host__ __device__ __forceinline__
#else
#define BGMOE_HD inline
#endif

// ---- 64-bit values from 32-bit halves ----------------------------------------------------------------------
// Both halves are taken as UNSIGNED 32-bit parameters, whatever the caller's expression type is: the wave
// builtins (readfirstlane, readlane) return `int`, and an `int` low half widened to 64 bits sign-extends, which
// turns every address with bit 31 set into an unmapped one.  Going through these parameters converts modulo 2^32
// first.
BGMOE_HD uint64_t bgmoe_compose_u64(uint32_t lo, uint32_t hi) { return ((uint64_t)hi << 32) | (uint64_t)lo; }

// Lowest and highest byte a launch addresses through `base`: rows [0, rows) of `row_bytes` bytes at a pitch of
// `pitch_bytes`.  Host-side launch checks compare this range with the allocation before anything is enqueued.
struct BgmoeByteRange { uint64_t lo, hi; };           // [lo, hi): hi == lo for an empty range
BGMOE_HD BgmoeByteRange bgmoe_rows_range(uint64_t base, uint64_t rows, uint64_t row_bytes, uint64_t pitch_bytes) {
  BgmoeByteRange r{base, base};
  if (rows != 0 && row_bytes != 0) r.hi = base + (rows - 1) * pitch_bytes + row_bytes;
  return r;
}
BGMOE_HD bool bgmoe_range_inside(BgmoeByteRange r, uint64_t alloc_base, uint64_t alloc_bytes) {
  return r.lo >= alloc_base && r.hi >= r.lo && r.hi <= alloc_base + alloc_bytes;
}

// ---- balanced (stream-K) weight-streaming GEMM: shares of the cumulative cost --------------------------------
// The launch's work is the sequence of units (item, K-block); an item is (group, row chunk, column slab) and its
// units follow each other in K.  Inside a group the order is row chunk by row chunk, each chunk slab by slab.
// Every unit has a cost; share r of G owns the units whose START cost lies in [bound(r), bound(r+1)).
struct BgmoeSkCost { int w, r, t; };   // per 2-KiB tile: weights first stream / re-stream for a later chunk / tokens
struct BgmoeSkShape { int tt, wc; };   // token tiles (16 rows) per row chunk; weight tiles per K-block of an item

// cost of ONE K-block of ALL chunks of one slab of a group with c rows
BGMOE_HD uint32_t bgmoe_sk_group_cost_per_kb(BgmoeSkShape s, BgmoeSkCost k, int c) {
  if (c <= 0) return 0;
  const int chunks = (c + 16 * s.tt - 1) / (16 * s.tt);
  const int tiles_g = (c + 15) >> 4;
  return (uint32_t)(s.wc * (k.w + (chunks - 1) * k.r) + tiles_g * k.t);
}
// the most a single unit can cost (a full first chunk), and the figure the share count is sized with: that plus one
// weight tile, so that the rounding of a share's two bounds cannot take it below a whole unit
BGMOE_HD uint32_t bgmoe_sk_max_unit_cost(BgmoeSkShape s, BgmoeSkCost k) { return (uint32_t)(s.wc * k.w + s.tt * k.t); }
BGMOE_HD uint32_t bgmoe_sk_share_unit(BgmoeSkShape s, BgmoeSkCost k) { return bgmoe_sk_max_unit_cost(s, k) + (uint32_t)k.w; }

// Shares are numbered XCD by XCD (n8 per XCD); a share of XCD x weighs w[x].  Weight of shares 0..r-1:
BGMOE_HD uint32_t bgmoe_sk_cum_weight(const int (&w)[8], uint32_t n8, uint32_t r) {
  uint32_t sum = 0, left = r;
#if defined(__HIPCC__)
#pragma unroll
#endif
  for (int x = 0; x < 8; ++x) {
    const uint32_t take = left < n8 ? left : n8;
    sum += take * (uint32_t)w[x];
    left -= take;
  }
  return sum;
}
// the last share r with cum_weight(r) <= t (t < the total weight)
BGMOE_HD uint32_t bgmoe_sk_share_of_weight(const int (&w)[8], uint32_t n8, uint32_t t) {
  uint32_t r = 0;
#if defined(__HIPCC__)
#pragma unroll
#endif
  for (int x = 0; x < 8; ++x) {
    const uint32_t seg = n8 * (uint32_t)w[x];
    if (t >= seg && x < 7) {
      t -= seg;
      r += n8;
    } else {
      const uint32_t q = t / (uint32_t)w[x];
      return r + (q < n8 - 1 ? q : n8 - 1);
    }
  }
  return r;
}
// Number of shares for a launch of cumulative cost C on `grid` blocks: a multiple of 8 (or 1), every share at
// least min_units times share_unit (bgmoe_sk_share_unit) ON AVERAGE.  Weighted shares are smaller than the average by up to
// 8 * wmin / sum(w); bgmoe_sk_weights_ok() bounds that factor so that the smallest share still holds a unit.
BGMOE_HD uint32_t bgmoe_sk_num_shares(uint32_t C, uint32_t grid, uint32_t share_unit, uint32_t min_units) {
  uint32_t G = C / (share_unit * min_units);
  return G < 8 ? 1u : (G > grid ? grid : G) & ~7u;
}
// With min_units = 8 the smallest share is >= 8 * max_unit * 8 * wmin / sum(w) minus one for the rounding of
// its two bounds; requiring sum(w) <= 32 * wmin leaves it at two units' cost or more.
BGMOE_HD bool bgmoe_sk_weights_ok(const int (&w)[8]) {
  int sum = 0, wmin = w[0];
  for (int x = 0; x < 8; ++x) {
    if (w[x] < 1 || w[x] > 64) return false;
    sum += w[x];
    if (w[x] < wmin) wmin = w[x];
  }
  return sum <= 32 * wmin;
}
// cost at which share r begins (r == G: the total cost C); Wg = cum_weight(G)
BGMOE_HD uint32_t bgmoe_sk_bound(const int (&w)[8], uint32_t n8, uint32_t Wg, uint32_t C, uint32_t r) {
  return (uint32_t)(((uint64_t)bgmoe_sk_cum_weight(w, n8, r) * C + Wg - 1) / Wg);
}
// share that holds cost position x (the share an item "begins in" / "ends in")
BGMOE_HD uint32_t bgmoe_sk_share_of_cost(const int (&w)[8], uint32_t n8, uint32_t Wg, uint32_t C, uint32_t x) {
  return bgmoe_sk_share_of_weight(w, n8, (uint32_t)(((uint64_t)x * Wg) / C));
}

// One contiguous run of K-blocks [kb_lo, kb_hi) of one item.
struct BgmoeSkPart {
  int grp, ntile, chunk, cnt;
  int kb_lo, kb_hi;
  uint32_t start;             // cumulative cost at the item's first K-block
  int cpk;                    // cost of one K-block of this item
};
// The unit search inside group g (c rows, its first unit at cost gpre): the first unit whose start cost is >= x,
// cut at x1 (exclusive).  Returns 1 and fills p; or returns 0 with *next = the start cost of the next item when x
// lies inside the last K-block of an item (the caller looks again from there, possibly in the next group).
BGMOE_HD int bgmoe_sk_locate_in_group(BgmoeSkShape s, BgmoeSkCost k, int g, int c, uint32_t gpre, int ntiles, int KB,
                                      uint32_t x, uint32_t x1, BgmoeSkPart* p, uint32_t* next) {
  const int chunks = (c + 16 * s.tt - 1) / (16 * s.tt);
  const int tiles_g = (c + 15) >> 4;
  const uint32_t slabs = (uint32_t)ntiles * (uint32_t)KB;
  const uint32_t f0 = slabs * (uint32_t)(s.wc * k.w + s.tt * k.t);             // a full first chunk, all slabs
  const uint32_t fl = slabs * (uint32_t)(s.wc * k.r + s.tt * k.t);             // a full later chunk
  uint32_t r = x - gpre;
  uint32_t ch = 0;
  if (chunks > 1 && r >= f0) {
    r -= f0;
    ch = r / fl;
    if (ch > (uint32_t)(chunks - 2)) ch = (uint32_t)(chunks - 2);
    r -= ch * fl;
    ch += 1;
  }
  const int rest = tiles_g - (int)ch * s.tt;
  const int tl = s.tt < rest ? s.tt : rest;
  const int cpk = s.wc * (ch == 0 ? k.w : k.r) + tl * k.t;
  const uint32_t ci = (uint32_t)KB * (uint32_t)cpk;                            // one item of this chunk
  const uint32_t nt = r / ci;
  r -= nt * ci;
  const uint32_t kb = (r + (uint32_t)cpk - 1) / (uint32_t)cpk;
  const uint32_t start = x - r;
  if (kb >= (uint32_t)KB) {             // x lies inside the item's last K-block: the next item's first unit
    *next = start + (uint32_t)KB * (uint32_t)cpk;
    return 0;
  }
  const uint32_t hi = (x1 - start + (uint32_t)cpk - 1) / (uint32_t)cpk;
  p->grp = g;
  p->ntile = (int)nt;
  p->chunk = (int)ch;
  p->cnt = c;
  p->kb_lo = (int)kb;
  p->kb_hi = (int)(hi < (uint32_t)KB ? hi : (uint32_t)KB);
  p->start = start;
  p->cpk = cpk;
  return 1;
}

// ---- weight-streaming grouped GEMMs: work items ------------------------------------------------------------------------
// A group's rows are cut into chunks of chunk_rows rows; an item is (group, chunk, n-tile) and streams the n-tile's
// weights once.  Groups with more than tall.min_rows rows (0: no such groups) are cut into chunks of tall.rows rows
// instead: half as many passes over their weights for twice the accumulators.
struct BgmoeTall { int min_rows, rows; };
BGMOE_HD int bgmoe_item_rows(int cnt, int chunk_rows, BgmoeTall tall) {
  return tall.min_rows > 0 && cnt > tall.min_rows ? tall.rows : chunk_rows;
}
BGMOE_HD int bgmoe_item_chunks(int cnt, int chunk_rows, BgmoeTall tall) {
  const int r = bgmoe_item_rows(cnt, chunk_rows, tall);
  return (cnt + r - 1) / r;
}
// XCD-aware slot -> (n-tile, chunk) map inside one group.  Blocks are dispatched round-robin over the 8 XCDs (block b
// runs on XCD b % 8), each with its own L2.  A group with several chunks streams the same weight tile once per chunk;
// the map puts all chunks of one n-tile on the SAME XCD in neighbouring blocks: slot q of the group (q = chunk-row *
// ntiles_pad + block % ntiles_pad, ntiles_pad = n-tiles rounded up to 8 so that every group starts on XCD 0) ->
// n-tile 8 * (q / (8 * chunks)) + q % 8, chunk (q / 8) % chunks.  An n-tile >= the real count is padding.
struct BgmoeItemSlot { int ntile, chunk; };
BGMOE_HD BgmoeItemSlot bgmoe_item_slot(int crow, int chunks, int ntiles_pad, unsigned block) {
  const int q = crow * ntiles_pad + (int)(block % (unsigned)ntiles_pad);
  return BgmoeItemSlot{8 * (q / (8 * chunks)) + (q & 7), (q >> 3) % chunks};
}
// Upper bound on the virtual blocks of a launch from host-side knowledge only: `row_bound` bounds the total live
// rows, `max_rows` the rows of any group the launch serves.  Tall items only lower the count (tall.rows >= chunk_rows).
BGMOE_HD unsigned bgmoe_item_grid(int ntiles, int groups, int64_t row_bound, int max_rows, int chunk_rows) {
  int64_t items = groups + row_bound / chunk_rows;                 // >= sum of ceil(count / chunk_rows)
  const int64_t per_group = (int64_t)groups * (((int64_t)max_rows + chunk_rows - 1) / chunk_rows);
  if (per_group < items) items = per_group;
  return (unsigned)(((ntiles + 7) & ~7) * items);
}

// ---- LDS-tiled grouped GEMM: the persistent blocks' walk over the work items ------------------------------------------
// Work items are (group, m-tile, n-tile); `tiles` is the exclusive prefix of m-tiles per group (tiles[groups] = all),
// ntn the n-tiles of the output.  The flat item list is cut into eight contiguous parts, one per XCD (block b runs on
// XCD b % 8); the bstep blocks of an XCD take its items round-robin.  Inside a group items come in panels of `panel`
// m-tiles, and inside a panel with the m-tile running fastest, so that the items an XCD works on at one time form a
// compact (m, n) patch whose token and weight streams its L2 can share.
// Tail of the static walk: an XCD's items are dealt to its bstep blocks in rounds.  When the last round is at most
// half full, each of its items is split into two 128-token halves taken by different blocks (a half keeps one wave
// per SIMD busy and takes little more than half the time), so the launch ends half a round earlier.  `virt` counts
// the XCD's virtual items (whole items, then the halves of the last round's items).
struct BgmoeTiledWalk { int64_t first; int count; int bstep; int split_base; int virt; };
BGMOE_HD BgmoeTiledWalk bgmoe_tiled_walk(int64_t total_items, unsigned grid, unsigned block) {
  const int nx = 8;
  const int xcd = (int)(block % nx);
  const int per_x = (int)((total_items + nx - 1) / nx);
  BgmoeTiledWalk w;
  w.bstep = (int)((grid + nx - 1 - xcd) / nx);
  w.first = (int64_t)xcd * per_x;
  int64_t left = total_items - w.first;
  if (left < 0) left = 0;
  w.count = (int)(left < per_x ? left : per_x);
  const int rounds = w.bstep > 0 ? (w.count + w.bstep - 1) / w.bstep : 0;
  w.split_base = rounds > 0 ? (rounds - 1) * w.bstep : 0;
  const int rem = w.count - w.split_base;
  w.virt = (rounds > 0 && 2 * rem <= w.bstep) ? w.split_base + 2 * rem : w.count;
  return w;
}
// virtual item itx of the XCD's walk -> flat item and half (-1: the whole 256-token tile; 0, 1: tokens 128 * half ..)
BGMOE_HD bool bgmoe_tiled_walk_item(const BgmoeTiledWalk& w, int64_t itx, int64_t* item, int* half) {
  if (itx >= w.virt) return false;
  *half = -1;
  *item = w.first + itx;
  if (w.virt != w.count && itx >= w.split_base) {
    *item = w.first + w.split_base + ((itx - w.split_base) >> 1);
    *half = (int)((itx - w.split_base) & 1);
  }
  return true;
}
struct BgmoeTiledItem { int grp, mtile, ntile; };
// flat item -> (group, m-tile of the group, n-tile); tiles[] may live in LDS
BGMOE_HD BgmoeTiledItem bgmoe_tiled_decode(const int* tiles, int groups, int ntn, int panel, int64_t item) {
  int lo = 0, hi = groups - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if ((int64_t)tiles[mid] * ntn <= item) lo = mid; else hi = mid - 1;
  }
  BgmoeTiledItem it;
  it.grp = lo;
  const int mt_g = tiles[lo + 1] - tiles[lo];
  const int64_t rel = item - (int64_t)tiles[lo] * ntn;
  const int pnl = (int)(rel / ((int64_t)panel * ntn));
  const int left = mt_g - pnl * panel;
  const int pm = panel < left ? panel : left;
  const int r2 = (int)(rel - (int64_t)pnl * panel * ntn);
  it.ntile = r2 / pm;
  it.mtile = pnl * panel + (r2 - it.ntile * pm);
  return it;
}
