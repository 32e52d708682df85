// Device-side work scheduling shared by the weight-streaming GEMM kernels.
#pragma once
#include "bgmoe_common.h"
#include "bgmoe_hostdev.h"

// Which kernel serves a group.  The weight-streaming kernel re-streams a group's weights once per
// 32-row chunk; the LDS-tiled kernel works in 256-row tiles and needs enough of them to fill the chip.
// Groups with at most small_rows rows always stream; groups with more than max_rows rows are always
// tiled; groups in between are tiled only when all groups above small_rows together make at least
// min_tiles 256-row tiles.  Both kernels evaluate this on the device from the same counts.
struct BgmoeSplit { int small_rows, max_rows, min_tiles; };

// Wave-uniform; every wave runs it redundantly.  Returns the row limit of the weight-streaming kernel.
__device__ __forceinline__ int bgmoe_split_limit(const int32_t* seqlens, int groups, BgmoeSplit s) {
  if (s.small_rows >= s.max_rows) return s.max_rows;
  const int lane = threadIdx.x & 63;
  int tiles = 0;
  for (int g0 = lane; g0 < groups; g0 += 64) {
    const int c = seqlens[g0];
    tiles += c > s.small_rows ? (c + 255) >> 8 : 0;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) tiles += __shfl_xor(tiles, off, BGMOE_WAVE);
  return tiles >= s.min_tiles ? s.small_rows : s.max_rows;
}

// Row chunks of all groups with lo < count <= hi (the number of items per n-tile).  Wave-uniform; every wave
// runs it redundantly.
__device__ __forceinline__ int bgmoe_total_chunks(const int32_t* seqlens, int groups, int lo, int hi, int chunk_rows,
                                                  BgmoeTall tall = BgmoeTall{0, 0}) {
  const int lane = threadIdx.x & 63;
  int chunks = 0;
  for (int g0 = lane; g0 < groups; g0 += 64) {
    const int c = seqlens[g0];
    chunks += (c > lo && c <= hi) ? bgmoe_item_chunks(c, chunk_rows, tall) : 0;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) chunks += __shfl_xor(chunks, off, BGMOE_WAVE);
  return __builtin_amdgcn_readfirstlane(chunks);
}

// Work items of one launch: every group with lo < count <= hi contributes bgmoe_item_chunks(count)
// items (ascending group, ascending chunk).  Returns the group of item `item` and its chunk index,
// or -1 when there are fewer items.  Wave-uniform; every wave of the block runs it redundantly.
__device__ __forceinline__ int nth_active_item(const int32_t* seqlens, int groups, int lo, int hi,
                                               int chunk_rows, int item, int* chunk,
                                               BgmoeTall tall = BgmoeTall{0, 0}) {
  const int lane = threadIdx.x & 63;
  int base = 0;
  for (int g0 = 0; g0 < groups; g0 += 64) {
    const int gi = g0 + lane;
    const int c = gi < groups ? seqlens[gi] : 0;
    const int mine = (c > lo && c <= hi) ? bgmoe_item_chunks(c, chunk_rows, tall) : 0;
    int inc = mine;                                  // inclusive prefix sum over the wave
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(inc, off, BGMOE_WAVE);
      if (lane >= off) inc += up;
    }
    const int total = __shfl(inc, 63, BGMOE_WAVE);
    if (item < base + total) {
      const int rel = item - base;
      const unsigned long long hit = __ballot(mine > 0 && rel >= inc - mine && rel < inc);
      const int src = __ffsll((long long)hit) - 1;
      *chunk = rel - __shfl(inc - mine, src, BGMOE_WAVE);
      return g0 + src;
    }
    base += total;
  }
  return -1;
}


// Virtual block -> work item.  The (n-tile, chunk) map inside a group is bgmoe_item_slot (bgmoe_hostdev.h): all
// chunks of one n-tile on the same XCD in neighbouring blocks.  `block` is the virtual block index (blockIdx.x, or
// blockIdx.x + i * gridDim.x in a persistent kernel whose grid is a multiple of 8, which keeps block % 8 == XCD).
// grp == BGMOE_ITEM_END: `block` lies past the last item (so do all larger ones); grp == BGMOE_ITEM_PAD: a padding
// n-tile, nothing to do.  rows: the item's height (chunk_rows, or tall.rows for a tall group); its rows are
// [chunk * rows, min(cnt, (chunk + 1) * rows)).
struct BgmoeItem { int grp, ntile, chunk, cnt, rows; };
constexpr int BGMOE_ITEM_PAD = -1;
constexpr int BGMOE_ITEM_END = -2;

__device__ __forceinline__ BgmoeItem bgmoe_decode_item(const int32_t* seqlens, int groups, int lo, int hi,
                                                       int chunk_rows, int ntiles, unsigned block,
                                                       BgmoeTall tall = BgmoeTall{0, 0}) {
  BgmoeItem it;
  const int ntiles_pad = (ntiles + 7) & ~7;
  int crow = 0;
  it.grp = nth_active_item(seqlens, groups, lo, hi, chunk_rows, (int)(block / ntiles_pad), &crow, tall);
  it.ntile = it.chunk = it.cnt = 0;
  it.rows = chunk_rows;
  if (__builtin_amdgcn_readfirstlane(it.grp) < 0) {
    it.grp = BGMOE_ITEM_END;
    return it;
  }
  it.cnt = seqlens[it.grp];
  const BgmoeItemSlot slot = bgmoe_item_slot(crow, bgmoe_item_chunks(it.cnt, chunk_rows, tall), ntiles_pad, block);
  it.ntile = slot.ntile;
  it.chunk = slot.chunk;
  it.rows = bgmoe_item_rows(it.cnt, chunk_rows, tall);
  if (it.ntile >= ntiles) it.grp = BGMOE_ITEM_PAD;
  // the fields are wave-uniform by construction; say so, so that everything derived from them (pointers,
  // loop bounds, branches) is scalar code
  it.grp = __builtin_amdgcn_readfirstlane(it.grp);
  it.ntile = __builtin_amdgcn_readfirstlane(it.ntile);
  it.chunk = __builtin_amdgcn_readfirstlane(it.chunk);
  it.cnt = __builtin_amdgcn_readfirstlane(it.cnt);
  it.rows = __builtin_amdgcn_readfirstlane(it.rows);
  return it;
}
