// Device-side work scheduling shared by the weight-streaming GEMM kernels.
#pragma once
#include "bgmoe_common.h"

// Work items of one launch: every group with lo < count <= hi contributes ceil(count / chunk_rows)
// items (ascending group, ascending chunk).  Returns the group of item `item` and its chunk index,
// or -1 when there are fewer items.  Wave-uniform; every wave of the block runs it redundantly.
__device__ __forceinline__ int nth_active_item(const int32_t* seqlens, int groups, int lo, int hi,
                                               int chunk_rows, int item, int* chunk) {
  const int lane = threadIdx.x & 63;
  int base = 0;
  for (int g0 = 0; g0 < groups; g0 += 64) {
    const int gi = g0 + lane;
    const int c = gi < groups ? seqlens[gi] : 0;
    const int mine = (c > lo && c <= hi) ? (c + chunk_rows - 1) / chunk_rows : 0;
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


// XCD-aware block -> (n-tile, token chunk) map inside one group.  Blocks are dispatched round-robin
// over the 8 XCDs (block b runs on XCD b % 8), each with its own L2.  A group with several token
// chunks streams the same weight tile once per chunk; the map puts all chunks of one n-tile on the
// SAME XCD in neighbouring blocks: block q of the group -> n-tile 8*(q / (8*chunks)) + q % 8,
// chunk (q / 8) % chunks.  `ntiles_pad` = n-tile count rounded up to 8 so every group starts on XCD 0.
struct BgmoeItem { int grp, ntile, chunk, cnt; };

__device__ __forceinline__ BgmoeItem bgmoe_decode_item(const int32_t* seqlens, int groups, int lo, int hi,
                                                       int chunk_rows, int ntiles) {
  BgmoeItem it;
  const int ntiles_pad = (ntiles + 7) & ~7;
  int crow = 0;
  it.grp = nth_active_item(seqlens, groups, lo, hi, chunk_rows, blockIdx.x / ntiles_pad, &crow);
  it.ntile = it.chunk = it.cnt = 0;
  if (it.grp < 0) return it;
  it.cnt = seqlens[it.grp];
  const int chunks = (it.cnt + chunk_rows - 1) / chunk_rows;
  const int q = crow * ntiles_pad + blockIdx.x % ntiles_pad;
  it.ntile = 8 * (q / (8 * chunks)) + (q & 7);
  it.chunk = (q >> 3) % chunks;
  if (it.ntile >= ntiles) it.grp = -1;
  return it;
}

static inline unsigned bgmoe_item_grid(int ntiles, int groups, int64_t row_bound, int chunk_rows) {
  const int64_t items = groups + row_bound / chunk_rows;          // >= sum of ceil(count / chunk_rows)
  return (unsigned)(((ntiles + 7) & ~7) * items);
}
