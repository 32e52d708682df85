// Host-compiled checks of the arithmetic the kernels share with the host (bgmoe_hostdev.h, bgmoe_tilemap.h).
//
// Built with g++ (no HIP, no GPU) into lib/libbgmoe_hostcheck.so and called from the CPU tests through ctypes.
// Nothing here is part of the product path: each function drives the SAME inline functions the kernels call, the
// way the kernels call them, and hands the result to a test that checks invariants (every unit of work owned
// exactly once, no share without work, addresses inside their buffers, operand bytes where the matrix
// instruction expects them).
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <vector>

#include "bgmoe_hostdev.h"
#include "bgmoe_tilemap.h"

extern "C" {

// A 64-bit value rebuilt from two halves that arrive as `int`, as the wave builtins return them.
uint64_t hc_compose_from_int_halves(int lo, int hi) { return bgmoe_compose_u64(lo, hi); }

// [lo, hi) a launch addresses through `base`, and whether it lies inside the allocation.
int hc_rows_range_inside(uint64_t base, uint64_t rows, uint64_t row_bytes, uint64_t pitch_bytes, uint64_t alloc_base,
                         uint64_t alloc_bytes, uint64_t* lo, uint64_t* hi) {
  const BgmoeByteRange r = bgmoe_rows_range(base, rows, row_bytes, pitch_bytes);
  *lo = r.lo;
  *hi = r.hi;
  return bgmoe_range_inside(r, alloc_base, alloc_bytes) ? 1 : 0;
}

int hc_sk_weights_ok(const int* w8) {
  int w[8];
  memcpy(w, w8, sizeof(w));
  return bgmoe_sk_weights_ok(w) ? 1 : 0;
}

// The balanced launch's share walk, as fp8_streamk_kernel runs it: the cost table of the launch, the share count
// and bounds, and for every share the parts it owns (the kernel's load and compute cursors both advance this way).
// out: 10 ints per part {share, grp, ntile, chunk, cnt, kb_lo, kb_hi, first_share, last_share, cpk}; at most
// max_parts parts.  info: {C, G, n8, Wg}.  Returns the number of parts, -(r + 1) when share r owns no unit, or
// -1000000 when max_parts is too small.
int hc_sk_walk(const int32_t* seqlens, int groups, int hi_rows, int ntiles, int KB, int tt, int wc, int cost_w,
               int cost_r, int cost_t, const int* w8, unsigned grid, unsigned min_units, int* out, int max_parts,
               uint32_t* info) {
  const BgmoeSkShape shape{tt, wc};
  const BgmoeSkCost cost{cost_w, cost_r, cost_t};
  int w[8];
  memcpy(w, w8, sizeof(w));
  std::vector<uint32_t> gpre(groups + 1, 0);
  std::vector<int> cnt(groups, 0);
  for (int g = 0; g < groups; ++g) {
    int c = seqlens[g];
    if (c < 0 || c > hi_rows) c = 0;
    cnt[g] = c;
    gpre[g + 1] = gpre[g] + (uint32_t)ntiles * (uint32_t)KB * bgmoe_sk_group_cost_per_kb(shape, cost, c);
  }
  const uint32_t C = gpre[groups];
  info[0] = C;
  info[1] = info[2] = info[3] = 0;
  if (C == 0) return 0;
  const uint32_t G = bgmoe_sk_num_shares(C, grid, bgmoe_sk_share_unit(shape, cost), min_units);
  const uint32_t n8 = G >= 8 ? G >> 3 : 1;
  const uint32_t Wg = bgmoe_sk_cum_weight(w, n8, G);
  info[1] = G;
  info[2] = n8;
  info[3] = Wg;
  auto locate = [&](uint32_t x, uint32_t x1, BgmoeSkPart* p) {
    for (int iter = 0; iter < 2; ++iter) {
      if (x >= x1) return false;
      int g = 0;
      for (int gi = 0; gi < groups; ++gi) g += gpre[gi + 1] <= x ? 1 : 0;
      uint32_t next = 0;
      if (bgmoe_sk_locate_in_group(shape, cost, g, cnt[g], gpre[g], ntiles, KB, x, x1, p, &next)) return true;
      x = next;
    }
    return false;
  };
  int n = 0;
  for (uint32_t r = 0; r < G; ++r) {
    const uint32_t x0 = bgmoe_sk_bound(w, n8, Wg, C, r), x1 = bgmoe_sk_bound(w, n8, Wg, C, r + 1);
    BgmoeSkPart p;
    if (!locate(x0, x1, &p)) return -(int)(r + 1);
    for (;;) {
      if (n >= max_parts) return -1000000;
      int* o = out + 10 * n++;
      o[0] = (int)r; o[1] = p.grp; o[2] = p.ntile; o[3] = p.chunk; o[4] = p.cnt; o[5] = p.kb_lo; o[6] = p.kb_hi;
      o[7] = (int)bgmoe_sk_share_of_cost(w, n8, Wg, C, p.start);
      o[8] = (int)bgmoe_sk_share_of_cost(w, n8, Wg, C, p.start + (uint32_t)(KB - 1) * (uint32_t)p.cpk);
      o[9] = p.cpk;
      if (!locate(p.start + (uint32_t)p.kb_hi * (uint32_t)p.cpk, x1, &p)) break;
    }
  }
  return n;
}

// ---- the LDS-tiled kernels' walk over work items -----------------------------------------------------------------
// Every block's walk as the K = 64 kernel runs it: counts -> m-tiles of 256 rows for groups above `lo` rows, the
// XCD-wise split of the flat item list, round-robin over an XCD's blocks, item -> (group, m-tile, n-tile).
// out: 6 ints per visit {block, round, grp, mtile, ntile, half}; returns the number of visits or -1 (out too small).
int hc_tiled_walk(const int32_t* counts, int groups, int lo, int ntn, int panel, unsigned grid, int* out, int max_items) {
  std::vector<int> tiles(groups + 1, 0);
  for (int g = 0; g < groups; ++g) tiles[g + 1] = tiles[g] + (counts[g] > lo ? (counts[g] + 255) / 256 : 0);
  const int64_t total = (int64_t)tiles[groups] * ntn;
  int n = 0;
  for (unsigned b = 0; b < grid; ++b) {
    const BgmoeTiledWalk w = bgmoe_tiled_walk(total, grid, b);
    int round = 0;
    int64_t item = 0;
    int half = -1;
    for (int64_t itx = b / 8; bgmoe_tiled_walk_item(w, itx, &item, &half); itx += w.bstep, ++round) {
      if (n >= max_items) return -1;
      const BgmoeTiledItem it = bgmoe_tiled_decode(tiles.data(), groups, ntn, panel, item);
      int* o = out + 6 * n++;
      o[0] = (int)b; o[1] = round; o[2] = it.grp; o[3] = it.mtile; o[4] = it.ntile; o[5] = half;
    }
  }
  return n;
}

// ---- operand tile images of the K = 64 LDS-tiled GEMM (bgmoe_tilemap.h) ----------------------------------------
// Emulates one wave's asynchronous load of half a tile image (64 lanes x 16 bytes into 1 KiB of LDS) from a
// row-major source with `pitch` bytes per row, then one wave's operand read of the whole 32-row image.
// src: 32 rows of at least 64 bytes at the given pitch; got: [64 lanes][32 bytes] what each lane feeds to the
// matrix instruction.  The test compares `got` with the layout the instruction defines (lane l: row l % 32,
// K bytes of half l / 32).
void hc_k64_tile_roundtrip(const uint8_t* src, uint32_t pitch, uint8_t* got) {
  uint8_t lds[BGMOE_K64_TILE_BYTES];
  memset(lds, 0xEE, sizeof(lds));
  for (int half = 0; half < 2; ++half)
    for (uint32_t lane = 0; lane < 64; ++lane) {
      const uint32_t goff = bgmoe_k64_load_src_offset(lane, half, pitch);
      const uint32_t loff = bgmoe_k64_load_lds_offset(lane, half);
      memcpy(lds + loff, src + goff, 16);
    }
  for (uint32_t lane = 0; lane < 64; ++lane) {
    memcpy(got + 32 * lane, lds + bgmoe_k64_operand_lo(lane), 16);
    memcpy(got + 32 * lane + 16, lds + bgmoe_k64_operand_hi(lane), 16);
  }
}
// The same for tile-major weights: `halves` = the two contiguous KiB (16 rows x 64 K-bytes each, [piece][row] order)
// that one step loads linearly for a 32-row image.
void hc_k64_tm_tile_roundtrip(const uint8_t* halves, uint8_t* got) {
  uint8_t lds[BGMOE_K64_TILE_BYTES];
  for (int half = 0; half < 2; ++half)
    for (uint32_t lane = 0; lane < 64; ++lane)
      memcpy(lds + bgmoe_k64_load_lds_offset(lane, half), halves + 1024 * half + 16 * lane, 16);
  for (uint32_t lane = 0; lane < 64; ++lane) {
    memcpy(got + 32 * lane, lds + bgmoe_k64_tm_operand_lo(lane), 16);
    memcpy(got + 32 * lane + 16, lds + bgmoe_k64_tm_operand_hi(lane), 16);
  }
}
// the 16-byte LDS offsets one operand read touches, for the bank-conflict check: out[0..64) lo offsets, out[64..128) hi
void hc_k64_operand_offsets(uint32_t* out, int tile_major) {
  for (uint32_t lane = 0; lane < 64; ++lane) {
    out[lane] = tile_major ? bgmoe_k64_tm_operand_lo(lane) : bgmoe_k64_operand_lo(lane);
    out[64 + lane] = tile_major ? bgmoe_k64_tm_operand_hi(lane) : bgmoe_k64_operand_hi(lane);
  }
}
// accumulator register v (0..15) of lane l of a 32x32 product: which (A row, B row) it holds
void hc_k64_acc_coord(uint32_t lane, uint32_t v, uint32_t* a_row, uint32_t* b_row) {
  *a_row = bgmoe_mfma32_acc_a_row(lane, v);
  *b_row = bgmoe_mfma32_acc_b_row(lane);
}


// ---- weight-streaming kernels: virtual block -> work item ----------------------------------------------------------------
// The device finds the group of item number block / ntiles_pad with a wave-wide prefix scan of bgmoe_item_chunks over
// the groups with lo < count <= hi; here the same search is a loop.  out: 5 ints per virtual block (grp or -1 for a
// padding n-tile, ntile, chunk, rows, count) for blocks 0, 1, ... until the list ends; returns the number of
// virtual blocks before the end, or -1 when it exceeds cap.
int64_t hc_item_walk(const int32_t* counts, int groups, int lo, int hi, int chunk_rows, int tall_min, int tall_rows,
                     int ntiles, int32_t* out, int64_t cap) {
  const BgmoeTall tall{tall_min, tall_rows};
  const int ntiles_pad = (ntiles + 7) & ~7;
  for (int64_t block = 0;; ++block) {
    const int item = (int)(block / ntiles_pad);
    int base = 0, grp = -1, crow = 0;
    for (int g = 0; g < groups && grp < 0; ++g) {
      const int c = counts[g];
      const int mine = (c > lo && c <= hi) ? bgmoe_item_chunks(c, chunk_rows, tall) : 0;
      if (item < base + mine) { grp = g; crow = item - base; }
      base += mine;
    }
    if (grp < 0) return block;
    if (block >= cap) return -1;
    const int c = counts[grp];
    const BgmoeItemSlot slot = bgmoe_item_slot(crow, bgmoe_item_chunks(c, chunk_rows, tall), ntiles_pad, (unsigned)block);
    int32_t* o = out + 5 * block;
    o[0] = slot.ntile >= ntiles ? -1 : grp;
    o[1] = slot.ntile; o[2] = slot.chunk; o[3] = bgmoe_item_rows(c, chunk_rows, tall); o[4] = c;
  }
}
unsigned hc_item_grid(int ntiles, int groups, int64_t row_bound, int max_rows, int chunk_rows) {
  return bgmoe_item_grid(ntiles, groups, row_bound, max_rows, chunk_rows);
}

// ---- bf16 GEMM with 128 x 64 block tiles: one K step's loads and operand reads -----------------------------------------
// experts [64][64] and tokens [128][64] bf16 values of one K step (given as uint16); the 24 issues of the block land
// them in a stage; got_e [4 tiles][64 lanes][2 halves][8 values] and got_t [8 token tiles][64 lanes][2][8] are what the
// lanes read.  Returns 0, or -1 when an issue leaves the stage's 24 KB or two lanes write one place.
int hc_rg64_step(const uint16_t* experts, const uint16_t* tokens, uint16_t* got_e, uint16_t* got_t) {
  std::vector<uint8_t> stage(192 * 128, 0xEE), hit(192 * 8, 0);
  for (uint32_t wave = 0; wave < 8; ++wave)
    for (uint32_t i = 0; i < 3; ++i)
      for (uint32_t lane = 0; lane < 64; ++lane) {
        const bool tok = bgmoe_rg64_issue_is_token(wave, i);
        const uint32_t row = bgmoe_rg64_lane_row(wave, i, lane);
        const uint32_t piece = bgmoe_rg64_lane_piece(row, lane);
        const uint32_t dst = bgmoe_rg64_issue_lds(wave, i) + 16 * lane;
        if (dst + 16 > stage.size() || row >= (tok ? 128u : 64u)) return -1;
        if (hit[dst / 16]++) return -1;
        memcpy(&stage[dst], reinterpret_cast<const uint8_t*>(tok ? tokens : experts) + row * 128 + piece * 16, 16);
      }
  for (size_t k = 0; k < hit.size(); ++k)
    if (hit[k] != 1) return -1;
  for (uint32_t lane = 0; lane < 64; ++lane)
    for (uint32_t jj = 0; jj < 2; ++jj) {
      for (uint32_t tn = 0; tn < 4; ++tn)
        memcpy(got_e + ((tn * 64 + lane) * 2 + jj) * 8, &stage[bgmoe_rg64_read_expert(tn, lane, jj)], 16);
      for (uint32_t wt = 0; wt < 8; ++wt)
        memcpy(got_t + ((wt * 64 + lane) * 2 + jj) * 8, &stage[bgmoe_rg64_read_token(wt, lane, jj)], 16);
    }
  return 0;
}

// ---- the K = 64 kernel's dataflow on one macro tile ----------------------------------------------------------------
// Walks what fp8_tiled_k64_kernel does for ONE work item with the kernel's own maps (bgmoe_tilemap.h): per K-step
// every wave's asynchronous loads into a ring slot (token image `wave`, weight image `wave`, clamped rows, swizzle
// or tile-major order), every wave's operand reads, the 32x32x64 products accumulated in place with the scale
// change at even steps, and the epilogue's (token, column) of every accumulator register.  The matrix instruction
// itself is taken from its definition: lane l supplies row l % 32 and K half l / 32 of each operand, register v of
// lane l receives D[8 (v / 4) + 4 (l / 32) + v % 4][l % 32].
//
// x: the group's tokens [cnt][K] e4m3 bytes, xs [cnt][KB] scales; w0 (and w1 when fused): [n][K] bytes, row-major or
// tile-major; ws0 / ws1: the K-row of weight scales per 128-row block [n / 128][KB]; (m0, n0): the macro tile.
// out [cnt][ncols_total] and written [cnt][ncols_total] (1 where the kernel stores): fused: ncols_total = n (values
// silu(gate) * up before the bf16 rounding); plain: n.  Returns 0, or a negative number when an address left its
// buffer.
static float e4m3_to_float(uint8_t b) {
  const int sign = b >> 7, e = (b >> 3) & 15, m = b & 7;
  float v;
  if (e == 0) v = ldexpf((float)m / 8.0f, -6);
  else if (e == 15 && m == 7) v = NAN;
  else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return sign ? -v : v;
}

int hc_k64_emulate_item(const uint8_t* x, const float* xs, int cnt, int K, const uint8_t* w0, const uint8_t* w1,
                        const float* ws0, const float* ws1, int n, int fused, int tile_major, int regroup, int m0, int n0,
                        float* out, uint8_t* written) {
  const int KB = K / 128, steps = 2 * KB;
  const bool F = fused != 0;
  float dec[256];
  for (int i = 0; i < 256; ++i) dec[i] = e4m3_to_float((uint8_t)i);
  const uint64_t x_bytes = (uint64_t)cnt * K, w_bytes = (uint64_t)n * K;
  std::vector<uint8_t> slot(2 * 8 * BGMOE_K64_TILE_BYTES);            // tokens, then weights
  std::vector<float> acc(8 * 64 * 4 * 2 * 16, 0.0f), prev(8 * 64 * 4 * 2, 0.0f);   // [wave][lane][b][a][v]
  auto ACC = [&](uint32_t wave, uint32_t lane, int b, int a, int v) -> float& {
    return acc[((((size_t)wave * 64 + lane) * 4 + b) * 2 + a) * 16 + v];
  };
  auto PREV = [&](uint32_t wave, uint32_t lane, int b, int a) -> float& { return prev[(((size_t)wave * 64 + lane) * 4 + b) * 2 + a]; };
  const uint32_t last = (uint32_t)(cnt - 1 - m0);
  for (int ks = 0; ks < steps; ++ks) {
    // ---- loads ----
    memset(slot.data(), 0xEE, slot.size());
    for (uint32_t wave = 0; wave < 8; ++wave) {
      const int nrow_raw = n0 + (int)bgmoe_k64_image_wrow(F, wave);
      const int nrow = nrow_raw < n - 32 ? nrow_raw : n - 32;
      const uint8_t* wbase = bgmoe_k64_image_matrix(F, wave) ? w1 : w0;
      for (uint32_t h = 0; h < 2; ++h)
        for (uint32_t lane = 0; lane < 64; ++lane) {
          const uint64_t src = (uint64_t)m0 * K + (uint64_t)ks * 64 + bgmoe_k64_token_src_offset(lane, h, wave, last, (uint32_t)K);
          if (src + 16 > x_bytes) return -1;
          memcpy(&slot[wave * BGMOE_K64_TILE_BYTES + bgmoe_k64_load_lds_offset(lane, h)], x + src, 16);
          uint64_t wsrc;
          if (tile_major) wsrc = (uint64_t)((nrow >> 4) + (int)h) * K * 16 + (uint64_t)ks * 1024 + lane * 16u;
          else wsrc = (uint64_t)nrow * K + (uint64_t)ks * 64 + bgmoe_k64_load_src_offset(lane, h, (uint32_t)K);
          if (wsrc + 16 > w_bytes) return -2;
          memcpy(&slot[(8 + wave) * BGMOE_K64_TILE_BYTES + bgmoe_k64_load_lds_offset(lane, h)], wbase + wsrc, 16);
        }
    }
    // ---- compute ----
    const int kb = ks >> 1;
    for (uint32_t wave = 0; wave < 8; ++wave) {
      const uint32_t wn = bgmoe_k64_wave_wn(wave), wm = bgmoe_k64_wave_wm(wave);
      if (!(m0 + 128 * (int)wm < cnt)) continue;                       // the kernel's wave_live
      if ((ks & 1) == 0) {
        const int nb0 = (n0 >> 7), nb1 = ((n0 + 128 < n ? n0 + 128 : n - 1) >> 7);
        const float wsc0 = F ? ws0[(size_t)nb0 * KB + kb] : ws0[(size_t)nb0 * KB + kb];
        const float wsc1 = F ? ws1[(size_t)nb0 * KB + kb] : ws0[(size_t)nb1 * KB + kb];
        const float wa0 = F ? wsc0 : (wn >= 2u ? wsc1 : wsc0), wa1 = F ? wsc1 : wa0;
        for (uint32_t lane = 0; lane < 64; ++lane)
          for (int b = 0; b < 4; ++b) {
            uint32_t t = bgmoe_k64_out_token(wm, b, lane);             // token scale the lane reads (clamped like the load)
            const uint32_t tc = t < last ? t : last;
            const float s = xs[(size_t)(m0 + tc) * KB + kb];
            const float c[2] = {s * wa0, s * wa1};
            for (int a = 0; a < 2; ++a) {
              if (kb > 0) {
                const float r = PREV(wave, lane, b, a) * (1.0f / c[a]);
                for (int v = 0; v < 16; ++v) ACC(wave, lane, b, a, v) *= r;
              }
              PREV(wave, lane, b, a) = c[a];
            }
          }
      }
      // operands as the lanes read them
      uint8_t A[2][64][32], B[4][64][32];
      for (uint32_t lane = 0; lane < 64; ++lane) {
        for (int a = 0; a < 2; ++a) {
          const uint8_t* img = &slot[(8 + bgmoe_k64_a_image(F, wn, a)) * BGMOE_K64_TILE_BYTES];
          memcpy(A[a][lane], img + (tile_major ? bgmoe_k64_tm_operand_lo(lane) : bgmoe_k64_operand_lo(lane)), 16);
          memcpy(A[a][lane] + 16, img + (tile_major ? bgmoe_k64_tm_operand_hi(lane) : bgmoe_k64_operand_hi(lane)), 16);
        }
        for (int b = 0; b < 4; ++b) {
          const uint8_t* img = &slot[bgmoe_k64_b_image(wm, b) * BGMOE_K64_TILE_BYTES];
          memcpy(B[b][lane], img + bgmoe_k64_operand_lo(lane), 16);
          memcpy(B[b][lane] + 16, img + bgmoe_k64_operand_hi(lane), 16);
        }
      }
      for (int b = 0; b < 4; ++b)
        for (int a = 0; a < 2; ++a) {
          float D[32][32];
          for (int i = 0; i < 32; ++i)
            for (int j = 0; j < 32; ++j) {
              double sum = 0.0;
              for (int h = 0; h < 2; ++h)
                for (int k = 0; k < 32; ++k)
                  sum += (double)dec[A[a][i + 32 * h][k]] * (double)dec[B[b][j + 32 * h][k]];
              D[i][j] = (float)sum;
            }
          for (uint32_t lane = 0; lane < 64; ++lane)
            for (uint32_t v = 0; v < 16; ++v)
              ACC(wave, lane, b, a, (int)v) += D[bgmoe_mfma32_acc_a_row(lane, v)][bgmoe_mfma32_acc_b_row(lane)];
        }
    }
  }
  // ---- epilogue ----
  auto value = [&](uint32_t wave, uint32_t lane, int b, int a, uint32_t v) {
    if (F) {
      const float gt = ACC(wave, lane, b, 0, (int)v) * PREV(wave, lane, b, 0);
      const float up = ACC(wave, lane, b, 1, (int)v) * PREV(wave, lane, b, 1);
      return gt / (1.0f + expf(-gt)) * up;
    }
    return ACC(wave, lane, b, a, (int)v) * PREV(wave, lane, b, a);
  };
  auto emit = [&](int tok, int col, float val) {
    const size_t o = (size_t)tok * n + col;
    if (written[o]) return false;                                       // two places claim one output element
    written[o] = 1;
    out[o] = val;
    return true;
  };
  for (uint32_t wave = 0; wave < 8; ++wave) {
    const uint32_t wn = bgmoe_k64_wave_wn(wave), wm = bgmoe_k64_wave_wm(wave);
    if (!regroup) {
      for (uint32_t lane = 0; lane < 64; ++lane)
        for (int b = 0; b < 4; ++b) {
          const int tok = m0 + (int)bgmoe_k64_out_token(wm, b, lane);
          if (tok >= cnt) continue;
          for (int a = 0; a < (F ? 1 : 2); ++a)
            for (uint32_t v = 0; v < 16; ++v) {
              const int col = n0 + (int)bgmoe_k64_out_col(F, wn, (uint32_t)a, lane, v);
              if (col >= n) continue;
              if (!emit(tok, col, value(wave, lane, b, a, v))) return -3;
            }
        }
      continue;
    }
    // through the wave's patch: one slot per output element (e4m3: one byte; bf16: two bytes), addressed with the
    // kernel's byte offsets
    const uint32_t esz = F ? 1u : 2u;
    std::vector<float> patch(BGMOE_K64_PATCH_BYTES / esz, NAN);
    if (F) {
      for (int b = 0; b < 4; ++b) {
        for (uint32_t lane = 0; lane < 64; ++lane)
          for (uint32_t q = 0; q < 4; ++q) {
            const uint32_t off = bgmoe_k64_qpatch_write_off(lane, q);
            if (off + 4 > BGMOE_K64_PATCH_BYTES) return -4;
            for (uint32_t i = 0; i < 4; ++i) patch[off + i] = value(wave, lane, b, 0, 4 * q + i);
          }
        for (uint32_t lane = 0; lane < 64; ++lane) {
          const uint32_t off = bgmoe_k64_qpatch_read_off(lane);
          if (off % 16 != 0 || off + 16 > BGMOE_K64_PATCH_BYTES) return -5;
          const int rtok = m0 + 128 * (int)wm + 32 * b + (int)bgmoe_k64_qpatch_read_token(lane);
          if (rtok >= cnt) continue;
          for (uint32_t i = 0; i < 16; ++i)
            if (!emit(rtok, n0 + 32 * (int)wn + (int)bgmoe_k64_qpatch_read_col(lane) + (int)i, patch[off + i])) return -3;
        }
      }
    } else {
      const int colw = n0 + 64 * (int)wn;
      if (colw >= n) continue;
      for (int b = 0; b < 4; ++b) {
        if (m0 + 128 * (int)wm + 32 * b >= cnt) continue;
        for (uint32_t p = 0; p < 4; ++p) {
          for (uint32_t lane = 0; lane < 64; ++lane) {
            if (!bgmoe_k64_patch_writer(lane, p)) continue;
            for (uint32_t a = 0; a < 2; ++a)
              for (uint32_t q = 0; q < 4; ++q) {
                const uint32_t off = bgmoe_k64_patch_write_off(lane, a, q);
                if (off % 8 != 0 || off + 8 > BGMOE_K64_PATCH_BYTES) return -4;
                for (uint32_t i = 0; i < 4; ++i) patch[off / 2 + i] = value(wave, lane, b, (int)a, 4 * q + i);
              }
          }
          for (uint32_t lane = 0; lane < 64; ++lane) {
            const uint32_t off = bgmoe_k64_patch_read_off(lane);
            if (off % 16 != 0 || off + 16 > BGMOE_K64_PATCH_BYTES) return -5;
            const int rtok = m0 + 128 * (int)wm + 32 * b + (int)bgmoe_k64_patch_read_token(p, lane);
            if (rtok >= cnt) continue;
            for (uint32_t i = 0; i < 8; ++i)
              if (!emit(rtok, colw + (int)bgmoe_k64_patch_read_col(lane) + (int)i, patch[off / 2 + i])) return -3;
          }
        }
      }
    }
  }
  return 0;
}

}  // extern "C"
