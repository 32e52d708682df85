// Host-compiled checks of the arithmetic the kernels share with the host (bgmoe_hostdev.h, bgmoe_tilemap.h).
//
// Built with g++ (no HIP, no GPU) into lib/libbgmoe_hostcheck.so and called from the CPU tests through ctypes.
// Nothing here is part of the product path: each function drives the SAME inline functions the kernels call, the
// way the kernels call them, and hands the result to a test that checks invariants (every unit of work owned
// exactly once, no share without work, addresses inside their buffers, operand bytes where the matrix
// instruction expects them).
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

}  // extern "C"
