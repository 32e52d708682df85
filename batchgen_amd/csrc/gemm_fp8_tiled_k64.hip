// Block-scaled FP8 grouped GEMM for MANY rows per group (prefill), K = 64 variant of the LDS-tiled kernel
// (gemm_fp8_tiled.hip).  Opt-in (bgmoe_set_tiled_variant): it exists to put more bytes in flight per CU.
//
// The K = 128 kernel's ring has two 65 KB slots in the 160 KB of LDS, so one K-step is in flight while the other is
// computed, and the CU's fill rate (bytes in flight / loaded latency) bounds it.  Here a K-step is 64 bytes wide:
// a slot is 32 KB (256 tokens + 256 weight rows, 64 bytes each), the ring has FOUR slots and THREE K-steps are in
// flight while one is computed -- 1.5x the bytes in flight at the same flops per byte.
//
// What makes 64-byte steps possible is a different way of applying the per-128-K scales.  The K = 128 kernel
// multiplies a whole scale block with zero-initialised products and promotes them (acc += product * scale, one VALU
// fma per accumulator and block); a product that spans two K-steps would have to stay in registers next to the
// accumulators, which do not leave room for it.  This kernel keeps the accumulators in units of the CURRENT
// block's scale and lets the matrix instruction accumulate into them directly:
//     block kb:  acc *= s[kb-1] / s[kb]            (VALU, once per block and accumulator; skipped for kb = 0)
//                acc += A_lo . B_lo ; acc += A_hi . B_hi      (two chained v_mfma_f32_32x32x64_f8f6f4)
//     at the end:  out = acc * s[KB-1]
// with s[kb] = token_scale[row, kb] * weight_scale[kb].  Same VALU count as the promotion, no product registers.
// The sums differ from the K = 128 kernel's in rounding only (one more rounding per block: the quotient of two
// scales, taken with the hardware reciprocal).  Scales must be POSITIVE: every quantiser of this path produces
// amax / 448 with a positive floor (>= 1e-12 / 448 for tokens, 1e-10 / 448 for weights), so the quotients stay far
// inside the fp32 range; a zero scale (which the K = 128 kernel would treat as a zero contribution) gives NaN here.
//
// Geometry: macro tile 256 tokens x 256 weight rows (fused stage 1: 128 gate + 128 up rows), 8 waves = 4 (weight
// rows) x 2 (tokens); a wave owns 64 weight rows x 128 tokens = 2 x 4 products of 32 x 32, 128 fp32 accumulators per
// lane; two waves per SIMD.  Tile images, lane maps and output coordinates: bgmoe_tilemap.h (checked on the CPU by
// emulating the loads and reads byte for byte).  Work list and XCD-aware item order: as in the K = 128 kernel.
//
// Streams: the load cursor runs three K-steps ahead of the compute cursor ACROSS item boundaries (it prepares the
// next item's sources and scales on its own), so the ring never drains between items.  Loads are issued from inline
// asm and waited for by count: every wave issues 4 loads per odd step and 5 per even step (the fifth brings the
// block's token scales), so "at most 9 outstanding" means the step about to be computed has landed; other
// vector-memory operations in between (scale rows, the epilogue's stores) only make that wait stricter.
#include "gemm_fp8_tiled.h"
#include "bgmoe_async.h"
#include "bgmoe_tilemap.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int TM = 256;            // tokens per macro tile
constexpr int TW = 256;            // weight rows per macro tile
constexpr int NS = 4;              // ring slots
constexpr int NT = 512;            // threads per block
constexpr int kTokBytes = TM * 64;
constexpr int kWBytes = TW * 64;
constexpr int kXsOff = kTokBytes + kWBytes;
constexpr int kSlotBytes = kXsOff + TM * 4;
constexpr int kLds = NS * kSlotBytes;
constexpr int kPanel = 8;          // m-tiles per panel of the work-item order
constexpr int kMaxGroups = kBgmoeTiledMaxGroups;
constexpr int kMaxKB = kBgmoeTiledMaxKB;
constexpr int kLoadsPerPair = 9;   // loads a wave issues per (even, odd) pair of K-steps

// REGROUP: the epilogue passes the e4m3 bytes (fused) / the bf16 values (plain GEMM) through a per-wave LDS patch and
// stores whole row segments (bgmoe_tilemap.h) instead of 4 / 8 bytes per lane and row.
template <bool FUSED, int LAYOUT, bool REGROUP>
__global__ __launch_bounds__(NT) void fp8_tiled_k64_kernel(BgmoeTiledArgs g) {
  extern __shared__ __align__(16) uint8_t smem[];      // NS slots
  __shared__ __align__(16) uint8_t s_patch[REGROUP ? NT / 64 : 1][REGROUP ? BGMOE_K64_PATCH_BYTES : 16];
  __shared__ int s_tiles[kMaxGroups + 1];              // exclusive prefix of m-tiles per group
  __shared__ float s_ws[2][2][kMaxKB];                 // [buffer][row] weight scales along K of an item
  __shared__ float s_amax[2][4][4][32];                // fused epilogue: [wm][wn][b][token] amax of 32 columns

  const int tid = threadIdx.x;
  const uint32_t wave = __builtin_amdgcn_readfirstlane((uint32_t)(tid >> 6));
  const uint32_t wn = bgmoe_k64_wave_wn(wave), wm = bgmoe_k64_wave_wm(wave);
  const uint32_t lane = (uint32_t)tid & 63u;
  const int K = g.k;
  const int KB = K >> 7;
  const int steps = 2 * KB;                            // K-steps of one item
  const int ncols = FUSED ? 128 : 256;                 // output columns per macro tile
  const int ntn = (g.n + ncols - 1) / ncols;
  const uint32_t smem_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem);
  const uint32_t ws_lds = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)&s_ws[0][0][0]);

  // ---- work list: m-tiles per group, prefix-summed (every block computes the same list) ----
  const int lo = bgmoe_split_limit(g.seqlens, g.groups, g.split);   // groups above this row count are ours
  for (int e = tid; e < g.groups; e += NT) {
    const int c = g.seqlens[e];
    s_tiles[e + 1] = c > lo ? (c + TM - 1) / TM : 0;
  }
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int e = 0; e < g.groups; ++e) {
      const int t = s_tiles[e + 1];
      s_tiles[e] = run;
      run += t;
    }
    s_tiles[g.groups] = run;
  }
  __syncthreads();
  const int total_m = s_tiles[g.groups];
  const int64_t total = (int64_t)total_m * ntn;
  // XCD-aware walk: block b (XCD b % 8) takes items of the b%8-th eighth of the list (bgmoe_hostdev.h)
  const BgmoeTiledWalk walk = bgmoe_tiled_walk(total, gridDim.x, blockIdx.x);
  const int bstep = walk.bstep;

  // ---- per-item state ----
  struct Meta { int cnt, m0, n0; int64_t row0; };
  struct Src {                                           // load sources of one item: wave-uniform bases + lane offsets
    const uint8_t* tok_base;
    uint32_t tok_off[2];
    const uint8_t* w_base[2];
    const float* xs_base;
    uint32_t xs_off;
    const float* ws_src;
  };
  // lane offsets of the weight loads do not depend on the item
  uint32_t w_off[2];
#pragma unroll
  for (uint32_t h = 0; h < 2; ++h)
    w_off[h] = LAYOUT == BGMOE_W_ROW_MAJOR ? bgmoe_k64_load_src_offset(lane, h, (uint32_t)K) : lane * 16u;

  // item index of this block's walk -> (group, n-tile, m-tile), its load sources and what the epilogue needs
  auto prepare = [&](int64_t itx, Meta& mt, Src& s) -> bool {
    int64_t item = 0;
    int half = -1;                                       // -1: the whole 256-token tile
    if (!bgmoe_tiled_walk_item(walk, itx, &item, &half)) return false;
    const BgmoeTiledItem it = bgmoe_tiled_decode(s_tiles, g.groups, ntn, kPanel, item);
    const int grp = __builtin_amdgcn_readfirstlane(it.grp);   // (LDS reads look divergent to the compiler)
    const int nt = __builtin_amdgcn_readfirstlane(it.ntile);
    const int mtile = __builtin_amdgcn_readfirstlane(it.mtile);
    int cnt = g.seqlens[grp];
    const int64_t row0 = g.cu[grp];
    int m0 = mtile * TM;
    if (half >= 0) {                                     // rows [m0 + 128 * half, + 128) of the tile
      m0 += 128 * half;
      if (m0 >= cnt) return false;                       // no live row in this half; a block has at most one split item
                                                         // and it is its last, so it is done
      cnt = min(cnt, m0 + 128);
    }
    const int n0 = nt * ncols;
    mt.cnt = cnt; mt.m0 = m0; mt.n0 = n0; mt.row0 = row0;

    const uint8_t* wb0 = g.w0.w_ptrs ? g.w0.w_ptrs[grp] : g.w0.w + (int64_t)grp * g.w0.w_group_stride;
    const float* ws0 = (g.w0.scale_ptrs ? g.w0.scale_ptrs[grp] : g.w0.scale + (int64_t)grp * g.w0.scale_group_stride);
    const uint8_t* wb1 = wb0;
    // weight scales along K: fused [0] gate, [1] up; else [0] columns 0..127, [1] columns 128..255 of the tile
    if constexpr (FUSED) {
      wb1 = g.w1.w_ptrs ? g.w1.w_ptrs[grp] : g.w1.w + (int64_t)grp * g.w1.w_group_stride;
      const float* ws1 = (g.w1.scale_ptrs ? g.w1.scale_ptrs[grp] : g.w1.scale + (int64_t)grp * g.w1.scale_group_stride) +
                         (int64_t)(n0 >> 7) * g.w1.scale_nb_stride;
      ws0 += (int64_t)(n0 >> 7) * g.w0.scale_nb_stride;
      s.ws_src = uniform_ptr(wave == 0 ? ws0 : ws1);
    } else {
      const int nb = min(n0 + (wave == 0 ? 0 : 128), g.n - 1) >> 7;
      s.ws_src = uniform_ptr(ws0 + (int64_t)nb * g.w0.scale_nb_stride);
    }

    // this wave's share of a K-step: token image `wave` and weight image `wave`, two half images (16 rows) each.
    // Tokens past the group's end re-read its last row (never stored).
    s.tok_base = uniform_ptr(g.a.x + (row0 + m0) * K);
#pragma unroll
    for (uint32_t h = 0; h < 2; ++h)
      s.tok_off[h] = bgmoe_k64_token_src_offset(lane, h, wave, (uint32_t)(cnt - 1 - m0), (uint32_t)K);
    // an image past N streams the last valid one instead; its products are never stored
    const int nrow = min(n0 + (int)bgmoe_k64_image_wrow(FUSED, wave), g.n - 32);
    const uint8_t* base = bgmoe_k64_image_matrix(FUSED, wave) ? wb1 : wb0;
    if constexpr (LAYOUT == BGMOE_W_ROW_MAJOR) {
      s.w_base[0] = s.w_base[1] = uniform_ptr(base + (int64_t)nrow * K);
    } else {                                             // two 16-row tiles of 16 * K bytes each
      s.w_base[0] = uniform_ptr(base + (int64_t)(nrow >> 4) * K * 16);
      s.w_base[1] = uniform_ptr(base + (int64_t)((nrow >> 4) + 1) * K * 16);
    }
    s.xs_base = uniform_ptr(g.a.scale_group_stride
                                ? g.a.scale + grp * g.a.scale_group_stride + (int64_t)m0 * g.a.scale_row_stride
                                : g.a.scale + (row0 + m0) * g.a.scale_row_stride);
    // every wave brings 64 token scales of an even step (waves 4..7 repeat what waves 0..3 bring: equal load
    // counts for all waves keep one wait count valid for the block)
    s.xs_off = (uint32_t)min((int)(64u * (wave & 3u) + lane), cnt - 1 - m0) * (uint32_t)g.a.scale_row_stride * 4u;
    return true;
  };

  // loads of K-step ks (64 bytes of K from byte 64 * ks) of the item described by s, into ring slot `slot`
  auto issue = [&](const Src& s, int ks, uint32_t slot) __attribute__((always_inline)) {
    const uint32_t sb = smem_base + slot * (uint32_t)kSlotBytes;
    const uint32_t dt = sb + wave * BGMOE_K64_TILE_BYTES;
    const uint8_t* tb = uniform_ptr(s.tok_base + (ks << 6));
    async_load16(tb, s.tok_off[0], dt);
    async_load16(tb, s.tok_off[1], dt + 1024u);
    const uint32_t dw = sb + (uint32_t)kTokBytes + wave * BGMOE_K64_TILE_BYTES;
    if constexpr (LAYOUT == BGMOE_W_ROW_MAJOR) {
      const uint8_t* wb = uniform_ptr(s.w_base[0] + (ks << 6));
      async_load16(wb, w_off[0], dw);
      async_load16(wb, w_off[1], dw + 1024u);
    } else {                                             // K half ks & 1 of K-block ks >> 1: KiB number ks of the tile
      async_load16(uniform_ptr(s.w_base[0] + ((int64_t)ks << 10)), w_off[0], dw);
      async_load16(uniform_ptr(s.w_base[1] + ((int64_t)ks << 10)), w_off[1], dw + 1024u);
    }
    if ((ks & 1) == 0)
      async_load4(uniform_ptr(s.xs_base + (int64_t)(ks >> 1) * g.a.scale_kb_stride), s.xs_off,
                  sb + (uint32_t)kXsOff + (wave & 3u) * 256u);
  };
  // waves 0 and 1 stage the item's two weight-scale rows (KB floats each) into s_ws[buf]
  auto issue_scales = [&](const Src& s, int buf) __attribute__((always_inline)) {
    if (wave < 2u) {
      for (int c = 0; c < KB; c += 64)
        async_load4(s.ws_src, (uint32_t)min(c + (int)lane, KB - 1) * 4u,
                    ws_lds + (uint32_t)(((buf * 2 + (int)wave) * kMaxKB + c) * 4));
    }
  };

  // ---- the two cursors ----
  Meta cur{}, nxt{};
  Src L{};
  int64_t l_itx = blockIdx.x / 8;
  int l_ks = 0, l_buf = 0;
  uint32_t lg = 0;                                       // global K-step the load cursor issues next (slot lg % NS)
  bool have = prepare(l_itx, cur, L);
  bool l_live = have, have_next = false;
  auto issue_next = [&]() __attribute__((always_inline)) {
    if (!l_live) return;
    issue(L, l_ks, lg & (NS - 1));
    ++lg;
    if (++l_ks == steps) {                               // the item's last step is on its way: on to the next item
      l_ks = 0;
      l_itx += bstep;
      have_next = l_live = prepare(l_itx, nxt, L);
      if (l_live) {
        l_buf ^= 1;
        issue_scales(L, l_buf);
      }
    }
  };
  if (have) {
    issue_scales(L, 0);
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) issue_next();       // steps >= 4 (K >= 256): all three lie inside the first item
  }

  // operand offsets inside a 2 KiB image
  const uint32_t b_lo = bgmoe_k64_operand_lo(lane), b_hi = bgmoe_k64_operand_hi(lane);
  const uint32_t a_lo = LAYOUT == BGMOE_W_ROW_MAJOR ? b_lo : bgmoe_k64_tm_operand_lo(lane);
  const uint32_t a_hi = LAYOUT == BGMOE_W_ROW_MAJOR ? b_hi : bgmoe_k64_tm_operand_hi(lane);
  auto load_image = [&](const uint8_t* img, uint32_t o_lo, uint32_t o_hi) __attribute__((always_inline)) {
    const intx4 lo4 = *reinterpret_cast<const intx4*>(img + o_lo);
    const intx4 hi4 = *reinterpret_cast<const intx4*>(img + o_hi);
    return intx8{lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
  };

  uint32_t gs = 0;                                       // global K-step of the compute cursor
  int buf = 0;
  while (have) {
    const int cnt = cur.cnt, m0 = cur.m0, n0 = cur.n0;
    const int64_t row0 = cur.row0;
    floatx16 acc[4][2];
    float prev[4][2];                                    // scale of the block the accumulators are expressed in
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        prev[b][a] = 0.0f;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[b][a][v] = 0.0f;
      }
    // a wave whose 128 tokens all lie past the group's end (the last m-tile of a ragged group) only keeps the
    // barriers and its share of the loads: the wave it shares a SIMD with gets the whole matrix pipe
    const bool wave_live = m0 + 128 * (int)wm < cnt;

    for (int kb = 0; kb < KB; ++kb) {
#pragma unroll
      for (int kh = 0; kh < 2; ++kh) {
        // this wave's loads of step gs have landed once at most the two younger steps' are outstanding; after the
        // load cursor has run out fewer steps are in flight than that count assumes, and the wait is for everything
        if (l_live) wait_vm<kLoadsPerPair>();
        else wait_vm<0>();
        block_barrier();                                 // ... and everybody's; everybody is done with step gs - 1
        issue_next();                                    // refill the slot step gs - 1 used with step gs + 3
        const uint32_t slot = gs & (NS - 1);
        ++gs;
        if (!wave_live) continue;
        const uint8_t* sl = smem + slot * kSlotBytes;
        const uint8_t* sw = sl + kTokBytes;
        if (kh == 0) {
          // into the units of block kb's scale
          const float* bxs = reinterpret_cast<const float*>(sl + kXsOff);
          const float wsc0 = s_ws[buf][0][kb], wsc1 = s_ws[buf][1][kb];
          const float wa0 = FUSED ? wsc0 : (wn >= 2u ? wsc1 : wsc0);
          const float wa1 = FUSED ? wsc1 : wa0;
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            const float xs = bxs[bgmoe_k64_out_token(wm, b, lane)];
            const float c0 = xs * wa0, c1 = xs * wa1;
            if (kb > 0) {
              const float r0 = prev[b][0] * __builtin_amdgcn_rcpf(c0);
              const float r1 = FUSED ? prev[b][1] * __builtin_amdgcn_rcpf(c1) : r0;
#pragma unroll
              for (int v = 0; v < 16; ++v) {
                acc[b][0][v] *= r0;
                acc[b][1][v] *= r1;
              }
            }
            prev[b][0] = c0;
            prev[b][1] = c1;
          }
        }
        intx8 A[2];
#pragma unroll
        for (int a = 0; a < 2; ++a)
          A[a] = load_image(sw + bgmoe_k64_a_image(FUSED, wn, a) * BGMOE_K64_TILE_BYTES, a_lo, a_hi);
        // token image b + 1 is fetched from LDS while image b is multiplied
        intx8 Bb[2];
        Bb[0] = load_image(sl + bgmoe_k64_b_image(wm, 0) * BGMOE_K64_TILE_BYTES, b_lo, b_hi);
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          if (b < 3) Bb[(b + 1) & 1] = load_image(sl + bgmoe_k64_b_image(wm, b + 1) * BGMOE_K64_TILE_BYTES, b_lo, b_hi);
          // (the scheduler would otherwise sink the prefetch below the products that do not need it)
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int a = 0; a < 2; ++a)
            acc[b][a] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(A[a], Bb[b & 1], acc[b][a], 0, 0, 0, 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }

    // ---- epilogue of the current item (the next item's first steps are in flight) -------------------------
    const uint32_t hsel = lane >> 5;                     // which 4 of every 8 columns this lane holds
    if constexpr (FUSED) {
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int tok = m0 + (int)bgmoe_k64_out_token(wm, b, lane);
        const float sg = prev[b][0], su = prev[b][1];
        float am = 0.0f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float h = bf16_round_f32(silu_rcp_f32(acc[b][0][v] * sg) * (acc[b][1][v] * su));
          acc[b][0][v] = h;
          am = fmaxf(am, fabsf(h));
        }
        if (g.out != nullptr && tok < cnt) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {                  // registers 4q .. 4q+3: columns 8q + 4*hsel .. + 3 of the wave's 32
            uint2 o;
            o.x = pack2_bf16(acc[b][0][4 * q], acc[b][0][4 * q + 1]);
            o.y = pack2_bf16(acc[b][0][4 * q + 2], acc[b][0][4 * q + 3]);
            *reinterpret_cast<uint2*>(g.out + (row0 + tok) * g.n + n0 + (int)bgmoe_k64_out_col(true, wn, 0, lane, 4 * q)) = o;
          }
        }
        if (g.out_q != nullptr) {
          am = fmaxf(am, __shfl_xor(am, 32, BGMOE_WAVE));
          if (lane < 32u) s_amax[wm][wn][b][lane] = am;
        }
      }
      if (g.out_q != nullptr) {
        lds_exchange_barrier();                          // s_amax only: the next item's loads stay in flight
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const uint32_t t32 = lane & 31u;
          const float am = fmaxf(fmaxf(s_amax[wm][0][b][t32], s_amax[wm][1][b][t32]),
                                 fmaxf(s_amax[wm][2][b][t32], s_amax[wm][3][b][t32]));
          const float sc = quant_scale_from_amax(am);
          const int tok = m0 + (int)bgmoe_k64_out_token(wm, b, lane);
          if constexpr (REGROUP) {
            // every lane quantises and writes its bytes into the wave's patch (rows past the group's end included:
            // they are simply not stored), then reads 16 bytes of one row and stores them
            uint8_t* const patch = s_patch[wave];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float hv[4] = {acc[b][0][4 * q], acc[b][0][4 * q + 1], acc[b][0][4 * q + 2], acc[b][0][4 * q + 3]};
              float qv[4];
              quant_div_clamp(hv, sc, qv);
              *reinterpret_cast<uint32_t*>(patch + bgmoe_k64_qpatch_write_off(lane, (uint32_t)q)) =
                  pack4_e4m3(qv[0], qv[1], qv[2], qv[3]);
            }
            // (the patch goes from lane to lane inside the wave: LDS serves a wave's accesses in order, so no wait is
            // needed; the wave barrier is no instruction, it keeps the compiler from moving accesses across it)
            __builtin_amdgcn_wave_barrier();
            const uint4 v = *reinterpret_cast<const uint4*>(patch + bgmoe_k64_qpatch_read_off(lane));
            __builtin_amdgcn_wave_barrier();
            const int rtok = m0 + 128 * (int)wm + 32 * b + (int)bgmoe_k64_qpatch_read_token(lane);
            if (rtok < cnt)
              *reinterpret_cast<uint4*>(g.out_q + (row0 + rtok) * g.n + n0 + 32 * (int)wn +
                                        (int)bgmoe_k64_qpatch_read_col(lane)) = v;
            if (tok < cnt && wn == 0u && lane < 32u) g.out_s[(row0 + tok) * g.os_row + (int64_t)(n0 >> 7) * g.os_nb] = sc;
          } else if (tok < cnt) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float hv[4] = {acc[b][0][4 * q], acc[b][0][4 * q + 1], acc[b][0][4 * q + 2], acc[b][0][4 * q + 3]};
              float qv[4];
              quant_div_clamp(hv, sc, qv);
              *reinterpret_cast<uint32_t*>(g.out_q + (row0 + tok) * g.n + n0 +
                                           (int)bgmoe_k64_out_col(true, wn, 0, lane, 4 * q)) =
                  pack4_e4m3(qv[0], qv[1], qv[2], qv[3]);
            }
            if (wn == 0u && lane < 32u) g.out_s[(row0 + tok) * g.os_row + (int64_t)(n0 >> 7) * g.os_nb] = sc;
          }
        }
        // s_amax is written again by the next item's epilogue, at least 2 * KB >= 4 barriers from here
      }
    } else {
      // the wave's 64 columns lie inside N or past it as a whole when N is a multiple of 64 (the launcher takes the
      // regrouping form only then, and only for a 16-byte aligned output)
      if constexpr (REGROUP) {
        uint8_t* const patch = s_patch[wave];
        const int colw = n0 + 64 * (int)wn;
        if (colw < g.n) {                                  // wave-uniform
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            if (m0 + 128 * (int)wm + 32 * b >= cnt) continue;          // no live token in this image (wave-uniform)
#pragma unroll
            for (uint32_t p = 0; p < 4; ++p) {
              if (bgmoe_k64_patch_writer(lane, p)) {
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                  const float s = prev[b][a];
#pragma unroll
                  for (int q = 0; q < 4; ++q) {
                    uint2 o;
                    o.x = pack2_bf16(acc[b][a][4 * q] * s, acc[b][a][4 * q + 1] * s);
                    o.y = pack2_bf16(acc[b][a][4 * q + 2] * s, acc[b][a][4 * q + 3] * s);
                    *reinterpret_cast<uint2*>(patch + bgmoe_k64_patch_write_off(lane, (uint32_t)a, (uint32_t)q)) = o;
                  }
                }
              }
              __builtin_amdgcn_wave_barrier();
              const uint4 v = *reinterpret_cast<const uint4*>(patch + bgmoe_k64_patch_read_off(lane));
              __builtin_amdgcn_wave_barrier();
              const int rtok = m0 + 128 * (int)wm + 32 * b + (int)bgmoe_k64_patch_read_token(p, lane);
              if (rtok < cnt)
                *reinterpret_cast<uint4*>(g.out + (row0 + rtok) * g.n + colw + (int)bgmoe_k64_patch_read_col(lane)) = v;
            }
          }
        }
      } else {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const int tok = m0 + (int)bgmoe_k64_out_token(wm, b, lane);
          if (tok >= cnt) continue;
#pragma unroll
          for (int a = 0; a < 2; ++a) {
            const int col0 = n0 + (int)bgmoe_k64_out_col(false, wn, a, lane, 0);   // this product's first column
            if (col0 - 4 * (int)hsel >= g.n) continue;     // the whole 32-column image lies past N (wave-uniform)
            const float s = prev[b][a];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              uint2 o;
              o.x = pack2_bf16(acc[b][a][4 * q] * s, acc[b][a][4 * q + 1] * s);
              o.y = pack2_bf16(acc[b][a][4 * q + 2] * s, acc[b][a][4 * q + 3] * s);
              *reinterpret_cast<uint2*>(g.out + (row0 + tok) * g.n + n0 + (int)bgmoe_k64_out_col(false, wn, a, lane, 4 * q)) = o;
            }
          }
        }
      }
    }
    have = have_next;
    cur = nxt;
    buf ^= 1;
  }
  wait_vm<0>();                                          // no asynchronous LDS write may outlive the block
}

bool g_ready = false;

}  // namespace

// the dynamic-LDS opt-in of every variant, once
int bgmoe_internal_init_fp8_tiled_k64() {
  static int state = 0;                                  // 0 = not tried, 1 = ready, -1 = failed
  if (state == 0) {
    const void* fns[8] = {reinterpret_cast<const void*>(&fp8_tiled_k64_kernel<true, 0, false>),
                          reinterpret_cast<const void*>(&fp8_tiled_k64_kernel<false, 0, false>),
                          reinterpret_cast<const void*>(&fp8_tiled_k64_kernel<true, 1, false>),
                          reinterpret_cast<const void*>(&fp8_tiled_k64_kernel<false, 1, false>),
                          reinterpret_cast<const void*>(&fp8_tiled_k64_kernel<true, 0, true>),
                          reinterpret_cast<const void*>(&fp8_tiled_k64_kernel<false, 0, true>),
                          reinterpret_cast<const void*>(&fp8_tiled_k64_kernel<true, 1, true>),
                          reinterpret_cast<const void*>(&fp8_tiled_k64_kernel<false, 1, true>)};
    hipError_t e1 = hipSuccess;
    for (const void* f : fns) {
      const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
      if (e != hipSuccess) e1 = e;
    }
    if (e1 != hipSuccess) (void)hipGetLastError();
    state = e1 == hipSuccess ? 1 : -1;
    g_ready = state == 1;
  }
  return BGMOE_OK;
}

template <bool FUSED, int LAYOUT>
void launch_k64(const BgmoeTiledArgs& g, bool regroup, dim3 grid, hipStream_t st) {
  if (regroup) hipLaunchKernelGGL((fp8_tiled_k64_kernel<FUSED, LAYOUT, true>), grid, dim3(NT), kLds, st, g);
  else hipLaunchKernelGGL((fp8_tiled_k64_kernel<FUSED, LAYOUT, false>), grid, dim3(NT), kLds, st, g);
}

int bgmoe_launch_fp8_tiled_k64(const BgmoeTiledArgs& g, bool fused, bool regroup, int64_t m, int num_cu, hipStream_t st) {
  bgmoe_internal_init_fp8_tiled_k64();
  // K >= 256: the load cursor runs three K-steps ahead and may be at most one item ahead of the compute cursor.
  // N a multiple of 32: weight images are 32 rows.  Everything else is the K = 128 kernel's contract.
  if (!g_ready || g.k < 256 || g.k % 128 != 0 || g.n % 32 != 0 || g.n < 32) return BGMOE_ERR_WORKSPACE;
  if (g.groups > kMaxGroups || (g.k >> 7) > kMaxKB) return BGMOE_ERR_WORKSPACE;
  const int ncols = fused ? 128 : 256;
  const int64_t ntn = (g.n + ncols - 1) / ncols;
  const int64_t max_items = ((m + TM - 1) / TM + g.groups) * ntn;
  int64_t blocks = (int64_t)(num_cu > 0 ? num_cu : 256);
  if (blocks > max_items) blocks = max_items;
  if (blocks < 8) blocks = 8;
  const dim3 grid((unsigned)blocks);
  const bool tm = g.w0.layout == BGMOE_W_TILE_MAJOR;
  // the regrouping epilogue stores 16 bytes per lane: e4m3 rows need a 16-byte aligned base (N is a multiple of 128
  // for stage 1), bf16 rows a 16-byte aligned base and the wave's 64 columns inside or past N as a whole
  if (regroup) {
    if (fused) regroup = g.out_q != nullptr && ((uintptr_t)g.out_q & 15) == 0 && g.n % 16 == 0;
    else regroup = ((uintptr_t)g.out & 15) == 0 && g.n % 64 == 0;
  }
  if (fused) {
    if (tm) launch_k64<true, 1>(g, regroup, grid, st);
    else launch_k64<true, 0>(g, regroup, grid, st);
  } else {
    if (tm) launch_k64<false, 1>(g, regroup, grid, st);
    else launch_k64<false, 0>(g, regroup, grid, st);
  }
  return bgmoe_check_launch("fp8 grouped gemm (tiled, K = 64)");
}
