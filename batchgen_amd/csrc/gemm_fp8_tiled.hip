// Block-scaled FP8 grouped GEMM for MANY rows per group (prefill): an LDS-tiled MFMA kernel.
//
// Macro tile: 256 tokens x 256 weight rows x 128 K per step (fused stage 1: 128 gate + 128 up rows, so
// SwiGLU and the requant of one 128-column group stay inside the block).  8 waves = 4 (weight rows) x
// 2 (tokens); a wave owns 64 weight rows (fused: 32 gate + 32 up) x 128 tokens = 8 x 4 MFMA 16x16x128
// tiles, 128 fp32 accumulators per lane.  Two waves share a SIMD, so the fp32 promotion
// (acc += partial * token_scale * weight_scale, VALU) of one overlaps the MFMAs of the other, and with
// <= 256 registers per lane the compiler emits the MFMAs with VGPR destinations (no AGPR copies).
//
// Operand staging: a 2-slot LDS ring (2 x 65 KB) filled by ASYNCHRONOUS global -> LDS loads
// (global_load_lds_dwordx4: every lane supplies its own global address, the wave's 64 x 16 bytes land
// contiguously at the LDS address in M0).  The lane -> address map is chosen so that each 1 KiB wave
// load is half of an MFMA operand "tile image": lane l = q*16 + r carries row r, bytes 16q..16q+15 of
// the 64-byte half-segment, which is exactly what lane l feeds to v_mfma_f32_16x16x128_f8f6f4 -- so
// operand reads from LDS are plain lane*16 accesses (conflict free, no swizzle), for row-major tokens,
// row-major weights and tile-major weights alike.  The next K-step is in flight while the current one
// is computed; completion is tracked by hand with s_waitcnt vmcnt (the loads are issued from inline
// asm, which keeps the compiler from draining the queue before every LDS read) and one s_barrier per
// K-step.
//
// Scheduling: a fixed grid of persistent blocks walks a device-built list of (group, n-tile, m-tile)
// work items ordered so that the blocks of one XCD (block b runs on XCD b % 8) work on a compact patch
// of m- and n-tiles and share their operands through that XCD's L2.  Groups at or below the row limit
// of bgmoe_split_limit() are left to the weight-streaming kernel; empty groups cost nothing.
#include "gemm_fp8_tiled.h"
#include "bgmoe_async.h"

namespace {

using TiledArgs = BgmoeTiledArgs;

constexpr int TM = 256;            // tokens per macro tile
constexpr int TW = 256;            // weight rows per macro tile
constexpr int NS = 2;              // LDS ring slots
constexpr int NT = 512;            // threads per block
constexpr int kTokBytes = TM * 128;
constexpr int kWBytes = TW * 128;
constexpr int kXsOff = kTokBytes + kWBytes;
constexpr int kSlotBytes = kXsOff + TM * 4;
constexpr int kPanel = 8;          // m-tiles per panel of the work-item order
constexpr int kMaxGroups = kBgmoeTiledMaxGroups;
constexpr int kMaxKB = kBgmoeTiledMaxKB;        // K <= 32768

template <bool FUSED, int LAYOUT>
__global__ __launch_bounds__(NT) void fp8_tiled_kernel(TiledArgs g) {
  extern __shared__ __align__(16) uint8_t smem[];      // NS slots
  __shared__ int s_tiles[kMaxGroups + 1];              // exclusive prefix of m-tiles per group
  __shared__ float s_ws[2][2][kMaxKB];                 // [buffer][row] weight scales along K of an item
  // the fused epilogue's amax exchange [2][4][8][16] floats, or the plain epilogue's per-wave transpose
  // patches (16 token rows x 144 B each): never both
  constexpr int kEpiPitch = 144;
  __shared__ __align__(16) uint8_t s_scratch[NT / 64 * 16 * kEpiPitch];
  float (*s_amax)[4][8][16] = reinterpret_cast<float (*)[4][8][16]>(s_scratch);

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int wn = wave & 3;                             // which 64 weight rows
  const int wm = wave >> 2;                            // which 128 tokens
  const int lane = tid & 63;
  const int r16 = lane & 15;
  const int kq = lane >> 4;
  const int K = g.k;
  const int KB = K >> 7;
  const int ncols = FUSED ? 128 : 256;                 // output columns per macro tile
  const int ntn = (g.n + ncols - 1) / ncols;
  const uint32_t smem_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem);
  const uint32_t wave_u = __builtin_amdgcn_readfirstlane((uint32_t)wave);

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
  // XCD-aware walk: block b (XCD b % 8) takes items of the b%8-th eighth of the list
  const int nx = 8;
  const int xcd = blockIdx.x % nx;
  const int per_x = (int)((total + nx - 1) / nx);
  const int bstep = (gridDim.x + nx - 1 - xcd) / nx;   // blocks living on this XCD
  const int bidx = blockIdx.x / nx;
  // Tail of the static walk: this XCD's items are dealt to its bstep blocks in rounds.  When the last round
  // is at most half full, each of its items is split into two 128-token halves handled by different blocks
  // (a half keeps one wave per SIMD busy and takes little more than half the time), so the kernel ends
  // half a round earlier.
  const int64_t first_x = (int64_t)xcd * per_x;
  const int cnt_x = (int)max((int64_t)0, min((int64_t)per_x, total - first_x));
  const int rounds_x = (cnt_x + bstep - 1) / bstep;
  const int split_base = rounds_x > 0 ? (rounds_x - 1) * bstep : 0;
  const int split_rem = cnt_x - split_base;
  const bool split_tail = rounds_x > 0 && 2 * split_rem <= bstep;
  const int walk_x = split_tail ? split_base + 2 * split_rem : cnt_x;      // virtual items of this XCD

  // ---- per-item state ----
  struct Meta { int cnt, m0, n0; int64_t row0; };
  const uint32_t ws_lds = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)&s_ws[0][0][0]);
  const int lrow = lane >> 3;
  const int lchunk = ((lane & 7) ^ lrow) * 16;
  // load sources of the item whose K-loop runs (or is about to run): wave-uniform bases + lane offsets
  const uint8_t* tok_base = nullptr;
  uint32_t tok_off[2][2] = {{0u, 0u}, {0u, 0u}};
  const uint8_t* w_base[2] = {nullptr, nullptr};
  const uint32_t w_off = LAYOUT == BGMOE_W_ROW_MAJOR ? (uint32_t)lrow * (uint32_t)K + lchunk : lane * 16;
  const float* xs_base = nullptr;
  uint32_t xs_off = 0u;
  const float* ws_src = nullptr;                       // waves 0 and 1: the weight-scale row each stages

  // item index of this block's walk -> (group, n-tile, m-tile) and its load sources
  auto prepare = [&](int64_t itx, Meta& mt) -> bool {
    if (itx >= walk_x) return false;
    int half = -1;                                         // -1: the whole 256-token tile
    int64_t item = first_x + itx;
    if (split_tail && itx >= split_base) {
      item = first_x + split_base + ((itx - split_base) >> 1);
      half = (int)((itx - split_base) & 1);
    }
    int lo_g = 0, hi_g = g.groups - 1;
    while (lo_g < hi_g) {
      const int mid = (lo_g + hi_g + 1) >> 1;
      if ((int64_t)s_tiles[mid] * ntn <= item) lo_g = mid; else hi_g = mid - 1;
    }
    const int grp = __builtin_amdgcn_readfirstlane(lo_g);   // (LDS reads look divergent to the compiler)
    const int mt_g = __builtin_amdgcn_readfirstlane(s_tiles[grp + 1] - s_tiles[grp]);
    const int64_t rel = item - (int64_t)__builtin_amdgcn_readfirstlane(s_tiles[grp]) * ntn;
    // panels of kPanel m-tiles; inside a panel n-tiles advance with m fastest, so the 32 items an XCD works
    // on at one time form a compact (m, n) patch: few distinct token and weight streams per L2
    const int panel = (int)(rel / ((int64_t)kPanel * ntn));
    const int pm = min(kPanel, mt_g - panel * kPanel);
    const int r2 = (int)(rel - (int64_t)panel * kPanel * ntn);
    const int nt = r2 / pm;
    const int mtile = panel * kPanel + (r2 - nt * pm);
    int cnt = g.seqlens[grp];
    const int64_t row0 = g.cu[grp];
    int m0 = mtile * TM;
    if (half >= 0) {                                       // rows [m0 + 128*half, +128) of the tile
      m0 += 128 * half;
      if (m0 >= cnt) return false;                         // no live row in this half; a block has at most one
                                                           // split item and it is its last, so it is done
      cnt = min(cnt, m0 + 128);
    }
    const int n0 = nt * ncols;
    mt.cnt = cnt; mt.m0 = m0; mt.n0 = n0; mt.row0 = row0;

    const uint8_t* wb0 = g.w0.w_ptrs ? g.w0.w_ptrs[grp] : g.w0.w + (int64_t)grp * g.w0.w_group_stride;
    const float* ws0 = (g.w0.scale_ptrs ? g.w0.scale_ptrs[grp] : g.w0.scale + (int64_t)grp * g.w0.scale_group_stride);
    const uint8_t* wb1 = nullptr;
    // weight scales along K: fused [0] gate, [1] up; else [0] columns 0..127, [1] columns 128..255 of the tile
    if constexpr (FUSED) {
      wb1 = g.w1.w_ptrs ? g.w1.w_ptrs[grp] : g.w1.w + (int64_t)grp * g.w1.w_group_stride;
      const float* ws1 = (g.w1.scale_ptrs ? g.w1.scale_ptrs[grp] : g.w1.scale + (int64_t)grp * g.w1.scale_group_stride) +
                         (int64_t)(n0 >> 7) * g.w1.scale_nb_stride;
      ws0 += (int64_t)(n0 >> 7) * g.w0.scale_nb_stride;
      ws_src = uniform_ptr(wave_u == 0 ? ws0 : ws1);
    } else {
      const int nb = min(n0 + (wave_u == 0 ? 0 : 128), g.n - 1) >> 7;
      ws_src = uniform_ptr(ws0 + (int64_t)nb * g.w0.scale_nb_stride);
    }

    // this wave's share of a stage: token tiles 2w, 2w+1; weight tiles 2w, 2w+1; waves 0..3: 64 token scales.
    // Row-major sources: load j of a tile covers rows 8j..8j+7, lane p = (row p>>3, LDS chunk p&7) fetches
    // the row's 16-byte chunk (p&7) ^ (p>>3): whole 128-byte lines per 8 lanes, XOR-swizzled in LDS
    tok_base = uniform_ptr(g.a.x + (row0 + m0) * K);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int tok = min(16 * (2 * wave + i) + 8 * j + lrow, cnt - 1 - m0);
        tok_off[i][j] = (uint32_t)tok * (uint32_t)K + lchunk;
      }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int lt = 2 * wave_u + i;               // LDS weight tile 0..15 (16 rows each)
      const int r = lt * 16;
      const int nrow = FUSED ? min(n0 + (r & 127), g.n - 16) : min(n0 + r, g.n - 16);
      const uint8_t* base = (FUSED && r >= 128) ? wb1 : wb0;
      // row-major: row nrow; tile-major: tile nrow / 16 (16 x K bytes per row of tiles)
      w_base[i] = uniform_ptr(base + (int64_t)(LAYOUT == BGMOE_W_ROW_MAJOR ? nrow : (nrow & ~15)) * K);
    }
    xs_base = uniform_ptr(g.a.scale_group_stride
                              ? g.a.scale + grp * g.a.scale_group_stride + (int64_t)m0 * g.a.scale_row_stride
                              : g.a.scale + (row0 + m0) * g.a.scale_row_stride);
    xs_off = (uint32_t)min(64 * wn + lane, cnt - 1 - m0) * (uint32_t)g.a.scale_row_stride * 4u;
    return true;
  };

  auto issue = [&](int kb, int slot) {
    const uint32_t sb = smem_base + (uint32_t)slot * kSlotBytes;
    const int ko = kb << 7;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const uint32_t d = sb + (2 * wave_u + i) * 2048;
      async_load16(tok_base + ko, tok_off[i][0], d);
      async_load16(tok_base + ko, tok_off[i][1], d + 1024);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const uint32_t d = sb + kTokBytes + (2 * wave_u + i) * 2048;
      if constexpr (LAYOUT == BGMOE_W_ROW_MAJOR) {
        async_load16(w_base[i] + ko, w_off, d);
        async_load16(w_base[i] + ko + 8 * (int64_t)K, w_off, d + 1024);
      } else {
        async_load16(w_base[i] + ((int64_t)kb << 11), w_off, d);
        async_load16(w_base[i] + ((int64_t)kb << 11) + 1024, w_off, d + 1024);
      }
    }
    if (wave_u < 4)
      async_load4(xs_base + (int64_t)kb * g.a.scale_kb_stride, xs_off, sb + kXsOff + wave_u * 256);
  };
  // waves 0 and 1 stage the item's two weight-scale rows (KB floats each) into s_ws[buf]
  auto issue_scales = [&](int buf) {
    if (wave_u < 2) {
      for (int c = 0; c < KB; c += 64)
        async_load4(ws_src, (uint32_t)min(c + lane, KB - 1) * 4u,
                    ws_lds + (uint32_t)(((buf * 2 + (int)wave_u) * kMaxKB + c) * 4));
    }
  };

  // The walk is software-pipelined across items: the first K-step and the scales of the next item are
  // requested before the epilogue of the current one, into the ring slot and scale buffer it no longer uses.
  Meta cur{}, nxt{};
  int64_t itx = bidx;
  bool have = prepare(itx, cur);
  int sbase = 0, buf = 0;
  if (have) {
    issue_scales(buf);
    issue(0, sbase);
  }
  while (have) {
    const int cnt = cur.cnt, m0 = cur.m0, n0 = cur.n0;
    const int64_t row0 = cur.row0;
    floatx4 acc[8][4];
#pragma unroll
    for (int tt = 0; tt < 8; ++tt)
#pragma unroll
      for (int t = 0; t < 4; ++t) acc[tt][t] = floatx4{0.f, 0.f, 0.f, 0.f};

    const bool wave_live = m0 + 128 * (int)(wave_u >> 2) < cnt;
    for (int kb = 0; kb < KB; ++kb) {
      const int slot = (sbase + kb) & 1;
      wait_vm<0>();                              // this wave's loads of step kb have landed ...
      block_barrier();                           // ... and everybody's; everybody is done with step kb-1
      if (kb + 1 < KB) issue(kb + 1, slot ^ 1);  // refill the slot step kb-1 used

      // a wave whose 128 tokens all lie past the group's end (the last m-tile of a ragged group) only keeps
      // the barriers and its share of the loads: the wave it shares a SIMD with gets the whole MFMA pipe
      if (!wave_live) continue;
      const uint8_t* b = smem + slot * kSlotBytes;
      const uint8_t* bw = b + kTokBytes;
      const float* bxs = reinterpret_cast<const float*>(b + kXsOff);
      const float wsc0 = s_ws[buf][0][kb], wsc1 = s_ws[buf][1][kb];

      // operand offsets inside a 2 KiB tile image: swizzled row-major (tokens, row-major weights) or lane order
      const int sw_lo = r16 * 128 + ((kq ^ (r16 & 7)) * 16);
      const int a_lo = LAYOUT == BGMOE_W_ROW_MAJOR ? sw_lo : lane * 16;
      const int a_hi = LAYOUT == BGMOE_W_ROW_MAJOR ? (sw_lo ^ 64) : lane * 16 + 1024;
      const uint8_t* bt = b + 8 * wm * 2048;
      const float* bx = bxs + 128 * wm + r16;
      auto load_b = [&](int tt) {
        const intx4 lo = *reinterpret_cast<const intx4*>(bt + tt * 2048 + sw_lo);
        const intx4 hi = *reinterpret_cast<const intx4*>(bt + tt * 2048 + (sw_lo ^ 64));
        return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      };
      // LDS returns data in request order: the first token tile and the first weight tile are requested
      // first, so the first MFMA waits for 4 reads instead of 10
      intx8 Bb[2];
      float xb[2];
      Bb[0] = load_b(0);
      xb[0] = bx[0];
      intx8 A[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int lt = FUSED ? ((t >> 1) * 8 + 2 * wn + (t & 1)) : (4 * wn + t);
        const intx4 lo = *reinterpret_cast<const intx4*>(bw + lt * 2048 + a_lo);
        const intx4 hi = *reinterpret_cast<const intx4*>(bw + lt * 2048 + a_hi);
        A[t] = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
      // 32 MFMAs (token tile tt = idx/4, weight tile t = idx%4) in one software pipeline: token tile tt+1
      // is fetched from LDS while tile tt is multiplied, and the promotion of product idx-2
      // (acc += partial * scale, VALU) is issued behind MFMA idx
      floatx4 P[3];
      float psc[2][2];
#pragma unroll
      for (int idx = 0; idx < 34; ++idx) {
        if (idx < 32) {
          const int tt = idx >> 2, t = idx & 3;
          if (t == 0) {
            if (tt < 7) {
              Bb[(tt + 1) & 1] = load_b(tt + 1);
              xb[(tt + 1) & 1] = bx[16 * (tt + 1)];
            }
            // fused: tiles 0,1 gate (scale 0), 2,3 up (scale 1); else all four tiles share one 128-column block
            psc[tt & 1][0] = xb[tt & 1] * (FUSED ? wsc0 : ((wn >= 2) ? wsc1 : wsc0));
            psc[tt & 1][1] = xb[tt & 1] * (FUSED ? wsc1 : ((wn >= 2) ? wsc1 : wsc0));
          }
          P[idx % 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
              A[t], Bb[tt & 1], floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
        }
        if (idx >= 2) {
          const int j = idx - 2, tt = j >> 2, t = j & 3;
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[tt][t][i] = fmaf(P[j % 3][i], psc[tt & 1][t >> 1], acc[tt][t][i]);
        }
      }
    }

    // ---- next item: sources, scales and first K-step (the slot used by step KB-2 is free) ----
    itx += bstep;
    const int nslot = (sbase + KB) & 1;
    have = prepare(itx, nxt);
    if (have) {
      issue_scales(buf ^ 1);
      issue(0, nslot);
    }

    // ---- epilogue of the current item -----------------------------------------------
    if constexpr (FUSED) {
#pragma unroll
      for (int tt = 0; tt < 8; ++tt) {
        float am = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float h = bf16_round_f32(silu_rcp_f32(acc[tt][j][i]) * acc[tt][j + 2][i]);
            acc[tt][j][i] = h;
            am = fmaxf(am, fabsf(h));
          }
        const int tok = m0 + 128 * wm + 16 * tt + r16;
        if (g.out != nullptr && tok < cnt) {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            uint2 o;
            o.x = pack2_bf16(acc[tt][j][0], acc[tt][j][1]);
            o.y = pack2_bf16(acc[tt][j][2], acc[tt][j][3]);
            *reinterpret_cast<uint2*>(g.out + (row0 + tok) * g.n + n0 + 32 * wn + 16 * j + 4 * kq) = o;
          }
        }
        if (g.out_q != nullptr) {
          am = fmaxf(am, __shfl_xor(am, 16, BGMOE_WAVE));
          am = fmaxf(am, __shfl_xor(am, 32, BGMOE_WAVE));
          if (kq == 0) s_amax[wm][wn][tt][r16] = am;
        }
      }
      if (g.out_q != nullptr) {
        __syncthreads();
#pragma unroll
        for (int tt = 0; tt < 8; ++tt) {
          const float am = fmaxf(fmaxf(s_amax[wm][0][tt][r16], s_amax[wm][1][tt][r16]),
                                 fmaxf(s_amax[wm][2][tt][r16], s_amax[wm][3][tt][r16]));
          const float sc = quant_scale_from_amax(am);
          const int tok = m0 + 128 * wm + 16 * tt + r16;
          if (tok < cnt) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const float hv[4] = {acc[tt][j][0], acc[tt][j][1], acc[tt][j][2], acc[tt][j][3]};
              float qv[4];
              quant_div_clamp(hv, sc, qv);
              const uint32_t q = pack4_e4m3(qv[0], qv[1], qv[2], qv[3]);
              *reinterpret_cast<uint32_t*>(g.out_q + (row0 + tok) * g.n + n0 + 32 * wn + 16 * j + 4 * kq) = q;
            }
            if (wn == 0 && kq == 0)
              g.out_s[(row0 + tok) * g.os_row + (int64_t)(n0 >> 7) * g.os_nb] = sc;
          }
        }
      }
    } else {
      // A lane holds 4 consecutive output columns of one token: stored as they are, a store instruction
      // would touch 16 token rows with 32 bytes each.  Each 16-token tile goes through a per-wave LDS patch
      // instead (written 8 B per lane, read back 16 B per lane with 8 lanes per token row), so that a store
      // instruction writes 8 whole 128-byte row segments.  LDS operations of one wave execute in order: no
      // barrier is needed between the patch's write, its read and the next tile's write.
      uint8_t* const patch = s_scratch + wave * (16 * kEpiPitch);
      const int col0 = n0 + 64 * wn;                       // this wave's 64 columns: all inside or all outside N
      const bool wide = ((uintptr_t)g.out & 15) == 0;
#pragma unroll
      for (int tt = 0; tt < 8; ++tt) {
        const int tok0 = m0 + 128 * wm + 16 * tt;
        if (tok0 >= cnt || col0 >= g.n) continue;          // wave-uniform
        if (wide) {
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            uint2 o;
            o.x = pack2_bf16(acc[tt][t][0], acc[tt][t][1]);
            o.y = pack2_bf16(acc[tt][t][2], acc[tt][t][3]);
            *reinterpret_cast<uint2*>(patch + r16 * kEpiPitch + (16 * t + 4 * kq) * 2) = o;
          }
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const int row = (lane >> 3) + 8 * i;
            const uint4 v = *reinterpret_cast<const uint4*>(patch + row * kEpiPitch + (lane & 7) * 16);
            if (tok0 + row < cnt)
              *reinterpret_cast<uint4*>(g.out + (row0 + tok0 + row) * g.n + col0 + (lane & 7) * 8) = v;
          }
        } else {
          const int tok = tok0 + r16;
          if (tok >= cnt) continue;
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            uint2 o;
            o.x = pack2_bf16(acc[tt][t][0], acc[tt][t][1]);
            o.y = pack2_bf16(acc[tt][t][2], acc[tt][t][3]);
            *reinterpret_cast<uint2*>(g.out + (row0 + tok) * g.n + col0 + 16 * t + 4 * kq) = o;
          }
        }
      }
    }
    cur = nxt;
    sbase = nslot;
    buf ^= 1;
  }
}

int g_num_cu = 0;
int g_variant = 0;                 // 0: this file's K = 128 kernel; 1, 2: the K = 64 kernel where it applies

}  // namespace

// Which LDS-tiled kernel serves the groups above the streaming limit (no reference counterpart): 0 = the K = 128
// kernel (16x16x128 products, two 65 KB ring slots), 1 = the K = 64 kernel (32x32x64 products accumulated in
// place, four 33 KB slots) for K >= 256, the K = 128 kernel otherwise; 2 = the same with plain per-lane stores in its
// epilogue instead of the regrouped ones (for comparison).  Results of the two kernels differ in rounding only; 1
// and 2 give the same bits.
extern "C" int bgmoe_set_tiled_variant(int variant) {
  BGMOE_REQUIRE(variant >= 0 && variant <= 2, "set_tiled_variant: variant must be 0 (K = 128), 1 or 2 (K = 64), got %d", variant);
  g_variant = variant;
  return BGMOE_OK;
}

// device query and the dynamic-LDS opt-in of every variant, once
int bgmoe_internal_init_fp8_tiled() {
  static bool attr_set = false;
  if (attr_set) return BGMOE_OK;
  constexpr int kLds = NS * kSlotBytes;
  hipDeviceProp_t prop;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
    bgmoe_set_error("fp8 tiled gemm: cannot query the device");
    return BGMOE_ERR_HIP;
  }
  g_num_cu = prop.multiProcessorCount;
  hipError_t e1 = hipSuccess;
  const void* fns[4] = {reinterpret_cast<const void*>(&fp8_tiled_kernel<true, 0>),
                        reinterpret_cast<const void*>(&fp8_tiled_kernel<false, 0>),
                        reinterpret_cast<const void*>(&fp8_tiled_kernel<true, 1>),
                        reinterpret_cast<const void*>(&fp8_tiled_kernel<false, 1>)};
  for (const void* f : fns) {
    hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) e1 = e;
  }
  if (e1 != hipSuccess) {
    bgmoe_set_error("fp8 tiled gemm: cannot reserve %d bytes of LDS", kLds);
    return BGMOE_ERR_HIP;
  }
  attr_set = true;
  return BGMOE_OK;
}

int bgmoe_launch_fp8_tiled(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* w0, const bgmoe_fp8_weight* w1,
                           const int32_t* seqlens, const int32_t* cu, int groups, int64_t m, int n, int k,
                           uint16_t* out, uint8_t* out_q, float* out_s, int64_t os_row, int64_t os_nb,
                           BgmoeSplit split, hipStream_t st) {
  if (groups == 0 || m == 0) return BGMOE_OK;
  if (groups > kMaxGroups) {
    bgmoe_set_error("fp8 tiled gemm: groups=%d exceeds %d", groups, kMaxGroups);
    return BGMOE_ERR_ARG;
  }
  if ((k >> 7) > kMaxKB) {
    bgmoe_set_error("fp8 tiled gemm: K=%d exceeds %d", k, kMaxKB * 128);
    return BGMOE_ERR_ARG;
  }
  TiledArgs g{};
  g.a = *a; g.w0 = *w0; if (w1) g.w1 = *w1;
  g.seqlens = seqlens; g.cu = cu; g.groups = groups; g.n = n; g.k = k;
  g.out = out; g.out_q = out_q; g.out_s = out_s; g.os_row = os_row; g.os_nb = os_nb; g.split = split;
  constexpr int kLds = NS * kSlotBytes;
  const int irc = bgmoe_internal_init_fp8_tiled();
  if (irc != BGMOE_OK) return irc;
  // upper bound on work items from host shapes only
  const int ncols = w1 ? 128 : 256;
  const int64_t ntn = (n + ncols - 1) / ncols;
  const int64_t max_items = ((m + TM - 1) / TM + groups) * ntn;
  int64_t blocks = (int64_t)(g_num_cu > 0 ? g_num_cu : 256);
  if (blocks > max_items) blocks = max_items;
  if (blocks < 8) blocks = 8;
  BgmoeProf prof(w1 ? BGMOE_K_S1_TILED : BGMOE_K_GEMM_TILED, st);
  if (g_variant != 0) {
    const int rc = bgmoe_launch_fp8_tiled_k64(g, w1 != nullptr, g_variant == 1, m, g_num_cu, st);
    if (rc != BGMOE_ERR_WORKSPACE) return rc;            // (without a message: the variant does not apply here)
  }
  const dim3 grid((unsigned)blocks), block(NT);
  const bool tm = w0->layout == BGMOE_W_TILE_MAJOR;
  if (w1) {
    if (tm) hipLaunchKernelGGL((fp8_tiled_kernel<true, 1>), grid, block, kLds, st, g);
    else hipLaunchKernelGGL((fp8_tiled_kernel<true, 0>), grid, block, kLds, st, g);
  } else {
    if (tm) hipLaunchKernelGGL((fp8_tiled_kernel<false, 1>), grid, block, kLds, st, g);
    else hipLaunchKernelGGL((fp8_tiled_kernel<false, 0>), grid, block, kLds, st, g);
  }
  return bgmoe_check_launch("fp8 grouped gemm (tiled)");
}
