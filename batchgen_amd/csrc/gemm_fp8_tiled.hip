// Block-scaled FP8 grouped GEMM for MANY rows per group (prefill, the shared
// expert): an LDS-tiled MFMA kernel.
//
// Macro tile: 128 tokens x 256 weight rows x 128 K per step (fused stage 1:
// 128 gate + 128 up rows, so SwiGLU and the requant of one 128-column group
// stay inside the block).  4 waves; wave w owns 64 weight rows (fused: 32 gate
// + 32 up) for all 128 tokens = 8 x 4 MFMA 16x16x128 tiles, 128 accumulator
// registers.  Global -> registers -> LDS double buffering, one barrier per K
// step.  LDS rows are 128 B with the 16-byte chunk index XOR-swizzled by
// (row & 7), which makes both the 16-byte stores and the MFMA operand reads
// (16 rows x 16 B per quarter-wave) conflict free.
//
// Scheduling: a fixed grid of persistent blocks walks a device-built list of
// (group, n-tile, m-tile) work items, m fastest, so the blocks of one XCD
// (block b runs on XCD b % 8) work on neighbouring m-tiles of the same weight
// tile and share it through that XCD's L2.  Groups with <= `lo` rows are left
// to the weight-streaming kernel; empty groups cost nothing.
#include "bgmoe_common.h"

namespace {

constexpr int TM = 128;            // tokens per macro tile
constexpr int TW = 256;            // weight rows per macro tile
constexpr int kTokBytes = TM * 128;
constexpr int kWBytes = TW * 128;
constexpr int kBufBytes = kTokBytes + kWBytes + TM * 4;
constexpr int kMaxGroups = 1024;

struct TiledArgs {
  bgmoe_fp8_act a;
  bgmoe_fp8_weight w0, w1;
  const int32_t* seqlens;
  const int32_t* cu;
  int groups, n, k;
  uint16_t* out;
  uint8_t* out_q;
  float* out_s;
  int64_t os_row, os_nb;
  int lo;
  int fused;
};

__device__ __forceinline__ int swz(int row, int chunk) { return row * 128 + ((chunk ^ (row & 7)) << 4); }

template <bool FUSED, int LAYOUT>
__global__ __launch_bounds__(256) void fp8_tiled_kernel(TiledArgs g) {
  extern __shared__ __align__(16) uint8_t smem[];
  __shared__ int s_tiles[kMaxGroups + 1];       // exclusive prefix of m-tiles per group
  __shared__ float s_amax[4][8][16];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int r16 = lane & 15;
  const int kq = lane >> 4;
  const int K = g.k;
  const int KB = K >> 7;
  const int ncols = FUSED ? 128 : 256;           // output columns per macro tile
  const int ntn = (g.n + ncols - 1) / ncols;

  // ---- work list: m-tiles per group, prefix-summed (every block computes the same list) ----
  if (tid == 0) {
    int run = 0;
    for (int e = 0; e < g.groups; ++e) {
      s_tiles[e] = run;
      const int c = g.seqlens[e];
      run += c > g.lo ? (c + TM - 1) / TM : 0;
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

  for (int64_t it = (int64_t)bidx; it < per_x; it += bstep) {
    const int64_t item = (int64_t)xcd * per_x + it;
    if (item >= total) break;
    // item -> (group, n-tile, m-tile): within a group, m fastest
    int lo_g = 0, hi_g = g.groups - 1;
    {
      // find group: largest e with s_tiles[e]*ntn <= item
      while (lo_g < hi_g) {
        const int mid = (lo_g + hi_g + 1) >> 1;
        if ((int64_t)s_tiles[mid] * ntn <= item) lo_g = mid; else hi_g = mid - 1;
      }
    }
    const int grp = lo_g;
    const int mt_g = s_tiles[grp + 1] - s_tiles[grp];
    const int64_t rel = item - (int64_t)s_tiles[grp] * ntn;
    const int nt = (int)(rel / mt_g);
    const int mt = (int)(rel - (int64_t)nt * mt_g);
    const int cnt = g.seqlens[grp];
    const int64_t row0 = g.cu[grp];
    const int m0 = mt * TM;
    const int n0 = nt * ncols;

    const uint8_t* wb0 = g.w0.w_ptrs ? g.w0.w_ptrs[grp] : g.w0.w + (int64_t)grp * g.w0.w_group_stride;
    const float* ws0 = (g.w0.scale_ptrs ? g.w0.scale_ptrs[grp] : g.w0.scale + (int64_t)grp * g.w0.scale_group_stride);
    const uint8_t* wb1 = nullptr;
    const float* ws1 = nullptr;
    if constexpr (FUSED) {
      wb1 = g.w1.w_ptrs ? g.w1.w_ptrs[grp] : g.w1.w + (int64_t)grp * g.w1.w_group_stride;
      ws1 = (g.w1.scale_ptrs ? g.w1.scale_ptrs[grp] : g.w1.scale + (int64_t)grp * g.w1.scale_group_stride) +
            (int64_t)(n0 >> 7) * g.w1.scale_nb_stride;
      ws0 += (int64_t)(n0 >> 7) * g.w0.scale_nb_stride;
    }
    const float* wsw = nullptr;                    // non-fused: this wave's 128-row block
    if constexpr (!FUSED) wsw = ws0 + (int64_t)(min(n0 + 64 * wave, g.n - 1) >> 7) * g.w0.scale_nb_stride;

    // ---- global -> register staging: 4 token chunks + 8 weight chunks per thread per step ----
    const int lrow = tid >> 3;                     // 0..31
    const int chunk = tid & 7;
    const uint8_t* tok_src[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int tok = min(m0 + i * 32 + lrow, cnt - 1);
      tok_src[i] = g.a.x + (row0 + tok) * K + chunk * 16;
    }
    const uint8_t* w_src[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if constexpr (LAYOUT == BGMOE_W_ROW_MAJOR) {
        const int r = i * 32 + lrow;               // LDS weight row 0..255
        if constexpr (FUSED) {
          const int nrow = min(n0 + (r & 127), g.n - 1);
          w_src[i] = (r < 128 ? wb0 : wb1) + (int64_t)nrow * K + chunk * 16;
        } else {
          const int nrow = min(n0 + r, g.n - 1);
          w_src[i] = wb0 + (int64_t)nrow * K + chunk * 16;
        }
      } else {
        // tile-major source: LDS keeps the 2 KiB tile image; this thread moves 16 bytes of LDS tile
        // 2*i + (tid >> 7) (16 weight rows each), a contiguous 2 KiB per 128 threads
        const int lt = 2 * i + (tid >> 7);         // LDS tile 0..15
        const int r = lt * 16;
        const int nrow = FUSED ? min(n0 + (r & 127), g.n - 16) : min(n0 + r, g.n - 16);
        w_src[i] = ((FUSED && r >= 128) ? wb1 : wb0) + (int64_t)(nrow >> 4) * K * 16 + (tid & 127) * 16;
      }
    }
    const float* xs_src = nullptr;
    if (tid < TM) xs_src = g.a.scale + (row0 + min(m0 + tid, cnt - 1)) * g.a.scale_row_stride;

    intx4 rt[4], rw[8];
    float rxs = 0.0f;
    auto gload = [&](int kb) {
      const int ko = kb << 7;
#pragma unroll
      for (int i = 0; i < 4; ++i) rt[i] = gload_x4(tok_src[i] + ko);
#pragma unroll
      for (int i = 0; i < 8; ++i)
        rw[i] = gload_x4(w_src[i] + (LAYOUT == BGMOE_W_ROW_MAJOR ? (int64_t)ko : ((int64_t)kb << 11)));
      if (tid < TM) rxs = xs_src[(int64_t)kb * g.a.scale_kb_stride];
    };
    auto lstore = [&](int buf) {
      uint8_t* b = smem + buf * kBufBytes;
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<intx4*>(b + swz(i * 32 + lrow, chunk)) = rt[i];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if constexpr (LAYOUT == BGMOE_W_ROW_MAJOR)
          *reinterpret_cast<intx4*>(b + kTokBytes + swz(i * 32 + lrow, chunk)) = rw[i];
        else
          *reinterpret_cast<intx4*>(b + kTokBytes + i * 4096 + tid * 16) = rw[i];
      }
      if (tid < TM) reinterpret_cast<float*>(b + kTokBytes + kWBytes)[tid] = rxs;
    };

    floatx4 acc[8][4];
#pragma unroll
    for (int tt = 0; tt < 8; ++tt)
#pragma unroll
      for (int t = 0; t < 4; ++t) acc[tt][t] = floatx4{0.f, 0.f, 0.f, 0.f};

    __syncthreads();          // previous item's LDS reads are done
    gload(0);
    lstore(0);
    __syncthreads();

    for (int kb = 0; kb < KB; ++kb) {
      const int cur = kb & 1;
      if (kb + 1 < KB) gload(kb + 1);
      const uint8_t* b = smem + cur * kBufBytes;
      const uint8_t* bw = b + kTokBytes;
      const float* bxs = reinterpret_cast<const float*>(b + kTokBytes + kWBytes);
      float wsc[2];
      if constexpr (FUSED) { wsc[0] = ws0[kb]; wsc[1] = ws1[kb]; }
      else { wsc[0] = wsw[kb]; wsc[1] = wsc[0]; }

      intx8 A[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int wr = FUSED ? ((t >> 1) * 128 + 32 * wave + 16 * (t & 1) + r16) : (64 * wave + 16 * t + r16);
        intx4 lo, hi;
        if constexpr (LAYOUT == BGMOE_W_ROW_MAJOR) {
          lo = *reinterpret_cast<const intx4*>(bw + swz(wr, kq));
          hi = *reinterpret_cast<const intx4*>(bw + swz(wr, 4 + kq));
        } else {
          lo = *reinterpret_cast<const intx4*>(bw + (wr >> 4) * 2048 + lane * 16);
          hi = *reinterpret_cast<const intx4*>(bw + (wr >> 4) * 2048 + 1024 + lane * 16);
        }
        A[t] = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
#pragma unroll
      for (int tt = 0; tt < 8; ++tt) {
        const int tr = 16 * tt + r16;
        const intx4 lo = *reinterpret_cast<const intx4*>(b + swz(tr, kq));
        const intx4 hi = *reinterpret_cast<const intx4*>(b + swz(tr, 4 + kq));
        const intx8 B = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        const float xs = bxs[tr];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const floatx4 p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
              A[t], B, floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
          const float sc = xs * wsc[FUSED ? (t >> 1) : 0];
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[tt][t][i] = fmaf(p[i], sc, acc[tt][t][i]);
        }
      }
      if (kb + 1 < KB) lstore(cur ^ 1);
      __syncthreads();
    }

    // ---- epilogue ----------------------------------------------------------------
    if constexpr (FUSED) {
      // h = bf16(silu(gate) * up), kept in acc[tt][0..1]
#pragma unroll
      for (int tt = 0; tt < 8; ++tt) {
        float am = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float h = bf16_round_f32(silu_f32(acc[tt][j][i]) * acc[tt][j + 2][i]);
            acc[tt][j][i] = h;
            am = fmaxf(am, fabsf(h));
          }
        const int tok = m0 + 16 * tt + r16;
        if (g.out != nullptr && tok < cnt) {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            uint2 o;
            o.x = f32_to_bf16_bits(acc[tt][j][0]) | (f32_to_bf16_bits(acc[tt][j][1]) << 16);
            o.y = f32_to_bf16_bits(acc[tt][j][2]) | (f32_to_bf16_bits(acc[tt][j][3]) << 16);
            *reinterpret_cast<uint2*>(g.out + (row0 + tok) * g.n + n0 + 32 * wave + 16 * j + 4 * kq) = o;
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
        for (int tt = 0; tt < 8; ++tt) {
          const float am = fmaxf(fmaxf(s_amax[0][tt][r16], s_amax[1][tt][r16]),
                                 fmaxf(s_amax[2][tt][r16], s_amax[3][tt][r16]));
          const float sc = quant_scale_from_amax(am);
          const int tok = m0 + 16 * tt + r16;
          if (tok < cnt) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const uint32_t q = pack4_e4m3(clamp448(acc[tt][j][0] / sc), clamp448(acc[tt][j][1] / sc),
                                            clamp448(acc[tt][j][2] / sc), clamp448(acc[tt][j][3] / sc));
              *reinterpret_cast<uint32_t*>(g.out_q + (row0 + tok) * g.n + n0 + 32 * wave + 16 * j + 4 * kq) = q;
            }
            if (wave == 0 && kq == 0)
              g.out_s[(row0 + tok) * g.os_row + (int64_t)(n0 >> 7) * g.os_nb] = sc;
          }
        }
      }
    } else {
#pragma unroll
      for (int tt = 0; tt < 8; ++tt) {
        const int tok = m0 + 16 * tt + r16;
        if (tok >= cnt) continue;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int col = n0 + 64 * wave + 16 * t + 4 * kq;
          if (col >= g.n) continue;
          uint2 o;
          o.x = f32_to_bf16_bits(acc[tt][t][0]) | (f32_to_bf16_bits(acc[tt][t][1]) << 16);
          o.y = f32_to_bf16_bits(acc[tt][t][2]) | (f32_to_bf16_bits(acc[tt][t][3]) << 16);
          *reinterpret_cast<uint2*>(g.out + (row0 + tok) * g.n + col) = o;
        }
      }
    }
  }
}

int g_num_cu = 0;

}  // namespace

int bgmoe_launch_fp8_tiled(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* w0, const bgmoe_fp8_weight* w1,
                           const int32_t* seqlens, const int32_t* cu, int groups, int64_t m, int n, int k,
                           uint16_t* out, uint8_t* out_q, float* out_s, int64_t os_row, int64_t os_nb,
                           int lo, hipStream_t st) {
  if (groups == 0 || m == 0) return BGMOE_OK;
  if (groups > kMaxGroups) {
    bgmoe_set_error("fp8 tiled gemm: groups=%d exceeds %d", groups, kMaxGroups);
    return BGMOE_ERR_ARG;
  }
  TiledArgs g{};
  g.a = *a; g.w0 = *w0; if (w1) g.w1 = *w1;
  g.seqlens = seqlens; g.cu = cu; g.groups = groups; g.n = n; g.k = k;
  g.out = out; g.out_q = out_q; g.out_s = out_s; g.os_row = os_row; g.os_nb = os_nb; g.lo = lo;
  static bool attr_set = false;
  if (!attr_set) {
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
      hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * kBufBytes);
      if (e != hipSuccess) e1 = e;
    }
    if (e1 != hipSuccess) {
      bgmoe_set_error("fp8 tiled gemm: cannot reserve %d bytes of LDS", 2 * kBufBytes);
      return BGMOE_ERR_HIP;
    }
    attr_set = true;
  }
  // upper bound on work items from host shapes only
  const int ncols = w1 ? 128 : 256;
  const int64_t ntn = (n + ncols - 1) / ncols;
  const int64_t max_items = ((m + TM - 1) / TM + groups) * ntn;
  int64_t blocks = (int64_t)(g_num_cu > 0 ? g_num_cu : 256);
  if (blocks > max_items) blocks = max_items;
  if (blocks < 8) blocks = 8;
  BgmoeProf prof(w1 ? BGMOE_K_S1_TILED : BGMOE_K_GEMM_TILED, st);
  const dim3 grid((unsigned)blocks), block(256);
  const bool tm = w0->layout == BGMOE_W_TILE_MAJOR;
  if (w1) {
    if (tm) hipLaunchKernelGGL((fp8_tiled_kernel<true, 1>), grid, block, 2 * kBufBytes, st, g);
    else hipLaunchKernelGGL((fp8_tiled_kernel<true, 0>), grid, block, 2 * kBufBytes, st, g);
  } else {
    if (tm) hipLaunchKernelGGL((fp8_tiled_kernel<false, 1>), grid, block, 2 * kBufBytes, st, g);
    else hipLaunchKernelGGL((fp8_tiled_kernel<false, 0>), grid, block, 2 * kBufBytes, st, g);
  }
  return bgmoe_check_launch("fp8 grouped gemm (tiled)");
}
