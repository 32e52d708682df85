// Expert permute for gfx950: a STABLE counting sort of the (token, k) pairs by
// local expert id.  Slot of pair i inside its expert = number of pairs j < i of
// the same expert, so the permutation is a pure function of topk_ids (the
// reference claims slots with a global atomic counter, i.e. arrival order).
//
// Pairs are cut into chunks of 2048; a block owns a chunk, each of its four
// waves owns 512 consecutive pairs and walks them 64 at a time.  Ranks come
// from ballots (which lanes hold my expert?) plus wave-private LDS counters --
// LDS atomics are used only for histograms, never to claim a slot.
//
//   nk <= 2048 : one launch does histogram, prefix and ranks (decode).
//   otherwise  : hist per chunk -> one-block scan -> ranks per chunk.
// The row copy (or the quantising copy) is a separate one-wave-per-pair launch.
#include "bgmoe_common.h"

namespace {

constexpr int kChunk = 2048;       // pairs per block
constexpr int kWavePairs = 512;    // pairs per wave
constexpr int kMaxLocal = 1024;    // local experts

struct PermArgs {
  const int32_t* ids;      // [nk]
  int64_t nk;
  int expert_start, e_local;
  int mtp;                 // masked layout stride, or 0 for ragged
  int row_align;           // ragged
  int32_t* counts;         // [e_local]
  int32_t* counters;       // [e_local] (may be null)
  int32_t* cu;             // [e_local+1] (ragged; may be null for masked)
  int32_t* pos;            // [nk]
  int32_t* row_pair;       // optional inverse map: row_pair[pos[i]] = i for every placed pair (rows without a pair keep
                           // what they held)
  int32_t* chunk_hist;     // workspace [nchunks][e_local]
  int nchunks;
  int extra_count;         // >= 0: one more group (counts[e_local] = extra_count,
  int64_t extra_start;     //       cu[e_local] = extra_start, cu[e_local+1] = extra_start + extra_count)
};

__device__ __forceinline__ void write_tail(const PermArgs& a, int64_t off) {
  if (a.extra_count >= 0) {
    a.counts[a.e_local] = a.extra_count;
    if (a.cu) {
      a.cu[a.e_local] = (int32_t)a.extra_start;
      a.cu[a.e_local + 1] = (int32_t)(a.extra_start + a.extra_count);
    }
  } else if (a.cu) {
    a.cu[a.e_local] = (int32_t)off;
  }
}

__device__ __forceinline__ int local_id(const PermArgs& a, int64_t i) {
  if (i >= a.nk) return -1;
  const int64_t le = (int64_t)a.ids[i] - a.expert_start;
  return (le >= 0 && le < a.e_local) ? (int)le : -1;
}

__global__ __launch_bounds__(256) void perm_hist_kernel(PermArgs a) {
  __shared__ int32_t hist[kMaxLocal];
  for (int e = threadIdx.x; e < a.e_local; e += 256) hist[e] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kChunk;
  for (int j = threadIdx.x; j < kChunk; j += 256) {
    const int le = local_id(a, base + j);
    if (le >= 0) atomicAdd(&hist[le], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < a.e_local; e += 256)
    a.chunk_hist[(int64_t)blockIdx.x * a.e_local + e] = hist[e];
}

// exclusive scan over chunks per expert (in place), then counts / cu_seqlens.  One wave per expert (16 at a
// time): lane = chunk, a shuffle scan per 64 chunks with a running carry.
__global__ __launch_bounds__(1024) void perm_scan_kernel(PermArgs a) {
  __shared__ int32_t tot[kMaxLocal];
  const int wave = threadIdx.x >> 6;
  const int lane = lane_id();
  for (int e = wave; e < a.e_local; e += 16) {
    int run = 0;
    for (int c0 = 0; c0 < a.nchunks; c0 += 64) {
      const int c = c0 + lane;
      const int64_t o = (int64_t)c * a.e_local + e;
      const int t = c < a.nchunks ? a.chunk_hist[o] : 0;
      int inc = t;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(inc, off, BGMOE_WAVE);
        if (lane >= off) inc += up;
      }
      if (c < a.nchunks) a.chunk_hist[o] = run + inc - t;
      run += __shfl(inc, 63, BGMOE_WAVE);
    }
    if (lane == 0) {
      const int cnt = a.mtp > 0 ? min(run, a.mtp) : run;
      tot[e] = cnt;
      a.counts[e] = cnt;
      if (a.counters) a.counters[e] = run;       // before clipping: counters[e] > counts[e] = rows were dropped
    }
  }
  __syncthreads();
  if (wave == 0) {
    int64_t base = 0;
    for (int g0 = 0; g0 < a.e_local; g0 += 64) {
      const int g = g0 + lane;
      const int64_t span = g < a.e_local ? (a.mtp > 0 ? (int64_t)a.mtp
                                                      : (((int64_t)tot[g] + a.row_align - 1) & ~(int64_t)(a.row_align - 1)))
                                         : 0;
      int64_t inc = span;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int64_t up = __shfl_up(inc, off, BGMOE_WAVE);
        if (lane >= off) inc += up;
      }
      if (g < a.e_local && a.cu) a.cu[g] = (int32_t)(base + inc - span);
      base += __shfl(inc, 63, BGMOE_WAVE);
    }
    if (lane == 0) write_tail(a, a.cu ? base : 0);
  }
}

template <bool SINGLE>
__global__ __launch_bounds__(256) void perm_rank_kernel(PermArgs a) {
  __shared__ int32_t whist[4][kMaxLocal];   // per-wave histogram, then per-wave next-slot counter
  __shared__ int32_t s_cu[SINGLE ? kMaxLocal + 1 : 1];
  const int wave = threadIdx.x >> 6;
  const int lane = lane_id();
  const int el = a.e_local;
  for (int e = threadIdx.x; e < 4 * el; e += 256) whist[e / el][e % el] = 0;
  __syncthreads();
  const int64_t wbase = (int64_t)blockIdx.x * kChunk + (int64_t)wave * kWavePairs;
  for (int s = 0; s < kWavePairs / 64; ++s) {
    const int le = local_id(a, wbase + s * 64 + lane);
    if (le >= 0) atomicAdd(&whist[wave][le], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < el; e += 256) {
    int run = SINGLE ? 0 : a.chunk_hist[(int64_t)blockIdx.x * el + e];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const int t = whist[w][e];
      whist[w][e] = run;
      run += t;
    }
    if constexpr (SINGLE) {
      const int cnt = a.mtp > 0 ? min(run, a.mtp) : run;
      a.counts[e] = cnt;
      if (a.counters) a.counters[e] = run;       // before clipping: counters[e] > counts[e] = rows were dropped
      s_cu[e + 1] = cnt;
    }
  }
  __syncthreads();
  if constexpr (SINGLE) {
    if (threadIdx.x == 0) {
      int64_t off = 0;
      for (int g = 0; g < el; ++g) {
        const int cnt = s_cu[g + 1];
        s_cu[g] = (int32_t)off;
        if (a.cu) a.cu[g] = (int32_t)off;
        off += a.mtp > 0 ? (int64_t)a.mtp
                         : (((int64_t)cnt + a.row_align - 1) & ~(int64_t)(a.row_align - 1));
      }
      write_tail(a, off);
    }
    __syncthreads();
  }

  int nbits = 0;
  while ((1 << nbits) < el) ++nbits;
  const unsigned long long lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  for (int s = 0; s < kWavePairs / 64; ++s) {
    const int64_t i = wbase + s * 64 + lane;
    const int le = local_id(a, i);
    unsigned long long peers = __ballot(le >= 0);
    for (int b = 0; b < nbits; ++b) {
      const bool bit = (le >> b) & 1;
      const unsigned long long m = __ballot(bit);
      peers &= bit ? m : ~m;
    }
    int slot = -1;
    if (le >= 0) slot = whist[wave][le] + __popcll(peers & lt);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (le >= 0 && (peers & lt) == 0ull) whist[wave][le] += __popcll(peers);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (i < a.nk) {
      int p = -1;
      if (le >= 0) {
        if (a.mtp > 0) p = slot < a.mtp ? le * a.mtp + slot : -1;
        else p = (SINGLE ? s_cu[le] : a.cu[le]) + slot;
      }
      a.pos[i] = p;
      if (a.row_pair != nullptr && p >= 0) a.row_pair[p] = (int32_t)i;
    }
  }
}

// Decode-sized problems (nk <= 64*16*S pairs, <= 256 local experts) in ONE block of 16 waves: every lane reads
// its S ids once (S = 2: up to 2048 pairs, S = 8: up to 8192), ranks inside a wave come from ballots, one pass
// over the 16 per-wave histograms turns them into offsets, a single wave scans the experts.  Latency chain:
// one global load, a few LDS round trips per sub-step.
constexpr int kSmallLocal = 256;
constexpr int kSmallPairsMax = 64 * 16 * 8;
// `global`: this block writes counts, offsets and positions to memory; `s_pos` (optional): the positions in LDS.
template <int S>
__device__ __forceinline__ void perm_small_body(const PermArgs& a, int32_t (*whist)[kSmallLocal], int32_t* s_cu,
                                                int32_t* s_pos, bool global) {
  const int wave = threadIdx.x >> 6;
  const int lane = lane_id();
  const int el = a.e_local;
  int le[S];
#pragma unroll
  for (int s = 0; s < S; ++s) le[s] = local_id(a, (int64_t)wave * (64 * S) + s * 64 + lane);
  for (int e = threadIdx.x; e < 16 * el; e += 1024) whist[e / el][e % el] = 0;
  __syncthreads();
  int nbits = 0;
  while ((1 << nbits) < el) ++nbits;
  const unsigned long long lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  int off[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    unsigned long long peers = __ballot(le[s] >= 0);
    for (int b = 0; b < nbits; ++b) {
      const bool bit = (le[s] >> b) & 1;
      const unsigned long long m = __ballot(bit);
      peers &= bit ? m : ~m;
    }
    off[s] = -1;
    if (le[s] >= 0) off[s] = whist[wave][le[s]] + __popcll(peers & lt);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (le[s] >= 0 && (peers & lt) == 0ull) whist[wave][le[s]] += __popcll(peers);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  __syncthreads();
  for (int e = threadIdx.x; e < el; e += 1024) {
    int run = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int t = whist[w][e];
      whist[w][e] = run;
      run += t;
    }
    const int cnt = a.mtp > 0 ? min(run, a.mtp) : run;
    if (global) {
      a.counts[e] = cnt;
      if (a.counters) a.counters[e] = run;       // before clipping: counters[e] > counts[e] = rows were dropped
    }
    s_cu[e + 1] = cnt;
  }
  __syncthreads();
  if (wave == 0) {
    int64_t base = 0;
    for (int g0 = 0; g0 < el; g0 += 64) {
      const int g = g0 + lane;
      const int cnt = g < el ? s_cu[g + 1] : 0;
      const int64_t span = g < el ? (a.mtp > 0 ? (int64_t)a.mtp
                                              : (((int64_t)cnt + a.row_align - 1) & ~(int64_t)(a.row_align - 1)))
                                  : 0;
      int64_t inc = span;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int64_t up = __shfl_up(inc, o, BGMOE_WAVE);
        if (lane >= o) inc += up;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();          // everybody has read s_cu[g + 1] before s_cu[g] is overwritten
      if (g < el) {
        s_cu[g] = (int32_t)(base + inc - span);
        if (a.cu && global) a.cu[g] = (int32_t)(base + inc - span);
      }
      base += __shfl(inc, 63, BGMOE_WAVE);
    }
    if (lane == 0 && global) write_tail(a, base);
  }
  __syncthreads();
#pragma unroll
  for (int s = 0; s < S; ++s) {
    const int64_t i = (int64_t)wave * (64 * S) + s * 64 + lane;
    if (i < a.nk) {
      int p = -1;
      if (le[s] >= 0) {
        const int slot = whist[wave][le[s]] + off[s];
        if (a.mtp > 0) p = slot < a.mtp ? le[s] * a.mtp + slot : -1;
        else p = s_cu[le[s]] + slot;
      }
      if (global) a.pos[i] = p;
      if (global && a.row_pair != nullptr && p >= 0) a.row_pair[p] = (int32_t)i;
      if (s_pos) s_pos[i] = p;
    }
  }
}

template <int S>
__global__ __launch_bounds__(1024) void perm_small_kernel(PermArgs a) {
  __shared__ int32_t whist[16][kSmallLocal];   // per-wave counts, then exclusive offsets over the waves
  __shared__ int32_t s_cu[kSmallLocal + 1];
  perm_small_body<S>(a, whist, s_cu, nullptr, true);
}

// Decode-sized batches (at most 2048 pairs): permutation indices, FP8 quantisation and the scatter in ONE launch.
// Every block repeats the whole (small) index computation above and keeps the positions in LDS -- cheaper than a
// second launch that waits for them -- block 0 also writes counts, offsets and positions to memory; then each
// wave quantises one (token, 512 columns) piece once and writes bytes and scales to every row the token is routed
// to and to its identity row (the shared expert), exactly as scatter_quant_kernel does.
struct FusedQuantArgs {
  const uint16_t* x;
  uint8_t* y;
  float* scale;
  int64_t srow, skb;
  int n, topk, h, steps, extra_rows;
  int64_t extra_start;
};

__global__ __launch_bounds__(1024) void perm_quant_small_kernel(PermArgs a, FusedQuantArgs q) {
  __shared__ int32_t whist[16][kSmallLocal];
  __shared__ int32_t s_cu[kSmallLocal + 1];
  __shared__ int32_t s_pos[kChunk];
  perm_small_body<2>(a, whist, s_cu, s_pos, blockIdx.x == 0);
  __syncthreads();
  const int wave = threadIdx.x >> 6;
  const int lane = lane_id();
  const int k = q.h;
  const int64_t njobs = (int64_t)q.n * q.steps;
  for (int64_t job = (int64_t)blockIdx.x * 16 + wave; job < njobs; job += (int64_t)gridDim.x * 16) {
    const int64_t tok = job / q.steps;
    const int c0 = (int)(job - tok * q.steps) * 512 + lane * 8;
    const bool in = c0 < k;
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = 0.0f;
    if (in) {
      const uint4 raw = *reinterpret_cast<const uint4*>(q.x + tok * (int64_t)k + c0);
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[2 * i] = bf16_bits_to_f32(w[i] & 0xffffu);
        v[2 * i + 1] = bf16_bits_to_f32(w[i] >> 16);
      }
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
    amax = wave_max_xor<16>(amax);
    const float sc = quant_scale_from_amax(amax);
    uint2 o;
    {
      float qv[8];
      quant_div_clamp(v, sc, qv);
      o.x = pack4_e4m3(qv[0], qv[1], qv[2], qv[3]);
      o.y = pack4_e4m3(qv[4], qv[5], qv[6], qv[7]);
    }
    const bool lead = (lane & 15) == 0;
    int mine = -1;
    if (lane < q.topk) mine = s_pos[tok * q.topk + lane];
    else if (lane == q.topk && tok < q.extra_rows) mine = (int)(q.extra_start + tok);
    unsigned long long live = __ballot(mine >= 0);
    while (live) {
      const int j = __ffsll((long long)live) - 1;
      live &= live - 1;
      const int64_t dst = __builtin_amdgcn_readlane(mine, j);
      if (in) {
        *reinterpret_cast<uint2*>(q.y + dst * (int64_t)k + c0) = o;
        if (lead) q.scale[dst * q.srow + (int64_t)(c0 >> 7) * q.skb] = sc;
      }
    }
  }
}


// one wave per pair: act[pos] = x[token]
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint16_t* __restrict__ x,
                                                          const int32_t* __restrict__ pos,
                                                          uint16_t* __restrict__ act, int64_t nk,
                                                          int k, int h, int vec) {
  const int wave = threadIdx.x >> 6;
  const int lane = lane_id();
  const int64_t stride = (int64_t)gridDim.x * 4;
  for (int64_t i = (int64_t)blockIdx.x * 4 + wave; i < nk; i += stride) {
    const int p = pos[i];
    if (p < 0) continue;
    const uint16_t* src = x + (i / k) * (int64_t)h;
    uint16_t* dst = act + (int64_t)p * h;
    if (vec) {
      const uint4* s4 = reinterpret_cast<const uint4*>(src);
      uint4* d4 = reinterpret_cast<uint4*>(dst);
      for (int v = lane; v < h / 8; v += BGMOE_WAVE) d4[v] = s4[v];
    } else {
      for (int c = lane; c < h; c += BGMOE_WAVE) dst[c] = src[c];
    }
  }
}

__global__ __launch_bounds__(64) void compact_kernel(const int32_t* __restrict__ counts, int e,
                                                     int32_t* group_size, int32_t* active_idx,
                                                     int32_t* starts, int32_t* num_active) {
  const int lane = lane_id();
  const unsigned long long lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  int written = 0, cumulative = 0;
  for (int base = 0; base < e; base += 64) {
    const int g = base + lane;
    const int c = g < e ? counts[g] : 0;
    const unsigned long long m = __ballot(c > 0);
    // inclusive scan of c over the wave
    int inc = c;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(inc, off, BGMOE_WAVE);
      if (lane >= off) inc += up;
    }
    if (c > 0) {
      const int w = written + __popcll(m & lt);
      active_idx[w] = g;
      group_size[w] = c;
      starts[w] = cumulative + inc - c;
    }
    written += __popcll(m);
    cumulative += __shfl(inc, 63, BGMOE_WAVE);
  }
  if (lane == 0) *num_active = written;
}

int run_index(PermArgs& a, void* workspace, size_t workspace_bytes, hipStream_t st) {
  if (a.nk <= kChunk || (a.nk <= kSmallPairsMax && a.e_local <= kSmallLocal)) {
    a.nchunks = 1;
    BgmoeProf prof(BGMOE_K_PERM_RANK, st);
    if (a.e_local <= kSmallLocal && a.nk <= kChunk) hipLaunchKernelGGL(perm_small_kernel<2>, dim3(1), dim3(1024), 0, st, a);
    else if (a.e_local <= kSmallLocal) hipLaunchKernelGGL(perm_small_kernel<8>, dim3(1), dim3(1024), 0, st, a);
    else hipLaunchKernelGGL((perm_rank_kernel<true>), dim3(1), dim3(256), 0, st, a);
    return bgmoe_check_launch("dispatch(single)");
  }
  a.nchunks = (int)((a.nk + kChunk - 1) / kChunk);
  const size_t need = (size_t)a.nchunks * a.e_local * sizeof(int32_t);
  if (workspace == nullptr || workspace_bytes < need) {
    bgmoe_set_error("dispatch: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    return BGMOE_ERR_WORKSPACE;
  }
  a.chunk_hist = (int32_t*)workspace;
  { BgmoeProf prof(BGMOE_K_PERM_HIST, st); hipLaunchKernelGGL(perm_hist_kernel, dim3(a.nchunks), dim3(256), 0, st, a); }
  { BgmoeProf prof(BGMOE_K_PERM_SCAN, st); hipLaunchKernelGGL(perm_scan_kernel, dim3(1), dim3(1024), 0, st, a); }
  { BgmoeProf prof(BGMOE_K_PERM_RANK, st); hipLaunchKernelGGL((perm_rank_kernel<false>), dim3(a.nchunks), dim3(256), 0, st, a); }
  return bgmoe_check_launch("dispatch");
}

int run_gather(const uint16_t* x, const int32_t* pos, uint16_t* act, int64_t nk, int k, int h,
               hipStream_t st) {
  if (nk == 0 || h == 0) return BGMOE_OK;
  int64_t blocks = (nk + 3) / 4;
  if (blocks > 65536) blocks = 65536;
  const int vec = (h % 8 == 0) && ((uintptr_t)x % 16 == 0) && ((uintptr_t)act % 16 == 0);
  BgmoeProf prof(BGMOE_K_GATHER_ROWS, st);
  hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, st, x, pos, act, nk,
                     k, h, vec);
  return bgmoe_check_launch("dispatch(gather)");
}

}  // namespace

int bgmoe_internal_dispatch_index(const int32_t* ids, int64_t nk, int expert_start, int e_local, int mtp,
                                  int row_align, int32_t* counts, int32_t* counters, int32_t* cu,
                                  int32_t* pos, int extra_count, int64_t extra_start, void* ws,
                                  size_t ws_bytes, hipStream_t st) {
  PermArgs a{};
  a.ids = ids; a.nk = nk; a.expert_start = expert_start; a.e_local = e_local; a.mtp = mtp;
  a.row_align = row_align; a.counts = counts; a.counters = counters; a.cu = cu; a.pos = pos;
  a.extra_count = extra_count; a.extra_start = extra_start;
  return run_index(a, ws, ws_bytes, st);
}

// Index + quantise + scatter in one launch for decode-sized batches.  BGMOE_ERR_WORKSPACE (no message): does not
// apply (too many pairs or experts, odd shapes), the caller runs the two steps separately.
int bgmoe_internal_dispatch_scatter_quant(const int32_t* ids, int n, int k, int h, int expert_start, int e_local, int mtp,
                                          int row_align, int32_t* counts, int32_t* counters, int32_t* cu, int32_t* pos,
                                          int extra_count, int64_t extra_start, const uint16_t* x, uint8_t* y,
                                          float* scale, int64_t srow, int64_t skb, hipStream_t st) {
  const int64_t nk = (int64_t)n * k;
  if (nk <= 0 || nk > kChunk || e_local > kSmallLocal || k >= 64 || h <= 0 || h % 8 != 0 ||
      (uintptr_t)x % 16 != 0 || (uintptr_t)y % 8 != 0 || extra_count > n)
    return BGMOE_ERR_WORKSPACE;
  PermArgs a{};
  a.ids = ids; a.nk = nk; a.expert_start = expert_start; a.e_local = e_local; a.mtp = mtp;
  a.row_align = row_align; a.counts = counts; a.counters = counters; a.cu = cu; a.pos = pos;
  a.extra_count = extra_count; a.extra_start = extra_start; a.nchunks = 1;
  FusedQuantArgs q{};
  q.x = x; q.y = y; q.scale = scale; q.srow = srow; q.skb = skb; q.n = n; q.topk = k; q.h = h;
  q.steps = (h + 511) / 512; q.extra_rows = extra_count > 0 ? extra_count : 0; q.extra_start = extra_start;
  const int64_t blocks = ((int64_t)n * q.steps + 15) / 16;
  BgmoeProf prof(BGMOE_K_ACT_QUANT, st);
  hipLaunchKernelGGL(perm_quant_small_kernel, dim3((unsigned)blocks), dim3(1024), 0, st, a, q);
  return bgmoe_check_launch("dispatch + scatter_quant");
}

extern "C" size_t bgmoe_dispatch_workspace_bytes(int64_t nk, int num_local_experts) {
  if (nk <= kChunk || num_local_experts <= 0) return 0;
  if (nk <= kSmallPairsMax && num_local_experts <= kSmallLocal) return 0;
  return (size_t)((nk + kChunk - 1) / kChunk) * (size_t)num_local_experts * sizeof(int32_t);
}

extern "C" int bgmoe_dispatch_scatter_3d(const uint16_t* x, const int32_t* topk_ids, int n, int k,
                                         int h, uint16_t* act_buffer, int expert_start,
                                         int num_local_experts, int max_tokens_padded,
                                         int32_t* expert_counts, int32_t* expert_counters,
                                         int32_t* topk_pos, void* workspace, size_t workspace_bytes,
                                         bgmoe_stream_t stream) {
  BGMOE_REQUIRE(n >= 0 && k > 0 && h >= 0, "dispatch_scatter_3d: bad sizes n=%d k=%d h=%d", n, k, h);
  BGMOE_REQUIRE(num_local_experts > 0 && num_local_experts <= kMaxLocal,
                "dispatch_scatter_3d: num_local_experts=%d outside [1,%d]", num_local_experts, kMaxLocal);
  BGMOE_REQUIRE(max_tokens_padded > 0, "dispatch_scatter_3d: max_tokens_padded must be positive");
  BGMOE_REQUIRE((int64_t)num_local_experts * max_tokens_padded <= 2147483647LL,
                "dispatch_scatter_3d: E_local*max_tokens_padded exceeds int32");
  BGMOE_REQUIRE(expert_counts && topk_pos, "dispatch_scatter_3d: null output");
  BGMOE_REQUIRE(n == 0 || topk_ids, "dispatch_scatter_3d: null topk_ids");
  PermArgs a{};
  a.ids = topk_ids; a.nk = (int64_t)n * k; a.expert_start = expert_start;
  a.e_local = num_local_experts; a.mtp = max_tokens_padded; a.row_align = 1;
  a.counts = expert_counts; a.counters = expert_counters; a.cu = nullptr; a.pos = topk_pos;
  a.extra_count = -1;
  int rc = run_index(a, workspace, workspace_bytes, bgmoe_stream(stream));
  if (rc != BGMOE_OK || act_buffer == nullptr) return rc;
  BGMOE_REQUIRE(n == 0 || x, "dispatch_scatter_3d: null x");
  return run_gather(x, topk_pos, act_buffer, a.nk, k, h, bgmoe_stream(stream));
}

extern "C" int bgmoe_dispatch_index_3d(const int32_t* topk_ids, int n, int k, int expert_start, int num_local_experts,
                                       int max_tokens_padded, int32_t* expert_counts, int32_t* expert_counters,
                                       int32_t* topk_pos, int32_t* row_pair, void* workspace, size_t workspace_bytes,
                                       bgmoe_stream_t stream) {
  BGMOE_REQUIRE(n >= 0 && k > 0, "dispatch_index_3d: bad sizes n=%d k=%d", n, k);
  BGMOE_REQUIRE(num_local_experts > 0 && num_local_experts <= kMaxLocal,
                "dispatch_index_3d: num_local_experts=%d outside [1,%d]", num_local_experts, kMaxLocal);
  BGMOE_REQUIRE(max_tokens_padded > 0, "dispatch_index_3d: max_tokens_padded must be positive");
  BGMOE_REQUIRE((int64_t)num_local_experts * max_tokens_padded <= 2147483647LL && (int64_t)n * k <= 2147483647LL,
                "dispatch_index_3d: E_local*max_tokens_padded or n*k exceeds int32");
  BGMOE_REQUIRE(expert_counts && topk_pos && row_pair, "dispatch_index_3d: null output");
  BGMOE_REQUIRE(n == 0 || topk_ids, "dispatch_index_3d: null topk_ids");
  PermArgs a{};
  a.ids = topk_ids; a.nk = (int64_t)n * k; a.expert_start = expert_start;
  a.e_local = num_local_experts; a.mtp = max_tokens_padded; a.row_align = 1;
  a.counts = expert_counts; a.counters = expert_counters; a.cu = nullptr; a.pos = topk_pos; a.row_pair = row_pair;
  a.extra_count = -1;
  return run_index(a, workspace, workspace_bytes, bgmoe_stream(stream));
}

extern "C" int bgmoe_dispatch_scatter_ragged(const uint16_t* x, const int32_t* topk_ids, int n, int k,
                                             int h, uint16_t* act_buffer, int64_t act_rows,
                                             int expert_start, int num_local_experts,
                                             int32_t* expert_counts, int32_t* expert_counters,
                                             int32_t* topk_pos, int32_t* cu_seqlens, int row_align,
                                             void* workspace, size_t workspace_bytes,
                                             bgmoe_stream_t stream) {
  BGMOE_REQUIRE(row_align > 0 && (row_align & (row_align - 1)) == 0,
                "dispatch_scatter_ragged: row_align must be a positive power of two, got %d", row_align);
  BGMOE_REQUIRE(n >= 0 && k > 0 && h >= 0, "dispatch_scatter_ragged: bad sizes n=%d k=%d h=%d", n, k, h);
  BGMOE_REQUIRE(num_local_experts > 0 && num_local_experts <= kMaxLocal,
                "dispatch_scatter_ragged: num_local_experts=%d outside [1,%d]", num_local_experts, kMaxLocal);
  BGMOE_REQUIRE(expert_start >= 0, "dispatch_scatter_ragged: expert_start out of range: %d", expert_start);
  const int64_t nk = (int64_t)n * k;
  const int64_t cap_rows = (nk + (int64_t)(row_align - 1) * (nk < num_local_experts ? nk : num_local_experts)) /
                           row_align * row_align;
  BGMOE_REQUIRE(cap_rows <= 2147483647LL, "dispatch_scatter_ragged: N*K too large: %lld", (long long)nk);
  if (act_buffer)
    BGMOE_REQUIRE(act_rows >= cap_rows, "dispatch_scatter_ragged: act_buffer rows (%lld) must be in [%lld, INT32_MAX]",
                  (long long)act_rows, (long long)cap_rows);
  BGMOE_REQUIRE(expert_counts && topk_pos && cu_seqlens, "dispatch_scatter_ragged: null output");
  BGMOE_REQUIRE(n == 0 || topk_ids, "dispatch_scatter_ragged: null topk_ids");
  PermArgs a{};
  a.ids = topk_ids; a.nk = nk; a.expert_start = expert_start; a.e_local = num_local_experts;
  a.mtp = 0; a.row_align = row_align; a.counts = expert_counts; a.counters = expert_counters;
  a.cu = cu_seqlens; a.pos = topk_pos; a.extra_count = -1;
  int rc = run_index(a, workspace, workspace_bytes, bgmoe_stream(stream));
  if (rc != BGMOE_OK || act_buffer == nullptr) return rc;
  BGMOE_REQUIRE(n == 0 || x, "dispatch_scatter_ragged: null x");
  return run_gather(x, topk_pos, act_buffer, nk, k, h, bgmoe_stream(stream));
}

// ---- allocation-free variant: the chunk histograms live in a file-scope device array --------------------
// One copy of the array exists per GPU, at its own address; the address is looked up once per device with
// that device current (bgmoe_init, else the first call on the device) and only that pointer is ever handed
// to kernels: the array's name is a host-side stand-in, not a device address.
namespace {
constexpr size_t kStaticHistInts = 262144;                 // 1 MiB per GPU, held until the process ends
constexpr int kMaxDevices = 64;
}  // namespace
static __device__ __align__(256) int32_t scratch[kStaticHistInts];
static int32_t* g_scratch_ptr[kMaxDevices] = {};

static int static_hist_ptr(int32_t** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    bgmoe_set_error("dispatch_scatter_ragged_static: no current HIP device (or device index >= %d)", kMaxDevices);
    return BGMOE_ERR_HIP;
  }
  if (g_scratch_ptr[dev] == nullptr) {
    int32_t* p = nullptr;
    const hipError_t err = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess || p == nullptr) {
      bgmoe_set_error("dispatch_scatter_ragged_static: hipGetSymbolAddress failed: %s", hipGetErrorString(err));
      return BGMOE_ERR_HIP;
    }
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return BGMOE_OK;
}

int bgmoe_internal_init_permute() {
  int32_t* p = nullptr;
  return static_hist_ptr(&p);
}

extern "C" size_t bgmoe_dispatch_static_max_pairs(int num_local_experts) {
  if (num_local_experts <= 0 || num_local_experts > kMaxLocal) return 0;
  return (kStaticHistInts / (size_t)num_local_experts) * (size_t)kChunk;
}

extern "C" int bgmoe_dispatch_scatter_ragged_static(const uint16_t* x, const int32_t* topk_ids, int n, int k, int h,
                                                    uint16_t* act_buffer, int64_t act_rows, int expert_start,
                                                    int num_local_experts, int32_t* expert_counts,
                                                    int32_t* expert_counters, int32_t* topk_pos,
                                                    int32_t* cu_seqlens, int row_align, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(n >= 0 && k > 0, "dispatch_scatter_ragged_static: bad sizes n=%d k=%d", n, k);
  BGMOE_REQUIRE(num_local_experts > 0 && num_local_experts <= kMaxLocal,
                "dispatch_scatter_ragged_static: num_local_experts=%d outside [1,%d]", num_local_experts, kMaxLocal);
  const size_t need = bgmoe_dispatch_workspace_bytes((int64_t)n * k, num_local_experts);
  if (need > kStaticHistInts * sizeof(int32_t)) {
    bgmoe_set_error("dispatch_scatter_ragged_static: %lld pairs x %d local experts need %zu bytes of histograms, the "
                    "static buffer holds %zu (at most %zu pairs at this expert count); use "
                    "bgmoe_dispatch_scatter_ragged with a workspace",
                    (long long)n * k, num_local_experts, need, kStaticHistInts * sizeof(int32_t),
                    bgmoe_dispatch_static_max_pairs(num_local_experts));
    return BGMOE_ERR_WORKSPACE;
  }
  int32_t* hist = nullptr;
  const int rc = static_hist_ptr(&hist);
  if (rc != BGMOE_OK) return rc;
  // every histogram entry the scan and rank kernels read is written by the histogram kernel of the same call,
  // so nothing has to start at zero
  return bgmoe_dispatch_scatter_ragged(x, topk_ids, n, k, h, act_buffer, act_rows, expert_start, num_local_experts,
                                       expert_counts, expert_counters, topk_pos, cu_seqlens, row_align, hist,
                                       kStaticHistInts * sizeof(int32_t), stream);
}

namespace {
// Per-row metadata of a tight (align 1) dispatch: row topk_pos[i] of pair i = (token i / k, slot i % k) gets the
// pair's expert id, token and slot; rows at or past *total (the last entry of the offsets) get -1.  Every row
// has exactly one writer.
__global__ __launch_bounds__(256) void row_metadata_kernel(const int32_t* __restrict__ ids, const int32_t* __restrict__ pos,
                                                           int64_t nk, int k, const int32_t* __restrict__ total, int64_t rows,
                                                           int32_t* __restrict__ eids, int32_t* __restrict__ toks,
                                                           int32_t* __restrict__ slots) {
  const int64_t live = *total;
  const int64_t span = nk > rows ? nk : rows;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < span; i += (int64_t)gridDim.x * 256) {
    if (i < nk) {
      const int p = pos[i];
      if (p >= 0 && p < rows) {
        eids[p] = ids[i];
        toks[p] = (int32_t)(i / k);
        slots[p] = (int32_t)(i % k);
      }
    }
    if (i < rows && i >= live) eids[i] = toks[i] = slots[i] = -1;
  }
}
}  // namespace

extern "C" int bgmoe_dispatch_row_metadata(const int32_t* topk_ids, const int32_t* topk_pos, int64_t nk, int k,
                                           const int32_t* total_rows, int64_t rows, int32_t* out_eids,
                                           int32_t* out_token_idx, int32_t* out_topk_pos, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(nk >= 0 && k > 0 && rows >= 0, "dispatch_row_metadata: bad sizes nk=%lld k=%d rows=%lld", (long long)nk, k,
                (long long)rows);
  if (rows == 0) return BGMOE_OK;
  BGMOE_REQUIRE(total_rows && out_eids && out_token_idx && out_topk_pos && (nk == 0 || (topk_ids && topk_pos)),
                "dispatch_row_metadata: null pointer");
  const int64_t span = nk > rows ? nk : rows;
  int64_t blocks = (span + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(row_metadata_kernel, dim3((unsigned)blocks), dim3(256), 0, bgmoe_stream(stream), topk_ids, topk_pos, nk,
                     k, total_rows, rows, out_eids, out_token_idx, out_topk_pos);
  return bgmoe_check_launch("dispatch_row_metadata");
}

extern "C" int bgmoe_compact_expert_data(const int32_t* expert_counts, int e, int32_t* group_size,
                                         int32_t* activated_group_idx, int32_t* group_start_indices,
                                         int32_t* num_active, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(e >= 0, "compact_expert_data: e < 0");
  BGMOE_REQUIRE(num_active, "compact_expert_data: null num_active");
  BGMOE_REQUIRE(e == 0 || (expert_counts && group_size && activated_group_idx && group_start_indices),
                "compact_expert_data: null pointer");
  BgmoeProf prof(BGMOE_K_COMPACT, bgmoe_stream(stream));
  hipLaunchKernelGGL(compact_kernel, dim3(1), dim3(64), 0, bgmoe_stream(stream), expert_counts, e,
                     group_size, activated_group_idx, group_start_indices, num_active);
  return bgmoe_check_launch("compact_expert_data");
}

namespace {
// Row -> group map (one contiguous run of rows per group, -1 on padding rows) -> (first row, live rows) per
// group.  One block: the map is a few hundred KB at most and is read once; every output has a single writer.
__global__ __launch_bounds__(1024) void layout_segments_kernel(const int32_t* __restrict__ layout, int64_t m, int groups,
                                                               int32_t* __restrict__ seqlens, int32_t* __restrict__ starts,
                                                               int32_t* __restrict__ status) {
  __shared__ int32_t s_first[1024], s_end[1024], s_bad;
  if (threadIdx.x == 0) s_bad = 0;
  for (int g = threadIdx.x; g < groups; g += 1024) { s_first[g] = 0; s_end[g] = 0; }
  __syncthreads();
  for (int64_t r = threadIdx.x; r < m; r += 1024) {
    const int32_t g = layout[r];
    if (g < 0) continue;
    if (g >= groups) { s_bad = 1; continue; }
    if (r == 0 || layout[r - 1] != g) {
      if (atomicAdd(&s_first[g], (int32_t)r + 1) != 0) s_bad = 2;       // a second run of the same group
    }
    if (r == m - 1 || layout[r + 1] != g) atomicAdd(&s_end[g], (int32_t)r + 1);
  }
  __syncthreads();
  for (int g = threadIdx.x; g < groups; g += 1024) {
    const bool live = s_first[g] != 0;
    starts[g] = live ? s_first[g] - 1 : 0;
    seqlens[g] = live && s_bad == 0 ? s_end[g] - (s_first[g] - 1) : 0;
  }
  if (threadIdx.x == 0) {
    starts[groups] = (int32_t)m;
    if (status) *status = s_bad;
  }
}
}  // namespace

extern "C" int bgmoe_layout_to_segments(const int32_t* grouped_layout, int64_t m, int groups, int32_t* seqlens,
                                        int32_t* starts, int32_t* status, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(m >= 0 && m <= 0x7fffffffLL && groups >= 1 && groups <= 1024,
                "layout_to_segments: m=%lld rows / %d groups out of range (groups in [1, 1024])", (long long)m, groups);
  BGMOE_REQUIRE(seqlens && starts && (m == 0 || grouped_layout), "layout_to_segments: null pointer");
  hipLaunchKernelGGL(layout_segments_kernel, dim3(1), dim3(1024), 0, bgmoe_stream(stream), grouped_layout, m, groups,
                     seqlens, starts, status);
  return bgmoe_check_launch("layout_to_segments");
}

