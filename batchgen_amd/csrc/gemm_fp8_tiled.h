// Arguments and launchers shared by the LDS-tiled FP8 grouped GEMM kernels (gemm_fp8_tiled.hip: K = 128 steps,
// 16x16x128 products; gemm_fp8_tiled_k64.hip: K = 64 steps, 32x32x64 products).
#pragma once
#include "bgmoe_common.h"
#include "bgmoe_sched.h"

struct BgmoeTiledArgs {
  bgmoe_fp8_act a;
  bgmoe_fp8_weight w0, w1;
  const int32_t* seqlens;
  const int32_t* cu;
  int groups, n, k;
  uint16_t* out;
  uint8_t* out_q;
  float* out_s;
  int64_t os_row, os_nb;
  BgmoeSplit split;
};

constexpr int kBgmoeTiledMaxGroups = 1024;     // per-group tile counts live in LDS
constexpr int kBgmoeTiledMaxKB = 256;          // K <= 32768: an item's weight scales along K live in LDS

// K = 64 variant: BGMOE_ERR_WORKSPACE (without a message) = does not apply to these sizes, take the K = 128 kernel
int bgmoe_internal_init_fp8_tiled_k64();
// regroup: its epilogue stores whole row segments through per-wave LDS patches where alignment allows
int bgmoe_launch_fp8_tiled_k64(const BgmoeTiledArgs& g, bool fused, bool regroup, int64_t m, int num_cu, hipStream_t st);
