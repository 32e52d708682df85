// One-time weight re-layout: row-major [groups, n, k] e4m3 bytes -> tile-major (see bgmoe.h).
// Each thread moves 16 bytes; reads are 64-byte runs of 16 rows, writes are fully contiguous.
#include "bgmoe_common.h"

namespace {
__global__ __launch_bounds__(256) void repack_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                     int64_t chunks, int n, int k) {
  const int kb_n = k >> 7;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < chunks; c += stride) {
    // destination chunk index: ((group * n/16 + nt) * kb_n + kb) * 128 + half*64 + lane
    const int in_tile = (int)(c & 127);
    const int64_t tile = c >> 7;
    const int half = in_tile >> 6, lane = in_tile & 63, r = lane & 15, q = lane >> 4;
    const int kb = (int)(tile % kb_n);
    const int64_t nt_all = tile / kb_n;                 // group * (n/16) + nt
    const int64_t row = nt_all * 16 + r;                // row in the [groups*n, k] matrix
    const int col = kb * 128 + half * 64 + q * 16;
    *reinterpret_cast<uint4*>(dst + c * 16) = *reinterpret_cast<const uint4*>(src + row * k + col);
  }
}
}  // namespace

extern "C" int bgmoe_fp8_weight_repack(const uint8_t* src_row_major, uint8_t* dst_tile_major, int groups, int n,
                                       int k, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(groups >= 0 && n > 0 && k > 0, "fp8_weight_repack: bad sizes");
  BGMOE_REQUIRE(n % 16 == 0 && k % 128 == 0, "fp8_weight_repack: N=%d must be a multiple of 16 and K=%d of 128", n, k);
  if (groups == 0) return BGMOE_OK;
  BGMOE_REQUIRE(src_row_major && dst_tile_major && src_row_major != dst_tile_major,
                "fp8_weight_repack: needs distinct non-null source and destination");
  BGMOE_REQUIRE((uintptr_t)src_row_major % 16 == 0 && (uintptr_t)dst_tile_major % 16 == 0,
                "fp8_weight_repack: buffers must be 16-byte aligned");
  const int64_t chunks = (int64_t)groups * n * k / 16;
  int64_t blocks = (chunks + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(repack_kernel, dim3((unsigned)blocks), dim3(256), 0, bgmoe_stream(stream), src_row_major,
                     dst_tile_major, chunks, n, k);
  return bgmoe_check_launch("fp8_weight_repack");
}
