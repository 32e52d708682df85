// Operand tile images of the K = 64 LDS-tiled FP8 GEMM (v_mfma_f32_32x32x64_f8f6f4): where a 16-byte piece of an
// operand goes on its way global memory -> LDS -> matrix-instruction registers.  Plain C++ (see bgmoe_hostdev.h):
// the kernel and the host-compiled checks share this text, so the lane maps are tested on the CPU by emulating a
// wave's loads and reads byte for byte.
//
// A tile image is 32 rows x 64 K-bytes = 2 KiB.  The matrix instruction takes, from lane l, 32 bytes of row
// l % 32: K half l / 32 of the image's 64 bytes (which 32 bytes a half holds is immaterial as long as both operands
// use the same split, which they do: one map for tokens and weights).  A lane reads them as two 16-byte pieces.
//
// Row-major sources (tokens, row-major weights): a wave's asynchronous load moves 64 lanes x 16 bytes to 1 KiB of
// LDS in lane order, so lane p lands at 16 * p of a half image (16 rows): row p / 4, stored piece p % 4.  The piece
// it FETCHES is (p % 4) ^ swizzle(row): four lanes still fetch one row's 64 contiguous bytes, and the operand
// reads of any 8 consecutive lanes (8 rows, one logical piece) fall into 8 different 16-byte bank groups of the
// 256-byte bank row: position 4 * (row % 4) + (piece ^ (row / 4 % 4)).
//
// Tile-major weights (16 rows x 128 K-bytes per 2 KiB tile, stored as [K half][16-byte piece][row] so that the
// K = 128 kernels read it with two linear 1 KiB loads): K half h of a tile is one contiguous KiB in
// [piece][row] order, loaded linearly; a 32-row image is two of them (rows 0..15, 16..31).
#pragma once
#include "bgmoe_hostdev.h"

constexpr uint32_t BGMOE_K64_TILE_BYTES = 2048;

BGMOE_HD uint32_t bgmoe_k64_swizzle(uint32_t row) { return (row >> 2) & 3u; }

// ---- row-major sources ------------------------------------------------------------------------------------------
// lane `lane` of the load of half image `half` (rows 16*half .. 16*half+15): byte offset in the source relative
// to the image's first row and K-byte, and byte offset inside the 2 KiB image in LDS
BGMOE_HD uint32_t bgmoe_k64_load_src_offset(uint32_t lane, uint32_t half, uint32_t pitch) {
  const uint32_t row = 16u * half + (lane >> 2);
  return row * pitch + (((lane & 3u) ^ bgmoe_k64_swizzle(row)) << 4);
}
BGMOE_HD uint32_t bgmoe_k64_load_lds_offset(uint32_t lane, uint32_t half) { return 1024u * half + 16u * lane; }
// the two 16-byte pieces lane `lane` feeds to the matrix instruction: row lane % 32, pieces 2h and 2h + 1 of K half
// h = lane / 32
BGMOE_HD uint32_t bgmoe_k64_operand_lo(uint32_t lane) {
  const uint32_t row = lane & 31u, h = lane >> 5;
  return row * 64u + (((2u * h) ^ bgmoe_k64_swizzle(row)) << 4);
}
BGMOE_HD uint32_t bgmoe_k64_operand_hi(uint32_t lane) {
  const uint32_t row = lane & 31u, h = lane >> 5;
  return row * 64u + (((2u * h + 1u) ^ bgmoe_k64_swizzle(row)) << 4);
}

// ---- tile-major weights -------------------------------------------------------------------------------------------
// Source: K half `kh` (0, 1) of K-block kb of the 16-row tile starts at tile_base + kb * 2048 + kh * 1024 and is
// copied linearly (lane p: 16 * p) to half image `half`.  Inside that KiB piece q (0..3) of row r sits at 16 * (16 * q + r).
BGMOE_HD uint32_t bgmoe_k64_tm_operand_lo(uint32_t lane) {
  const uint32_t row = lane & 31u, h = lane >> 5;
  return 1024u * (row >> 4) + 16u * (16u * (2u * h) + (row & 15u));
}
BGMOE_HD uint32_t bgmoe_k64_tm_operand_hi(uint32_t lane) {
  const uint32_t row = lane & 31u, h = lane >> 5;
  return 1024u * (row >> 4) + 16u * (16u * (2u * h + 1u) + (row & 15u));
}

// ---- accumulator of a 32 x 32 product (16 fp32 registers per lane) ---------------------------------------------------
// register v of lane l holds D[a_row][b_row]: a_row from the first operand (weights: the output column), b_row
// from the second (tokens: the output row)
BGMOE_HD uint32_t bgmoe_mfma32_acc_a_row(uint32_t lane, uint32_t v) { return 8u * (v >> 2) + 4u * (lane >> 5) + (v & 3u); }
BGMOE_HD uint32_t bgmoe_mfma32_acc_b_row(uint32_t lane) { return lane & 31u; }
