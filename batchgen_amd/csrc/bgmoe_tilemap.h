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
// the same for token image `image` of a macro tile whose group has only rows 0 .. last_row of the tile left: rows
// past the end re-read the last row (their products are never stored); the swizzle follows the image row, not the
// row that is read
BGMOE_HD uint32_t bgmoe_k64_token_src_offset(uint32_t lane, uint32_t half, uint32_t image, uint32_t last_row, uint32_t pitch) {
  const uint32_t img_row = 16u * half + (lane >> 2);
  const uint32_t tok = 32u * image + img_row;
  return (tok < last_row ? tok : last_row) * pitch + (((lane & 3u) ^ bgmoe_k64_swizzle(img_row)) << 4);
}
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

// ---- block geometry of the K = 64 kernel -------------------------------------------------------------------------------
// Macro tile: 256 tokens x 256 weight rows (fused stage 1: 128 gate + 128 up rows = 128 output columns), 8 waves =
// 4 (weight rows: wn) x 2 (tokens: wm).  A ring slot holds one K-step of 64 bytes: 8 token images (image i = tokens
// 32 i .. 32 i + 31 of the macro tile) and 8 weight images (plain: rows 32 i ..; fused: images 0..3 = gate rows
// 32 i .., images 4..7 = up rows 32 (i - 4) ..).  Wave w loads token image w and weight image w.
BGMOE_HD uint32_t bgmoe_k64_wave_wn(uint32_t wave) { return wave & 3u; }
BGMOE_HD uint32_t bgmoe_k64_wave_wm(uint32_t wave) { return wave >> 2; }
// weight image a (0, 1) and token image b (0..3) that wave (wn, wm) multiplies
BGMOE_HD uint32_t bgmoe_k64_a_image(bool fused, uint32_t wn, uint32_t a) { return fused ? 4u * a + wn : 2u * wn + a; }
BGMOE_HD uint32_t bgmoe_k64_b_image(uint32_t wm, uint32_t b) { return 4u * wm + b; }
// first weight row of image i relative to the macro tile's first row n0, and the matrix it comes from (fused: 0 gate, 1 up)
BGMOE_HD uint32_t bgmoe_k64_image_wrow(bool fused, uint32_t image) { return fused ? 32u * (image & 3u) : 32u * image; }
BGMOE_HD uint32_t bgmoe_k64_image_matrix(bool fused, uint32_t image) { return fused ? image >> 2 : 0u; }
// where accumulator register v of lane `lane` of product (b, a) belongs: token and output column relative to the
// macro tile's (m0, n0).  Fused: products a = 0 (gate) and a = 1 (up) of one b hold the SAME (token, column): SwiGLU
// pairs them in the lane.
BGMOE_HD uint32_t bgmoe_k64_out_token(uint32_t wm, uint32_t b, uint32_t lane) { return 128u * wm + 32u * b + (lane & 31u); }
BGMOE_HD uint32_t bgmoe_k64_out_col(bool fused, uint32_t wn, uint32_t a, uint32_t lane, uint32_t v) {
  const uint32_t r = bgmoe_mfma32_acc_a_row(lane, v);
  return fused ? 32u * wn + r : 64u * wn + 32u * a + r;
}

// ---- epilogue regrouping through a per-wave LDS patch -------------------------------------------------------------------
// A lane holds 4 consecutive output columns of 16 different places of one token, and the 32 lanes of a half wave hold
// 32 different tokens: stored as they are, one store instruction touches 32 rows with 8 (bf16) or 4 (e4m3) bytes
// each.  Each wave therefore passes its results through a private LDS patch (LDS operations of one wave execute in
// order: no barrier) and stores whole row segments.
constexpr uint32_t BGMOE_K64_PATCH_BYTES = 1536;
// Plain GEMM, bf16: pass p (0..3) of token image b moves its tokens 8p .. 8p+7: 8 rows x the wave's 64 columns
// (128 bytes) at a pitch of 144 bytes.  Writers are the 16 lanes that hold those tokens; each writes, per product a
// and register group q, 8 bytes (registers 4q .. 4q+3 = columns 32a + 8q + 4 (lane / 32) .. + 3).  Then every lane
// reads 16 bytes: row lane / 8, columns 8 (lane % 8) .. + 7, and a store instruction writes 8 whole 128-byte segments.
BGMOE_HD bool bgmoe_k64_patch_writer(uint32_t lane, uint32_t p) { return ((lane & 31u) >> 3) == p; }
BGMOE_HD uint32_t bgmoe_k64_patch_write_off(uint32_t lane, uint32_t a, uint32_t q) {
  return (lane & 7u) * 144u + 64u * a + 16u * q + 8u * (lane >> 5);
}
BGMOE_HD uint32_t bgmoe_k64_patch_read_off(uint32_t lane) { return (lane >> 3) * 144u + (lane & 7u) * 16u; }
BGMOE_HD uint32_t bgmoe_k64_patch_read_token(uint32_t p, uint32_t lane) { return 8u * p + (lane >> 3); }   // of the image's 32
BGMOE_HD uint32_t bgmoe_k64_patch_read_col(uint32_t lane) { return (lane & 7u) * 8u; }                     // of the wave's 64
// Fused stage 1, e4m3 bytes: all 32 tokens of token image b at once: 32 rows x the wave's 32 columns (32 bytes) at a
// pitch of 48 bytes; a lane writes 4 bytes per register group q and reads 16 bytes: row lane / 2, columns
// 16 (lane % 2) .. + 15; a store instruction writes 32 segments of 32 bytes.
BGMOE_HD uint32_t bgmoe_k64_qpatch_write_off(uint32_t lane, uint32_t q) { return (lane & 31u) * 48u + 8u * q + 4u * (lane >> 5); }
BGMOE_HD uint32_t bgmoe_k64_qpatch_read_off(uint32_t lane) { return (lane >> 1) * 48u + (lane & 1u) * 16u; }
BGMOE_HD uint32_t bgmoe_k64_qpatch_read_token(uint32_t lane) { return lane >> 1; }                          // of the image's 32
BGMOE_HD uint32_t bgmoe_k64_qpatch_read_col(uint32_t lane) { return (lane & 1u) * 16u; }                    // of the wave's 32

// ---- bf16 GEMM with 128-token x 64-output block tiles (router_gemm_lds64_kernel) ----------------------------------------
// A K step holds 64 output ("expert") rows then 128 token rows, 128 bytes (64 bf16) each, in one LDS stage:
// experts at byte 0, tokens at byte 64 * 128.  The block's 8 waves issue 3 loads each; issue j = 3 * wave + i covers
// rows 8j .. 8j+7 of the list [64 expert rows; 128 token rows]; lane p of an issue moves row p / 8's 16-byte piece
// (p % 8) ^ (row % 8) to position p % 8 of the row (XOR swizzle).  Lane (r, q) of a wave then reads logical pieces
// 2q and 2q + 1 of row r of a 16-row tile.
constexpr uint32_t BGMOE_RG64_EXPERTS = 64;
BGMOE_HD bool bgmoe_rg64_issue_is_token(uint32_t wave, uint32_t i) { return 8u * (3u * wave + i) >= BGMOE_RG64_EXPERTS; }
// first row (inside its half of the stage) of issue (wave, i)
BGMOE_HD uint32_t bgmoe_rg64_issue_row0(uint32_t wave, uint32_t i) {
  const uint32_t j = 3u * wave + i;
  return bgmoe_rg64_issue_is_token(wave, i) ? 8u * j - BGMOE_RG64_EXPERTS : 8u * j;
}
BGMOE_HD uint32_t bgmoe_rg64_lane_row(uint32_t wave, uint32_t i, uint32_t lane) { return bgmoe_rg64_issue_row0(wave, i) + (lane >> 3); }
BGMOE_HD uint32_t bgmoe_rg64_lane_piece(uint32_t row, uint32_t lane) { return (lane & 7u) ^ (row & 7u); }   // fetched piece
// LDS byte offset (inside the stage) of the issue's first byte; lane p lands at + 16 p
BGMOE_HD uint32_t bgmoe_rg64_issue_lds(uint32_t wave, uint32_t i) {
  return (bgmoe_rg64_issue_is_token(wave, i) ? BGMOE_RG64_EXPERTS * 128u : 0u) + bgmoe_rg64_issue_row0(wave, i) * 128u;
}
// operand reads: output tile tn (0..3), token tile wt (0..7), lane (r = lane % 16, q = lane / 16), half jj (0, 1)
BGMOE_HD uint32_t bgmoe_rg64_read_expert(uint32_t tn, uint32_t lane, uint32_t jj) {
  const uint32_t r = lane & 15u, q = lane >> 4;
  return (16u * tn + r) * 128u + (((2u * q + jj) ^ (r & 7u)) << 4);
}
BGMOE_HD uint32_t bgmoe_rg64_read_token(uint32_t wt, uint32_t lane, uint32_t jj) {
  const uint32_t r = lane & 15u, q = lane >> 4;
  return BGMOE_RG64_EXPERTS * 128u + (16u * wt + r) * 128u + (((2u * q + jj) ^ (r & 7u)) << 4);
}
