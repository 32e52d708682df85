/*
 * bgmoe.h -- C ABI of libbgmoe.so: the MoE expert-layer hot path for AMD
 * MI355X (gfx950).  Plain pointers and sizes only; every pointer that is not
 * marked "host" is DEVICE memory on the current HIP device; every call
 * enqueues on `stream` (a hipStream_t passed as void*) and returns without
 * synchronising, reading nothing back from the device, with a launch geometry
 * that depends on host arguments only (so a call sequence can be captured in
 * a HIP graph and replayed with different device-side counts).
 *
 * Return value: BGMOE_OK, or an error code with a message available from
 * bgmoe_last_error() (thread-local).  Argument errors are detected before
 * anything is launched.
 *
 * "reference" below = batchgen-project/batchgen; each entry point names the
 * reference op it replaces.  Paths are relative to the reference tree.
 */
#ifndef BGMOE_H
#define BGMOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* bgmoe_stream_t; /* hipStream_t */

enum {
  BGMOE_OK = 0,
  BGMOE_ERR_ARG = 1,         /* bad shape / alignment / unsupported value */
  BGMOE_ERR_HIP = 2,         /* a HIP runtime call failed                 */
  BGMOE_ERR_WORKSPACE = 3    /* workspace too small                       */
};

const char* bgmoe_last_error(void);
int bgmoe_version(void);

/* Optional one-time set-up on the current device: the occupancy and device-property queries and the
 * dynamic-LDS opt-in that the GEMM entry points otherwise perform at their first call.  After it (or after
 * one eager call of each entry point) every call is a pure sequence of enqueues, which is what HIP-graph
 * capture needs.  No counterpart in the reference (its TMA plans play this role,
 * batchgen/moe/grouped_fp8_blockwise_moe.py, `fp8_blockwise_prepare_s1_s3_tma`). */
int bgmoe_init(void);

/* Per-launch timing for benchmarks.  bgmoe_prof_enable(1) brackets every kernel
 * launch with HIP events on its stream; bgmoe_prof_collect synchronises the
 * device and returns, per kernel id in [0, bgmoe_prof_kernel_count()), the total
 * elapsed milliseconds and number of launches since the last collect.  No
 * reference counterpart (the reference times spans with CUDA-event pairs in
 * Python, batchgen/timing.py:1-60). */
int bgmoe_prof_enable(int on);
int bgmoe_prof_kernel_count(void);
const char* bgmoe_prof_kernel_name(int id);
int bgmoe_prof_collect(double* total_ms, int64_t* launches, int n);

/* ------------------------------------------------------------------ router */

/* Group-limited top-k on (optionally already sigmoided) scores.
 * Replaces `moe_fused_gate` (batchgen_kernels/common/mgn.py:32-65,
 * batchgen_kernels/src/moe/mgn/moe_fused_gate.cu:83-329).
 * scores [n,e] fp32 contiguous; bias [e]; ids [n,top_k] int32 in descending
 * biased-score order; weights [n,top_k] fp32 = raw*rsf/(sum(raw)+1e-20).
 * apply_sigmoid != 0: `scores` holds logits; the correctly rounded fp32
 * sigmoid is applied first (the reference caller does torch.sigmoid before the
 * op, batchgen/models/deepseek/deepseekv3/modeling_deepseek_v3.py:893-914).
 * e <= 1024, n_group <= 64, e % n_group == 0, top_k <= 32. */
int bgmoe_fused_gate(const float* scores, const float* bias, int n, int e, int n_group,
                     int topk_group, int top_k, float routed_scaling_factor, int apply_sigmoid,
                     int32_t* topk_ids, float* topk_weights, bgmoe_stream_t stream);

/* Ungrouped sigmoid + bias top-k.
 * Replaces `gate_sigmoid_topk` / `gate_sigmoid_topk_warp`
 * (batchgen/moe/routing/cuda_routing.py:124-304,
 * batchgen_kernels/src/moe/routing/gate_sigmoid_topk.cu:71-213, 546-714).
 * logits rows may be strided (logits_stride elements, >= e).
 * ids: int32 or int64 [n,k] (ids_are_int64).  num_valid_tokens (device int32
 * scalar) or rank_token_counts (device int64 [ceil(n/rows_per_rank)]) mark
 * padding rows, which get id -1 / weight 0; both may be NULL.
 * latent_out (bf16 [n, latent_size]) optionally receives
 * bf16(row[latent_offset : latent_offset+latent_size]); NULL to skip. */
int bgmoe_gate_sigmoid_topk(const float* logits, int64_t logits_stride, const float* bias, int n,
                            int e, int k, float routed_scaling_factor, void* topk_ids,
                            int ids_are_int64, float* topk_weights,
                            const int32_t* num_valid_tokens, const int64_t* rank_token_counts,
                            int rows_per_rank, uint16_t* latent_out, int latent_offset,
                            int latent_size, bgmoe_stream_t stream);

/* ------------------------------------------------------------ router GEMM */

/* Bytes of device workspace for the router GEMM at these sizes: the split-K planes
 * (ceil(h/512) * n * e * 4) when few tokens make split-K the launch shape, else n * e * 4.  Without it
 * bgmoe_router_gemm still works (one block walks all of K: the same bits, slower when n is small);
 * bgmoe_router_gemm_gate needs it. */
size_t bgmoe_router_gemm_workspace_bytes(int n, int h, int e);

/* logits[n,e] fp32 = hidden[n,h] bf16 x router_weight[e,h]^T bf16, fp32 accumulation.
 * Replaces `glm5_router_gemm_cuda` (batchgen/moe/routing/cuda_routing.py:318-366,
 * batchgen_kernels/src/moe/routing/glm5_router_gemm.cu:35-180) and its contract: a row's logits do not
 * depend on the number of rows in the call (batchgen/models/glm5/model.py:1135-1140), and with
 * rank_token_counts (device int64 [world_size]) row i is padding when
 * i % bucket_size >= rank_token_counts[i / bucket_size]: its logits are 0 and its hidden row may hold
 * anything (NaN included).  The summation order differs from the reference kernel's (MFMA chains per
 * 512-element K segment, segments added in order), so the fp32 bits differ in the last places; the order
 * is fixed, so results are reproducible and equal between this entry point and
 * bgmoe_router_gemm_gate.  h % 8 == 0.  rank_token_counts may be NULL. */
int bgmoe_router_gemm(const uint16_t* hidden, const uint16_t* router_weight, int n, int h, int e,
                      const int64_t* rank_token_counts, int bucket_size, int world_size, float* logits,
                      void* workspace, size_t workspace_bytes, bgmoe_stream_t stream);

/* out[n,e] bf16 = bf16(x[n,h] bf16 x weight[e,h]^T bf16), fp32 accumulation in the router GEMM's fixed order: a
 * bias-free linear layer on the same kernels (`nn.Linear` of the bf16 shared expert and of the latent projections,
 * batchgen/moe/fused_moe_mxfp4_resident.py:905-944, kimi_linear/model.py:585-603, which the reference runs on the
 * vendor GEMM).  workspace: bgmoe_router_gemm_workspace_bytes(n,h,e) (optional, as for bgmoe_router_gemm). */
int bgmoe_bf16_linear(const uint16_t* x, const uint16_t* weight, int n, int h, int e, uint16_t* out, void* workspace,
                      size_t workspace_bytes, bgmoe_stream_t stream);

/* Router GEMM + top-k in two launches without materialising the logits: identical ids and weights to
 * bgmoe_router_gemm followed by bgmoe_fused_gate(apply_sigmoid=1) (n_group >= 1) or by
 * bgmoe_gate_sigmoid_topk (n_group == 0; rank_token_counts / rows_per_rank as there).  The reference
 * runs the GEMM and the gate as separate ops (batchgen/models/glm5/model.py:1119-1161); fusing them is
 * this build's choice.  workspace: bgmoe_router_gemm_workspace_bytes(n,h,e). */
int bgmoe_router_gemm_gate(const uint16_t* hidden, const uint16_t* router_weight, const float* bias,
                           int n, int h, int e, int n_group, int topk_group, int top_k,
                           float routed_scaling_factor, int32_t* topk_ids, float* topk_weights,
                           const int64_t* rank_token_counts, int rows_per_rank, void* workspace,
                           size_t workspace_bytes, bgmoe_stream_t stream);

/* Tuning/test knob (no reference counterpart): force the router GEMM's launch shape.  token_tiles in
 * {1,2,4} = 16-token tiles per wave; split 0 = one block walks all of K, 1 = one block per 512-element
 * K segment, 2 = the same with one-wave blocks (the shape for few tokens), 3 = all of K with the operands
 * shared through LDS (the shape for many tokens; h % 64 == 0), 4 = one LDS block per K segment, 5 = all of K
 * through LDS with block tiles of 128 tokens x 64 outputs instead of 128 x 128 (twice as many blocks: for shapes
 * whose wide tiles number fewer than the CUs, e.g. a 512-row linear layer; h % 64 == 0; never chosen from the
 * sizes yet); -1 = choose from the sizes.
 * Results do not depend on it, bit for bit. */
int bgmoe_set_router_gemm_plan(int token_tiles, int split);

/* ------------------------------------------- producer: add + RMSNorm + FP8 */

/* residual += hidden (bf16, in place); normed = RMSNorm(residual) * weight (bf16); and, when quant_out is
 * not NULL, the per-token 128-block e4m3fn cast of `normed` in the same pass, so that the MoE layer's FP8
 * activation never makes a second trip through memory.
 * Replaces `cuda_add_rmsnorm_fp8_quant` (batchgen_kernels/attention/add_rmsnorm_fp8_quant.py:33-83,
 * batchgen_kernels/src/attention/csrc/add_rmsnorm_fp8_quant.cu:242-541) with its thread partition and
 * reduction tree (8 columns per thread, fma chain, 32-lane trees), its gates and its contract: `normed`
 * and `residual` equal the unfused add+RMSNorm, and (quant_out, quant_scale) equal the standalone 1-D
 * quantiser applied to the bf16 `normed` (batchgen_kernels/triton/fp8_quantize.py:252-331: amax floored
 * at 2^-16, scale = max(amax/448, 1e-12)), bit for bit -- which for blocks with amax >= 2^-16 is also
 * bgmoe_act_quant_rows(normed).  The CUDA kernel's rsqrtf and div.full.f32 are approximate instructions;
 * here both are correctly rounded, so `normed` can differ from the CUDA bytes in the last bf16 place.
 * h: a multiple of 128 up to 8192 (the reference is compiled for 6144 only).  Scale element (r,kb) at
 * quant_scale[r*scale_row_stride + kb*scale_kb_stride]: (h/128, 1) is the contiguous form,
 * (1, align4(rows)) the MN-major one.  Gates (device int32 scalars / bf16 [rows], any may be NULL):
 * rows >= *norm_num_valid_tokens are not touched by the norm; rows >= *quant_num_valid_tokens get bytes 0
 * and scales 1e-12; row_valid_mask[r] == 0 drops hidden row r from the sum (a predicate: NaN rows are
 * safe).  norm_num_valid_tokens must be the same pointer as quant_num_valid_tokens when quantising. */
int bgmoe_add_rmsnorm_fp8_quant(uint16_t* residual, const uint16_t* hidden, const uint16_t* weight,
                                int64_t rows, int h, float eps, uint16_t* normed_out, uint8_t* quant_out,
                                float* quant_scale, int64_t scale_row_stride, int64_t scale_kb_stride,
                                const int32_t* norm_num_valid_tokens, const int32_t* quant_num_valid_tokens,
                                const uint16_t* row_valid_mask, bgmoe_stream_t stream);

/* --------------------------------------------------------- FP8 act quant */

/* Per-row, per-128 e4m3fn quantisation of plain rows:
 *   s = fmaxf(amax,1e-12f)*(1/448.f); q = clamp(x/s, +-448) -> RNE e4m3fn.
 * Replaces `act_quant` (batchgen/quantization/act_quant.py:78-128; identical
 * bytes and, for amax >= 2^-16, identical scales).  x [rows,k] bf16;
 * y [rows,k] bytes; scale element (r,kb) at scale[r*srow + kb*skb]. */
int bgmoe_act_quant_rows(const uint16_t* x, int64_t rows, int k, uint8_t* y, float* scale,
                         int64_t scale_row_stride, int64_t scale_kb_stride, bgmoe_stream_t stream);

/* The 1-D quantiser exactly: replaces `per_token_blocked_quantize_bf16_to_fp8_1d`
 * (batchgen_kernels/triton/fp8_quantize.py:252-391): amax floored at 2^-16, s = fmaxf(amax * (1/448.f), 1e-12f),
 * q = clamp(x/s, +-448) -> RNE e4m3fn; equals bgmoe_act_quant_rows wherever a block's amax is >= 2^-16.
 * num_valid_tokens (optional, device int32 scalar): rows at or past it get zero bytes and scale 1e-12.
 * Scale element (r,kb) at scale[r*srow + kb*skb]: (k/128, 1) contiguous, (1, align4(rows)) MN-major. */
int bgmoe_act_quant_rows_1d(const uint16_t* x, int64_t rows, int k, uint8_t* y, float* scale,
                            int64_t scale_row_stride, int64_t scale_kb_stride, const int32_t* num_valid_tokens,
                            bgmoe_stream_t stream);

/* Masked layout.  Replaces `act_quant_3d`
 * (batchgen_kernels/src/moe/fp8_blockwise/fp8_blockwise_ops.cu:39-111, 519-556).
 * x [e,mtp,k]; rows >= tokens_per_expert[e] are neither read nor written;
 * scale [e,mtp,ceil(k/128)]. */
int bgmoe_act_quant_3d(const uint16_t* x, const int32_t* tokens_per_expert, int e, int mtp, int k,
                       uint8_t* y, float* scale, bgmoe_stream_t stream);

/* Ragged layout.  Replaces `act_quant_ragged` (fp8_blockwise_ops.cu:151-361,
 * 558-628).  Row r in [cu[0],cu[e]) owned by o = max{e: cu[e] <= r} is written
 * iff r-cu[o] < align(seqlens[o],row_align); rows past seqlens[o] inside the
 * span get bytes 0 and the all-zero-row scale; other rows are untouched and
 * their x is not read.  scale_t is TRANSPOSED [ceil(k/128), max_rows]. */
int bgmoe_act_quant_ragged(const uint16_t* x, const int32_t* seqlens, const int32_t* cu_seqlens,
                           int e, int64_t max_rows, int k, uint8_t* y, float* scale_t,
                           int row_align, bgmoe_stream_t stream);

/* silu(gate)*up -> bf16 on the masked layout.  Replaces `silu_mul_3d`
 * (fp8_blockwise_ops.cu:391-438).  gate, up, out [e,mtp,k] bf16. */
int bgmoe_silu_mul_3d(const uint16_t* gate, const uint16_t* up, const int32_t* tokens_per_expert,
                      int e, int mtp, int k, uint16_t* out, bgmoe_stream_t stream);

/* silu(gate)*up then quantise.  Replaces `fused_silu_quant_3d`
 * (fp8_blockwise_ops.cu:445-513) with this build's canonical rounding:
 * h = bf16(silu_f32(gate)*up) then the act-quant above (so that the result is
 * bit-identical to bgmoe_silu_mul_3d followed by bgmoe_act_quant_3d). */
int bgmoe_fused_silu_quant_3d(const uint16_t* gate, const uint16_t* up,
                              const int32_t* tokens_per_expert, int e, int mtp, int k, uint8_t* y,
                              float* scale, bgmoe_stream_t stream);

/* Replaces `deepep_ll_scale_repack` (fp8_blockwise_ops.cu:685-797; wrapper batchgen/models/glm/glm5/moe_ragged.py:330-352):
 * the low-latency exchange returns activation scales as a contiguous [E, KB, S] fp32 block (KB = hidden/128,
 * S = rows per expert); out is the [KB, E*S] matrix with expert e at column e*S.  Per expert, columns
 * [0, ceil(recv_count[e] / span_align) * span_align) of every row are copied bit for bit and the rest of `out`
 * is left as it is.  span_align: positive multiple of 4 dividing S.  Both buffers 16-byte aligned and disjoint.
 * A count outside [0, S] copies nothing for that expert and ORs 1 into *status (optional, device; never
 * cleared here) where the reference traps the device.  The grouped GEMMs of this library also read the
 * exchange's block in place (bgmoe_fp8_act.scale_group_stride), which needs no repack. */
int bgmoe_deepep_ll_scale_repack(const float* recv_scales, const int32_t* recv_count, float* out, int experts,
                                 int kb, int s, int span_align, int32_t* status, bgmoe_stream_t stream);

/* bf16(silu(gate)) * up in bf16, then the per-row, per-128-column FP8 cast, in one pass: the activation
 * between the two grouped GEMMs of the DeepGEMM chains and of the dense shared expert.  Replaces
 *   form 1 (D): `silu_mul_masked_group_quant` / `silu_mul_ragged_group_quant`
 *               (batchgen_kernels/triton/moe_masked_act_quant.py:43-376; oracle `act_reference`,
 *               tests/test_glm52_deepgemm_masked_parity_gpu.py:128-149):
 *               amax = max(max|p|, 1e-10), scale = amax / 448, q = clamp(p / scale, +-448);
 *   form 0 (A): `silu_mul_per_token_blocked_quantize_bf16_to_fp8_1d`
 *               (batchgen_kernels/triton/fp8_quantize.py:394-526): the 1-D quantiser of
 *               bgmoe_act_quant_rows (amax floor 2^-16, scale = max(amax * (1/448), 1e-12), non-finite -> 0).
 * In both, p = bf16( bf16(s) * up ) with s = g / (1 + exp(-g)) evaluated as the fp32 sequence
 * exp (correctly rounded), add, IEEE division (PyTorch's SiLU, fp8_quantize.py:414-424).
 * Row r of group e lives at element offset e*stride_e + (start_e + r)*stride_s, start_e = starts[e] or 0 when
 * starts is NULL; rows r >= counts[e] (all max_rows rows when counts is NULL) are neither read nor written.
 * masked [E,S,I]: stride_e = S*stride_s, starts NULL, counts = masked_m, max_rows = S;
 * ragged [m,I]:   stride_e = 0, starts = cu_seqlens, counts = live rows, max_rows = bound on any count;
 * 1-D [M,2I]:     groups 1, counts NULL, gate = x, up = x + I, in_stride_s = 2I, max_rows = M.
 * Scale of (e, r, group g) at scale[e*scale_stride_e + (start_e + r)*scale_stride_s + g*scale_stride_g].
 * prod_out (bf16, addressed like out) optionally receives p.  n a multiple of 128; 16-byte aligned rows. */
int bgmoe_silu_mul_group_quant(const uint16_t* gate, const uint16_t* up, int64_t in_stride_e,
                               int64_t in_stride_s, const int32_t* counts, const int32_t* starts, int groups,
                               int64_t max_rows, int n, int form, uint8_t* out, int64_t out_stride_e,
                               int64_t out_stride_s, float* scale, int64_t scale_stride_e,
                               int64_t scale_stride_s, int64_t scale_stride_g, uint16_t* prod_out,
                               bgmoe_stream_t stream);

/* The same activation fed by bgmoe_fp8_dense_gemm_partials: gate | up arrive as `slices` fp32 planes of
 * [rows, 2n] (plane stride slice_stride floats); the planes are added in ascending order and rounded to bf16, which
 * is what the GEMM's own second launch would have stored, then processed as above (form 0 or 1).  out [rows, n]
 * bytes with row stride out_stride_s, scale element (r, g) at scale[r*scale_stride_s + g*scale_stride_g]. */
int bgmoe_silu_mul_group_quant_partials(const float* partials, int slices, int64_t slice_stride, int64_t rows, int n,
                                        int form, uint8_t* out, int64_t out_stride_s, float* scale,
                                        int64_t scale_stride_s, int64_t scale_stride_g, bgmoe_stream_t stream);

/* ------------------------------------------------------ permute / unpermute */

/* Bytes of device workspace the dispatch calls need for n*k pairs. */
size_t bgmoe_dispatch_workspace_bytes(int64_t nk, int num_local_experts);

/* Masked [E_l, mtp, H] layout.  Replaces `dispatch_scatter_3d`
 * (batchgen/moe/dispatch_scatter_3d.py:76-109,
 * batchgen_kernels/src/moe/dispatch_scatter_3d.cu:15-137).
 * Pair i = t*k + j with local id le = ids[i]-expert_start in [0,E_l) goes to
 * row le*mtp + slot, slot = number of earlier pairs (smaller i) of the same
 * expert (deterministic; the reference uses arrival order).  topk_pos[i] = row
 * or -1.  Pairs with slot >= mtp are dropped (-1) and counts are clipped.
 * expert_counters[e] is written with the number of pairs routed to expert e
 * BEFORE clipping (what the reference's atomic counter holds at the end):
 * expert_counters[e] > expert_counts[e] tells the caller that rows of expert e
 * were dropped.  act_buffer may be NULL to compute indices only. */
int bgmoe_dispatch_scatter_3d(const uint16_t* x, const int32_t* topk_ids, int n, int k, int h,
                              uint16_t* act_buffer, int expert_start, int num_local_experts,
                              int max_tokens_padded, int32_t* expert_counts,
                              int32_t* expert_counters, int32_t* topk_pos, void* workspace,
                              size_t workspace_bytes, bgmoe_stream_t stream);

/* The index part of bgmoe_dispatch_scatter_3d alone, plus the inverse map (no counterpart in the reference): same
 * expert_counts / expert_counters / topk_pos, no rows are moved, and row_pair[topk_pos[i]] = i for every placed pair
 * i = token * k + slot (rows of the masked layout that hold no pair keep what they held).  For consumers that read
 * a row's data from its token instead of from a gathered copy (bgmoe_mxfp4_fused_s1_gather). */
int bgmoe_dispatch_index_3d(const int32_t* topk_ids, int n, int k, int expert_start, int num_local_experts,
                            int max_tokens_padded, int32_t* expert_counts, int32_t* expert_counters, int32_t* topk_pos,
                            int32_t* row_pair, void* workspace, size_t workspace_bytes, bgmoe_stream_t stream);

/* Contiguous ragged layout.  Replaces `dispatch_scatter_ragged`
 * (dispatch_scatter_3d.py:112-156, dispatch_scatter_3d.cu:152-358) and, with
 * row_align = 1, `dispatch_count_gather`
 * (batchgen_kernels/src/moe/routing/dispatch_count_gather.cu:32-251) and
 * `fused_moe_token_dispatch` (batchgen_kernels/src/moe/mgn/fused_moe_token_dispatch.cu:172-292).
 * cu_seqlens[e+1]-cu_seqlens[e] = align(count[e], row_align); act_rows is the
 * capacity of act_buffer, checked against the worst case. */
int bgmoe_dispatch_scatter_ragged(const uint16_t* x, const int32_t* topk_ids, int n, int k, int h,
                                  uint16_t* act_buffer, int64_t act_rows, int expert_start,
                                  int num_local_experts, int32_t* expert_counts,
                                  int32_t* expert_counters, int32_t* topk_pos,
                                  int32_t* cu_seqlens, int row_align, void* workspace,
                                  size_t workspace_bytes, bgmoe_stream_t stream);

/* bgmoe_dispatch_scatter_ragged for callers that cannot allocate device memory or pass a workspace (code under
 * HIP-graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same arguments, outputs and results, bit for bit; the chunk histograms that the other entry
 * point keeps in `workspace` live in a 1 MiB device array that is part of the library image (one copy per
 * GPU, held until the process ends), so the call allocates nothing and frees nothing.  Limit:
 * ceil(n*k / 2048) * num_local_experts <= 262144 (bgmoe_dispatch_static_max_pairs(num_local_experts) pairs:
 * 2 097 152 at 256 local experts); larger problems are rejected with BGMOE_ERR_WORKSPACE before anything is
 * launched.  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams,
 * two host threads) race; calls ordered on one stream, or separated by an event, are safe, and nothing has to
 * be cleared between them. */
size_t bgmoe_dispatch_static_max_pairs(int num_local_experts);
int bgmoe_dispatch_scatter_ragged_static(const uint16_t* x, const int32_t* topk_ids, int n, int k, int h,
                                         uint16_t* act_buffer, int64_t act_rows, int expert_start,
                                         int num_local_experts, int32_t* expert_counts,
                                         int32_t* expert_counters, int32_t* topk_pos, int32_t* cu_seqlens,
                                         int row_align, bgmoe_stream_t stream);

/* The per-row outputs of `fused_moe_token_dispatch` (batchgen_kernels/src/moe/mgn/fused_moe_token_dispatch.cu:59-88:
 * output_eids / output_token_idx / output_topk_pos) from the indices of a tight (row_align 1) ragged dispatch:
 * row topk_pos[i] of pair i receives its expert id topk_ids[i], its token i / k and its slot i % k.  Rows at or
 * past *total_rows (device int32: the last entry of the dispatch's cu_seqlens) receive -1, where the reference
 * leaves them uninitialised.  One launch, nothing read back. */
int bgmoe_dispatch_row_metadata(const int32_t* topk_ids, const int32_t* topk_pos, int64_t nk, int k,
                                const int32_t* total_rows, int64_t rows, int32_t* out_eids,
                                int32_t* out_token_idx, int32_t* out_topk_pos, bgmoe_stream_t stream);

/* Quantise-while-scattering: for every pair with topk_pos[i] >= 0 write the
 * act-quant of x[i/k] to row topk_pos[i] of y / scale.  Bit-identical to a
 * scatter followed by bgmoe_act_quant_*.  No reference counterpart as one op:
 * it fuses `dispatch_scatter_*` with `act_quant_*` (the reference's DeepEP
 * receive path delivers the same quantised masked layout,
 * batchgen/moe/deepep_ll.py:331-364). */
int bgmoe_scatter_quant(const uint16_t* x, const int32_t* topk_pos, int n, int k, int h,
                        uint8_t* y, float* scale, int64_t scale_row_stride,
                        int64_t scale_kb_stride, bgmoe_stream_t stream);

/* The same permutation for tokens that arrive ALREADY quantised (bgmoe_add_rmsnorm_fp8_quant upstream):
 * bytes xq [n,h] and scales (t,kb) at xs[t*xs_row_stride + kb*xs_kb_stride] are copied to every row the
 * token is routed to.  Replaces the hand-down of `x_fp8`/`x_scale` into the expert chain
 * (batchgen/models/glm/glm5/wrappers.py:409-447).  h % 16 == 0, k < 64. */
int bgmoe_scatter_fp8_rows(const uint8_t* xq, const float* xs, int64_t xs_row_stride, int64_t xs_kb_stride,
                           const int32_t* topk_pos, int n, int k, int h, uint8_t* y, float* scale,
                           int64_t scale_row_stride, int64_t scale_kb_stride, bgmoe_stream_t stream);

/* out[t] = bf16(sum_k float(y[pos[t,k]])*w[t,k]), k ascending, pos<0 skipped; every term is one fp32 fused
 * multiply-add, acc = fma(value, weight, acc), as the reference kernel's `acc += val * w[k]` compiles.
 * Replaces `reduce_weighted_scatter` (dispatch_scatter_3d.cu:365-395, 527-556;
 * batchgen_kernels/src/moe/routing/reduce_weighted_scatter.cu:26-131).
 * num_valid_tokens > 0 limits the rows written.  shared (bf16 [n,h], may be
 * NULL) is the shared expert's output: shared_mode 0 -> bf16(bf16(sum)+shared)
 * (the reference's bf16 tensor add), 1 -> bf16(sum+shared). */
int bgmoe_reduce_weighted_scatter(const uint16_t* expert_out, const int32_t* topk_pos,
                                  const float* topk_weights, int n, int h, int k, uint16_t* out,
                                  int num_valid_tokens, const uint16_t* shared, int shared_mode,
                                  bgmoe_stream_t stream);

/* fp32 output.  Replaces `reduce_weighted_scatter_fp32` (dispatch_scatter_3d.cu:402-434). */
int bgmoe_reduce_weighted_scatter_fp32(const uint16_t* expert_out, const int32_t* topk_pos,
                                       const float* topk_weights, int n, int h, int k, float* out,
                                       bgmoe_stream_t stream);

/* Expert-id-ordered bf16 accumulation.  Replaces
 * `reduce_weighted_scatter_bf16_ordered` (dispatch_scatter_3d.cu:436-525). */
int bgmoe_reduce_weighted_scatter_bf16_ordered(const uint16_t* expert_out, const int32_t* topk_pos,
                                               const int32_t* topk_ids, const float* topk_weights,
                                               int n, int h, int k, uint16_t* out,
                                               bgmoe_stream_t stream);

/* Active-expert compaction.  Replaces `compact_expert_data`
 * (batchgen_kernels/src/moe/mgn/expert_bin_count.cu:332-385): ascending expert
 * id; outputs int32 [e]: group_size, activated_group_idx, group_start_indices;
 * num_active int32 [1]. */
int bgmoe_compact_expert_data(const int32_t* expert_counts, int e, int32_t* group_size,
                              int32_t* activated_group_idx, int32_t* group_start_indices,
                              int32_t* num_active, bgmoe_stream_t stream);

/* ------------------------------------------------------------ grouped GEMM */

/* Operands of one block-scaled FP8 grouped GEMM
 *   Y[r,n] = sum_kb (sum_{k in kb} Xq[r,k]*Wq[g,n,k]) * xs[r,kb] * ws[g,n/128,kb]
 * for rows r in [cu_seqlens[g], cu_seqlens[g]+seqlens[g]).
 * Weights: either a stack (w + g*w_group_stride bytes) or, when w_ptrs != NULL,
 * a device table of per-group pointers (the reference's *_ptrs forms). */
typedef struct bgmoe_fp8_weight {
  const uint8_t* w;              /* [groups, n, k] e4m3fn                      */
  int64_t w_group_stride;        /* bytes between groups                      */
  const uint8_t* const* w_ptrs;  /* device int64[groups] or NULL              */
  const float* scale;            /* [groups, n/128, kb_stride] fp32           */
  int64_t scale_group_stride;    /* elements between groups                   */
  int64_t scale_nb_stride;       /* elements between 128-row blocks (>= k/128)*/
  const float* const* scale_ptrs;/* device table or NULL                      */
  int32_t layout;                /* BGMOE_W_ROW_MAJOR or BGMOE_W_TILE_MAJOR   */
  int32_t reserved;
} bgmoe_fp8_weight;

/* Weight byte layouts.  ROW_MAJOR is the checkpoint layout [n, k] the reference
 * ops take.  TILE_MAJOR is this build's resident layout for weight streaming:
 * the matrix is cut into 16-row x 128-column tiles of 2048 bytes, tile (nt, kb)
 * at byte ((nt * k/128) + kb) * 2048; inside a tile, byte
 * half*1024 + (q*16 + r)*16 + j holds row nt*16 + r, column kb*128 + half*64 +
 * q*16 + j (r < 16, q < 4, j < 16, half < 2) -- the order in which one wave64
 * reads an MFMA 16x16x128 operand with two fully contiguous 1 KiB loads.
 * bgmoe_fp8_weight_repack converts (one-time, at weight load; the reference has
 * the same kind of step for its own kernels: Marlin repack,
 * batchgen/moe/fused_moe_mxfp4_resident.py:13-15, and TMA plans,
 * batchgen/moe/grouped_fp8_blockwise_moe.py:195-247). */
enum { BGMOE_W_ROW_MAJOR = 0, BGMOE_W_TILE_MAJOR = 1 };
int bgmoe_fp8_weight_repack(const uint8_t* src_row_major, uint8_t* dst_tile_major, int groups, int n,
                            int k, bgmoe_stream_t stream);

typedef struct bgmoe_fp8_act {
  const uint8_t* x;              /* [m, k] e4m3fn                              */
  const float* scale;            /* element (r,kb) at r*row_stride+kb*kb_stride */
  int64_t scale_row_stride;
  int64_t scale_kb_stride;
  /* 0: r is the row of x (cu_seqlens[g] + t).  Non-zero: scales are stored per group, token t of group g at
   * g*scale_group_stride + t*row_stride + kb*kb_stride -- DeepGEMM's masked A-scale form, a contiguous
   * [E, K/128, S] block viewed as [E, S, K/128]: group stride K/128*S, row stride 1, kb stride S
   * (batchgen/models/glm/glm5/moe_deepgemm_masked.py:46-70). */
  int64_t scale_group_stride;
} bgmoe_fp8_act;

/* Single grouped GEMM, bf16 output [m,n].  Replaces
 * `fp8_blockwise_grouped_gemm` / `_ptrs` (batchgen/moe/grouped_fp8_blockwise_moe.py:292-420,
 * batchgen_kernels/src/moe/fp8_blockwise/fp8_blockwise_gemm.cu:564-900).
 * k % 128 == 0, n % 128 == 0, groups <= 1024.  Rows outside every group's
 * live range are not written. */
int bgmoe_fp8_grouped_gemm(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* b,
                           const int32_t* seqlens, const int32_t* cu_seqlens, int groups,
                           int64_t m, int n, int k, uint16_t* out, bgmoe_stream_t stream);

/* One weight matrix against few rows: out[m, n] = bf16(dequant(a) @ dequant(w)^T), w [n, k] e4m3fn (row-major, or the
 * tile-major resident layout) with block scales w_scale[(r/128)*scale_nb_stride + c/128].  Replaces
 * `deep_gemm.fp8_gemm_nt` as the reference calls it for the dense MLP and the shared expert at decode
 * (batchgen/attention/mla/fa3_backend.py:525-590, batchgen/models/glm/glm5/wrappers.py:448-461).  A grouped launch has
 * too few work items for one group, so K is the parallel axis here, in one of two forms chosen from m, k and the
 * layout (never from n).  Wave split: the 8 waves of a block own one K-slice each and add their partial sums through
 * LDS in wave order (no workspace).  Block split: the weight-streaming kernel of the grouped GEMM on K-slices, fp32
 * partial sums in `workspace` (bgmoe_fp8_dense_gemm_workspace(m, n, k, layout) bytes, 0 for the wave split; 16-byte
 * aligned, caller-owned, contents irrelevant before and after), added in ascending slice order by a second launch.
 * Every call is deterministic, and the gate and up halves of a stacked [gate; up] weight equal two separate
 * calls bit for bit.  a->scale_group_stride is ignored.  Weights are streamed once per 64 rows: measured faster than
 * bgmoe_fp8_grouped_gemm with one group up to 64 rows for any n, and up to 512 rows for n <= 8192.
 * k % 128 == 0, n % 128 == 0. */
int64_t bgmoe_fp8_dense_gemm_workspace(int64_t m, int n, int k, int layout);
int bgmoe_fp8_dense_gemm(const bgmoe_fp8_act* a, const uint8_t* w, const float* w_scale, int64_t scale_nb_stride,
                         int layout, int64_t m, int n, int k, uint16_t* out, void* workspace, int64_t workspace_bytes,
                         bgmoe_stream_t stream);

/* The block-split form of bgmoe_fp8_dense_gemm without its second launch, for a consumer that adds the K-slices
 * itself: writes *slices planes of m*n floats (plane stride m*n) into `workspace` and sets *slices.  Fails when
 * (m, k, layout) is served without partial sums (bgmoe_fp8_dense_gemm_workspace == 0).  No reference counterpart:
 * it exists so that the shared expert's chain (glm5/wrappers.py:448-461) needs no launch between its first GEMM
 * and the activation. */
int bgmoe_fp8_dense_gemm_partials(const bgmoe_fp8_act* a, const uint8_t* w, const float* w_scale,
                                  int64_t scale_nb_stride, int layout, int64_t m, int n, int k, void* workspace,
                                  int64_t workspace_bytes, int* slices, bgmoe_stream_t stream);

/* Which LDS-tiled kernel serves the groups above the streaming limit (tuning switch, no reference counterpart;
 * the reference's own tile choice is `num_seq_per_group_avg` -> TileM, batchgen/moe/grouped_fp8_blockwise_moe.py:143-190):
 * 0 (default) = K steps of 128 bytes, 16x16x128 products promoted with one fma per accumulator and scale block,
 * two 65 KB ring slots; 1 = K steps of 64 bytes, 32x32x64 products accumulated in place in units of the current
 * block's scale, four 33 KB ring slots (three K-steps in flight), taken for K >= 256 and the other kernel
 * otherwise; its epilogue stores whole row segments through per-wave LDS patches; 2 = the same kernel with plain
 * per-lane stores (for comparison; same bits as 1).  Results of 0 and 1 differ in rounding only.  Token and
 * weight scales must be positive for 1 and 2.  Process-wide; not meant to be switched while launches are being
 * enqueued from another thread. */
int bgmoe_set_tiled_variant(int variant);

/* Workspace of the balanced form of the weight-streaming grouped GEMM (no reference counterpart).  A decode launch
 * has a few hundred work items of 0.25-1.8 MB for ~512 resident blocks, so whole items leave CUs idle; the
 * balanced form cuts the sequence of all items' K-blocks into one equal share per block, streams each share
 * without a gap across item boundaries, and finishes an item that was cut over several blocks in the block that
 * arrives last (fp32 partial sums in this workspace, added in block order; no block waits for another).  A cut
 * item's K-chain is summed in as many pieces as it was cut into, so its last bits depend on the group sizes of the
 * launch (never on timing).  Layout: 4096 bytes of counters (zero before the first use, left zero by every launch)
 * followed by the partial-sum slots. */
size_t bgmoe_fp8_streamk_workspace_bytes(void);
/* Tuning aid: with a device buffer of 4 * 1024 uint64 set, every share (block) of the following balanced launches
 * records the constant-rate clock (100 MHz) at its start, before its first unit, at the end of its stream and at its
 * end, at [4 * share .. 4 * share + 3].  NULL switches it off. */
int bgmoe_debug_streamk_trace(uint64_t* device_buffer);
/* Tuning knob: relative sizes of the shares of XCD 0..7 (8 ints, each in [1, 64], their sum at most 32 times the
 * smallest, so that the lightest share still holds a whole unit of work; default 23/21 alternating: on MI355X
 * the odd XCDs were measured to stream about 9% slower than the even ones). */
int bgmoe_set_streamk_xcd_weights(const int* weights);
/* Debug aid: copies the device's sticky status word of the balanced launches to *host_out and clears it
 * (synchronises the device; not for the hot path).  Bit 0: a share of some launch found no unit of work, which
 * the share arithmetic rules out for accepted XCD weights; rows of the items that spanned it would be stale. */
int bgmoe_debug_streamk_status(int32_t* host_out);

/* bgmoe_fp8_grouped_gemm / bgmoe_fp8_fused_s1 (same operands, outputs and checks) in the balanced form when it
 * applies: tile-major weights, workspace of bgmoe_fp8_streamk_workspace_bytes() bytes, and max_group_rows -- the
 * caller's bound on the rows of any one group (a decode batch: the number of tokens) -- within the streaming
 * kernel's row limit.  Otherwise (max_group_rows 0 = unknown, row-major weights, NULL workspace) they are the plain
 * calls.  No reference counterpart: the reference's ops take no workspace (fp8_blockwise_gemm.cu:564-900). */
int bgmoe_fp8_grouped_gemm_balanced(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* b, const int32_t* seqlens,
                                    const int32_t* cu_seqlens, int groups, int64_t m, int n, int k, uint16_t* out,
                                    int64_t max_group_rows, void* workspace, size_t workspace_bytes,
                                    bgmoe_stream_t stream);
int bgmoe_fp8_fused_s1_balanced(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* gate, const bgmoe_fp8_weight* up,
                                const int32_t* seqlens, const int32_t* cu_seqlens, int groups, int64_t m, int n, int k,
                                uint16_t* out, uint8_t* out_q, float* out_scale, int64_t out_scale_row_stride,
                                int64_t out_scale_nb_stride, int64_t max_group_rows, void* workspace,
                                size_t workspace_bytes, bgmoe_stream_t stream);

/* Tuning knob (no reference counterpart): groups with at most `rows` rows are served by the
 * weight-streaming kernel, larger ones by the LDS-tiled kernel.  0 sends everything to the tiled
 * kernel.  Default 256 (or the environment variable BGMOE_SKINNY_MAX_ROWS at first use).
 * Results do not depend on it beyond fp32 summation order. */
int bgmoe_set_skinny_max_rows(int rows);

/* Stage 1 of the weight-streaming kernel with tall work items (process-wide, opt-in; no counterpart in the reference).
 * Groups with more than `rows` rows are cut into 64-row items instead of 32-row items, so that their weights are
 * passed over half as often (a 256-row shared expert folded into a decode step: 4 passes instead of 8); the other
 * groups keep the 32-row items and their three-stage prefetch.  rows = 0 (the default) turns it off; otherwise
 * rows >= 32.  Every output element is computed by the same chain of operations either way: the results are the
 * same bits.  Returns BGMOE_OK or BGMOE_ERR_ARG. */
int bgmoe_set_skinny_tall_min_rows(int rows);

/* Prefetch depth of the plain weight-streaming grouped GEMM, the down projection of a decode step (process-wide,
 * opt-in; no counterpart in the reference).  stages = 2 (the default): an item loads one K-block ahead of the one it
 * computes; 3, 4 or 6: two, three or five ahead, i.e. as many times the weight bytes in flight per block (the kernel
 * keeps three blocks per CU with 3 stages, two with 4 or 6; bgmoe_fp8_dense_gemm takes 6 as 4).  Every output element is computed by the same chain of operations
 * whatever the depth: the results are the same bits.  The block-split form of bgmoe_fp8_dense_gemm follows the switch
 * (its 128-row chunks take three stages at most).  Fused stage 1 is not affected (its three stages fill the register file).  Returns BGMOE_OK or
 * BGMOE_ERR_ARG. */
int bgmoe_set_skinny_gemm_stages(int stages);

/* Prefetch depth of fused stage 1 of the weight-streaming kernel (process-wide, opt-in; no counterpart in the
 * reference).  stages = 3 (the default): an item loads two K-blocks ahead of the one it computes; 4: three ahead (half
 * again the weight bytes in flight per block, at the same two blocks per CU).  Same chain of operations per output
 * element, same bits.  With tall items switched on (bgmoe_set_skinny_tall_min_rows) their form is used instead.
 * Returns BGMOE_OK or BGMOE_ERR_ARG. */
int bgmoe_set_skinny_s1_stages(int stages);

/* Fused stage 1: out = bf16( silu(X*Wg^T) * (X*Wu^T) ), fp32 gate and up.
 * Replaces `fp8_blockwise_fused_s1` / `_ptrs`
 * (grouped_fp8_blockwise_moe.py:423-560, fp8_blockwise_s1_kernel.cuh:425-607).
 * If out_q != NULL the bf16 result is quantised in the epilogue (act-quant of
 * each row's 128-blocks) into out_q [m,n] bytes + out_scale (strided), and
 * `out` may be NULL: this replaces the S1 -> `act_quant_ragged` pair
 * (batchgen/models/glm/glm5/model.py:2560-2573) bit for bit. */
int bgmoe_fp8_fused_s1(const bgmoe_fp8_act* a, const bgmoe_fp8_weight* gate,
                       const bgmoe_fp8_weight* up, const int32_t* seqlens,
                       const int32_t* cu_seqlens, int groups, int64_t m, int n, int k,
                       uint16_t* out, uint8_t* out_q, float* out_scale,
                       int64_t out_scale_row_stride, int64_t out_scale_nb_stride,
                       bgmoe_stream_t stream);

/* ------------------------------------------------------- MXFP4 (W4A16) GEMM */

/* MXFP4 weights: e2m1 values packed two per byte (low nibble = even K), one e8m0 scale byte per 32
 * consecutive K, scale = 2^(byte-127) (batchgen/moe/mxfp4_oracle_vector.py:48-115).
 * ROW_MAJOR: packed [n, k/2], scales [n, k/32] (the checkpoint layout,
 * batchgen/models/moonshotai/kimi_linear/k3/mxfp4_expert.py:239-285).
 * TILE_MAJOR: per (16 rows x 128 K) tile, 1024 packed bytes in wave-lane order and 64 scale bytes
 * [row][4]; produced by bgmoe_mxfp4_weight_repack.  It plays the role of the reference's Marlin
 * repack (batchgen/moe/fused_moe_mxfp4_resident.py:13-15), whose NVIDIA register layout is not
 * reproduced. */
typedef struct bgmoe_mxfp4_weight {
  const uint8_t* w;               /* [groups, ...] packed values                 */
  int64_t w_group_stride;         /* bytes between groups (n*k/2)               */
  const uint8_t* const* w_ptrs;   /* device table or NULL                       */
  const uint8_t* scale;           /* [groups, ...] e8m0 bytes                   */
  int64_t scale_group_stride;     /* bytes between groups (n*k/32)              */
  const uint8_t* const* scale_ptrs;
  int32_t layout;
  int32_t reserved;
} bgmoe_mxfp4_weight;

int bgmoe_mxfp4_weight_repack(const uint8_t* w_packed, const uint8_t* scales, uint8_t* w_out,
                              uint8_t* scales_out, int groups, int n, int k, bgmoe_stream_t stream);

/* out[r, :] = bf16( x[r, :] (bf16) * dequant(W[g])^T ), fp32 accumulation, for rows of group g.
 * Replaces `marlin_grouped_m16_mxfp4` (batchgen/moe/marlin_grouped_moe.py:476-543,
 * batchgen_kernels/src/moe/marlin_grouped_gemm.cu).  row_bound: host-side upper bound on the live
 * rows (0 = m); groups with more than 32 rows stream their weights once per 32-row chunk.
 * Output: row r of x -> row r of `out`, or, when out_ptrs (device table, the reference's C_ptrs)
 * is given, token t of group g -> out_ptrs[g] + t*n. */
int bgmoe_mxfp4_grouped_gemm(const uint16_t* x, const bgmoe_mxfp4_weight* w, const int32_t* seqlens,
                             const int32_t* cu_seqlens, int groups, int64_t m, int n, int k,
                             uint16_t* out, uint16_t* const* out_ptrs, int64_t row_bound,
                             bgmoe_stream_t stream);

/* Stage-1 activations.  SWIGLU: out = bf16( silu(g) * u ) on the fp32 accumulators (the benchmark's
 * Kimi-K3-shaped config).  SITU: the Kimi-K3 model's own activation, with the constants the reference
 * kernel compiles in (batchgen_kernels/src/moe/marlin_grouped_gemm.cu:243-256; asserted against the
 * config at kimi_linear/k3/mxfp4_expert.py:302-312): g and u are rounded to bf16 first (:1055-1069), then
 *   out = bf16( 4*tanh(g/4)*sigmoid(g) * 25*tanh(u/25) )   in fp32. */
enum { BGMOE_ACT_SWIGLU = 0, BGMOE_ACT_SITU = 1 };

/* out = act(x Wg^T, x Wu^T).  Replaces `marlin_grouped_stage1_fused_mxfp4_situ`
 * (batchgen/moe/marlin_grouped_moe.py:411-470) with activation = BGMOE_ACT_SITU. */
int bgmoe_mxfp4_fused_s1(const uint16_t* x, const bgmoe_mxfp4_weight* gate,
                         const bgmoe_mxfp4_weight* up, const int32_t* seqlens,
                         const int32_t* cu_seqlens, int groups, int64_t m, int n, int k, uint16_t* out,
                         uint16_t* const* out_ptrs, int activation, int64_t row_bound,
                         bgmoe_stream_t stream);

/* The same with the rows read where the tokens lie (no counterpart in the reference, whose dispatch always copies
 * the rows into the expert-major buffer first): x_tokens is the [n_tokens, k] token matrix, and row r of group g
 * (r in [cu_seqlens[g], cu_seqlens[g] + seqlens[g])) is token row_pair[r] / top_k -- row_pair as written by
 * bgmoe_dispatch_index_3d.  A token index is clamped to n_tokens - 1, so that no map entry can make the kernel read
 * outside x_tokens; n_tokens * k * 2 must not exceed 4 GiB.  Same results as bgmoe_mxfp4_fused_s1 on the gathered rows. */
int bgmoe_mxfp4_fused_s1_gather(const uint16_t* x_tokens, int64_t n_tokens, const int32_t* row_pair, int top_k,
                                const bgmoe_mxfp4_weight* gate, const bgmoe_mxfp4_weight* up, const int32_t* seqlens,
                                const int32_t* cu_seqlens, int groups, int64_t m, int n, int k, uint16_t* out,
                                uint16_t* const* out_ptrs, int activation, int64_t row_bound, bgmoe_stream_t stream);

/* Which shape of the MXFP4 weight-streaming kernel serves the calls above (process-wide, opt-in; no counterpart in
 * the reference): 0 = 64-row work items with a three-stage weight prefetch (the default), 1 = 32-row items with a
 * six-stage prefetch (2.5 times the weight bytes in flight per wave, groups above 32 rows pass over their weights
 * once per 32 rows), 2 = the item height chosen per group on the device, in one launch: groups of at most 32 rows as
 * 32-row items with a five-stage prefetch, larger groups as 64-row items with three stages (the 64-row items'
 * accumulators and the 32-row items' stages share the register file, hence five), 3 = the default's 64-row items with a
 * four-stage prefetch (a 64 KB token ring).  Every output element is computed by
 * the same chain of operations: same bits.  Returns BGMOE_OK or BGMOE_ERR_ARG. */
int bgmoe_set_mxfp4_variant(int variant);

/* DeepGEMM's contiguous m-grouped API describes the rows by a map `grouped_layout` [m] (row -> group, -1 on
 * alignment padding; batchgen/moe/grouped_fp8_deepgemm_moe.py:9-22, built by `build_grouped_layout`, :118-186).
 * This call turns the map into what the grouped GEMMs here take: starts[g] = first row of group g (starts has
 * groups + 1 entries, the last one m) and seqlens[g] = its live rows (0 for a group without rows).  Each group
 * must own ONE contiguous run of rows; *status (optional, device) is set to 0, or to 1 for a group index
 * >= groups and 2 for a group with two runs, in which case every seqlens entry is 0 and the GEMM that follows
 * does nothing.  One small launch, no host synchronisation. */
int bgmoe_layout_to_segments(const int32_t* grouped_layout, int64_t m, int groups, int32_t* seqlens,
                             int32_t* starts, int32_t* status, bgmoe_stream_t stream);

/* ---------------------------------------------------------------- self-check */

/* The routers' sigmoid is the correctly rounded fp32 one (fp64 evaluation rounded once: the reference
 * compiles its gate with fast-math, batchgen_kernels/setup.py:245, so its own `1/(1+expf(-x))`,
 * gate_sigmoid_topk.cu:88, is not a reproducible function).  The kernels take a short fp64 evaluation when
 * it provably rounds the same way and the library evaluation otherwise; this call runs both on the `count`
 * float bit patterns starting at `first_bits` and adds the number of inputs whose results differ in any bit
 * to *mismatches (device memory, caller-zeroed; 0 is the only acceptable value) and, when fallbacks is not
 * NULL, the number of inputs the short evaluation hands to the library one to *fallbacks.  No counterpart
 * in the reference. */
int bgmoe_selfcheck_sigmoid(uint32_t first_bits, uint64_t count, uint64_t* mismatches, uint64_t* fallbacks,
                            bgmoe_stream_t stream);

/* The quantisers divide by the block scale exactly as IEEE fp32 division does (the reference's forms A-D
 * all use a true division or `x * (1/s)`; see bgmoe_act_quant_rows) but compute the quotient as
 * q0 = x*r, e = fma(-q0, s, x), q = fma(e, r, q0) with r = 1/s once per block.  This call draws `count`
 * pseudo-random (s, x) pairs from the quantisers' domain (s in (1e-30, 1e30), |x| <= 448.5 s, x fp32 or
 * bf16, signed zeros) and adds to *byte_mismatches the pairs whose e4m3 byte differs between the two
 * divisions and to *bit_mismatches those whose normal-range quotients differ in any bit (device memory,
 * caller-zeroed; both must stay 0).  No counterpart in the reference. */
int bgmoe_selfcheck_scale_division(uint64_t seed, uint64_t count, uint64_t* byte_mismatches,
                                   uint64_t* bit_mismatches, bgmoe_stream_t stream);

/* ------------------------------------------------- Kimi-K3 latent-MoE seam */

/* out[r, c] = bf16( beta*tanh(g/beta)*sigmoid(g) * u' ),  g = x[r, c], u = x[r, d + c] (bf16 -> fp32),
 * u' = linear_beta*tanh(u/linear_beta) when linear_beta > 0, else u.  One rounding, to bf16.
 * Replaces `situ_and_mul_triton` (batchgen/models/moonshotai/kimi_linear/situ_triton.py:55-77), the
 * activation of the Kimi-K3 shared expert and dense MLP (`SituAndMul`, kimi_linear/model.py:84-115).
 * x is [rows, 2d] with row stride x_row_stride (elements), out [rows, d] with out_row_stride. */
int bgmoe_situ_and_mul(const uint16_t* x, int64_t rows, int d, int64_t x_row_stride, float beta,
                       float linear_beta, uint16_t* out, int64_t out_row_stride, bgmoe_stream_t stream);

/* out[r, c] = bf16( bf16(silu(g)) * u ): PyTorch's `F.silu(gate) * up` on bf16 tensors (the SwiGLU of a bf16 shared
 * expert, batchgen/moe/fused_moe_mxfp4_resident.py:905-944), same layout and strides as above. */
int bgmoe_silu_and_mul(const uint16_t* x, int64_t rows, int d, int64_t x_row_stride, uint16_t* out,
                       int64_t out_row_stride, bgmoe_stream_t stream);

/* out[r, :] = bf16( x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * weight ): fp32 math, one rounding.
 * Replaces `triton_rmsnorm` / `cuda_rmsnorm` as used by `KimiRMSNorm.forward`
 * (batchgen/models/moonshotai/kimi_linear/rmsnorm_triton.py:24-44, kimi_linear/model.py:192-205): the norm
 * between the combined latent rows and the latent -> hidden projection.  The sum of squares follows the
 * same fixed tree as bgmoe_add_rmsnorm_fp8_quant and the reciprocal square root is the correctly rounded
 * one.  h a multiple of 8, at most 8192; x, weight and out bf16, 16-byte aligned; out may alias x. */
int bgmoe_rmsnorm(const uint16_t* x, const uint16_t* weight, int64_t rows, int h, float eps, uint16_t* out,
                  bgmoe_stream_t stream);

/* ------------------------------------------------------------ whole layer */

/* One FP8 MoE layer forward on one GPU's share of the experts:
 *   router (sigmoid + bias, group-limited when n_group > 1, else ungrouped)
 *   -> stable permute into the masked [E_l, max_tokens, H] layout (layout 0) or
 *      the contiguous ragged layout (layout 1, starts aligned to row_align)
 *   -> act-quant fused into the scatter -> fused gate_up/SwiGLU/requant GEMM
 *   -> down GEMM -> top-k weighted combine + shared expert -> out [n,h] bf16.
 * Replaces the op sequence of `WGMMAMoEBuffers.forward`
 * (batchgen/moe/fp8_wgmma_pipeline.py:294-372) plus the gate and shared expert
 * of `DeepseekV3MoE_Decoding_FP8.forward`
 * (batchgen/models/deepseek/deepseekv3/modeling_deepseek_v3.py:1924-1940).
 * Every buffer is caller-owned; nothing is allocated and nothing is read back.
 *
 * Row space of xq/xs/hq/hs/y: [0, cap_rows) routed rows, then n rows of the
 * shared expert (identity permutation) when has_shared.
 *   masked: cap_rows = e_local*max_tokens; ragged: cap_rows >= worst case of
 *   bgmoe_dispatch_scatter_ragged.
 * Weights: routed = groups [0,e_local).  shared_folded != 0: gate/up/down are
 * pointer tables with e_local+1 entries, entry e_local being the shared expert
 * (same inter), and all experts run in one grouped launch.  Otherwise the
 * shared expert comes in sh_* (1 group) and runs as launches of its own. */
typedef struct bgmoe_moe_fp8_layer {
  int32_t n, h, inter, e_total, e_local, expert_start;
  int32_t top_k, n_group, topk_group;
  float routed_scaling_factor;
  int32_t layout, max_tokens, row_align;
  int32_t has_shared, shared_folded, shared_inter, shared_mode;
  int64_t cap_rows;
  const uint16_t* x;          /* [n,h] bf16            */
  const float* logits;        /* [n,e_total] fp32      */
  const float* bias;          /* [e_total] fp32        */
  bgmoe_fp8_weight gate, up, down;
  bgmoe_fp8_weight sh_gate, sh_up, sh_down;
  int32_t* topk_ids;          /* [n,top_k]             */
  float* topk_weights;        /* [n,top_k]             */
  int32_t* expert_counts;     /* [e_local+1]           */
  int32_t* cu_seqlens;        /* [e_local+2]           */
  int32_t* topk_pos;          /* [n*top_k]             */
  uint8_t* xq;                /* [rows,h]              */
  float* xs;                  /* [rows,h/128]          */
  uint8_t* hq;                /* [rows,inter]          */
  float* hs;                  /* [rows,inter/128]      */
  uint8_t* shq;               /* [n,shared_inter]  (unfolded shared only) */
  float* shs;                 /* [n,shared_inter/128]                     */
  uint16_t* y;                /* [rows,h] bf16         */
  void* workspace;            /* bgmoe_dispatch_workspace_bytes(n*top_k, e_local) */
  size_t workspace_bytes;
  uint16_t* out;              /* [n,h] bf16            */
  /* Optional upstream fusions; all NULL/0 = the plain layer above.
   * x_fp8/x_scale: the tokens already quantised (bgmoe_add_rmsnorm_fp8_quant): step 3 copies them instead
   * of quantising x (x may then be NULL).  Scale (t,kb) at x_scale[t*x_scale_row_stride + kb*x_scale_kb_stride].
   * router_weight: bf16 [e_total,h]; with logits == NULL the layer computes them itself from
   * router_hidden (bf16 [n,h]; NULL = x) with bgmoe_router_gemm_gate, and needs router_workspace of
   * bgmoe_router_gemm_workspace_bytes(n,h,e_total) bytes. */
  const uint8_t* x_fp8;
  const float* x_scale;
  int64_t x_scale_row_stride, x_scale_kb_stride;
  const uint16_t* router_weight;
  const uint16_t* router_hidden;
  void* router_workspace;
  size_t router_workspace_bytes;
  /* non-zero: the routes are given -- topk_ids [n,top_k] and topk_weights [n,top_k] are INPUTS, the router is
   * skipped and logits / router_weight are not read (the form of `WGMMAMoEBuffers.forward(layer_id, global_x,
   * topk_idx, topk_weight)`, batchgen/moe/fp8_wgmma_pipeline.py:294-372).  Ids outside the local expert range
   * (and -1) contribute nothing.  BGMOE_ROUTES_GIVEN: a row of topk_ids may name one expert several times (a
   * group is then bounded by n*top_k rows only).  BGMOE_ROUTES_GIVEN_DISTINCT: the caller promises that the ids
   * of a row are pairwise different, as every top-k gate's are: a group then holds at most n rows, and a decode
   * batch keeps the weight-streaming kernels it would get with the layer's own router.  A broken promise loses
   * no row and touches no memory outside the buffers (groups above the streaming limit are then served by the
   * tiled kernel only when one is launched, i.e. their rows may be left uncomputed): it is the caller's bug. */
  int32_t routes_given;
  /* Optional: bgmoe_fp8_streamk_workspace_bytes() bytes, 16-byte aligned, its first 4096 bytes zero before the
   * first call (every call leaves them zero).  With it, a batch in which no group can exceed the streaming
   * kernel's row limit (n <= 256) runs both grouped GEMMs in their balanced form (see
   * bgmoe_fp8_streamk_workspace_bytes); NULL / 0 = the item-per-block form.  One workspace per stream: calls that
   * overlap on one workspace race. */
  void* gemm_workspace;
  size_t gemm_workspace_bytes;
} bgmoe_moe_fp8_layer;

enum { BGMOE_ROUTES_GIVEN = 1, BGMOE_ROUTES_GIVEN_DISTINCT = 2 };
int bgmoe_moe_fp8_layer_forward(const bgmoe_moe_fp8_layer* layer, bgmoe_stream_t stream);

/* One MXFP4 (W4A16) MoE layer forward on one GPU's share of the experts, masked layout:
 *   ungrouped sigmoid top-k -> masked dispatch of bf16 rows -> MXFP4 gate_up + SwiGLU -> MXFP4 down ->
 *   weighted combine (+ the shared expert's output, computed by the caller: a dense bf16 MLP).
 * Mirrors `ResidentEPMXFP4MoELayer._expert_path` / `forward`
 * (batchgen/moe/fused_moe_mxfp4_resident.py:709-944) without its collectives and latent projections.
 * stages: BGMOE_MXFP4_ROUTED runs everything up to the down projection, BGMOE_MXFP4_COMBINE the combine,
 * their sum both -- so that a caller can run the shared expert on another stream beside the routed part
 * and join before the combine.  All buffers caller-owned; capturable. */
enum { BGMOE_MXFP4_ROUTED = 1, BGMOE_MXFP4_COMBINE = 2 };
typedef struct bgmoe_moe_mxfp4_layer {
  int32_t n, h, inter, e_total, e_local, expert_start, top_k, max_tokens;
  float routed_scaling_factor;
  int32_t shared_mode;            /* as bgmoe_reduce_weighted_scatter                        */
  const uint16_t* x;              /* [n,h] bf16                                               */
  const float* logits;            /* [n,e_total] fp32                                         */
  const float* bias;              /* [e_total] fp32                                           */
  bgmoe_mxfp4_weight gate, up, down;
  int32_t* topk_ids;              /* [n,top_k]                                                */
  float* topk_weights;            /* [n,top_k]                                                */
  int32_t* expert_counts;         /* [e_local]                                                */
  int32_t* expert_counters;       /* [e_local]                                                */
  const int32_t* cu_seqlens;      /* [e_local+1], cu[e] = e*max_tokens (filled by the caller) */
  int32_t* topk_pos;              /* [n*top_k]                                                */
  uint16_t* act;                  /* [e_local*max_tokens, h] bf16                             */
  uint16_t* hmid;                 /* [e_local*max_tokens, inter] bf16                         */
  uint16_t* y;                    /* [e_local*max_tokens, h] bf16                             */
  void* workspace;                /* bgmoe_dispatch_workspace_bytes(n*top_k, e_local)         */
  size_t workspace_bytes;
  const uint16_t* shared_out;     /* [n,h] bf16 or NULL                                       */
  uint16_t* out;                  /* [n,h] bf16                                               */
  int32_t activation;             /* BGMOE_ACT_SWIGLU or BGMOE_ACT_SITU                       */
  int32_t* row_pair;              /* NULL, or [e_local*max_tokens]: the dispatch only computes indices (this row ->
                                   * pair map included) and stage 1 reads its rows from x through the map; `act`
                                   * is then unused and may be NULL.  Same results.               */
} bgmoe_moe_mxfp4_layer;

int bgmoe_moe_mxfp4_layer_forward(const bgmoe_moe_mxfp4_layer* layer, int stages, bgmoe_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* BGMOE_H */
