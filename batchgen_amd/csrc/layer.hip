// Whole-layer driver: chains the kernels of one FP8 MoE layer on one stream
// with caller-owned buffers, no allocation and no device->host reads, so the
// sequence can be captured in a HIP graph.
#include "bgmoe_common.h"

extern "C" int bgmoe_moe_fp8_layer_forward(const bgmoe_moe_fp8_layer* L, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(L != nullptr, "moe_fp8_layer_forward: null layer");
  const int n = L->n, h = L->h, inter = L->inter, el = L->e_local, k = L->top_k;
  BGMOE_REQUIRE(n >= 0 && h > 0 && inter > 0 && el > 0 && k > 0, "moe_fp8_layer_forward: bad sizes");
  BGMOE_REQUIRE(h % 128 == 0 && inter % 128 == 0, "moe_fp8_layer_forward: H=%d and I=%d must be multiples of 128", h, inter);
  BGMOE_REQUIRE(L->layout == 0 || L->layout == 1, "moe_fp8_layer_forward: layout must be 0 (masked) or 1 (ragged)");
  BGMOE_REQUIRE(L->layout == 1 || L->max_tokens > 0, "moe_fp8_layer_forward: masked layout needs max_tokens");
  BGMOE_REQUIRE(L->layout == 0 || (L->row_align > 0 && (L->row_align & (L->row_align - 1)) == 0),
                "moe_fp8_layer_forward: row_align must be a positive power of two");
  const int64_t nk = (int64_t)n * k;
  int64_t need_rows;
  if (L->layout == 0) {
    need_rows = (int64_t)el * L->max_tokens;
  } else {
    const int64_t a = L->row_align;
    need_rows = (nk + (a - 1) * (nk < el ? nk : el)) / a * a;
  }
  BGMOE_REQUIRE(L->cap_rows >= need_rows, "moe_fp8_layer_forward: cap_rows=%lld < %lld rows needed",
                (long long)L->cap_rows, (long long)need_rows);
  BGMOE_REQUIRE(L->cap_rows + n <= 2147483647LL, "moe_fp8_layer_forward: row space exceeds int32");
  if (n == 0) return BGMOE_OK;
  const bool pre_quant = L->x_fp8 != nullptr;
  const bool routed = L->routes_given != 0;
  const bool own_logits = !routed && L->logits == nullptr;
  BGMOE_REQUIRE(L->bias && L->out, "moe_fp8_layer_forward: null input/output");
  BGMOE_REQUIRE(pre_quant ? L->x_scale != nullptr : L->x != nullptr,
                "moe_fp8_layer_forward: needs x, or x_fp8 together with x_scale");
  BGMOE_REQUIRE(!own_logits || (L->router_weight && (L->router_hidden || L->x)),
                "moe_fp8_layer_forward: without logits the layer needs router_weight and bf16 hidden states");
  BGMOE_REQUIRE(L->topk_ids && L->topk_weights && L->expert_counts && L->cu_seqlens && L->topk_pos &&
                L->xq && L->xs && L->hq && L->hs && L->y, "moe_fp8_layer_forward: null buffer");
  const bool shared = L->has_shared != 0;
  const bool folded = shared && L->shared_folded != 0;
  BGMOE_REQUIRE(!folded || L->shared_inter == inter, "moe_fp8_layer_forward: a folded shared expert needs shared_inter == inter");
  BGMOE_REQUIRE(!folded || (L->gate.w_ptrs && L->up.w_ptrs && L->down.w_ptrs),
                "moe_fp8_layer_forward: a folded shared expert needs pointer-table weights");
  BGMOE_REQUIRE(!shared || folded || (L->shq && L->shs), "moe_fp8_layer_forward: null shared-expert buffer");
  hipStream_t st = bgmoe_stream(stream);
  int rc;

  // 1. router (from logits, or from the hidden states through the router GEMM), unless the routes are given
  if (routed) {
    rc = BGMOE_OK;
  } else if (own_logits) {
    const bool grouped = L->n_group > 1;
    rc = bgmoe_router_gemm_gate(L->router_hidden ? L->router_hidden : L->x, L->router_weight, L->bias, n, h,
                                L->e_total, grouped ? L->n_group : 0, grouped ? L->topk_group : 0, k,
                                L->routed_scaling_factor, L->topk_ids, L->topk_weights, nullptr, 0,
                                L->router_workspace, L->router_workspace_bytes, stream);
  } else if (L->n_group > 1) {
    rc = bgmoe_fused_gate(L->logits, L->bias, n, L->e_total, L->n_group, L->topk_group, k,
                          L->routed_scaling_factor, 1, L->topk_ids, L->topk_weights, stream);
  } else {
    rc = bgmoe_gate_sigmoid_topk(L->logits, L->e_total, L->bias, n, L->e_total, k, L->routed_scaling_factor,
                                 L->topk_ids, 0, L->topk_weights, nullptr, nullptr, 0, nullptr, 0, 0, stream);
  }
  if (rc != BGMOE_OK) return rc;

  // 2 + 3. stable counting sort -> counts, cu_seqlens (+ the shared expert as one more group), topk_pos; quantise
  // while scattering (the shared expert's rows are the tokens themselves).  One launch for a decode-sized batch,
  // two otherwise.
  const int hb = h / 128, ib = inter / 128;
  rc = BGMOE_ERR_WORKSPACE;
  if (!pre_quant)
    rc = bgmoe_internal_dispatch_scatter_quant(L->topk_ids, n, k, h, L->expert_start, el,
                                               L->layout == 0 ? L->max_tokens : 0, L->layout == 0 ? 1 : L->row_align,
                                               L->expert_counts, nullptr, L->cu_seqlens, L->topk_pos, shared ? n : 0,
                                               L->cap_rows, L->x, L->xq, L->xs, hb, 1, st);
  if (rc == BGMOE_ERR_WORKSPACE) {
    rc = bgmoe_internal_dispatch_index(L->topk_ids, nk, L->expert_start, el, L->layout == 0 ? L->max_tokens : 0,
                                       L->layout == 0 ? 1 : L->row_align, L->expert_counts, nullptr,
                                       L->cu_seqlens, L->topk_pos, shared ? n : 0, L->cap_rows, L->workspace,
                                       L->workspace_bytes, st);
    if (rc != BGMOE_OK) return rc;
    if (pre_quant)
      rc = bgmoe_internal_scatter_fp8(L->x_fp8, L->x_scale, L->x_scale_row_stride, L->x_scale_kb_stride,
                                      L->topk_pos, n, k, h, L->xq, L->xs, hb, 1, shared ? n : 0, L->cap_rows, st);
    else
      rc = bgmoe_internal_scatter_quant(L->x, L->topk_pos, n, k, h, L->xq, L->xs, hb, 1, shared ? n : 0,
                                        L->cap_rows, st);
  }
  if (rc != BGMOE_OK) return rc;

  // 4/5. gate_up + SwiGLU + requant, then down
  const int64_t rows = L->cap_rows + (shared ? n : 0);
  const int groups = el + (folded ? 1 : 0);
  bgmoe_fp8_act ax{L->xq, L->xs, hb, 1};
  const int64_t live_bound = nk + (folded ? n : 0);       // rows that can be live in one pass
  // Rows one group can have: the router picks distinct experts per token, so at most n; routes handed in from
  // outside may name one expert several times in a token's row, so only n*k bounds them unless the caller
  // vouches for distinct ids (a top-k gate of its own).
  const int64_t group_bound = routed && L->routes_given != BGMOE_ROUTES_GIVEN_DISTINCT ? nk : n;
  rc = bgmoe_internal_fp8_gemm(&ax, &L->gate, &L->up, L->expert_counts, L->cu_seqlens, groups,
                               folded ? rows : L->cap_rows, inter, h, nullptr, L->hq, L->hs, ib, 1, live_bound, group_bound,
                               L->gemm_workspace, L->gemm_workspace_bytes, st);
  if (rc != BGMOE_OK) return rc;
  bgmoe_fp8_act ah{L->hq, L->hs, ib, 1};
  rc = bgmoe_internal_fp8_gemm(&ah, &L->down, nullptr, L->expert_counts, L->cu_seqlens, groups,
                               folded ? rows : L->cap_rows, h, inter, L->y, nullptr, nullptr, 0, 0, live_bound, group_bound,
                               L->gemm_workspace, L->gemm_workspace_bytes, st);
  if (rc != BGMOE_OK) return rc;
  if (shared && !folded) {
    const int si = L->shared_inter;
    BGMOE_REQUIRE(si > 0 && si % 128 == 0, "moe_fp8_layer_forward: shared_inter=%d must be a multiple of 128", si);
    // Group `el` of expert_counts / cu_seqlens describes the shared rows (n rows starting at
    // cap_rows).  shq/shs hold only those n rows, so their base pointers are shifted back by
    // cap_rows rows: the kernels address row cu_seqlens[el] + t.
    const int32_t* cnt1 = L->expert_counts + el;
    bgmoe_fp8_act sx0{L->xq, L->xs, hb, 1};
    rc = bgmoe_fp8_fused_s1(&sx0, &L->sh_gate, &L->sh_up, cnt1, L->cu_seqlens + el, 1, rows, si, h, nullptr,
                            L->shq - L->cap_rows * si, L->shs - L->cap_rows * (si / 128), si / 128, 1, stream);
    if (rc != BGMOE_OK) return rc;
    bgmoe_fp8_act sh{L->shq - L->cap_rows * si, L->shs - L->cap_rows * (si / 128), si / 128, 1};
    rc = bgmoe_fp8_grouped_gemm(&sh, &L->sh_down, cnt1, L->cu_seqlens + el, 1, rows, h, si, L->y, stream);
    if (rc != BGMOE_OK) return rc;
  }

  // 6. weighted combine + shared expert
  return bgmoe_reduce_weighted_scatter(L->y, L->topk_pos, L->topk_weights, n, h, k, L->out, -1,
                                       shared ? L->y + L->cap_rows * h : nullptr, L->shared_mode, stream);
}

extern "C" int bgmoe_moe_mxfp4_layer_forward(const bgmoe_moe_mxfp4_layer* L, int stages, bgmoe_stream_t stream) {
  BGMOE_REQUIRE(L != nullptr, "moe_mxfp4_layer_forward: null layer");
  BGMOE_REQUIRE(stages >= 1 && stages <= 3, "moe_mxfp4_layer_forward: stages must be ROUTED, COMBINE or both");
  const int n = L->n, h = L->h, inter = L->inter, el = L->e_local, k = L->top_k;
  BGMOE_REQUIRE(n >= 0 && h > 0 && inter > 0 && el > 0 && k > 0 && L->max_tokens > 0,
                "moe_mxfp4_layer_forward: bad sizes");
  if (n == 0) return BGMOE_OK;
  BGMOE_REQUIRE(L->topk_weights && L->topk_pos && L->y && L->out, "moe_mxfp4_layer_forward: null buffer");
  const int64_t rows = (int64_t)el * L->max_tokens;
  int rc;
  if (stages & BGMOE_MXFP4_ROUTED) {
    BGMOE_REQUIRE(L->x && L->logits && L->bias && L->topk_ids && L->expert_counts && L->expert_counters &&
                  L->cu_seqlens && (L->act || L->row_pair) && L->hmid, "moe_mxfp4_layer_forward: null input or buffer");
    rc = bgmoe_gate_sigmoid_topk(L->logits, L->e_total, L->bias, n, L->e_total, k, L->routed_scaling_factor,
                                 L->topk_ids, 0, L->topk_weights, nullptr, nullptr, 0, nullptr, 0, 0, stream);
    if (rc != BGMOE_OK) return rc;
    const int64_t bound = (int64_t)n * k;
    if (L->row_pair != nullptr) {
      // indices only; stage 1 reads each row from its token through the row -> pair map
      rc = bgmoe_dispatch_index_3d(L->topk_ids, n, k, L->expert_start, el, L->max_tokens, L->expert_counts,
                                   L->expert_counters, L->topk_pos, L->row_pair, L->workspace, L->workspace_bytes,
                                   stream);
      if (rc != BGMOE_OK) return rc;
      rc = bgmoe_mxfp4_fused_s1_gather(L->x, n, L->row_pair, k, &L->gate, &L->up, L->expert_counts, L->cu_seqlens,
                                       el, rows, inter, h, L->hmid, nullptr, L->activation, bound, stream);
    } else {
      rc = bgmoe_dispatch_scatter_3d(L->x, L->topk_ids, n, k, h, L->act, L->expert_start, el, L->max_tokens,
                                     L->expert_counts, L->expert_counters, L->topk_pos, L->workspace,
                                     L->workspace_bytes, stream);
      if (rc != BGMOE_OK) return rc;
      rc = bgmoe_mxfp4_fused_s1(L->act, &L->gate, &L->up, L->expert_counts, L->cu_seqlens, el, rows, inter, h,
                                L->hmid, nullptr, L->activation, bound, stream);
    }
    if (rc != BGMOE_OK) return rc;
    rc = bgmoe_mxfp4_grouped_gemm(L->hmid, &L->down, L->expert_counts, L->cu_seqlens, el, rows, h, inter, L->y,
                                  nullptr, bound, stream);
    if (rc != BGMOE_OK) return rc;
  }
  if (stages & BGMOE_MXFP4_COMBINE)
    return bgmoe_reduce_weighted_scatter(L->y, L->topk_pos, L->topk_weights, n, h, k, L->out, -1, L->shared_out,
                                         L->shared_mode, stream);
  return BGMOE_OK;
}
