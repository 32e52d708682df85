"""gfx950 implementation of the reference extension ``batchgen_kernels.moe._C_routing``
(bindings: batchgen_kernels/src/moe/routing/routing_extension.cc:12-105).

Exports gate_sigmoid_topk, gate_sigmoid_topk_warp, glm5_router_gemm,
dispatch_count_gather, reduce_weighted_scatter, and router_gemm_gate (GEMM +
top-k without the logits round trip; no counterpart in the reference).  The
softmax router and the bias epilogue of that extension are not part of this
build.
"""
from __future__ import annotations

import torch

from ..._lib import check, lib, ptr, stream
from .. import _checks as ck
from .._workspace import dispatch_workspace, router_gemm_workspace


def _padding(n, logits, num_valid_tokens, rank_token_counts, rows_per_rank):
    """resolve_gst_padding_shape (gate_sigmoid_topk.cu:500-540)."""
    nv = rc = None
    rpr = 0
    if num_valid_tokens is not None and num_valid_tokens.numel() > 0:
        if rank_token_counts is not None and rank_token_counts.numel() > 0:
            ck.fail("num_valid_tokens and rank_token_counts are mutually exclusive")
        ck.cuda_tensor(logits, num_valid_tokens, torch.int32, "num_valid_tokens")
        if num_valid_tokens.numel() != 1:
            ck.fail("num_valid_tokens must hold one int32")
        nv = num_valid_tokens
    elif rank_token_counts is not None and rank_token_counts.numel() > 0:
        ck.cuda_tensor(logits, rank_token_counts, torch.int64, "rank_token_counts")
        rpr = int(rows_per_rank or 0)
        if rpr <= 0:
            ck.fail("rows_per_rank must be positive when rank_token_counts is given")
        if rank_token_counts.numel() * rpr != n:
            ck.fail(f"rank_token_counts ({rank_token_counts.numel()}) x rows_per_rank ({rpr}) must equal N={n}")
        rc = rank_token_counts
    return nv, rc, rpr


def _gate(router_logits, e_score_correction, k, routed_scaling_factor, topk_indices, topk_weights,
          num_valid_tokens, latent_out, latent_offset, rank_token_counts, rows_per_rank, max_e, allow_i64):
    ck.gpu(router_logits, "router_logits")
    ck.dtype(router_logits, torch.float32, "router_logits")
    if router_logits.dim() != 2:
        ck.fail("router_logits must be 2-D")
    if router_logits.stride(1) != 1:
        ck.fail("router_logits rows must be contiguous")
    ck.cuda_tensor(router_logits, e_score_correction, torch.float32, "e_score_correction")
    n, e = router_logits.shape
    if e > max_e:
        ck.fail(f"E={e} exceeds MAX_EXPERTS={max_e}")
    if e < k:
        ck.fail(f"E={e} must be at least k={k}")
    if e_score_correction.numel() != e:
        ck.fail("e_score_correction must have E elements")
    dev = router_logits.device
    if topk_indices is None or topk_indices.numel() == 0:
        topk_indices = torch.empty((n, k), dtype=torch.int32, device=dev)
    if topk_weights is None or topk_weights.numel() == 0:
        topk_weights = torch.empty((n, k), dtype=torch.float32, device=dev)
    ck.cuda_tensor(router_logits, topk_indices, (torch.int32, torch.int64) if allow_i64 else torch.int32,
                   "topk_indices")
    ck.cuda_tensor(router_logits, topk_weights, torch.float32, "topk_weights")
    if tuple(topk_indices.shape) != (n, k) or tuple(topk_weights.shape) != (n, k):
        ck.fail(f"topk_indices / topk_weights must be contiguous [{n}, {k}] tensors")
    nv, rc, rpr = _padding(n, router_logits, num_valid_tokens, rank_token_counts, rows_per_rank)
    lat_ptr, lat_off, lat_size = None, 0, 0
    if latent_out is not None and latent_out.numel() > 0:
        ck.cuda_tensor(router_logits, latent_out, torch.bfloat16, "latent_out")
        if latent_out.dim() != 2 or latent_out.size(0) != n:
            ck.fail(f"latent_out must have {n} rows")
        lat_off = int(latent_offset or 0)
        lat_size = latent_out.size(1)
        lat_ptr = ptr(latent_out)
    if n == 0:
        return [topk_indices, topk_weights]
    with torch.cuda.device(dev):
        check(lib().bgmoe_gate_sigmoid_topk(
            ptr(router_logits), router_logits.stride(0), ptr(e_score_correction), n, e, int(k),
            float(routed_scaling_factor), ptr(topk_indices), int(topk_indices.dtype == torch.int64),
            ptr(topk_weights), ptr(nv), ptr(rc), rpr, lat_ptr, lat_off, lat_size, stream()))
    return [topk_indices, topk_weights]


def gate_sigmoid_topk(router_logits, e_score_correction, k, routed_scaling_factor, topk_indices,
                      topk_weights, num_valid_tokens=None, latent_out=None, latent_offset=None,
                      rank_token_counts=None, rows_per_rank=None):
    """Ungrouped sigmoid + bias top-k, E <= 1024 (gate_sigmoid_topk.cu:546-640)."""
    return _gate(router_logits, e_score_correction, k, routed_scaling_factor, topk_indices, topk_weights,
                 num_valid_tokens, latent_out, latent_offset, rank_token_counts, rows_per_rank, 1024, False)


def gate_sigmoid_topk_warp(router_logits, e_score_correction, k, routed_scaling_factor, topk_indices,
                           topk_weights, num_valid_tokens=None, rank_token_counts=None, rows_per_rank=None):
    """Same routing, E <= 256, int32 or int64 ids (gate_sigmoid_topk.cu:643-714).  On gfx950 both
    entry points run the same one-wave-per-token kernel."""
    if topk_indices is None or topk_weights is None:
        ck.fail("gate_sigmoid_topk_warp needs caller-owned topk_indices and topk_weights")
    return _gate(router_logits, e_score_correction, k, routed_scaling_factor, topk_indices, topk_weights,
                 num_valid_tokens, None, None, rank_token_counts, rows_per_rank, 256, True)


def _router_gemm_operands(hidden_states, router_weight):
    """The reference binding's operand checks (glm5_router_gemm.cu:116-133)."""
    ck.gpu(hidden_states, "hidden_states")
    ck.gpu(router_weight, "router_weight")
    if hidden_states.dtype != torch.bfloat16:
        ck.fail("hidden_states must be BF16")
    if router_weight.dtype != torch.bfloat16:
        ck.fail("router_weight must be BF16")
    if hidden_states.dim() != 2:
        ck.fail("hidden_states must be rank-2 [N, H]")
    if router_weight.dim() != 2:
        ck.fail("router_weight must be rank-2 [E, H]")
    ck.contiguous(hidden_states, "hidden_states")
    ck.contiguous(router_weight, "router_weight")
    ck.same_device(hidden_states, router_weight, "router_weight")
    n, h = hidden_states.shape
    e = router_weight.size(0)
    if router_weight.size(1) != h:
        ck.fail(f"router_weight hidden dim mismatch: got {router_weight.size(1)}, expected {h}")
    return n, h, e


def glm5_router_gemm(hidden_states, router_weight, rank_token_counts, output, bucket_size, world_size):
    """logits [N,E] fp32 = hidden [N,H] bf16 x router_weight [E,H]^T bf16 with a per-row summation order
    that does not depend on N; rows past their rank's count are zeroed (glm5_router_gemm.cu:107-180)."""
    n, h, e = _router_gemm_operands(hidden_states, router_weight)
    dev = hidden_states.device
    if output is None or output.numel() == 0:
        output = torch.empty((n, e), dtype=torch.float32, device=dev)
    ck.gpu(output, "output")
    if output.dtype != torch.float32:
        ck.fail("output must be FP32")
    if output.dim() != 2:
        ck.fail("output must be rank-2 [N, E]")
    if tuple(output.shape) != (n, e):
        ck.fail(f"output shape mismatch: got [{output.size(0)}, {output.size(1)}], expected [{n}, {e}]")
    ck.contiguous(output, "output")
    rc = None
    if rank_token_counts is not None and rank_token_counts.numel() > 0:
        ck.gpu(rank_token_counts, "rank_token_counts")
        if rank_token_counts.dtype != torch.int64:
            ck.fail("rank_token_counts must be int64")
        ck.contiguous(rank_token_counts, "rank_token_counts")
        if int(world_size) <= 0:
            ck.fail("world_size must be positive when rank_token_counts is provided")
        if rank_token_counts.numel() < int(world_size):
            ck.fail(f"rank_token_counts length {rank_token_counts.numel()} is smaller than world_size {world_size}")
        if int(bucket_size) <= 0:
            ck.fail("bucket_size must be positive when rank_token_counts is provided")
        rc = rank_token_counts
    if n == 0 or e == 0:
        return output
    ws, ws_bytes = router_gemm_workspace(dev, n, h, e)
    with torch.cuda.device(dev):
        check(lib().bgmoe_router_gemm(ptr(hidden_states), ptr(router_weight), n, h, e, ptr(rc), int(bucket_size),
                                      int(world_size), ptr(output), ptr(ws), ws_bytes, stream()))
    return output


def router_gemm_gate(hidden_states, router_weight, e_score_correction, k, routed_scaling_factor, topk_indices,
                     topk_weights, n_group=0, topk_group=0, rank_token_counts=None, rows_per_rank=None):
    """glm5_router_gemm followed by gate_sigmoid_topk (n_group == 0) or by the grouped gate on sigmoided
    logits (n_group >= 1), identical ids and weights, without writing the logits: the GEMM's split-K
    planes are summed by the router kernel.  Returns [topk_indices, topk_weights]."""
    n, h, e = _router_gemm_operands(hidden_states, router_weight)
    dev = hidden_states.device
    ck.cuda_tensor(hidden_states, e_score_correction, torch.float32, "e_score_correction")
    if e_score_correction.numel() != e:
        ck.fail("e_score_correction must have E elements")
    if topk_indices is None or topk_indices.numel() == 0:
        topk_indices = torch.empty((n, k), dtype=torch.int32, device=dev)
    if topk_weights is None or topk_weights.numel() == 0:
        topk_weights = torch.empty((n, k), dtype=torch.float32, device=dev)
    ck.cuda_tensor(hidden_states, topk_indices, torch.int32, "topk_indices")
    ck.cuda_tensor(hidden_states, topk_weights, torch.float32, "topk_weights")
    if tuple(topk_indices.shape) != (n, k) or tuple(topk_weights.shape) != (n, k):
        ck.fail(f"topk_indices / topk_weights must be contiguous [{n}, {k}] tensors")
    rc, rpr = None, 0
    if rank_token_counts is not None and rank_token_counts.numel() > 0:
        _, rc, rpr = _padding(n, hidden_states, None, rank_token_counts, rows_per_rank)
    if n == 0:
        return [topk_indices, topk_weights]
    ws, ws_bytes = router_gemm_workspace(dev, n, h, e)
    with torch.cuda.device(dev):
        check(lib().bgmoe_router_gemm_gate(ptr(hidden_states), ptr(router_weight), ptr(e_score_correction), n, h,
                                           e, int(n_group), int(topk_group), int(k), float(routed_scaling_factor),
                                           ptr(topk_indices), ptr(topk_weights), ptr(rc), rpr, ptr(ws), ws_bytes,
                                           stream()))
    return [topk_indices, topk_weights]


def dispatch_count_gather(x, topk_indices, expert_start, num_local_experts, expert_counts, expert_offsets,
                          expert_counters, dispatched_x, topk_pos, num_valid_tokens=-1):
    """Tight (align 1) counting-sort dispatch (dispatch_count_gather.cu:145-251).
    Returns [expert_counts, expert_offsets, topk_pos]."""
    ck.cuda_tensor(None, x, torch.bfloat16, "x")
    ck.cuda_tensor(x, topk_indices, torch.int32, "topk_indices")
    n, h = x.shape
    k = topk_indices.size(1)
    if 0 < int(num_valid_tokens) < n:
        n = int(num_valid_tokens)
    for t, name in ((expert_counts, "expert_counts"), (expert_offsets, "expert_offsets"),
                    (expert_counters, "expert_counters"), (topk_pos, "topk_pos")):
        ck.cuda_tensor(x, t, torch.int32, name)
    ck.cuda_tensor(x, dispatched_x, torch.bfloat16, "dispatched_x")
    if expert_offsets.numel() < num_local_experts + 1:
        ck.fail("expert_offsets must have num_local_experts + 1 elements")
    ws, ws_bytes = dispatch_workspace(x.device, n * k, num_local_experts)
    with torch.cuda.device(x.device):
        check(lib().bgmoe_dispatch_scatter_ragged(
            ptr(x), ptr(topk_indices), n, k, h, ptr(dispatched_x), dispatched_x.size(0), int(expert_start),
            int(num_local_experts), ptr(expert_counts), ptr(expert_counters), ptr(topk_pos),
            ptr(expert_offsets), 1, ptr(ws), ws_bytes, stream()))
    return [expert_counts, expert_offsets, topk_pos]


def reduce_weighted_scatter(expert_output, topk_pos, topk_weights, N, H, K, output, num_valid_tokens=-1):
    """out[t] = bf16(sum_k y[pos]*w), K in {2,4,8} (reduce_weighted_scatter.cu:26-131)."""
    if K not in (2, 4, 8):
        ck.fail(f"Unsupported K={K}")
    ck.gpu(expert_output, "expert_output")
    if output is None or output.numel() == 0:
        output = torch.zeros((N, H), dtype=torch.bfloat16, device=expert_output.device)
    ck.combine_args(expert_output, topk_pos, topk_weights, output, int(N), int(H), int(K), torch.bfloat16)
    with torch.cuda.device(expert_output.device):
        check(lib().bgmoe_reduce_weighted_scatter(ptr(expert_output), ptr(topk_pos), ptr(topk_weights), int(N),
                                                  int(H), int(K), ptr(output), int(num_valid_tokens), None, 0,
                                                  stream()))
    return output
