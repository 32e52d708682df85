"""gfx950 implementation of the reference extension ``batchgen_kernels.common._C_mgn_ops``
(bindings: batchgen_kernels/src/moe/mgn/mgn_extension.cc:19-62)."""
from __future__ import annotations

import torch

from ..._lib import check, lib, ptr, stream
from .. import _checks as ck
from .._workspace import dispatch_workspace


def moe_fused_gate(scores, e_score_correction_bias, n_group, topk_group, n_routed_experts, top_k,
                   routed_scaling_factor):
    """Group-limited top-k on already-sigmoided scores -> [topk_indices int32 [n,k],
    topk_weights fp32 [n,k]] (moe_fused_gate.cu:256-329; outputs allocated by the op)."""
    ck.gpu(scores, "scores")
    if scores.dim() != 2 or scores.size(1) != n_routed_experts:
        ck.fail(f"scores dimension 1 ({scores.size(1) if scores.dim() == 2 else '?'}) must match "
                f"n_routed_experts ({n_routed_experts})")
    if e_score_correction_bias.numel() != n_routed_experts:
        ck.fail(f"e_score_correction_bias size ({e_score_correction_bias.numel()}) must match "
                f"n_routed_experts ({n_routed_experts})")
    if n_routed_experts % n_group != 0:
        ck.fail(f"n_routed_experts ({n_routed_experts}) must be divisible by n_group ({n_group})")
    scores = scores.contiguous().to(torch.float32)
    bias = e_score_correction_bias.to(scores.device).contiguous().to(torch.float32)
    n = scores.size(0)
    ids = torch.empty((n, top_k), dtype=torch.int32, device=scores.device)
    w = torch.empty((n, top_k), dtype=torch.float32, device=scores.device)
    with torch.cuda.device(scores.device):
        check(lib().bgmoe_fused_gate(ptr(scores), ptr(bias), n, n_routed_experts, n_group, topk_group,
                                     top_k, float(routed_scaling_factor), 0, ptr(ids), ptr(w), stream()))
    return [ids, w]


def moe_fused_gate_logits(logits, e_score_correction_bias, n_group, topk_group, n_routed_experts, top_k,
                          routed_scaling_factor, topk_indices=None, topk_weights=None):
    """Same op with the correctly rounded sigmoid applied inside and optional
    caller-owned outputs (no reference counterpart: it fuses the caller's
    torch.sigmoid, modeling_deepseek_v3.py:893-914)."""
    ck.cuda_tensor(None, logits, torch.float32, "logits")
    ck.cuda_tensor(logits, e_score_correction_bias, torch.float32, "e_score_correction_bias")
    n = logits.size(0)
    if topk_indices is None:
        topk_indices = torch.empty((n, top_k), dtype=torch.int32, device=logits.device)
    if topk_weights is None:
        topk_weights = torch.empty((n, top_k), dtype=torch.float32, device=logits.device)
    with torch.cuda.device(logits.device):
        check(lib().bgmoe_fused_gate(ptr(logits), ptr(e_score_correction_bias), n, n_routed_experts, n_group,
                                     topk_group, top_k, float(routed_scaling_factor), 1,
                                     ptr(topk_indices), ptr(topk_weights), stream()))
    return [topk_indices, topk_weights]


def compact_expert_data(expert_counts):
    """-> [group_size, activated_group_idx, group_start_indices, num_active_experts]
    (expert_bin_count.cu:332-385)."""
    ck.gpu(expert_counts, "expert_counts")
    ck.dtype(expert_counts, torch.int32, "expert_counts")
    e = expert_counts.numel()
    dev = expert_counts.device
    idx = torch.empty(e, dtype=torch.int32, device=dev)
    size = torch.empty(e, dtype=torch.int32, device=dev)
    start = torch.empty(e, dtype=torch.int32, device=dev)
    num = torch.zeros(1, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        check(lib().bgmoe_compact_expert_data(ptr(expert_counts.contiguous()), e, ptr(size), ptr(idx),
                                              ptr(start), ptr(num), stream()))
    return [size, idx, start, num]


def expert_bincount(eids, routed_expert_start_idx, experts_per_rank, device):
    """Histogram of expert ids + the compaction above (expert_bin_count.cu:155-231)."""
    ck.gpu(eids, "eids")
    flat = eids.reshape(-1, 1).to(torch.int32).contiguous()
    n = flat.size(0)
    dev = flat.device
    counts = torch.empty(experts_per_rank, dtype=torch.int32, device=dev)
    counters = torch.empty(experts_per_rank, dtype=torch.int32, device=dev)
    pos = torch.empty(max(n, 1), dtype=torch.int32, device=dev)
    cu = torch.empty(experts_per_rank + 1, dtype=torch.int32, device=dev)
    ws, ws_bytes = dispatch_workspace(dev, n, experts_per_rank)
    with torch.cuda.device(dev):
        check(lib().bgmoe_dispatch_scatter_ragged(None, ptr(flat), n, 1, 0, None, 0, int(routed_expert_start_idx),
                                                  int(experts_per_rank), ptr(counts), ptr(counters), ptr(pos),
                                                  ptr(cu), 1, ptr(ws), ws_bytes, stream()))
    return compact_expert_data(counts)


def fused_moe_token_dispatch(global_x, topk_idx, token_idx, topk_pos, routed_expert_start_idx,
                             routed_expert_end_idx):
    """Tight expert-sorted gather -> [output_x, output_eids, output_token_idx, output_topk_pos,
    expert_counts, expert_offsets] (fused_moe_token_dispatch.cu:172-292).  Rows are in the
    stable (token, k) order; ``output_x`` is sized for all N*K pairs, the first
    expert_offsets[-1] rows are live (the reference sizes it after a host read)."""
    ck.gpu(global_x, "global_x")
    ck.gpu(topk_idx, "topk_idx")
    ck.contiguous(global_x, "global_x")
    ck.contiguous(topk_idx, "topk_idx")
    ck.dtype(global_x, torch.bfloat16, "global_x")
    n, h = global_x.shape
    k = topk_idx.size(1)
    e_l = int(routed_expert_end_idx - routed_expert_start_idx)
    dev = global_x.device
    ids32 = topk_idx.to(torch.int32).contiguous()
    nk = n * k
    if e_l <= 0:
        ck.fail(f"routed_expert_end_idx ({routed_expert_end_idx}) must exceed routed_expert_start_idx "
                f"({routed_expert_start_idx})")
    out_x = torch.empty((max(nk, 1), h), dtype=global_x.dtype, device=dev)
    counts = torch.empty(e_l, dtype=torch.int32, device=dev)
    counters = torch.empty(e_l, dtype=torch.int32, device=dev)
    pos = torch.empty(max(nk, 1), dtype=torch.int32, device=dev)
    offsets = torch.empty(e_l + 1, dtype=torch.int32, device=dev)
    ws, ws_bytes = dispatch_workspace(dev, nk, e_l)
    with torch.cuda.device(dev):
        check(lib().bgmoe_dispatch_scatter_ragged(ptr(global_x), ptr(ids32), n, k, h, ptr(out_x), out_x.size(0),
                                                  int(routed_expert_start_idx), e_l, ptr(counts), ptr(counters),
                                                  ptr(pos), ptr(offsets), 1, ptr(ws), ws_bytes, stream()))
    # per-row metadata: one more launch, no device -> host read (the reference's kernel writes them while it copies
    # the rows and ignores its token_idx / topk_pos arguments, fused_moe_token_dispatch.cu:59-88)
    rows = out_x.size(0)
    out_eids = torch.empty(rows, dtype=torch.int32, device=dev)
    out_tok = torch.empty(rows, dtype=torch.int32, device=dev)
    out_pos = torch.empty(rows, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        check(lib().bgmoe_dispatch_row_metadata(ptr(ids32), ptr(pos), nk, k, offsets[e_l:].data_ptr(), rows,
                                                ptr(out_eids), ptr(out_tok), ptr(out_pos), stream()))
    return [out_x, out_eids, out_tok, out_pos, counts, offsets]
