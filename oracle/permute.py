"""Expert permute (counting sort of (token, k) pairs by local expert) on the
CPU.  Oracle code: test infrastructure only.

The reference kernels claim a slot inside an expert with an atomic counter
(batchgen_kernels/src/moe/dispatch_scatter_3d.cu:66, :217), so their order
within an expert is arrival order.  The only deterministic definition in the
reference is its tests' sequential loop ``ref_dispatch``
(tests/gpu/test_moe_routing_kernels.py:40-73): walk the flat index
i = t*K + k in ascending order, slot = running counter of that expert.  That
stable order is the contract here.
"""
from __future__ import annotations

import numpy as np


def _stable_ranks(topk_ids: np.ndarray, expert_start: int, num_local: int):
    flat = np.asarray(topk_ids, dtype=np.int64).reshape(-1)
    local = flat - int(expert_start)
    is_local = (local >= 0) & (local < num_local)
    counts = np.bincount(local[is_local], minlength=num_local).astype(np.int32)
    rank = np.full(flat.shape, -1, dtype=np.int64)
    # stable: rank of pair i = number of earlier pairs with the same expert
    order = np.argsort(np.where(is_local, local, num_local), kind="stable")
    sorted_local = np.where(is_local, local, num_local)[order]
    starts = np.searchsorted(sorted_local, np.arange(num_local + 1), side="left")
    pos_in_sorted = np.arange(flat.size)
    rank_sorted = pos_in_sorted - starts[np.minimum(sorted_local, num_local)]
    rank[order] = rank_sorted
    rank = np.where(is_local, rank, -1)
    return local, is_local, counts, rank


def dispatch_masked(topk_ids, expert_start: int, num_local: int, max_tokens: int):
    """``dispatch_scatter_3d`` index part (dispatch_scatter_3d.cu:15-137).

    Returns (expert_counts int32 [E_l], topk_pos int32 [N*K]) with
    topk_pos = e*max_tokens + slot, or -1 for a non-local id.  A pair whose
    slot would be >= max_tokens is dropped (pos -1) and the count is clipped to
    max_tokens; the reference writes out of bounds in that case.
    """
    local, is_local, counts, rank = _stable_ranks(topk_ids, expert_start, num_local)
    keep = is_local & (rank < max_tokens)
    pos = np.where(keep, local * max_tokens + rank, -1).astype(np.int32)
    return np.minimum(counts, max_tokens).astype(np.int32), pos


def dispatch_masked_arrivals(topk_ids, expert_start: int, num_local: int, max_tokens: int):
    """``dispatch_masked`` plus what the scatter kernel's atomic slot counter holds when it has run
    (dispatch_scatter_3d.cu:66: every local pair bumps ``expert_counters[e]``, also the pairs beyond
    ``max_tokens``): the arrivals per expert before clipping.  ``arrivals[e] > counts[e]`` is the only
    sign a caller gets that rows of expert e were dropped.

    Returns (expert_counts, topk_pos, arrivals int32 [E_l]).
    """
    counts, pos = dispatch_masked(topk_ids, expert_start, num_local, max_tokens)
    _, _, arrivals, _ = _stable_ranks(topk_ids, expert_start, num_local)
    return counts, pos, arrivals.astype(np.int32)


def dispatch_ragged(topk_ids, expert_start: int, num_local: int, row_align: int = 1):
    """``dispatch_scatter_ragged`` index part (dispatch_scatter_3d.cu:152-358)
    and, with row_align=1, the tight forms ``dispatch_count_gather`` /
    ``fused_moe_token_dispatch``.

    cu_seqlens[e+1] - cu_seqlens[e] = align(count[e], row_align) (:182-190).
    Returns (expert_counts [E_l], cu_seqlens [E_l+1], topk_pos [N*K]) int32.
    """
    local, is_local, counts, rank = _stable_ranks(topk_ids, expert_start, num_local)
    aligned = (counts.astype(np.int64) + row_align - 1) // row_align * row_align
    cu = np.zeros(num_local + 1, dtype=np.int64)
    cu[1:] = np.cumsum(aligned)
    pos = np.where(is_local, cu[np.clip(local, 0, num_local - 1)] + rank, -1).astype(np.int32)
    return counts, cu.astype(np.int32), pos


def ragged_capacity_rows(num_tokens: int, top_k: int, num_local: int, row_align: int) -> int:
    """dispatch_scatter_3d.cu:229-243."""
    nk = num_tokens * top_k
    rows = nk + (row_align - 1) * min(num_local, nk)
    return rows // row_align * row_align


def gather_rows(x: np.ndarray, topk_pos: np.ndarray, top_k: int, num_rows: int, fill=0):
    """Materialise the permuted activation buffer: out[pos] = x[i // K]."""
    out = np.full((num_rows,) + x.shape[1:], fill, dtype=x.dtype)
    idx = np.nonzero(topk_pos >= 0)[0]
    out[topk_pos[idx]] = x[idx // top_k]
    return out


def dispatch_sequential(topk_ids, expert_start: int, num_local: int):
    """Literal per-pair loop of the reference test oracle
    (tests/gpu/test_moe_routing_kernels.py:40-73); used to pin the vectorised
    forms above on small inputs."""
    flat = np.asarray(topk_ids).reshape(-1)
    counts = np.zeros(num_local, dtype=np.int32)
    for eid in flat:
        if expert_start <= eid < expert_start + num_local:
            counts[eid - expert_start] += 1
    offs = np.zeros(num_local + 1, dtype=np.int32)
    for e in range(num_local):
        offs[e + 1] = offs[e] + counts[e]
    pos = np.full(flat.size, -1, dtype=np.int32)
    ctr = np.zeros(num_local, dtype=np.int32)
    for i, eid in enumerate(flat):
        if expert_start <= eid < expert_start + num_local:
            le = eid - expert_start
            pos[i] = offs[le] + ctr[le]
            ctr[le] += 1
    return counts, offs, pos
