"""Sigmoid + bias-corrected top-k routers on the CPU.  Oracle code: test
infrastructure only.

Two ops are restated:

* ``fused_gate``  -- the group-limited router ``moe_fused_gate``
  (batchgen_kernels/src/moe/mgn/moe_fused_gate.cu:83-253): input is ALREADY
  sigmoided scores.
* ``gate_sigmoid_topk`` -- the ungrouped router
  (batchgen_kernels/src/moe/routing/gate_sigmoid_topk.cu:71-213).

The reference compiles the second one with fast-math, so its sigmoid is not a
reproducible function.  This build defines the sigmoid as the correctly rounded
one: float32( 1 / (1 + exp(-float64(x))) ).
"""
from __future__ import annotations

import numpy as np

F32 = np.float32
NEG_BIG = F32(-1e9)


def sigmoid_f32(logits) -> np.ndarray:
    x = np.asarray(logits, dtype=np.float32).astype(np.float64)
    with np.errstate(over="ignore"):
        return (1.0 / (1.0 + np.exp(-x))).astype(F32)


def _argmax_rounds(vals: np.ndarray, rounds: int, floor: np.float32, tie_floor_ok: bool):
    """``rounds`` successive arg-max picks per row.

    A candidate must compare strictly greater than ``floor`` (NaN never does);
    among equal values the lowest index wins; a picked entry is retired.  When
    no candidate is left the pick is -1.  Returns int32 [rows, rounds].
    """
    v = np.array(vals, dtype=np.float32, copy=True)
    with np.errstate(invalid="ignore"):
        ok = v > floor
    if tie_floor_ok:
        ok = ok | (v == floor)
    work = np.where(ok, v.astype(np.float64), -np.inf)
    n = v.shape[0]
    out = np.full((n, rounds), -1, dtype=np.int32)
    rows = np.arange(n)
    for r in range(rounds):
        idx = np.argmax(work, axis=1)              # first occurrence == lowest index
        has = work[rows, idx] > -np.inf
        out[:, r] = np.where(has, idx, -1)
        work[rows[has], idx[has]] = -np.inf
    return out


def fused_gate(scores, bias, n_group: int, topk_group: int, top_k: int,
               routed_scaling_factor: float):
    """moe_fused_gate.cu:83-253.  scores [N,E] fp32 (sigmoided), bias [E].

    Returns (ids int32 [N,K] in descending biased-score order, w fp32 [N,K]).
    Steps: s = score + bias; group score = sum of the group's two largest s
    (strict '>' scan from -1e9, :128-140); ``topk_group`` arg-max rounds over
    groups (strict '>' so the lowest group index wins a tie, :46, :157);
    experts outside the chosen groups := -1e9 (:176-194); ``top_k`` arg-max
    rounds over all experts (:197-224); weights from the UN-biased scores:
    sum in route order from 0.0f, scale = rsf / (sum + 1e-20f), w = orig*scale
    (:230-251).
    """
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    bias = np.ascontiguousarray(bias, dtype=np.float32)
    n, e = scores.shape
    assert e % n_group == 0
    epg = e // n_group
    s = (scores + bias[None, :]).astype(F32)
    g = s.reshape(n, n_group, epg)
    with np.errstate(invalid="ignore"):
        geff = np.where(g > NEG_BIG, g, NEG_BIG).astype(F32)
    gs = -np.sort(-geff, axis=2)
    max1 = gs[:, :, 0]
    max2 = gs[:, :, 1] if epg > 1 else np.full_like(max1, NEG_BIG)
    group_scores = (max1 + max2).astype(F32)
    sel = _argmax_rounds(group_scores, topk_group, NEG_BIG, tie_floor_ok=False)   # [n, topk_group]
    gmask = np.zeros((n, n_group), dtype=bool)
    for r in range(topk_group):
        ok = sel[:, r] >= 0
        gmask[np.arange(n)[ok], sel[ok, r]] = True
    emask = np.repeat(gmask, epg, axis=1)
    masked = np.where(emask, s, NEG_BIG).astype(F32)
    ids = _argmax_rounds(masked, top_k, NEG_BIG, tie_floor_ok=False)
    safe = np.where(ids >= 0, ids, 0)
    orig = np.take_along_axis(scores, safe.astype(np.int64), axis=1)
    orig = np.where(ids >= 0, orig, F32(0.0)).astype(F32)
    total = np.zeros(n, dtype=F32)
    for k in range(top_k):
        total = (total + orig[:, k]).astype(F32)
    scale = (F32(routed_scaling_factor) / (total + F32(1e-20))).astype(F32)
    w = (orig * scale[:, None]).astype(F32)
    return ids, w


def gate_sigmoid_topk(logits, bias, k: int, routed_scaling_factor: float,
                      num_valid_tokens=None, rank_token_counts=None, rows_per_rank=None):
    """gate_sigmoid_topk.cu:71-213.  logits [N,E] fp32, bias [E].

    score = sigmoid(logit); biased = score + bias; K arg-max rounds with
    "larger wins, equal -> lower expert id" (:64, :160-166), winner retired to
    -FLT_MAX; weights: raw scores summed in route order from 0.0f,
    inv = 1/(sum+1e-20f), w = raw*inv*rsf (:193-211).  Padding rows (row >=
    num_valid_tokens, or local row >= rank_token_counts[rank]) get id -1 and
    weight 0 (:100-126).  A route with no candidate left (NaN logits) is id -1
    with raw weight 0, as the reference's one-warp kernel documents (:283-286).
    """
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    bias = np.ascontiguousarray(bias, dtype=np.float32)
    n, e = logits.shape
    score = sigmoid_f32(logits)
    biased = (score + bias[None, :]).astype(F32)
    fmax = np.finfo(np.float32).max
    ids = _argmax_rounds(biased, k, F32(-fmax), tie_floor_ok=False)
    safe = np.where(ids >= 0, ids, 0).astype(np.int64)
    raw = np.where(ids >= 0, np.take_along_axis(score, safe, axis=1), F32(0)).astype(F32)
    total = np.zeros(n, dtype=F32)
    for j in range(k):
        total = (total + raw[:, j]).astype(F32)
    inv = (F32(1.0) / (total + F32(1e-20))).astype(F32)
    w = ((raw * inv[:, None]).astype(F32) * F32(routed_scaling_factor)).astype(F32)
    pad = np.zeros(n, dtype=bool)
    if num_valid_tokens is not None:
        pad = np.arange(n) >= int(num_valid_tokens)
    elif rank_token_counts is not None:
        r = np.arange(n) // int(rows_per_rank)
        local = np.arange(n) - r * int(rows_per_rank)
        pad = local >= np.asarray(rank_token_counts, dtype=np.int64)[r]
    ids = np.where(pad[:, None], -1, ids).astype(np.int32)
    w = np.where(pad[:, None], F32(0), w).astype(F32)
    return ids, w


def grouped_router(logits, bias, n_group, topk_group, top_k, routed_scaling_factor):
    """The layer's router: correctly rounded sigmoid, then ``fused_gate``
    (``moe_gate_forward_hybrid``, batchgen/models/deepseek/deepseekv3/modeling_deepseek_v3.py:893-914)."""
    return fused_gate(sigmoid_f32(logits), bias, n_group, topk_group, top_k, routed_scaling_factor)
