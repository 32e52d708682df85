"""Top-k weighted combine (un-permute) on the CPU.  Oracle code: test
infrastructure only.

The bf16 and fp32 forms accumulate ``acc = fma(value, weight, acc)`` in fp32, k ascending: the reference
kernels' ``acc += val * w[k]`` (batchgen_kernels/src/moe/dispatch_scatter_3d.cu:386-392, 421-431;
routing/reduce_weighted_scatter.cu:58) compiles to one fused multiply-add per term (nvcc contracts by default,
and the extension is built with --use_fast_math, batchgen_kernels/setup.py:245).  The reference's test oracle
``ref_reduce`` (tests/gpu/test_moe_routing_kernels.py:76-86: ``acc += w * x.float()`` in torch) rounds product
and sum separately and is compared with a tolerance there; ``reduce_loop`` below keeps that form, and the two
differ by at most one fp32 rounding per term.
"""
from __future__ import annotations

import numpy as np

from .norm_quant import fma_f32
from .quant import as_f32, bf16_round

F32 = np.float32


def _weighted_sum_f32(y, topk_pos, w, n, k):
    y = as_f32(y)
    pos = np.asarray(topk_pos, dtype=np.int64).reshape(n, k)
    w = np.asarray(w, dtype=np.float32).reshape(n, k)
    acc = np.zeros((n, y.shape[1]), dtype=F32)
    for j in range(k):
        live = pos[:, j] >= 0
        rows = y[np.where(live, pos[:, j], 0)]
        acc = np.where(live[:, None], fma_f32(rows, np.broadcast_to(w[:, j:j + 1], rows.shape), acc), acc)
    return acc


def reduce_weighted_scatter(y, topk_pos, w, n: int, k: int, shared=None, shared_mode: str = "bf16_add"):
    """out[t] = bf16( sum_k float(y[pos[t,k]]) * w[t,k] ), pos < 0 skipped
    (dispatch_scatter_3d.cu:365-395).  Returns float32 holding bf16 values.

    ``shared`` [N,H] (bf16 values): the shared expert's output.
      "bf16_add": bf16( bf16(routed) + shared ) -- the reference's
                  ``out + self.shared_experts(identity)`` on bf16 tensors
                  (batchgen/models/deepseek/deepseekv3/modeling_deepseek_v3.py:1939).
      "fp32_add": bf16( routed_fp32 + shared ) -- one rounding.
      "fp32":     routed_fp32 + shared, nothing rounded to bf16 (the fp32 yardstick of the layer oracle).
    """
    acc = _weighted_sum_f32(y, topk_pos, w, n, k)
    if shared_mode == "fp32":
        return acc if shared is None else (acc + as_f32(shared)).astype(F32)
    if shared is None:
        return bf16_round(acc)
    sh = as_f32(shared)
    if shared_mode == "bf16_add":
        return bf16_round((bf16_round(acc) + sh).astype(F32))
    if shared_mode == "fp32_add":
        return bf16_round((acc + sh).astype(F32))
    raise ValueError(shared_mode)


def reduce_weighted_scatter_fp32(y, topk_pos, w, n: int, k: int):
    """K=16 form with fp32 output (dispatch_scatter_3d.cu:402-434)."""
    return _weighted_sum_f32(y, topk_pos, w, n, k)


def reduce_weighted_scatter_bf16_ordered(y, topk_pos, topk_ids, w, n: int, k: int):
    """Stable ascending expert-id order, every product and partial sum rounded
    to bf16: acc = bf16(acc + bf16(x * bf16(w))) (dispatch_scatter_3d.cu:436-525)."""
    y = as_f32(y)
    pos = np.asarray(topk_pos, dtype=np.int64).reshape(n, k)
    ids = np.asarray(topk_ids, dtype=np.int64).reshape(n, k)
    wb = bf16_round(np.asarray(w, dtype=np.float32).reshape(n, k))
    order = np.argsort(ids, axis=1, kind="stable")
    pos = np.take_along_axis(pos, order, axis=1)
    wb = np.take_along_axis(wb, order, axis=1)
    acc = np.zeros((n, y.shape[1]), dtype=F32)
    for j in range(k):
        live = pos[:, j] >= 0
        rows = y[np.where(live, pos[:, j], 0)]
        prod = bf16_round((rows * wb[:, j:j + 1]).astype(F32))
        acc = np.where(live[:, None], bf16_round((acc + prod).astype(F32)), acc)
    return acc


def _fma_f32_exact(a: float, b: float, c: float) -> np.float32:
    """fma(a, b, c) of three float32 values, rounded once to float32, by exact rational arithmetic."""
    from fractions import Fraction
    exact = Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c))
    r = np.float32(float(exact))                         # within one float32 ulp of the exact value
    best = r
    for cand in (np.nextafter(r, np.float32(-np.inf)), np.nextafter(r, np.float32(np.inf))):
        d_best, d_cand = abs(Fraction(float(best)) - exact), abs(Fraction(float(cand)) - exact)
        even = (np.float32(cand).view(np.uint32) & 1) == 0
        if d_cand < d_best or (d_cand == d_best and even):
            best = cand
    return np.float32(best)


def reduce_loop(y, topk_pos, w, n: int, k: int, fma: bool = True):
    """Literal per-token, per-route, per-column loop in the reference kernel's order
    (dispatch_scatter_3d.cu:386-392).  ``fma=True``: ``acc = fma(val, w, acc)`` evaluated in exact rational
    arithmetic and rounded once (what the compiled kernel does); ``fma=False``: the separately rounded product
    and sum of the reference's test oracle (tests/gpu/test_moe_routing_kernels.py:76-86)."""
    y = as_f32(y)
    pos = np.asarray(topk_pos).reshape(-1)
    w = np.asarray(w, dtype=np.float32).reshape(n, k)
    out = np.zeros((n, y.shape[1]), dtype=F32)
    for t in range(n):
        acc = np.zeros(y.shape[1], dtype=F32)
        for j in range(k):
            p = int(pos[t * k + j])
            if p >= 0:
                if fma:
                    acc = np.array([_fma_f32_exact(y[p, c], w[t, j], acc[c]) for c in range(y.shape[1])], dtype=F32)
                else:
                    acc = (acc + (w[t, j] * y[p]).astype(F32)).astype(F32)
        out[t] = bf16_round(acc)
    return out
