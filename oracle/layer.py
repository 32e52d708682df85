"""Whole MoE layer on the CPU.  Oracle code: test infrastructure only.

Two layer restatements:

* ``moe_layer_fp8`` / ``moe_layer_mxfp4`` -- the composition the HIP path is
  checked against: router -> stable permute -> act-quant (form C) -> fp32
  dequantise-then-matmul experts with SwiGLU and requant -> fp32 weighted
  combine -> + shared expert.  Op order follows the reference's FP8 pipeline
  class (batchgen/moe/fp8_wgmma_pipeline.py:294-372).
* ``moe_layer_l1_torch`` -- the reference's CPU-runnable pure-PyTorch path
  (``DeepseekV3MoE_Prefill.forward/moe_infer``,
  batchgen/models/deepseek/deepseekv3/modeling_deepseek_v3.py:1115-1236; experts
  ``DeepseekV3MLP.forward`` :614-617 on bf16 weights dequantised by
  ``deepseek_v3_dequantization``, batchgen_kernels/triton/fp8_quantize.py:624-656):
  activations are NOT quantised, matmuls run in bf16, the weighted sum in fp32.
  This is what ``bench.py`` times as the CPU baseline.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F

from . import combine as _cb
from . import gemm as _gm
from . import mxfp4 as _mx
from . import permute as _pm
from . import quant as _q
from . import router as _rt
from . import situ as _situ

F32 = np.float32


def route(logits, bias, rcfg):
    """rcfg: dict(top_k, n_group, topk_group, rsf).  n_group <= 1 -> ungrouped."""
    if rcfg.get("n_group", 1) > 1:
        return _rt.grouped_router(logits, bias, rcfg["n_group"], rcfg["topk_group"],
                                  rcfg["top_k"], rcfg["rsf"])
    return _rt.gate_sigmoid_topk(logits, bias, rcfg["top_k"], rcfg["rsf"])


def _permute(ids, expert_start, num_local, layout, max_tokens, row_align):
    if layout == "masked":
        counts, pos = _pm.dispatch_masked(ids, expert_start, num_local, max_tokens)
        cu = (np.arange(num_local + 1, dtype=np.int64) * max_tokens).astype(np.int32)
        rows = num_local * max_tokens
    else:
        counts, cu, pos = _pm.dispatch_ragged(ids, expert_start, num_local, row_align)
        rows = int(cu[-1])
    return counts, cu, pos, rows


def moe_layer_fp8(x, logits, bias, rcfg, w, expert_start, num_local,
                  layout="masked", max_tokens=0, row_align=64, shared=None,
                  shared_mode="bf16_add", routes=None, variant="i"):
    """x [N,H] bf16-valued; w = dict(gate_q,gate_s,up_q,up_s,down_q,down_s) for the
    LOCAL experts ([E_l,...] numpy); shared = same keys with a leading 1.

    ``variant`` picks the rounding of the intermediate (``oracle.gemm.expert_mlp_fp8``): "i" is what the HIP
    path computes; "ii" and "iii" emulate the reference's own kernels; "fp32" is the fp32
    dequantise-then-matmul yardstick (no bf16 rounding anywhere after the routing: fp32 expert outputs, fp32
    combine, fp32 shared-expert add, fp32 result).

    Returns a dict with every intermediate the parity tests compare.
    """
    x = _q.as_f32(x)
    n, h = x.shape
    # routes = (ids [N,K], weights [N,K]) from an external gate (fp8_wgmma_pipeline.py:294-307): the router is skipped
    ids, wt = route(logits, bias, rcfg) if routes is None else (np.asarray(routes[0], dtype=np.int32),
                                                                 np.asarray(routes[1], dtype=np.float32))
    k = ids.shape[1]
    counts, cu, pos, rows = _permute(ids, expert_start, num_local, layout, max_tokens, row_align)
    xq_tok, xs_tok = _q.act_quant(x)
    xq = _pm.gather_rows(xq_tok, pos, k, max(rows, 1))
    xs = _pm.gather_rows(xs_tok, pos, k, max(rows, 1))
    y, hmid, hq, hs = _gm.expert_mlp_fp8(xq, xs, w["gate_q"], w["gate_s"], w["up_q"], w["up_s"],
                                         w["down_q"], w["down_s"], counts, cu, variant=variant)
    y_sh = None
    if shared is not None:
        one = np.array([n], dtype=np.int32)
        zero = np.array([0, n], dtype=np.int32)
        y_sh, _, _, _ = _gm.expert_mlp_fp8(xq_tok, xs_tok, shared["gate_q"], shared["gate_s"],
                                           shared["up_q"], shared["up_s"], shared["down_q"],
                                           shared["down_s"], one, zero, variant=variant)
    if variant == "fp32":
        out = _cb.reduce_weighted_scatter(y, pos, wt, n, k, shared=y_sh, shared_mode="fp32")
    else:
        out = _cb.reduce_weighted_scatter(y, pos, wt, n, k, shared=y_sh, shared_mode=shared_mode)
    return dict(out=out, ids=ids, weights=wt, counts=counts, cu=cu, pos=pos, xq_tok=xq_tok,
                xs_tok=xs_tok, xq=xq, xs=xs, h=hmid, hq=hq, hs=hs, y=y, y_shared=y_sh)


def moe_layer_mxfp4(x, logits, bias, rcfg, w, expert_start, num_local,
                    layout="masked", max_tokens=0, row_align=16, shared_bf16=None,
                    shared_mode="bf16_add", activation="swiglu", latent=None):
    """bf16 activations, MXFP4 routed experts (w = dict(gate_p,gate_s,up_p,up_s,
    down_p,down_s)), bf16 shared expert (dict(gate,up,down) float32 holding bf16).

    ``latent`` = dict(down_proj [L,H], up_proj [H,L], norm_weight [L] or None, eps) selects the Kimi-K3
    latent-MoE data flow (kimi_linear/model.py:585-603, fused_moe_mxfp4_resident.py:922-944): the router sees
    the hidden rows, the experts the rows of bf16(x @ down_proj^T); their fp32-combined output is rounded to
    bf16, normalised, projected back with up_proj (bf16), and the shared expert's bf16 output -- computed from
    the hidden rows with the same activation -- is added in bf16."""
    x = _q.as_f32(x)
    n, h = x.shape
    ids, wt = route(logits, bias, rcfg)
    k = ids.shape[1]
    counts, cu, pos, rows = _permute(ids, expert_start, num_local, layout, max_tokens, row_align)
    x_exp = x if latent is None else _q.bf16_round(_gm._mm(x, _q.as_f32(latent["down_proj"])))
    xr = _pm.gather_rows(x_exp, pos, k, max(rows, 1))
    y, hmid = _gm.expert_mlp_mxfp4(xr, w["gate_p"], w["gate_s"], w["up_p"], w["up_s"],
                                   w["down_p"], w["down_s"], counts, cu, activation=activation)
    y_sh = None
    if shared_bf16 is not None:
        g = _gm._mm(x, shared_bf16["gate"])
        u = _gm._mm(x, shared_bf16["up"])
        if activation == "situ":       # the module form: bf16 [gate | up] -> SituAndMul -> bf16
            hh = _situ.situ_and_mul(np.concatenate([_q.bf16_round(g), _q.bf16_round(u)], axis=-1),
                                    _situ.K3_BETA, _situ.K3_LINEAR_BETA)
        else:
            hh = _q.swiglu_bf16(g, u)
        y_sh = _q.bf16_round(_gm._mm(hh, shared_bf16["down"]))
    if latent is None:
        out = _cb.reduce_weighted_scatter(y, pos, wt, n, k, shared=y_sh, shared_mode=shared_mode)
        y_lat = None
    else:
        y_lat = _cb.reduce_weighted_scatter(y, pos, wt, n, k)
        z = y_lat
        if latent.get("norm_weight") is not None:
            z = _situ.rmsnorm(z, latent["norm_weight"], latent["eps"])
        out = _q.bf16_round(_gm._mm(z, _q.as_f32(latent["up_proj"])))
        if y_sh is not None:
            out = _q.bf16_round(out + y_sh)
    return dict(out=out, ids=ids, weights=wt, counts=counts, cu=cu, pos=pos, x_rows=xr, h=hmid,
                y=y, y_shared=y_sh, y_latent=y_lat, x_latent=x_exp if latent is not None else None)


def moe_layer_dense_bruteforce(x, ids, wt, expert_fn, n_experts_start, num_local):
    """out[t] = sum_k w[t,k] * expert_fn(e, x[t]) over local experts only; one
    token and one route at a time.  Pins the permute/combine bookkeeping of the
    layer functions above."""
    x = _q.as_f32(x)
    n, h = x.shape
    out = np.zeros((n, h), dtype=F32)
    for t in range(n):
        acc = np.zeros(h, dtype=F32)
        for j in range(ids.shape[1]):
            le = int(ids[t, j]) - n_experts_start
            if 0 <= le < num_local:
                acc = (acc + (expert_fn(le, x[t:t + 1])[0] * wt[t, j]).astype(F32)).astype(F32)
        out[t] = acc
    return out


# ----------------------------------------------------------------------------
# the reference's CPU-runnable PyTorch path (bench.py's cpu_baseline)
# ----------------------------------------------------------------------------
def l1_dequant_weights(wq: np.ndarray, ws: np.ndarray) -> torch.Tensor:
    """deepseek_v3_dequantization -> bf16 (fp8_quantize.py:624-656)."""
    e = torch.from_numpy(_q.weight_block_dequant(wq, ws))
    return e.to(torch.bfloat16)


def l1_dequant_mxfp4(packed: np.ndarray, scales: np.ndarray) -> torch.Tensor:
    """MXFP4 weight -> bf16 with the reference recipe (``mxfp4_dequantize_oracle``,
    batchgen/moe/mxfp4_oracle_vector.py:80-115; every e2m1 value times a power of two is exact in bf16)."""
    return torch.from_numpy(_mx.dequant(packed, scales)).to(torch.bfloat16)


@torch.inference_mode()
def moe_layer_l1_torch(x: torch.Tensor, ids: np.ndarray, wt: np.ndarray, experts, expert_start: int,
                       shared=None) -> torch.Tensor:
    """x [N,H] bf16 torch; experts = list of (gate,up,down) bf16 torch weights
    for the local experts; returns [N,H] bf16.

    modeling_deepseek_v3.py:1133-1236: argsort pairs by expert, per-expert
    ``down(silu(gate(x)) * up(x))`` in bf16, fp32 weighted accumulation
    (pure-torch form of the combine at :1221-1231), ``+ shared_experts(x)``.
    """
    n, h = x.shape
    k = ids.shape[1]
    flat = torch.from_numpy(np.asarray(ids, dtype=np.int64).reshape(-1))
    idxs = flat.argsort(stable=True)
    sorted_e = flat[idxs]
    num_local = len(experts)
    local = (sorted_e >= expert_start) & (sorted_e < expert_start + num_local)
    w_flat = torch.from_numpy(np.asarray(wt, dtype=np.float32).reshape(-1))
    out = torch.zeros(n, h, dtype=torch.float32)
    bounds = torch.searchsorted(sorted_e, torch.arange(expert_start, expert_start + num_local + 1))
    for i in range(num_local):
        lo, hi = int(bounds[i]), int(bounds[i + 1])
        if hi == lo:
            continue
        pair = idxs[lo:hi]
        tok = pair // k
        g, u, d = experts[i]
        xe = x[tok]
        ye = F.linear(F.silu(F.linear(xe, g)) * F.linear(xe, u), d)
        out.index_add_(0, tok, ye.float() * w_flat[pair].unsqueeze(1))
    y = out.to(torch.bfloat16)
    if shared is not None:
        g, u, d = shared
        y = y + F.linear(F.silu(F.linear(x, g)) * F.linear(x, u), d)
    return y
