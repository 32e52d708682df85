"""The ops of the Kimi-K3 latent-MoE seam that are not GEMMs, with the reference's signatures.

* ``situ_and_mul(x, beta, linear_beta)``: ``situ_and_mul_triton``
  (batchgen/models/moonshotai/kimi_linear/situ_triton.py:55-77) and the module ``SituAndMul``
  (kimi_linear/model.py:84-115): ``[..., 2d] -> [..., d]``, gate in the first half.
* ``rmsnorm(x, weight, eps)``: ``triton_rmsnorm`` (kimi_linear/rmsnorm_triton.py:51-69), what
  ``KimiRMSNorm.forward`` calls on a CUDA tensor (kimi_linear/model.py:192-205).

Both run the HIP kernels of libbgmoe.so; there is no eager fallback.
"""
from __future__ import annotations

from typing import Optional

import torch

from .._lib import check, lib, ptr, stream


def bf16_linear(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None,
                workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x [n, h] @ weight [e, h]^T -> [n, e]`` bf16 on the router GEMM's kernels (``bgmoe_bf16_linear``): the
    bias-free ``nn.Linear`` of the bf16 shared expert and the latent projections.  With ``out`` and ``workspace``
    (``bgmoe_router_gemm_workspace_bytes(n, h, e)`` bytes) given the call allocates nothing."""
    if not x.is_cuda or x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or x.dim() != 2 or \
            weight.dim() != 2 or x.size(1) != weight.size(1) or not x.is_contiguous() or not weight.is_contiguous():
        raise RuntimeError("bf16_linear: x [n, h] and weight [e, h] must be contiguous CUDA BF16 tensors")
    n, h = x.shape
    e = weight.size(0)
    if out is None:
        out = torch.empty((n, e), dtype=torch.bfloat16, device=x.device)
    elif out.dtype != torch.bfloat16 or tuple(out.shape) != (n, e) or not out.is_contiguous():
        raise RuntimeError(f"bf16_linear: out must be contiguous BF16 [{n}, {e}]")
    if workspace is None:
        need = int(lib().bgmoe_router_gemm_workspace_bytes(n, h, e))
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=x.device)
    if n:
        with torch.cuda.device(x.device):
            check(lib().bgmoe_bf16_linear(ptr(x), ptr(weight), n, h, e, ptr(out), ptr(workspace), workspace.numel(),
                                          stream()))
    return out


def bf16_linear_workspace_bytes(n_max: int, h: int, e: int) -> int:
    """Bytes of workspace that serve ``bf16_linear`` for every row count up to ``n_max``: the launch shape depends
    on the row count (few rows: fp32 partial planes per 512-wide K segment, never more than 64 MiB of them; many
    rows: no planes), so the need is not monotonic in it and a layer sizes its buffer once with this bound."""
    nseg = (h + 511) // 512
    one = n_max * e * 4
    return max(16, one, min(nseg * one, 64 << 20))


def silu_and_mul(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``bf16(bf16(silu(x[:, :d])) * x[:, d:])``: ``F.silu(gate) * up`` on a bf16 ``[rows, 2d]`` tensor."""
    rows, d2 = x.shape
    d = d2 // 2
    if out is None:
        out = torch.empty((rows, d), dtype=x.dtype, device=x.device)
    if rows and d:
        with torch.cuda.device(x.device):
            check(lib().bgmoe_silu_and_mul(ptr(x), rows, d, x.stride(0), ptr(out), out.stride(0), stream()))
    return out


def situ_and_mul(x: torch.Tensor, beta: float, linear_beta: Optional[float] = None,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x[..., :d]`` = gate, ``x[..., d:]`` = up -> ``[..., d]`` bf16."""
    if not x.is_cuda or x.dtype != torch.bfloat16:
        raise RuntimeError("situ_and_mul: x must be a CUDA BF16 tensor")
    if x.shape[-1] % 2:
        raise RuntimeError("situ_and_mul: the last axis holds [gate, up] and must be even")
    d = x.shape[-1] // 2
    x2 = x.reshape(-1, 2 * d)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    rows = x2.shape[0]
    y = torch.empty((rows, d), dtype=x.dtype, device=x.device) if out is None else out.view(rows, d)
    if rows and d:
        with torch.cuda.device(x.device):
            check(lib().bgmoe_situ_and_mul(ptr(x2), rows, d, x2.stride(0) if rows > 1 else 2 * d, float(beta),
                                           float(linear_beta) if linear_beta is not None else 0.0, ptr(y), d,
                                           stream()))
    return y.reshape(*x.shape[:-1], d)


class SituAndMul(torch.nn.Module):
    """``beta * tanh(gate / beta) * sigmoid(gate) * up'`` with ``up' = linear_beta * tanh(up / linear_beta)``
    when ``linear_beta`` is set (kimi_linear/model.py:84-115)."""

    def __init__(self, beta: float = 1.0, linear_beta: Optional[float] = None):
        super().__init__()
        self.beta = beta
        self.linear_beta = linear_beta

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return situ_and_mul(x, self.beta, self.linear_beta)


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm over the last axis: fp32 math, one rounding to bf16.  ``out`` (contiguous, same shape): no allocation."""
    h = x.shape[-1]
    if not x.is_cuda or x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or weight.numel() != h:
        raise RuntimeError(f"rmsnorm: x must be CUDA BF16 [..., {h}] and weight BF16 [{h}]")
    x2 = x.reshape(-1, h)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    y = torch.empty_like(x2) if out is None else out.view(-1, h)
    if x2.shape[0]:
        with torch.cuda.device(x.device):
            check(lib().bgmoe_rmsnorm(ptr(x2), ptr(weight.contiguous()), x2.shape[0], h, float(eps), ptr(y), stream()))
    return y.view_as(x)
