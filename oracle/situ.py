"""SiTU-and-multiply and the latent-seam RMSNorm on the CPU.  Oracle code: test infrastructure only.

``SituAndMul._forward_eager`` (batchgen/models/moonshotai/kimi_linear/model.py:109-115):

    situ_a = beta * tanh(gate / beta) * sigmoid(gate)
    up'    = linear_beta * tanh(up / linear_beta)      (when linear_beta is set)
    out    = dtype(situ_a * up')

evaluated here in float64 and rounded once to bf16.  The reference's native forms are not functions another
machine can reproduce -- the Triton kernel writes tanh as 1 - 2/(exp(2x)+1) (situ_triton.py:24-27) and the
fused GEMM epilogue is compiled with fast-math tanhf/__expf (marlin_grouped_gemm.cu:243-256) -- so the
device is compared with this exact evaluation within one bf16 unit in the last place; the reference's own
bar is max|diff| <= max|ref| * 2^-7 + 1e-3 with < 2 % differing elements
(tests/test_kimi_k3_situ_triton.py:25-28).

``situ_fused`` is the stage-1 epilogue of the MXFP4 expert GEMM: both branches rounded to bf16 first
(marlin_grouped_gemm.cu:1055-1069), beta = 4, linear_beta = 25 compiled in (:253-254).

``rmsnorm`` is ``x * (1 / sqrt(mean(x^2) + eps)) * w`` rounded once (rmsnorm_triton.py:37-44), in float64.
The device's fixed summation order is restated by ``oracle.norm_quant.add_rmsnorm`` with a zero residual.
"""
from __future__ import annotations

import numpy as np

from .quant import as_f32, bf16_round

F64 = np.float64
K3_BETA = 4.0
K3_LINEAR_BETA = 25.0


def situ_f64(gate, up, beta: float, linear_beta=None) -> np.ndarray:
    g = np.asarray(gate, dtype=F64)
    u = np.asarray(up, dtype=F64)
    with np.errstate(over="ignore"):
        a = beta * np.tanh(g / beta) * (1.0 / (1.0 + np.exp(-g)))
    if linear_beta is not None:
        u = linear_beta * np.tanh(u / linear_beta)
    return a * u


def situ_and_mul(x, beta: float, linear_beta=None) -> np.ndarray:
    """[..., 2d] (gate | up), bf16-valued -> [..., d] bf16-valued float32."""
    x = as_f32(x)
    d = x.shape[-1] // 2
    return bf16_round(situ_f64(x[..., :d], x[..., d:], beta, linear_beta).astype(np.float32))


def situ_fused(g_f32, u_f32) -> np.ndarray:
    """fp32 GEMM results of the gate and up projections -> bf16-valued float32."""
    g = bf16_round(np.asarray(g_f32, dtype=np.float32))
    u = bf16_round(np.asarray(u_f32, dtype=np.float32))
    return bf16_round(situ_f64(g, u, K3_BETA, K3_LINEAR_BETA).astype(np.float32))


def rmsnorm(x, weight, eps: float) -> np.ndarray:
    x = as_f32(x).astype(F64)
    w = as_f32(weight).reshape(-1).astype(F64)
    inv = 1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return bf16_round((x * inv * w).astype(np.float32))
