"""Argument checks shared by the op modules (the reference's TORCH_CHECKs:
a violation raises RuntimeError before anything is launched)."""
from __future__ import annotations

import torch


def fail(msg: str):
    raise RuntimeError(msg)


def gpu(t: torch.Tensor, name: str):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        fail(f"{name} must be a CUDA tensor")


def same_device(ref: torch.Tensor, t: torch.Tensor, name: str):
    if t.device != ref.device:
        fail(f"{name} must be on {ref.device}, got {t.device}")


def contiguous(t: torch.Tensor, name: str):
    if not t.is_contiguous():
        fail(f"{name} must be contiguous")


def dtype(t: torch.Tensor, dt, name: str):
    dts = dt if isinstance(dt, (tuple, list)) else (dt,)
    if t.dtype not in dts:
        fail(f"{name} must be {' or '.join(str(d) for d in dts)}, got {t.dtype}")


def cuda_tensor(ref, t, dt, name):
    gpu(t, name)
    if ref is not None:
        same_device(ref, t, name)
    contiguous(t, name)
    if dt is not None:
        dtype(t, dt, name)


def combine_args(expert_output, topk_pos, topk_weights, output, n, h, k, out_dtype):
    """The weighted combines read ``topk_pos`` / ``topk_weights`` [n*k] and ``expert_output`` [rows, h] and write
    ``output`` [n, h]: dtype, device, contiguity and minimum sizes, so that no wrong-typed or short tensor is
    ever handed to the kernel as a raw pointer."""
    if n < 0 or h <= 0:
        fail(f"N must be >= 0 and H positive, got N={n} H={h}")
    cuda_tensor(None, expert_output, torch.bfloat16, "expert_output")
    cuda_tensor(expert_output, topk_pos, torch.int32, "topk_pos")
    cuda_tensor(expert_output, topk_weights, torch.float32, "topk_weights")
    cuda_tensor(expert_output, output, out_dtype, "output")
    if topk_pos.numel() < n * k or topk_weights.numel() < n * k:
        fail(f"topk_pos / topk_weights must hold N*K = {n * k} elements")
    if output.numel() < n * h:
        fail(f"output must hold N*H = {n * h} elements")
    if expert_output.dim() < 2 or expert_output.size(-1) != h:      # [rows, H] or the masked [E_local, max_tokens, H]
        fail(f"expert_output must have rows of H={h} elements")


FP8_BYTES = (torch.uint8, torch.float8_e4m3fn)
