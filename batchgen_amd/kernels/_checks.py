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


FP8_BYTES = (torch.uint8, torch.float8_e4m3fn)
