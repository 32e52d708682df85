"""Helpers shared by the tests."""
import numpy as np
import torch


def bf16(x: np.ndarray, device=None) -> torch.Tensor:
    t = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.bfloat16)
    return t.to(device) if device is not None else t


def rand_bf16(gen: torch.Generator, *shape, scale=1.0) -> torch.Tensor:
    return (torch.randn(*shape, generator=gen) * scale).to(torch.bfloat16)


def say(*a):
    print(*a, flush=True)
