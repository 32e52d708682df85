"""Per-device scratch for the multi-block dispatch path, allocated once per
size class and kept (graph-static address after the first call)."""
from __future__ import annotations

import torch

from .._lib import lib

_CACHE = {}


def dispatch_workspace(device, nk: int, e_local: int):
    need = int(lib().bgmoe_dispatch_workspace_bytes(int(nk), int(e_local)))
    if need == 0:
        return None, 0
    key = (device.type, device.index)
    buf = _CACHE.get(key)
    if buf is None or buf.numel() < need:
        buf = torch.empty(max(need, 1 << 20), dtype=torch.uint8, device=device)
        _CACHE[key] = buf
    return buf, buf.numel()


_ROUTER_CACHE = {}


def router_gemm_workspace(device, n: int, h: int, e: int):
    """Split-K planes of the router GEMM; grown on demand, kept per device."""
    need = int(lib().bgmoe_router_gemm_workspace_bytes(int(n), int(h), int(e)))
    if need == 0:
        return None, 0
    key = (device.type, device.index)
    buf = _ROUTER_CACHE.get(key)
    if buf is None or buf.numel() < need:
        buf = torch.empty(need, dtype=torch.uint8, device=device)
        _ROUTER_CACHE[key] = buf
    return buf, buf.numel()
