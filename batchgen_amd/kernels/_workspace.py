"""Scratch buffers of the op wrappers whose reference signatures carry no workspace argument (dispatch histograms,
router-GEMM split-K planes, dense-GEMM partial sums).

One buffer per (kind, device, stream): two streams never share scratch, so ops that overlap on different streams do
not race.  A buffer that has been handed out is never freed: when a call needs more, a larger buffer takes its
place for later calls and the old one stays alive, because a HIP graph captured earlier still writes to its address
on every replay (freeing it would let the allocator hand that memory to another tensor).  Growth at least doubles,
so the retired buffers together stay below the size of the live one.  Callers that own their scratch (the layer
objects) do not come through here."""
from __future__ import annotations

import torch

from .._lib import lib

_LIVE = {}
_RETIRED = []


def scratch(kind: str, device, need: int, floor: int = 0):
    """A uint8 buffer of at least ``need`` bytes for ``kind`` on the current stream of ``device``."""
    device = torch.device(device)
    index = device.index if device.index is not None else torch.cuda.current_device()
    key = (kind, index, torch.cuda.current_stream(index).cuda_stream)
    buf = _LIVE.get(key)
    if buf is None or buf.numel() < need:
        size = max(int(need), int(floor), 2 * buf.numel() if buf is not None else 0)
        if buf is not None:
            _RETIRED.append(buf)
        buf = torch.empty(size, dtype=torch.uint8, device=torch.device("cuda", index))
        _LIVE[key] = buf
    return buf


def retired_bytes() -> int:
    return sum(b.numel() for b in _RETIRED)


def dispatch_workspace(device, nk: int, e_local: int):
    need = int(lib().bgmoe_dispatch_workspace_bytes(int(nk), int(e_local)))
    if need == 0:
        return None, 0
    buf = scratch("dispatch", device, need, 1 << 20)
    return buf, buf.numel()


def router_gemm_workspace(device, n: int, h: int, e: int):
    """Split-K planes of the router GEMM."""
    need = int(lib().bgmoe_router_gemm_workspace_bytes(int(n), int(h), int(e)))
    if need == 0:
        return None, 0
    buf = scratch("router_gemm", device, need, 1 << 20)
    return buf, buf.numel()


def dense_gemm_workspace(device, nbytes: int):
    """Partial sums of the block-split dense GEMM."""
    if nbytes <= 0:
        return None
    return scratch("dense_gemm", device, int(nbytes), 1 << 24)
