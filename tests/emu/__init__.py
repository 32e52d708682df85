"""TEST INFRASTRUCTURE: loads the CPU-emulation build of the kernel sources (tests/emu/build_emu.py) with the
package's ctypes signatures.  "Device memory" is host memory here: tests pass numpy arrays."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_handle = None


def load():
    global _handle
    if _handle is None:
        from batchgen_amd import _lib
        from tests.emu.build_emu import build
        h = C.CDLL(build())
        for name, (res, args) in _lib._SIGS.items():
            fn = getattr(h, name, None)
            if fn is not None:
                fn.restype, fn.argtypes = res, args
        h.emu_set_async_mode.argtypes = [C.c_int]
        h.emu_set_schedule.argtypes = [C.c_int]
        h.emu_set_wait_slack.argtypes = [C.c_int]
        h.emu_stats.argtypes = [C.c_void_p]
        h.emu_guarded_alloc.restype, h.emu_guarded_alloc.argtypes = C.c_void_p, [C.c_size_t]
        h.emu_guarded_free.argtypes = [C.c_void_p]
        h.emu_e4m3_to_f32.restype, h.emu_e4m3_to_f32.argtypes = C.c_float, [C.c_uint8]
        h.emu_f32_to_e4m3.restype, h.emu_f32_to_e4m3.argtypes = C.c_uint8, [C.c_float]
        _handle = h
    return _handle


def p(a: np.ndarray):
    """Pointer to a C-contiguous array's data (the caller keeps the array alive)."""
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def ok(h, status: int):
    if status != 0:
        raise RuntimeError(h.bgmoe_last_error().decode())


def stats(h):
    out = (C.c_uint64 * 4)()
    h.emu_stats(out)
    return dict(zip(("launches", "blocks", "rendezvous", "async_loads"), [int(v) for v in out]))


class _NoDeviceContext:
    def __init__(self, *a, **k):
        pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


class _NullStream:
    cuda_stream = None

    def __init__(self, *a, **k):
        pass

    def wait_event(self, ev):
        pass

    def wait_stream(self, st):
        pass

    def synchronize(self):
        pass


class _NullEvent:
    """torch.cuda.Event stand-in: the host's clock (the time the emulation took, of no meaning for the GPU)."""

    def __init__(self, *a, **k):
        self.t = 0.0

    def record(self, stream=None):
        import time
        self.t = time.perf_counter()

    def elapsed_time(self, other):
        return max((other.t - self.t) * 1e3, 1e-6)

    def synchronize(self):
        pass

    def wait(self, stream=None):
        pass


def run_package_on_emulator(monkeypatch):
    """For a test: the package's host code (its ctypes layer classes) calls the emulation build instead of the GPU
    library, with CPU tensors standing for device memory.  Patches, through pytest's monkeypatch, the library
    handle, ``torch.cuda.current_stream`` / ``device`` / ``synchronize`` and the op wrappers' "is a CUDA tensor"
    check; everything is undone when the test ends."""
    import torch
    from batchgen_amd import _lib
    from batchgen_amd.kernels import _checks
    h = load()
    monkeypatch.setattr(_lib, "_lib", h)
    monkeypatch.setattr(torch.cuda, "current_stream", lambda *a, **k: _NullStream())
    monkeypatch.setattr(torch.cuda, "device", _NoDeviceContext)
    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a, **k: None)
    monkeypatch.setattr(torch.cuda, "Stream", _NullStream)
    monkeypatch.setattr(torch.cuda, "Event", _NullEvent)
    monkeypatch.setattr(torch.cuda, "stream", _NoDeviceContext)
    monkeypatch.setattr(torch.cuda, "set_device", lambda *a, **k: None)
    monkeypatch.setattr(torch.cuda, "empty_cache", lambda *a, **k: None)
    # host code that asks a tensor whether it lives on the GPU (the emulated device memory is host memory)
    monkeypatch.setattr(torch.Tensor, "is_cuda", property(lambda self: True))

    def tensor_only(t, name):
        if not isinstance(t, torch.Tensor):
            _checks.fail(f"{name} must be a tensor")
    monkeypatch.setattr(_checks, "gpu", tensor_only)

    from batchgen_amd.kernels import _workspace
    pool = {}

    def cpu_scratch(kind, device, need, floor=0):
        buf = pool.get(kind)
        if buf is None or buf.numel() < need:
            buf = pool[kind] = torch.empty(max(int(need), int(floor)), dtype=torch.uint8)
        return buf
    monkeypatch.setattr(_workspace, "scratch", cpu_scratch)
    return h


def guarded(a: np.ndarray) -> np.ndarray:
    """A copy of ``a`` in a buffer that ends at a page boundary with an inaccessible page behind it (and one in front):
    a kernel that reads or writes past the end of the array faults at once, with a message that says by how much,
    instead of quietly touching the neighbouring heap.  The size is rounded up to 16 bytes (slack at the front)."""
    import weakref
    h = load()
    a = np.ascontiguousarray(a)
    nbytes = max(a.nbytes, 16)
    addr = h.emu_guarded_alloc(nbytes)
    if not addr:
        raise MemoryError("guarded allocation failed")
    padded = (nbytes + 15) // 16 * 16
    buf = (C.c_uint8 * a.nbytes).from_address(addr + padded - nbytes if a.nbytes else addr)
    out = np.frombuffer(buf, dtype=a.dtype, count=a.size).reshape(a.shape)
    out[...] = a
    weakref.finalize(buf, h.emu_guarded_free, addr)
    return out
