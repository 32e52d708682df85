"""TEST INFRASTRUCTURE: loads the CPU-emulation build of the kernel sources (tests/emu/build_emu.py) with the
package's ctypes signatures.  "Device memory" is host memory here: tests pass numpy arrays."""
from __future__ import annotations

import ctypes as C

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
        h.emu_stats.argtypes = [C.c_void_p]
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
