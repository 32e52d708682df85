"""Host-side mirror of the reference's ``batchgen_kernels`` extension loader.

``load_extension("batchgen_kernels.moe._C_routing")`` (or the same name under
``batchgen_amd.kernels``) returns a module that exports the reference
extension's op names with the same positional argument order
(batchgen_kernels/__init__.py:24-45 is the loader this replaces).  The ops are
thin argument checkers over libbgmoe.so's C ABI; a missing library raises
ImportError, exactly what the reference callers treat as "kernel not built".
"""
from __future__ import annotations

import importlib

_PREFIXES = ("batchgen_kernels.", "batchgen_amd.kernels.")

AVAILABLE = (
    "common._C_mgn_ops",
    "moe._C_routing",
    "moe._C_dispatch_scatter_3d",
    "moe._C_fp8_blockwise_ops",
    "moe._C_fp8_blockwise_gemm",
    "moe._C_marlin_grouped_gemm",
    "attention._C_add_rmsnorm_fp8_quant",
)


def load_extension(module_name: str, allow_dev_jit: bool = True):
    """Import the gfx950 implementation of a reference extension module."""
    tail = module_name
    for p in _PREFIXES:
        if module_name.startswith(p):
            tail = module_name[len(p):]
            break
    if tail not in AVAILABLE:
        raise ImportError(f"No gfx950 implementation of {module_name}. Available: {list(AVAILABLE)}")
    return importlib.import_module("batchgen_amd.kernels." + tail)
