"""ctypes binding of libbgmoe.so (the C ABI declared in include/bgmoe.h).

There is no fallback: if the library is missing or a symbol is absent the
import of an op module fails with ImportError / RuntimeError, and every call
that returns a non-zero status raises RuntimeError with the library's message.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libbgmoe.so")

vp = C.c_void_p
i32 = C.c_int
i64 = C.c_int64
f32 = C.c_float
sz = C.c_size_t


class Fp8Weight(C.Structure):
    """bgmoe_fp8_weight"""
    _fields_ = [("w", vp), ("w_group_stride", i64), ("w_ptrs", vp), ("scale", vp),
                ("scale_group_stride", i64), ("scale_nb_stride", i64), ("scale_ptrs", vp),
                ("layout", i32), ("reserved", i32)]


class Mxfp4Weight(C.Structure):
    """bgmoe_mxfp4_weight"""
    _fields_ = [("w", vp), ("w_group_stride", i64), ("w_ptrs", vp), ("scale", vp), ("scale_group_stride", i64),
                ("scale_ptrs", vp), ("layout", i32), ("reserved", i32)]


class Fp8Act(C.Structure):
    """bgmoe_fp8_act"""
    _fields_ = [("x", vp), ("scale", vp), ("scale_row_stride", i64), ("scale_kb_stride", i64),
                ("scale_group_stride", i64)]


_SIGS = {
    "bgmoe_last_error": (C.c_char_p, []),
    "bgmoe_version": (i32, []),
    "bgmoe_init": (i32, []),
    "bgmoe_prof_enable": (i32, [i32]),
    "bgmoe_prof_kernel_count": (i32, []),
    "bgmoe_prof_kernel_name": (C.c_char_p, [i32]),
    "bgmoe_prof_collect": (i32, [C.POINTER(C.c_double), C.POINTER(i64), i32]),
    "bgmoe_fused_gate": (i32, [vp, vp, i32, i32, i32, i32, i32, f32, i32, vp, vp, vp]),
    "bgmoe_gate_sigmoid_topk": (i32, [vp, i64, vp, i32, i32, i32, f32, vp, i32, vp, vp, vp, i32, vp, i32, i32, vp]),
    "bgmoe_router_gemm_workspace_bytes": (sz, [i32, i32, i32]),
    "bgmoe_router_gemm": (i32, [vp, vp, i32, i32, i32, vp, i32, i32, vp, vp, sz, vp]),
    "bgmoe_router_gemm_gate": (i32, [vp, vp, vp, i32, i32, i32, i32, i32, i32, f32, vp, vp, vp, i32, vp, sz, vp]),
    "bgmoe_set_router_gemm_plan": (i32, [i32, i32]),
    "bgmoe_add_rmsnorm_fp8_quant": (i32, [vp, vp, vp, i64, i32, f32, vp, vp, vp, i64, i64, vp, vp, vp, vp]),
    "bgmoe_selfcheck_sigmoid": (i32, [C.c_uint32, C.c_uint64, vp, vp, vp]),
    "bgmoe_layout_to_segments": (i32, [vp, i64, i32, vp, vp, vp, vp]),
    "bgmoe_silu_mul_group_quant": (i32, [vp, vp, i64, i64, vp, vp, i32, i64, i32, i32, vp, i64, i64, vp, i64, i64, i64,
                                         vp, vp]),
    "bgmoe_selfcheck_scale_division": (i32, [C.c_uint64, C.c_uint64, vp, vp, vp]),
    "bgmoe_situ_and_mul": (i32, [vp, i64, i32, i64, f32, f32, vp, i64, vp]),
    "bgmoe_rmsnorm": (i32, [vp, vp, i64, i32, f32, vp, vp]),
    "bgmoe_act_quant_rows": (i32, [vp, i64, i32, vp, vp, i64, i64, vp]),
    "bgmoe_fp8_dense_gemm": (i32, [vp, vp, vp, i64, i32, i64, i32, i32, vp, vp, i64, vp]),
    "bgmoe_fp8_dense_gemm_partials": (i32, [vp, vp, vp, i64, i32, i64, i32, i32, vp, i64, C.POINTER(i32), vp]),
    "bgmoe_silu_mul_group_quant_partials": (i32, [vp, i32, i64, i64, i32, i32, vp, i64, vp, i64, i64, vp]),
    "bgmoe_fp8_dense_gemm_workspace": (i64, [i64, i32, i32, i32]),
    "bgmoe_act_quant_rows_1d": (i32, [vp, i64, i32, vp, vp, i64, i64, vp, vp]),
    "bgmoe_act_quant_3d": (i32, [vp, vp, i32, i32, i32, vp, vp, vp]),
    "bgmoe_act_quant_ragged": (i32, [vp, vp, vp, i32, i64, i32, vp, vp, i32, vp]),
    "bgmoe_silu_mul_3d": (i32, [vp, vp, vp, i32, i32, i32, vp, vp]),
    "bgmoe_fused_silu_quant_3d": (i32, [vp, vp, vp, i32, i32, i32, vp, vp, vp]),
    "bgmoe_deepep_ll_scale_repack": (i32, [vp, vp, vp, i32, i32, i32, i32, vp, vp]),
    "bgmoe_dispatch_workspace_bytes": (sz, [i64, i32]),
    "bgmoe_silu_and_mul": (i32, [vp, i64, i32, i64, vp, i64, vp]),
    "bgmoe_bf16_linear": (i32, [vp, vp, i32, i32, i32, vp, vp, sz, vp]),
    "bgmoe_fp8_streamk_workspace_bytes": (sz, []),
    "bgmoe_debug_streamk_trace": (i32, [vp]),
    "bgmoe_set_streamk_xcd_weights": (i32, [vp]),
    "bgmoe_debug_streamk_status": (i32, [vp]),
    "bgmoe_dispatch_scatter_3d": (i32, [vp, vp, i32, i32, i32, vp, i32, i32, i32, vp, vp, vp, vp, sz, vp]),
    "bgmoe_dispatch_scatter_ragged": (i32, [vp, vp, i32, i32, i32, vp, i64, i32, i32, vp, vp, vp, vp, i32, vp, sz, vp]),
    "bgmoe_dispatch_static_max_pairs": (sz, [i32]),
    "bgmoe_dispatch_scatter_ragged_static": (i32, [vp, vp, i32, i32, i32, vp, i64, i32, i32, vp, vp, vp, vp, i32, vp]),
    "bgmoe_dispatch_row_metadata": (i32, [vp, vp, i64, i32, vp, i64, vp, vp, vp, vp]),
    "bgmoe_scatter_fp8_rows": (i32, [vp, vp, i64, i64, vp, i32, i32, i32, vp, vp, i64, i64, vp]),
    "bgmoe_scatter_quant": (i32, [vp, vp, i32, i32, i32, vp, vp, i64, i64, vp]),
    "bgmoe_reduce_weighted_scatter": (i32, [vp, vp, vp, i32, i32, i32, vp, i32, vp, i32, vp]),
    "bgmoe_reduce_weighted_scatter_fp32": (i32, [vp, vp, vp, i32, i32, i32, vp, vp]),
    "bgmoe_reduce_weighted_scatter_bf16_ordered": (i32, [vp, vp, vp, vp, i32, i32, i32, vp, vp]),
    "bgmoe_set_skinny_max_rows": (i32, [i32]),
    "bgmoe_set_skinny_tall_min_rows": (i32, [i32]),
    "bgmoe_set_skinny_gemm_stages": (i32, [i32]),
    "bgmoe_set_skinny_s1_stages": (i32, [i32]),
    "bgmoe_set_mxfp4_variant": (i32, [i32]),
    "bgmoe_set_tiled_variant": (i32, [i32]),
    "bgmoe_fp8_weight_repack": (i32, [vp, vp, i32, i32, i32, vp]),
    "bgmoe_mxfp4_weight_repack": (i32, [vp, vp, vp, vp, i32, i32, i32, vp]),
    "bgmoe_mxfp4_grouped_gemm": (i32, [vp, C.POINTER(Mxfp4Weight), vp, vp, i32, i64, i32, i32, vp, vp, i64, vp]),
    "bgmoe_mxfp4_fused_s1": (i32, [vp, C.POINTER(Mxfp4Weight), C.POINTER(Mxfp4Weight), vp, vp, i32, i64, i32, i32, vp,
                                   vp, i32, i64, vp]),
    "bgmoe_mxfp4_fused_s1_gather": (i32, [vp, i64, vp, i32, C.POINTER(Mxfp4Weight), C.POINTER(Mxfp4Weight), vp, vp, i32,
                                          i64, i32, i32, vp, vp, i32, i64, vp]),
    "bgmoe_dispatch_index_3d": (i32, [vp, i32, i32, i32, i32, i32, vp, vp, vp, vp, vp, sz, vp]),
    "bgmoe_compact_expert_data": (i32, [vp, i32, vp, vp, vp, vp, vp]),
    "bgmoe_fp8_grouped_gemm": (i32, [C.POINTER(Fp8Act), C.POINTER(Fp8Weight), vp, vp, i32, i64, i32, i32, vp, vp]),
    "bgmoe_fp8_fused_s1": (i32, [C.POINTER(Fp8Act), C.POINTER(Fp8Weight), C.POINTER(Fp8Weight), vp, vp, i32,
                                 i64, i32, i32, vp, vp, vp, i64, i64, vp]),
    "bgmoe_fp8_grouped_gemm_balanced": (i32, [C.POINTER(Fp8Act), C.POINTER(Fp8Weight), vp, vp, i32, i64, i32, i32, vp,
                                              i64, vp, sz, vp]),
    "bgmoe_fp8_fused_s1_balanced": (i32, [C.POINTER(Fp8Act), C.POINTER(Fp8Weight), C.POINTER(Fp8Weight), vp, vp, i32,
                                          i64, i32, i32, vp, vp, vp, i64, i64, i64, vp, sz, vp]),
}

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is not built; run `python -m batchgen_amd.build` "
                "(hipcc, gfx950). There is no CPU fallback.")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGS.items():
            try:
                fn = getattr(handle, name)
            except AttributeError as exc:
                raise RuntimeError(f"libbgmoe.so has no symbol {name}; rebuild batchgen_amd") from exc
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def register(name: str, restype, argtypes):
    """Declare one more exported symbol (used by modules that add entry points)."""
    _SIGS[name] = (restype, argtypes)
    if _lib is not None:
        fn = getattr(_lib, name)
        fn.restype = restype
        fn.argtypes = argtypes


def check(status: int) -> None:
    if status != 0:
        msg = lib().bgmoe_last_error()
        raise RuntimeError((msg or b"unknown error").decode("utf-8", "replace"))


def ptr(t):
    """Device pointer of a torch tensor (None -> NULL)."""
    return None if t is None else t.data_ptr()


def stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def exported_symbols():
    return sorted(_SIGS)


def prof_enable(on: bool) -> None:
    check(lib().bgmoe_prof_enable(int(on)))


def prof_collect():
    """-> {kernel name: (total_ms, launches)} since the last collect (synchronises the device)."""
    n = lib().bgmoe_prof_kernel_count()
    ms = (C.c_double * n)()
    cnt = (i64 * n)()
    check(lib().bgmoe_prof_collect(ms, cnt, n))
    return {lib().bgmoe_prof_kernel_name(i).decode(): (ms[i], int(cnt[i])) for i in range(n) if cnt[i]}
