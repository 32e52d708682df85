"""TEST INFRASTRUCTURE: builds ``tests/emu/_build/libbgmoe_emu.so``, the library's kernel sources compiled as plain
C++ for the host against the CPU emulator of this directory (``shim/hip/hip_runtime.h``, ``emu_core.cc``).

The sources are staged unchanged except for what the host compiler cannot take -- ``bgmoe_async.h`` (gfx950 inline
assembly) is replaced by this directory's version with the same names, a dynamic-LDS declaration
(``extern __shared__ T name[];``) becomes a pointer to the emulator's LDS buffer, the stream-K form's assembly helpers
get plain C++ bodies -- and for what the emulator has to be told: the explicit global loads of ``bgmoe_common.h``
report themselves, and two lane-to-lane exchanges of a measured kernel get a rendezvous.  Only tests load the result.
"""
from __future__ import annotations

import os
import re
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "batchgen_amd", "csrc")
BUILD = os.path.join(HERE, "_build")
LIB = os.path.join(BUILD, "libbgmoe_emu.so")
CLANG = "/opt/rocm/llvm/bin/clang++"

# kernels that run under the emulator (their launch code and entry points included)
SOURCES = ["gemm_fp8_skinny.hip", "gemm_fp8_tiled.hip", "gemm_fp8_tiled_k64.hip", "gemm_mxfp4_skinny.hip", "permute.hip",
           "router_gemm.hip", "weight_repack.hip", "layer.hip", "act_quant.hip", "combine.hip", "router.hip",
           "activation.hip", "norm_quant.hip", "gemm_fp8_dense.hip", "runtime.hip", "gemm_fp8_streamk.hip"]
DYNAMIC_LDS = re.compile(r"extern\s+__shared__\s+(?:__align__\(\d+\)\s+)?(\w+)\s+(\w+)\[\];")
# Lanes of a wave are not in lockstep under the emulator.  Where a kernel that a GPU has run passes data from lane to
# lane through LDS with no rendezvous in between (on the GPU a wave's LDS accesses execute in order, and the source is
# left as it is because an extra compiler barrier there changes the register allocation of a measured kernel), the
# STAGED copy gets one: (file, text after which "emu::wave_sync();" is inserted).
# The stream-K form's five small helpers are gfx950 inline assembly (loads the compiler must not reorder, write-through
# stores, a per-lane asynchronous LDS load): the staged copy gets plain C++ bodies with the same meaning.
STREAMK_ASM = [
    (re.compile(r'asm volatile\("s_nop 4\\n\\tglobal_load_dwordx4 %0, %2, %3\\n\\tglobal_load_dwordx4 %1, %2, %3 offset:1024"\s*:[^;]*;'),
     "lo = *reinterpret_cast<const intx4*>(base + off); hi = *reinterpret_cast<const intx4*>(base + off + 1024);"),
    (re.compile(r'asm volatile\("s_nop 4\\n\\tglobal_load_dwordx4 %0, %2, %3 nt\\n\\tglobal_load_dwordx4 %1, %2, %3 offset:1024 nt"\s*:[^;]*;'),
     "lo = *reinterpret_cast<const intx4*>(base + off); hi = *reinterpret_cast<const intx4*>(base + off + 1024);"),
    (re.compile(r'asm volatile\("s_nop 4\\n\\tglobal_store_dwordx4 %0, %1, %2 sc0 sc1"[^;]*;'),
     "*reinterpret_cast<floatx4*>(reinterpret_cast<uint8_t*>(const_cast<floatx4*>(base)) + off) = v;"),
    (re.compile(r'asm volatile\("s_nop 4\\n\\tglobal_load_dwordx4 %0, %1, %2 sc0 sc1"[^;]*;'),
     "v = *reinterpret_cast<const floatx4*>(reinterpret_cast<const uint8_t*>(base) + off);"),
    (re.compile(r'asm volatile\("s_nop 4\\n\\ts_mov_b32 m0, %0\\n\\ts_nop 0\\n\\tglobal_load_lds_dword %1, off"[^;]*;'),
     "emu::async_load(lane_ptr, 0, lds_base, 4, false);"),
    (re.compile(r'asm volatile\(""\s*:\s*"\+v"[^;]*;'), "(void)0;"),
]
# The kernels' explicit global loads (bgmoe_common.h) report themselves to the emulator, which under its counted lazy
# model gives them a place in the lane's queue of outstanding vector-memory operations.
COUNTED_LOADS = re.compile(r"(__device__ __forceinline__ (?:intx4|float|uint32_t) gload_(?:x4|x4_stream|f32|u32)\([^)]*\) \{\n)")
LOCKSTEP_POINTS = [
    ("gemm_fp8_tiled.hip", "            *reinterpret_cast<uint2*>(patch + r16 * kEpiPitch + (16 * t + 4 * kq) * 2) = o;\n          }\n"),
    ("gemm_fp8_tiled.hip", "              *reinterpret_cast<uint4*>(g.out + (row0 + tok0 + row) * g.n + col0 + (lane & 7) * 8) = v;\n          }\n"),
]


def _inputs():
    files = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC)) if f.endswith((".h", ".hip"))]
    files += [os.path.join(HERE, f) for f in ("emu_core.cc", "bgmoe_async.h", "build_emu.py")]
    files += [os.path.join(HERE, "shim", "hip", "hip_runtime.h"), os.path.join(ROOT, "include", "bgmoe.h")]
    return files


def up_to_date() -> bool:
    if not os.path.exists(LIB):
        return False
    t = os.path.getmtime(LIB)
    return all(os.path.getmtime(f) <= t for f in _inputs())


def build(force: bool = False) -> str:
    if not force and up_to_date():
        return LIB
    stage = os.path.join(BUILD, "stage", "pkg", "csrc")          # two levels under include/, as in the package
    shutil.rmtree(os.path.join(BUILD, "stage"), ignore_errors=True)
    os.makedirs(stage)
    os.makedirs(os.path.join(BUILD, "stage", "include"))
    shutil.copy(os.path.join(ROOT, "include", "bgmoe.h"), os.path.join(BUILD, "stage", "include", "bgmoe.h"))
    for f in os.listdir(CSRC):
        if not f.endswith((".h", ".hip")) or f == "bgmoe_async.h":
            continue
        text = open(os.path.join(CSRC, f)).read()
        text = DYNAMIC_LDS.sub(r"\1* const \2 = reinterpret_cast<\1*>(emu::dynamic_lds());", text)
        if f == "bgmoe_common.h":
            text, hits = COUNTED_LOADS.subn(r"\1  emu::count_vm_load();\n", text)
            if hits != 4:
                raise RuntimeError(f"{f}: expected the four gload_* helpers, found {hits}")
        if f == "gemm_fp8_streamk.hip":
            for rx, body in STREAMK_ASM:
                text, hits = rx.subn(body, text)
                if hits == 0:
                    raise RuntimeError(f"{f}: an inline-assembly helper the emulation build replaces was not found: {rx.pattern[:60]}")
            if "asm volatile" in text:
                raise RuntimeError(f"{f}: inline assembly without an emulated body")
        for name, anchor in LOCKSTEP_POINTS:
            if name == f:
                if text.count(anchor) != 1:
                    raise RuntimeError(f"{f}: the lockstep point {anchor!r} is not unique in the source any more")
                text = text.replace(anchor, anchor + "          emu::wave_sync();\n")
        with open(os.path.join(stage, f.replace(".hip", ".cc")), "w") as out:
            out.write(text)
    shutil.copy(os.path.join(HERE, "bgmoe_async.h"), os.path.join(stage, "bgmoe_async.h"))
    cmd = [CLANG, "-std=c++17", "-O1", "-g", "-fPIC", "-shared", "-fno-strict-aliasing", "-ffp-contract=off",
           "-Wno-unknown-attributes", "-Wno-unused-value", "-Wno-ignored-attributes",
           f"-I{os.path.join(HERE, 'shim')}", f"-I{stage}", "-o", LIB,
           os.path.join(HERE, "emu_core.cc")]
    cmd += [os.path.join(stage, s.replace(".hip", ".cc")) for s in SOURCES]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout[-4000:] + r.stderr[-12000:])
        raise RuntimeError("emulation build failed")
    return LIB


if __name__ == "__main__":
    print("built", build(force=True))
