"""TEST INFRASTRUCTURE: builds ``tests/emu/_build/libbgmoe_emu.so``, the library's kernel sources compiled as plain
C++ for the host against the CPU emulator of this directory (``shim/hip/hip_runtime.h``, ``emu_core.cc``).

The sources are staged unchanged except for two things the host compiler cannot take: ``bgmoe_async.h`` (gfx950
inline assembly) is replaced by this directory's version with the same names, and a dynamic-LDS declaration
(``extern __shared__ T name[];``) becomes a pointer to the emulator's LDS buffer.  Only tests load the result.
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
           "activation.hip", "norm_quant.hip", "gemm_fp8_dense.hip", "runtime.hip"]
DYNAMIC_LDS = re.compile(r"extern\s+__shared__\s+(?:__align__\(\d+\)\s+)?(\w+)\s+(\w+)\[\];")
# Lanes of a wave are not in lockstep under the emulator.  Where a kernel that a GPU has run passes data from lane to
# lane through LDS with no rendezvous in between (on the GPU a wave's LDS accesses execute in order, and the source is
# left as it is because an extra compiler barrier there changes the register allocation of a measured kernel), the
# STAGED copy gets one: (file, text after which "emu::wave_sync();" is inserted).
LOCKSTEP_POINTS = [
    ("gemm_fp8_tiled.hip", "            *reinterpret_cast<uint2*>(patch + r16 * kEpiPitch + (16 * t + 4 * kq) * 2) = o;\n          }\n"),
    ("gemm_fp8_tiled.hip", "              *reinterpret_cast<uint4*>(g.out + (row0 + tok0 + row) * g.n + col0 + (lane & 7) * 8) = v;\n          }\n"),
]


def _inputs():
    files = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC)) if f.endswith((".h", ".hip"))]
    files += [os.path.join(HERE, f) for f in ("emu_core.cc", "emu_stubs.cc", "bgmoe_async.h", "build_emu.py")]
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
           os.path.join(HERE, "emu_core.cc"), os.path.join(HERE, "emu_stubs.cc")]
    cmd += [os.path.join(stage, s.replace(".hip", ".cc")) for s in SOURCES]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout[-4000:] + r.stderr[-12000:])
        raise RuntimeError("emulation build failed")
    return LIB


if __name__ == "__main__":
    print("built", build(force=True))
