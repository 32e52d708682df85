"""Build libbgmoe.so (HIP kernels + C ABI) for gfx950 with hipcc.

    python -m batchgen_amd.build            # incremental
    python -m batchgen_amd.build --force    # recompile everything

hipcc cross-compiles without a GPU.  Objects land in batchgen_amd/csrc/build/,
the library in batchgen_amd/lib/libbgmoe.so (both git-ignored).
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libbgmoe.so")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")

ARCH = "gfx950"
# -ffp-contract=off: the routers, the quantiser and the combine are specified as
#   sequences of individually rounded fp32 operations; kernels that want an FMA
#   call fmaf() explicitly.
# -fhip-fp32-correctly-rounded-divide-sqrt: x / s in the quantiser is IEEE division.
# packed-fp32-ops is disabled on purpose (the compiler must not form v_pk_*_f32).
FLAGS = [
    "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", f"-I{INCLUDE}",
]


def hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _newer(target: str, deps) -> bool:
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ, src[:-4] + ".o")
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers.append(os.path.join(INCLUDE, "bgmoe.h"))
    deps = [os.path.join(CSRC, src)] + headers
    if not force and _newer(obj, deps):
        return obj
    cmd = [hipcc()] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    if src in NO_SPILL:
        cmd.insert(-4, "-Rpass-analysis=kernel-resource-usage")
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    if src in NO_SPILL:
        _check_no_spill(src, r.stderr, obj)
    return obj


# Kernels whose weight loads are issued from inline asm and waited for by hand: a register that such a load is
# still writing must never be spilled or copied, so these files must compile without scratch memory.
NO_SPILL = {"gemm_fp8_streamk.hip": "fp8_streamk_kernel"}


def _check_no_spill(src: str, remarks: str, obj: str) -> None:
    import re
    name, bad, seen = None, [], 0
    for line in remarks.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
        if m and name and NO_SPILL[src] in name:
            seen += 1
            if int(m.group(1)) != 0:
                bad.append(f"{name}: {m.group(1)} bytes of scratch per lane")
    if bad or seen == 0:
        os.remove(obj)
        raise RuntimeError(f"{src}: kernels must not spill registers ({'; '.join(bad) or 'no resource remarks found'})")


def build(force: bool = False, jobs: int = 4, verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    if force or not _newer(LIB, objs):
        cmd = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-fno-gpu-rdc", "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources")
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-j", type=int, default=4)
    a = ap.parse_args()
    try:
        build(force=a.force, jobs=a.j)
    except RuntimeError as e:
        print(e, file=sys.stderr)
        sys.exit(1)
