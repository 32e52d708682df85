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
    asm_job = _start_asm(src, obj) if src in NO_FLAT else None       # beside the compile, not after it
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        if asm_job:
            asm_job.kill()
            asm_job.communicate()
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    if src in NO_SPILL:
        _check_no_spill(src, r.stderr, obj)
    if asm_job:
        _check_no_flat(src, obj, asm_job)
    return obj


# Kernels whose loads are issued from inline asm and waited for by hand: a register that such a load is still
# writing must never be spilled or copied, so these kernels must compile without scratch memory.  The LDS-tiled
# K = 64 kernel must also keep two waves per SIMD (at most 256 registers, no AGPR copies of its accumulators) and
# leave room for its 4 x 33 KB ring in the CU's 160 KB of LDS.  Checked on every build from the compiler's own
# resource remarks; a kernel over budget fails the build.
RESOURCE_GATES = {
    # the weight-streaming kernels keep their prefetch stages in registers: two blocks per CU and no spills, whatever
    # variant is added (a variant whose paths together need more than 256 registers drops to one block per CU)
    "gemm_fp8_skinny.hip": dict(kernel="fp8_skinny_kernel", min_occupancy=2),
    "gemm_mxfp4_skinny.hip": dict(kernel="mxfp4_skinny_kernel", min_occupancy=2),
    "gemm_fp8_streamk.hip": dict(kernel="fp8_streamk_kernel"),
    "gemm_fp8_tiled_k64.hip": dict(kernel="fp8_tiled_k64_kernel", max_vgprs=256, max_agprs=0,
                                   max_static_lds=163840 - 4 * (32768 + 1024), min_occupancy=2),
}
NO_SPILL = RESOURCE_GATES           # (the name the compile step tests membership with)


def _check_no_spill(src: str, remarks: str, obj: str) -> None:
    import re
    gate = RESOURCE_GATES[src]
    fields = {"ScratchSize [bytes/lane]": ("scratch", lambda v: v == 0, "must be 0"),
              "VGPRs": ("max_vgprs", None, None), "AGPRs": ("max_agprs", None, None),
              "LDS Size [bytes/block]": ("max_static_lds", None, None),
              "Occupancy [waves/SIMD]": ("min_occupancy", None, None)}
    name, bad, seen = None, [], 0
    for line in remarks.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            continue
        if not name or gate["kernel"] not in name:
            continue
        m = re.search(r"remark:\s+([A-Za-z \[\]/]+?): (\d+)", line)
        if not m or m.group(1) not in fields:
            continue
        key, _, _ = fields[m.group(1)]
        value = int(m.group(2))
        if key == "scratch":
            seen += 1
            if value != 0:
                bad.append(f"{name}: {value} bytes of scratch per lane")
        elif key in gate:
            limit = gate[key]
            over = value < limit if key.startswith("min_") else value > limit
            if over:
                bad.append(f"{name}: {m.group(1)} = {value}, limit {limit}")
    if bad or seen == 0:
        os.remove(obj)
        raise RuntimeError(f"{src}: kernel resource budget violated ({'; '.join(bad) or 'no resource remarks found'})")


# The weight-streaming kernels run one work item into the next; a flat memory instruction (an access through a pointer
# the compiler cannot place in the global address space) that is still pending makes the compiler wait for ALL loads at
# the next use of a loaded register, which drains the next item's prefetch ring.  Their device assembly must hold none.
NO_FLAT = ("gemm_fp8_skinny.hip", "gemm_mxfp4_skinny.hip")


def _start_asm(src: str, obj: str):
    cmd = [hipcc()] + FLAGS + ["--cuda-device-only", "-S", "-c", os.path.join(CSRC, src), "-o", obj[:-2] + ".s"]
    return subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)


def _check_no_flat(src: str, obj: str, job) -> None:
    import re
    asm = obj[:-2] + ".s"
    _, err = job.communicate()
    if job.returncode != 0:
        raise RuntimeError(f"hipcc -S failed for {src}:\n{err}")
    with open(asm) as f:
        found = sorted(set(re.findall(r"^\s*(flat_(?:load|store|atomic)\w*)", f.read(), re.M)))
    os.remove(asm)
    if found:
        os.remove(obj)
        raise RuntimeError(f"{src}: flat memory instructions in the device code ({', '.join(found)}): "
                           "load and store through the gload_* / gstore_* helpers")


# ---- PyTorch C++ extension modules (host code over the C ABI) --------------------------------------------------
EXT_SRC = os.path.join(HERE, "ext", "bgmoe_torch.cc")
EXT_ROOT = os.path.join(HERE, "ext", "build")              # put on sys.path: holds the batchgen_kernels/... tree
EXT_MODULES = (
    "moe/_C_routing", "common/_C_mgn_ops", "moe/_C_dispatch_scatter_3d", "moe/_C_fp8_blockwise_gemm",
    "moe/_C_fp8_blockwise_ops", "attention/_C_add_rmsnorm_fp8_quant",
)


def build_extensions(force: bool = False, verbose: bool = True) -> str:
    """Compile batchgen_amd/ext/bgmoe_torch.cc once (g++: host code only) against the torch headers and libbgmoe.so,
    and install the shared object as batchgen_kernels/<pkg>/<module>.so under batchgen_amd/ext/build: the module and
    op names of the reference's compiled extensions (batchgen_kernels/__init__.py:24-45 imports them by these
    names).  Returns the directory to put on sys.path."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension as ce
    if not os.path.exists(LIB):
        raise RuntimeError(f"{LIB} is missing: build the HIP library first")
    os.makedirs(EXT_ROOT, exist_ok=True)
    one = os.path.join(EXT_ROOT, "_bgmoe_torch.so")
    deps = [EXT_SRC, os.path.join(INCLUDE, "bgmoe.h")]
    if force or not _newer(one, deps):
        tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
        rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
        cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-w", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
               f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
        cmd += [f"-I{p}" for p in ce.include_paths()] + [f"-I{sysconfig.get_paths()['include']}", f"-I{rocm}/include"]
        cmd += [EXT_SRC, "-o", one, f"-L{tlib}", f"-L{LIB_DIR}", "-ltorch_python", "-ltorch", "-ltorch_cpu", "-lc10",
                "-lc10_hip", "-ltorch_hip", "-lbgmoe", f"-Wl,-rpath,{tlib}", "-Wl,-rpath,$ORIGIN/../../../lib",
                "-Wl,-rpath,$ORIGIN/../../../../lib"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"g++ failed for {EXT_SRC}:\n{r.stdout[-3000:]}\n{r.stderr[-6000:]}")
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    for mod in EXT_MODULES:
        pkg, name = mod.split("/")
        d = os.path.join(EXT_ROOT, "batchgen_kernels", pkg)
        os.makedirs(d, exist_ok=True)
        dst = os.path.join(d, name + suffix)
        if force or not _newer(dst, [one]):
            shutil.copyfile(one, dst)
    if verbose:
        print(f"built {len(EXT_MODULES)} extension modules under {EXT_ROOT}/batchgen_kernels")
    return EXT_ROOT


# ---- host-compiled checks of the arithmetic shared with the kernels (g++, no GPU) -----------------------------
HOSTCHECK_SRC = os.path.join(CSRC, "hostcheck.cc")
HOSTCHECK_LIB = os.path.join(LIB_DIR, "libbgmoe_hostcheck.so")


def build_hostcheck(force: bool = False, verbose: bool = True) -> str:
    """Compile csrc/hostcheck.cc with g++ into lib/libbgmoe_hostcheck.so: the index and address arithmetic of
    csrc/bgmoe_hostdev.h and csrc/bgmoe_tilemap.h (the very text the kernels include) behind a few C functions that
    the CPU tests drive.  Test infrastructure; the product library does not depend on it."""
    os.makedirs(LIB_DIR, exist_ok=True)
    deps = [HOSTCHECK_SRC] + [os.path.join(CSRC, f) for f in ("bgmoe_hostdev.h", "bgmoe_tilemap.h")]
    if force or not _newer(HOSTCHECK_LIB, deps):
        cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-Werror", HOSTCHECK_SRC, "-o",
               HOSTCHECK_LIB]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"g++ failed for {HOSTCHECK_SRC}:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {HOSTCHECK_LIB}")
    return HOSTCHECK_LIB


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
    ap.add_argument("--ext", action="store_true", help="also build the PyTorch C++ extension modules")
    ap.add_argument("-j", type=int, default=4)
    a = ap.parse_args()
    try:
        build(force=a.force, jobs=a.j)
        build_hostcheck(force=a.force)
        if a.ext:
            build_extensions(force=a.force)
    except RuntimeError as e:
        print(e, file=sys.stderr)
        sys.exit(1)
