"""GPU test files -- those that no GPU has executed yet, and the cheap ones among the proven -- rehearsed on the CPU emulator (tests/emu) as part of the CPU suite:
the same test functions, the package's own host code, CPU tensors standing for device memory (BGMOE_EMULATE=1, see
tests/conftest.py).  What cannot be rehearsed is left out: the compiled extension and the device-mismatch case skip
themselves off the GPU; allocation counters of torch's CUDA allocator and the full-size shapes (too slow here) are
deselected by name.  A rehearsal shows that the test code and the kernels' logic hold together; the GPU
run remains the parity test."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

REHEARSALS = [
    # files no GPU has executed yet
    ("tests/test_gpu_x_routes_and_argument_checks.py", ""),
    ("tests/test_gpu_x_moe_base.py", ""),
    ("tests/test_gpu_x_dense_backend.py", "not full_size and not allocates_nothing and not 4096 and not latent_small"),
    ("tests/test_gpu_x_streamk_status.py", ""),
    # files a GPU has run, the cheap ones: the same bit-exact gates against the oracle hold on the emulator (router ids
    # and weights, permutation indices, FP8 bytes and scales, combine), which is also what says that the emulator
    # executes these sources faithfully
    ("tests/test_gpu_router.py", ""),
    ("tests/test_gpu_permute_combine.py", ""),
    ("tests/test_gpu_quant.py", ""),
    ("tests/test_gpu_group_quant.py", ""),
    ("tests/test_gpu_scale_repack.py", ""),
    ("tests/test_gpu_moe_ragged.py", ""),
    ("tests/test_gpu_tight_dispatch.py", "not graph_capturable and not dispatch_errors"),
    ("tests/test_zz_no_alloc.py", ""),
    # the files that wait for their first GPU run under names pytest does not collect, at their smaller shapes (their
    # kernels are also driven directly in tests/test_emu_kernels.py): the test code itself must not rot while it waits
    ("tests/wip_gpu_mxfp4_fold_gather.py", ""),
    ("tests/wip_gpu_skinny_tall.py", "case2 or case3 or layer"),
    ("tests/wip_gpu_gemm_stages.py", "case2 or case3 or 100-1152-1024 or 300-1152-1024 or in_the_layer"),
    ("tests/wip_gpu_mxfp4_variant.py", "case0 or layer"),
]


WORKERS = 4          # children at a time (each is a python process with torch imported: about 1 GB)


@pytest.fixture(scope="module")
def rehearsals():
    """All files at once, WORKERS children at a time; each parametrised test below then reads its own result."""
    from concurrent.futures import ThreadPoolExecutor
    from tests.emu.build_emu import build
    build()                                                   # before the children, so that their time is the tests'
    env = dict(os.environ, BGMOE_EMULATE="1", OMP_NUM_THREADS="2")

    def run(item):
        path, select = item
        cmd = [sys.executable, "-m", "pytest", path, "-m", "gpu", "-q", "--tb=short", "-p", "no:cacheprovider"]
        if select:
            cmd += ["-k", select]
        try:
            return subprocess.run(cmd, cwd=ROOT, env=env, capture_output=True, text=True, timeout=1500)
        except subprocess.TimeoutExpired as e:
            return e

    with ThreadPoolExecutor(WORKERS) as ex:
        return dict(zip([p for p, _ in REHEARSALS], ex.map(run, REHEARSALS)))


@pytest.mark.parametrize("path", [p for p, _ in REHEARSALS], ids=[os.path.basename(p) for p, _ in REHEARSALS])
def test_gpu_test_files_pass_on_the_emulator(rehearsals, path):
    r = rehearsals[path]
    assert not isinstance(r, subprocess.TimeoutExpired), f"{path}: rehearsal timed out"
    tail = (r.stdout + r.stderr)[-3000:]
    assert r.returncode == 0, tail
    assert " passed" in r.stdout and "failed" not in r.stdout.splitlines()[-1], tail
