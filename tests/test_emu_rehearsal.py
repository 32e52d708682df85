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
]


@pytest.mark.parametrize("path,select", REHEARSALS, ids=[os.path.basename(p) for p, _ in REHEARSALS])
def test_gpu_test_files_pass_on_the_emulator(path, select):
    from tests.emu.build_emu import build
    build()                                                   # before the child, so that its time is the tests'
    cmd = [sys.executable, "-m", "pytest", path, "-m", "gpu", "-q", "--tb=short", "-p", "no:cacheprovider"]
    if select:
        cmd += ["-k", select]
    env = dict(os.environ, BGMOE_EMULATE="1")
    r = subprocess.run(cmd, cwd=ROOT, env=env, capture_output=True, text=True, timeout=1500)
    tail = (r.stdout + r.stderr)[-3000:]
    assert r.returncode == 0, tail
    assert " passed" in r.stdout and "failed" not in r.stdout.splitlines()[-1], tail
