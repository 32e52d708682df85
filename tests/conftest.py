import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def emulating() -> bool:
    """BGMOE_EMULATE=1 rehearses the GPU tests on the CPU emulator of tests/emu (no GPU visible, or not wanted): the
    `dev` fixture is the CPU, the package's library handle is the emulation build, and the few torch.cuda calls
    the tests and the host code make are stood in for.  A rehearsal of test and kernel logic, never a substitute
    for the GPU run: speed, the hardware's rounding inside a matrix instruction and real memory ordering are not
    what it shows."""
    return os.environ.get("BGMOE_EMULATE", "0") == "1"


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped (not failed) when no GPU is visible."""
    import torch
    if torch.cuda.is_available() or emulating():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def dev():
    import torch
    return torch.device("cpu" if emulating() else "cuda:0")


@pytest.fixture(autouse=True)
def _emulator_when_asked(request, monkeypatch):
    if emulating() and "gpu" in request.keywords:
        from tests import emu
        emu.run_package_on_emulator(monkeypatch)
    yield
