import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_addoption(parser):
    parser.addoption("--on-emulator", action="store_true",
                     help="rehearse GPU tests without a GPU: the Python wrappers call the CPU emulator build of the kernel "
                          "sources (tests/emu) on CPU tensors.  Checks the tests' and wrappers' logic at small sizes; "
                          "pick cases with -k, full-size ones take hours.  Never a substitute for the GPU run.")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def dev(request):
    import torch
    if request.config.getoption("--on-emulator"):
        _wrappers_onto_the_emulator(torch)
        return torch.device("cpu")
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _wrappers_onto_the_emulator(torch):
    """Test-side patching only: the product has no CPU path, and nothing in it knows of this."""
    sys.path.insert(0, os.path.join(ROOT, "tests", "emu"))
    import harness
    from flagtree_amd import _lib
    emu = harness.lib()
    _lib.load = lambda: emu
    _lib.on_device = lambda t: True
    _lib.stream_handle = lambda device: None
    torch.cuda.synchronize = lambda *a, **k: None
