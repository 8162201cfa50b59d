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


def pytest_collection_modifyitems(config, items):
    """The single-instruction probes run before every other GPU test: they take seconds, a kernel
    that faults can end the box and leave nothing behind, and what the probes print is what sorts
    such a failure into "an instruction differs from its model" or "something else".  The
    whole-kernel comparisons of the same file stay where the file name puts them: last."""
    first = [it for it in items if "test_primitive_on_the_gpu" in it.nodeid]
    if first:
        rest = [it for it in items if "test_primitive_on_the_gpu" not in it.nodeid]
        items[:] = first + rest


@pytest.fixture(scope="session")
def dev(request):
    import torch
    if request.config.getoption("--on-emulator"):
        _wrappers_onto_the_emulator(torch)
        return torch.device("cpu")
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _default_workspace_stays_healthy(request):
    """After every GPU test: the split workspace the wrappers keep for the current stream has not
    been flagged by any launch of the test (a merge that gave up marks rows with NaN, which a test
    that looks at other rows would not see)."""
    yield
    if request.node.get_closest_marker("gpu") is None or "dev" not in request.fixturenames:
        return
    import flagtree_amd as ft
    ft.workspace_status(None, request.getfixturevalue("dev"))


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
