"""Every machine-specific primitive the kernels use, run alone on the GPU (one wavefront, operands
handed to each lane, tests/hw_model/primitives.hip) and compared bit for bit with the CPU
emulator's model of it and with the documented behaviour stated in numpy.  A kernel test that
passes on the emulator and fails on the GPU points here first: either a primitive differs (this
file names it) or the fault is in what the emulator does not model (registers, timing, caches).
The file sorts after the kernel parity tests: the probes themselves are new to the hardware."""
import os
import sys

import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [os.path.join(HERE, "emu"), os.path.join(HERE, "hw_model")]
import cases      # noqa: E402
import harness    # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu_probes(dev, request):
    if request.config.getoption("--on-emulator"):
        pytest.skip("compares the GPU with the emulator: nothing to rehearse")
    return cases.gpu_lib()


def run_on_gpu(lib, dev, name, rec):
    src = torch.from_numpy(rec.copy()).to(dev)
    out = torch.full((cases.LANES, cases.RECORD), 0xCD, dtype=torch.uint8, device=dev)
    assert src.data_ptr() % 256 == 0 and out.data_ptr() % 256 == 0
    assert src.numel() == out.numel() == cases.LANES * cases.RECORD
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream(dev).cuda_stream
    assert lib.hwm_run(cases.PROBES[name], src.data_ptr(), out.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    return out.cpu().numpy()


def run_on_emulator(name, rec):
    lib = cases.bind(harness.lib())
    src = torch.from_numpy(rec.copy())
    out = torch.full((cases.LANES, cases.RECORD), 0xCD, dtype=torch.uint8)
    assert lib.hwm_run(cases.PROBES[name], src.data_ptr(), out.data_ptr(), None) == 0
    return out.numpy()


@pytest.mark.parametrize("seed", [0, 1, 2])
@pytest.mark.parametrize("name", cases.PROBE_NAMES)
def test_primitive_on_the_gpu_matches_the_emulator_and_the_documentation(dev, gpu_probes, name, seed):
    rec = cases.make_input(name, seed)
    print(f"probe {name} seed {seed}", flush=True)
    got = run_on_gpu(gpu_probes, dev, name, rec)
    against_emulator = cases.differences(name, got, run_on_emulator(name, rec))
    against_documentation = cases.differences(name, got, cases.expect(name, rec))
    assert not against_emulator and not against_documentation, (against_emulator, against_documentation)
