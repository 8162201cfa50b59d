"""The emulator's model of every machine-specific primitive the kernels use, against what the
instruction is documented to do (tests/hw_model/cases.py states that in numpy).  The probes are
one-wavefront kernels in tests/hw_model/primitives.hip; tests/test_gpu_y_hw_model.py runs the
same probes on the GPU and compares them with the emulator bit for bit."""
import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [os.path.join(HERE, "emu"), os.path.join(HERE, "hw_model")]
import cases      # noqa: E402
import harness    # noqa: E402


def run_on_emulator(name, rec):
    lib = cases.bind(harness.lib())
    src = torch.from_numpy(rec.copy())
    out = torch.full((cases.LANES, cases.RECORD), 0xCD, dtype=torch.uint8)
    assert lib.hwm_run(cases.PROBES[name], src.data_ptr(), out.data_ptr(), None) == 0
    return out.numpy()


def test_probe_numbers_agree_with_the_library():
    lib = cases.bind(harness.lib())
    assert lib.hwm_count() == cases.PROBES["COUNT"] == len(cases.PROBE_NAMES)
    assert sorted(cases.PROBES[n] for n in cases.PROBE_NAMES) == list(range(len(cases.PROBE_NAMES)))
    assert lib.hwm_run(999, None, None, None) != 0


@pytest.mark.parametrize("seed", [0, 1, 2])
@pytest.mark.parametrize("name", cases.PROBE_NAMES)
def test_emulated_primitive_does_what_the_instruction_is_documented_to_do(name, seed):
    rec = cases.make_input(name, seed)
    got = run_on_emulator(name, rec)
    diff = cases.differences(name, got, cases.expect(name, rec))
    assert not diff, diff


def test_a_wrong_answer_is_noticed():
    """Negative control: one changed byte of an output fails the comparison."""
    rec = cases.make_input("DMA_B128", 0)
    got = run_on_emulator("DMA_B128", rec)
    got[5, 3] ^= 1
    assert cases.differences("DMA_B128", got, cases.expect("DMA_B128", rec))


def test_the_gfx950_build_of_the_probes_exports_its_entry_points():
    if not os.path.exists(cases.GPU_LIB_PATH):
        pytest.skip("tests/hw_model/libhw_model.so not built")
    with open(cases.GPU_LIB_PATH, "rb") as f:
        blob = f.read()
    assert b"hwm_run" in blob and b"hwm_count" in blob and b"gfx950" in blob
