"""A fixed, seeded set of random cases through the emulator build of the kernels, every buffer
between inaccessible pages: 60 attention cases over all kernels, switches, formats, page sizes,
split counts and emulator schedules, and 40 cases of the other entry points (index producer, local
GEMM, cache writer, gather), each held against the numpy oracle.  tests/emu/fuzz_cases.py draws and
runs the cases; it runs in processes of its own (a stray access ends the process), several at a
time.  Further seeds: ``python tests/emu/fuzz_cases.py forward 60 1000``."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SCRIPT = os.path.join(HERE, "emu", "fuzz_cases.py")
RUNS = [("forward", 0, 15), ("forward", 15, 30), ("forward", 30, 45), ("forward", 45, 60), ("other", 0, 40)]


def test_seeded_random_cases_against_the_oracle():
    sys.path.insert(0, os.path.join(HERE, "emu"))
    import harness
    harness.lib()                                     # built once here, not by five processes at a time
    procs = [(r, subprocess.Popen([sys.executable, SCRIPT, r[0], str(r[1]), str(r[2])], stdout=subprocess.PIPE,
                                  stderr=subprocess.STDOUT, text=True)) for r in RUNS]
    failed = []
    for r, p in procs:
        try:
            out, _ = p.communicate(timeout=900)
        except subprocess.TimeoutExpired:
            p.kill()
            out, _ = p.communicate()
            out += "\n(timed out)"
        n_cases = sum(1 for line in out.splitlines() if line.startswith("seed "))
        if p.returncode != 0 or not out.rstrip().endswith("done, failures: 0") or n_cases != r[2] - r[1]:
            failed.append((r, p.returncode, out[-3000:]))
    assert not failed, failed
