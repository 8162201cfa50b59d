"""Build the hardware-model probes for gfx950 (test infrastructure): tests/hw_model/libhw_model.so.
The CPU emulator's build (tests/emu/build_emu.py) compiles the same source for the host.
``python tests/hw_model/build_hw_model.py``."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB_PATH = os.path.join(HERE, "libhw_model.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-int-to-pointer-cast",
         "-I", os.path.join(ROOT, "flagtree_amd", "csrc"), "-I", HERE]


def build(verbose=False):
    cmd = [HIPCC] + FLAGS + [os.path.join(HERE, "primitives.hip"), "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    if verbose and log.strip():
        print(log)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
