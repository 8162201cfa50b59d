"""Build recipe for libflagtree_smla.so (hipcc, gfx950 only).  ``python -m flagtree_amd.build``."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libflagtree_smla.so")
SOURCES = ["smla_api.hip", "smla_scalar.hip", "smla_mfma_tall.hip", "smla_mfma_short.hip", "smla_mfma_few_fp8.hip", "smla_mfma_few_f8.hip", "smla_mfma_group.hip", "gemm_rs.hip", "topk_select.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # keep hipcc from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # <smla_hw.h>: hardware-specific wrappers, found through the include path
    "-I", CSRC,
]


def build(verbose=False):
    """Compile every HIP source into the in-tree shared library; raises on failure."""
    cmd = [HIPCC] + FLAGS + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "packed-fp32-ops"
    log = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    if verbose and log.strip():
        print(log)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
