"""Build the kernel sources for the CPU emulator (test infrastructure; the product never loads it).

The very same .hip files the product compiles for gfx950 are compiled here as host C++ against
tests/emu/include (a stand-in <hip/hip_runtime.h> and <smla_hw.h>), together with the fiber
runtime, into tests/emu/libflagtree_smla_emu.so.  ``python tests/emu/build_emu.py``."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "flagtree_amd", "csrc")
LIB_PATH = os.path.join(HERE, "libflagtree_smla_emu.so")
SOURCES = ["smla_api.hip", "smla_scalar.hip", "smla_mfma_tall.hip", "smla_mfma_short.hip", "smla_mfma_few_fp8.hip", "smla_mfma_few_f8.hip", "smla_mfma_group.hip", "gemm_rs.hip", "topk_select.hip"]
HW_MODEL = os.path.join(os.path.dirname(HERE), "hw_model")      # probes of single instructions, built for both sides
CXX = os.environ.get("EMU_CXX", "/opt/rocm/llvm/bin/clang++")
FLAGS = ["-x", "c++", "-std=c++17", "-O2", "-g1", "-fPIC", "-ffp-contract=off", "-fno-strict-aliasing",
         "-Wno-unused-value", "-Wno-pass-failed", "-Wno-unknown-attributes", "-Wno-ignored-attributes",
         "-I", os.path.join(HERE, "include"), "-I", CSRC, "-I", HW_MODEL]


def _stale(outputs, inputs):
    if not all(os.path.exists(o) for o in outputs):
        return True
    newest = max(os.path.getmtime(i) for i in inputs)
    return any(os.path.getmtime(o) < newest for o in outputs)


STAMP_PATH = LIB_PATH + ".stamp"


def _digest(paths):
    """Hash of everything the library is made from (contents, not time stamps: a copy of the tree
    to another machine keeps the contents)."""
    import hashlib
    h = hashlib.sha256(" ".join([CXX] + FLAGS).replace(ROOT, "").encode())
    for p in sorted(paths):
        h.update(os.path.relpath(p, ROOT).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def build(verbose=False, force=False):
    # every header a kernel source may include (the product's own smla_hw.h is shadowed by the emulator's)
    headers = [os.path.join(HERE, "emu_runtime.h"), os.path.join(HERE, "include", "smla_hw.h"),
               os.path.join(HERE, "include", "hip", "hip_runtime.h"), os.path.join(ROOT, "include", "flagtree_smla.h"),
               os.path.abspath(__file__), os.path.join(HW_MODEL, "primitives.h")]
    headers += sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h") and f != "smla_hw.h")
    names = SOURCES + ["primitives.hip", "emu_runtime.cc"]
    paths = [os.path.join(HERE if n.endswith(".cc") else (HW_MODEL if n == "primitives.hip" else CSRC), n) for n in names]
    digest = _digest(paths + headers)
    # a library that was built from exactly these files is used as it is, also where the object
    # files did not travel with it (a GPU box runs what was built beforehand and compiles nothing)
    if not force and os.path.exists(LIB_PATH) and os.path.exists(STAMP_PATH) and open(STAMP_PATH).read().strip() == digest:
        return LIB_PATH
    objs = []
    procs = []
    for src, path in zip(names, paths):
        obj = os.path.join(HERE, "build", src + ".o")
        objs.append(obj)
        if not force and not _stale([obj], [path] + headers):
            continue
        os.makedirs(os.path.dirname(obj), exist_ok=True)
        cmd = [CXX] + FLAGS + ["-c", path, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for src, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError(f"emulator build of {src} failed:\n{out[-6000:]}")
        if verbose and out.strip():
            print(out)
    if procs or not os.path.exists(LIB_PATH):
        res = subprocess.run([CXX, "-shared", "-rdynamic", "-o", LIB_PATH] + objs, stdout=subprocess.PIPE,
                             stderr=subprocess.STDOUT, text=True)
        if res.returncode != 0:
            raise RuntimeError("emulator link failed:\n" + res.stdout[-4000:])
    with open(STAMP_PATH, "w") as f:
        f.write(digest + "\n")
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv, force="-f" in sys.argv))
