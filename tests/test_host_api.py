"""CPU checks of the host side: the C ABI library loads and exports every declared symbol, its
argument validation answers with the documented codes before touching a device, and the Python
surface rejects what the operator cannot take."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from flagtree_amd import _lib, build
    if not os.path.exists(build.LIB_PATH):
        build.build()
    return _lib.load()


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "flagtree_smla.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(smla_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(lib):
    from flagtree_amd import _lib
    names = _declared_functions()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/flagtree_smla.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names
    assert lib.smla_abi_version() == 4


def test_status_texts(lib):
    from flagtree_amd import _lib
    assert _lib.strerror(0) == "ok"
    for code in range(-8, 0):
        assert _lib.strerror(code) not in ("ok", "unknown status")
    with pytest.raises(ValueError):
        _lib.check(-2, "x")
    with pytest.raises(RuntimeError):
        _lib.check(-101, "x")


def test_validation_codes_without_a_device(lib):
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    p16 = (p + 15) & ~15
    ok = dict(fmt=0, q=p16, kv=p16, idx=p16, bt=None, out=p16, lse=p16, T=4, S=1, H=16, K=32, dqk=576, dv=512,
              page=64, bts=0, stride=0, rows=100, scale=0.04, ns=1, ws=None, wsb=0, stream=None)

    def call(**kw):
        a = dict(ok, **kw)
        return lib.smla_fwd(a["fmt"], a["q"], a["kv"], a["idx"], a["bt"], a["out"], a["lse"], a["T"], a["S"], a["H"],
                            a["K"], a["dqk"], a["dv"], a["page"], a["bts"], a["stride"], a["rows"], a["scale"],
                            a["ns"], a["ws"], a["wsb"], a["stream"])

    assert call(q=None) == -1 and call(lse=None) == -1
    assert call(dqk=512) == -2 and call(dv=256) == -2 and call(T=0) == -2 and call(T=5, S=2) == -2
    assert call(rows=0) == -2 and call(rows=2 ** 31) == -2 and call(bt=p16, bts=0) == -2 and call(fmt=9) == -2
    assert call(kv=p16 + 2) == -3
    assert call(ns=33) == -5 and call(ns=-1) == -5
    assert call(scale=0.0) == -7 and call(scale=-1.0) == -7 and call(scale=float("inf")) == -7
    assert call(ns=2, K=2048) == -4                           # split without a workspace
    assert lib.smla_gather_rows(None, 16, p16, None, p16, None, 1, 1, 1, 64, 0, 0, 10, None) == -1
    assert lib.smla_gather_rows(p16, 20, p16, None, p16, None, 1, 1, 1, 64, 0, 0, 10, None) == -2
    assert lib.smla_merge_splits(p16, p16, p16, p16, 1, 1, 256, 2, None) == -2
    assert lib.smla_merge_splits(p16, p16, p16, p16, 1, 1, 512, 40, None) == -5
    assert lib.smla_kv_quantize_fp8(None, None, p16, 1, 1, None) == -1
    assert lib.smla_gemm_rs_local(p16, p16, None, p16, 100, 256, 64, 1, 25600, None) == -2
    assert lib.smla_gemm_rs_local(p16, p16, None, p16, 128, 256, 64, 1, 100, None) == -2    # chunk stride too small
    assert lib.smla_workspace_init(None, 1 << 20, None) == -1
    assert lib.smla_workspace_init(p16, 100, None) == -4
    # cache writer, index producer, dense decode and the scalar cross-check reject bad arguments the same way
    assert lib.smla_kv_write(0, None, None, p16, 4, 64, None) == -1 and lib.smla_kv_write(0, p16, None, None, 4, 64, None) == -1
    assert lib.smla_kv_write(0, p16, None, p16, -1, 64, None) == -2 and lib.smla_kv_write(0, p16, None, p16, 4, 0, None) == -2
    assert lib.smla_kv_write(0, p16 + 4, None, p16, 4, 64, None) == -3
    assert lib.smla_kv_write(7, p16, None, p16, 4, 64, None) == -2                           # unknown cache format
    assert lib.smla_kv_quantize_fp8(p16, None, p16, 4, 0, None) == -2 and lib.smla_kv_quantize_fp8(p16 + 8, None, p16, 4, 8, None) == -3
    assert lib.smla_topk_indices(None, None, p16, 1, 64, 64, 8, None, 0, None) == -1 and lib.smla_topk_indices(p16, None, None, 1, 64, 64, 8, None, 0, None) == -1
    assert lib.smla_topk_indices(p16, None, p16, 1, 0, 64, 8, None, 0, None) == -2 and lib.smla_topk_indices(p16, None, p16, 1, 64, 64, 0, None, 0, None) == -2
    assert lib.smla_topk_indices(p16, None, p16, -1, 64, 64, 8, None, 0, None) == -2
    assert lib.smla_topk_indices(p16, None, p16, 1, 64, 32, 8, None, 0, None) == -2                   # row stride shorter than a row
    assert lib.smla_topk_indices(p16, None, p16, 1, 64, 64, 8, p16 + 2, 64, None) == -3               # workspace off a 4-byte boundary
    assert lib.smla_topk_rows(p16, None, None, p16, 2, 64, 64, 8, 1, 16, 4, 100, None, 0, None) == -1   # no page table
    assert lib.smla_topk_rows(p16, None, p16, p16, 3, 64, 64, 8, 2, 16, 4, 100, None, 0, None) == -2    # rows do not divide into sequences
    assert lib.smla_topk_rows(p16, None, p16, p16, 2, 64, 64, 8, 1, 0, 4, 100, None, 0, None) == -2     # page size
    assert lib.smla_topk_rows(p16, None, p16, p16, 2, 64, 64, 8, 1, 16, 4, 0, None, 0, None) == -2      # empty pool

    def dense(**kw):
        a = dict(ok, **kw)
        return lib.smla_decode_dense(a["fmt"], a["q"], a["kv"], a["idx"], a["bt"], a["out"], a["lse"], a["T"], a["S"], a["H"],
                                     a["K"], a["dqk"], a["dv"], a["page"], a["bts"], a["stride"], a["rows"], a["scale"],
                                     a.get("cap", 0.0), a["ns"], a["ws"], a["wsb"], a["stream"])

    assert dense(q=None) == -1 and dense(idx=None) == -1 and dense(dv=256) == -2 and dense(K=0) == -2
    assert dense(out=p16 + 2) == -3 and dense(ns=40) == -5 and dense(scale=float("nan")) == -7
    assert dense(cap=-1.0) == -7 and dense(cap=float("inf")) == -7 and dense(cap=float("nan")) == -7

    def scalar(**kw):
        a = dict(ok, **kw)
        return lib.smla_fwd_scalar(a["fmt"], a["q"], a["kv"], a["idx"], a["bt"], a["out"], a["lse"], a["T"], a["S"], a["H"],
                                   a["K"], a["dqk"], a["dv"], a["page"], a["bts"], a["stride"], a["rows"], a["scale"], a["stream"])

    assert scalar(kv=None) == -1 and scalar(dqk=64) == -2 and scalar(H=70000) == -2 and scalar(scale=0.0) == -7


def test_workspace_and_split_planning(lib):
    assert lib.smla_workspace_bytes(64, 128, 512, 1) == 0
    assert lib.smla_workspace_bytes(64, 128, 512, 2) == 262144 + 64 * 2 * 128 * 513 * 4
    ns = lib.smla_plan_splits(0, 64, 128, 2048)
    assert 1 <= ns <= 8
    assert lib.smla_plan_splits(0, 8192, 128, 2048) == 1       # plenty of tokens: no split
    assert lib.smla_plan_splits(2, 4, 16, 256) == 1            # fp32 plumbing path never splits


def test_split_planning_follows_the_kernel_switches(lib, monkeypatch):
    """A 128-heads-per-workgroup kernel has half as many (token, head block) units to fill the
    device with, so the planner doubles the splits; the switches are read at every call.
    (Without a GPU the library plans for 256 compute units.)"""
    BF16, FP8 = 0, 1
    monkeypatch.delenv("FLAGTREE_SMLA_HEAD_GROUPS", raising=False)
    monkeypatch.delenv("FLAGTREE_SMLA_FEW_FP8", raising=False)
    monkeypatch.delenv("FLAGTREE_SMLA_FP8_MFMA", raising=False)
    base = [lib.smla_plan_splits(BF16, 64, 128, 2048), lib.smla_plan_splits(FP8, 64, 128, 2048), lib.smla_plan_splits(FP8, 128, 16, 2048)]
    assert base == [2, 2, 2]
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1")          # a wavefront per head group: both formats
    assert [lib.smla_plan_splits(BF16, 64, 128, 2048), lib.smla_plan_splits(FP8, 64, 128, 2048)] == [4, 4]
    assert lib.smla_plan_splits(FP8, 128, 16, 2048) == 2           # few heads: not its business
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "0")
    monkeypatch.setenv("FLAGTREE_SMLA_FEW_FP8", "1")              # two workgroups per compute unit
    assert lib.smla_plan_splits(FP8, 128, 16, 2048) == 4 and lib.smla_plan_splits(BF16, 64, 128, 2048) == 2
    monkeypatch.setenv("FLAGTREE_SMLA_FEW_FP8", "0")
    monkeypatch.setenv("FLAGTREE_SMLA_FP8_MFMA", "1")             # the fp8-MFMA kernel: two workgroups per compute unit as well
    assert lib.smla_plan_splits(FP8, 128, 16, 2048) == 4 and lib.smla_plan_splits(BF16, 128, 16, 2048) == 2


def test_python_surface_rejects_bad_input():
    import flagtree_amd as ft
    q = torch.zeros((1, 2, 16, 576), dtype=torch.bfloat16)
    kv = torch.zeros((64, 576), dtype=torch.bfloat16)
    idx = torch.zeros((1, 2, 8), dtype=torch.int32)
    with pytest.raises(ValueError, match="device tensor"):
        ft.sparse_mla_fwd(q, kv, idx, 0.04, 512)
    with pytest.raises(ValueError, match="d_qk"):
        ft.sparse_mla_fwd(q[..., :512], kv, idx, 0.04, 512)
    with pytest.raises(ValueError, match="d_qk"):
        ft.sparse_mla_fwd(q, kv, idx, 0.04, 256)
    with pytest.raises(ValueError, match="q must be"):
        ft.sparse_mla_fwd(q.float(), kv, idx, 0.04, 512)
    with pytest.raises(ValueError, match="kv_cache"):
        ft.sparse_mla_fwd(q, kv[:, :500], idx, 0.04, 512)
    with pytest.raises(ValueError, match="indices"):
        ft.sparse_mla_fwd(q, kv, idx.float(), 0.04, 512)
    with pytest.raises(ValueError, match="indices"):
        ft.sparse_mla_fwd(q, kv, idx[:, :1], 0.04, 512)
    with pytest.raises(ValueError):
        ft.gemm_rs_local(torch.zeros((8, 8)), torch.zeros((8, 8)))
    with pytest.raises(ValueError):
        ft.quantize_kv_fp8(torch.zeros((4, 576), dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="no CPU path"):
        ft.topk_indices(torch.zeros((2, 64)), 8)
    with pytest.raises(ValueError, match="no CPU path"):
        ft.reshape_and_cache(torch.zeros((4, 576), dtype=torch.bfloat16), torch.zeros((8, 576), dtype=torch.bfloat16),
                             torch.zeros(4, dtype=torch.int64))
    with pytest.raises(ValueError, match="indices must be"):
        ft.sparse_mla_fwd(q, kv, idx.view(2, 1, 1, 8), 0.04, 512)         # [B, S, 1, topk] with the wrong B, S
    with pytest.raises(ValueError, match="kv_format"):
        ft.sparse_mla_fwd(q, kv, idx, 0.04, 512, kv_format="int4")
    with pytest.raises(ValueError, match="multiple"):
        ft.sparse_mla_fwd(q.view(2, 16, 576)[:1].expand(3, 16, 576), kv, idx.view(2, 8), 0.04, 512,
                          block_table=torch.zeros((2, 4), dtype=torch.int32))


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "flagtree_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), f
                assert "_work/" not in text, f


def test_workload_accounting():
    from flagtree_amd import workloads
    cfg = workloads.plumbing_f32(device="cpu")
    flops, nbytes, n_valid = workloads.attention_work(cfg)
    assert n_valid == 4 * 231 and flops == 2.0 * 924 * 16 * 1088      # 10 % of 256 = 25 padded per token
    assert cfg["indices"].shape == (1, 4, 256) and (cfg["indices"][0, :, -25:] == -1).all()


def test_header_is_plain_c_and_matches_the_library(tmp_path):
    """include/flagtree_smla.h must compile as C99 on its own (a cgo / JNI / ctypes binding sees
    nothing else), and a C program that takes the address of every declared entry point must link
    against the built library."""
    import shutil
    import subprocess
    from flagtree_amd import build
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    if not os.path.exists(build.LIB_PATH):
        build.build()
    inc = os.path.join(ROOT, "include")
    lib_dir = os.path.dirname(build.LIB_PATH)
    names = _declared_functions()
    assert len(names) >= 14
    src = tmp_path / "use_header.c"
    src.write_text('#include "flagtree_smla.h"\n#include <stdio.h>\ntypedef void (*entry_fn)(void);\nint main(void) {\n'
                   '  entry_fn f[] = {' + ", ".join("(entry_fn)" + n for n in names) + '};\n'
                   '  printf("%d %d\\n", (int)(sizeof f / sizeof f[0]), SMLA_MAX_SPLITS);\n  return f[0] == 0;\n}\n')
    exe = tmp_path / "use_header"
    r = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-I", inc, str(src), "-o", str(exe),
                        "-L", lib_dir, "-lflagtree_smla", "-Wl,-rpath," + lib_dir,
                        "-Wl,--unresolved-symbols=ignore-in-shared-libs"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
