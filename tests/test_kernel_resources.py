"""CPU check of what the compiled gfx950 kernels occupy (hipcc cross-compiles without a GPU):
every kernel's LDS fits the CU's 160 KB, and only the kernels named below use scratch at all.
A spill in any other kernel is a performance regression.  Loads issued from inline assembly into
registers are banned outright: the compiler takes an asm output as written when the statement
ends, while the load is still in flight, so any copy or spill it places before the wait reads
registers the hardware has not filled yet."""
import os
import re
import subprocess
import tempfile

import pytest

from flagtree_amd import build

LDS_PER_CU = 160 * 1024
# Kernels that may park registers in scratch memory OUTSIDE their inner loops (checked below):
#  * the two-workgroups-per-CU fp8 kernel is capped at 256 registers and parks a few across the
#    per-chunk set-up.
#  * the wavefront-per-head-group kernel holds 144 Q and 256 accumulator registers; it parks values
#    across the per-chunk set-up and in the epilogue's merge.
#  * the persistent GEMM kernel holds the whole-tile and the half-tile code; four lane-derived
#    offsets of the half-tile part are parked at the kernel's start and fetched once, before it.
MAY_SPILL = ("fwd_few_fp8_kernel", "fwd_group_kernel", "gemm_rs_chain_kernel")

_cache = {}


def _compile(source):
    """(kernel name -> resource figures, assembly text) of one source file, from a single compile."""
    if source in _cache:
        return _cache[source]
    flags = [f for f in build.FLAGS if f not in ("-fPIC", "-shared")]
    with tempfile.TemporaryDirectory() as tmp:
        asm = os.path.join(tmp, "out.s")
        cmd = [build.HIPCC] + flags + ["--cuda-device-only", "-S", "-Rpass-analysis=kernel-resource-usage", "-I",
                                       os.path.join(os.path.dirname(build.HERE), "include"),
                                       os.path.join(build.CSRC, source), "-o", asm]
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=900)
        assert res.returncode == 0, res.stdout[-2000:]
        text = open(asm).read()
    kernels, cur = {}, None
    for line in res.stdout.splitlines():
        m = re.search(r"remark: \s*Function Name: (\S+)", line)
        if m:
            cur = kernels.setdefault(m.group(1), {})
            continue
        m = re.search(r"remark: \s*([A-Za-z ]+?)(?: \[[^\]]*\])?: (\d+)", line)
        if m and cur is not None:
            cur[m.group(1).strip()] = int(m.group(2))
    _cache[source] = (kernels, text)
    return _cache[source]


def _resource_usage(source):
    return _compile(source)[0]


def _scratch_in_inner_loops(asm_text):
    """{kernel: number of scratch loads / stores inside innermost loops}.  The compiler annotates
    basic blocks with the loop they belong to; an innermost loop's header says 'Inner Loop Header'."""
    out, kernel, inner, block_loop = {}, None, set(), None
    lines = asm_text.splitlines()
    last_label = None
    for line in lines:                                    # first pass: the innermost loop headers
        m = re.match(r"^(\.LBB\d+_\d+):", line)
        if m:
            last_label = m.group(1)[2:]                   # 'BB3_195'
        elif not re.match(r"^\s+;", line):
            last_label = None if line.strip() else last_label
        # (a nested loop's header carries the note on a continuation line under its 'Parent Loop' lines)
        if "This Inner Loop Header" in line and last_label:
            inner.add(last_label)
    for line in lines:
        m = re.match(r"^(_Z\w+):", line)
        if m:
            kernel, block_loop = m.group(1), None
            out.setdefault(kernel, 0)
            continue
        if line.startswith(".Lfunc_end"):
            kernel = None
            continue
        m = re.match(r"^\.L(BB\d+_\d+):(.*)", line)
        if m:
            label, note = m.group(1), m.group(2)
            h = re.search(r"in Loop: Header=(BB\d+_\d+)", note)
            block_loop = label if label in inner else (h.group(1) if h and h.group(1) in inner else None)
            continue
        m = re.match(r"^; %bb\.\d+:(.*)", line)          # fall-through blocks carry the same annotation
        if m:
            h = re.search(r"in Loop: Header=(BB\d+_\d+)", m.group(1))
            block_loop = h.group(1) if h and h.group(1) in inner else None
            continue
        if kernel and block_loop and re.match(r"^\s+scratch_(load|store)", line):
            out[kernel] += 1
    return out


@pytest.mark.parametrize("source", [s for s in build.SOURCES if s != "smla_api.hip"])
def test_kernels_fit_the_cu_and_do_not_spill(source):
    kernels, asm = _compile(source)
    assert kernels, "no kernel found in " + source
    for name, use in kernels.items():
        assert use["LDS Size"] <= LDS_PER_CU, (name, use)
        assert use["VGPRs"] <= 256 and use["AGPRs"] <= 256, (name, use)
        if not any(tag in name for tag in MAY_SPILL):
            assert use["ScratchSize"] == 0 and use["VGPRs Spill"] == 0, (name, use)
    hot = _scratch_in_inner_loops(asm)
    assert hot and all(n == 0 for n in hot.values()), {k: v for k, v in hot.items() if v}


def test_two_workgroups_of_the_column_split_fp8_kernel_fit_a_cu():
    few = _resource_usage("smla_mfma_few_fp8.hip")
    assert few and all(u["Occupancy"] >= 2 and u["LDS Size"] <= LDS_PER_CU // 2 and u["VGPRs"] + u["AGPRs"] <= 256
                       for u in few.values()), few


def test_one_wavefront_per_simd_kernels_use_the_whole_register_file():
    """The forward kernels are built around one wavefront per SIMD (accumulators + Q resident);
    the 256 x 256 GEMM runs 16 wavefronts per workgroup, so 4 per SIMD, 128 registers each."""
    tall = _resource_usage("smla_mfma_tall.hip")
    assert all(u["Occupancy"] == 1 for u in tall.values()), tall
    group = _resource_usage("smla_mfma_group.hip")
    assert group and all(u["Occupancy"] == 1 and u["AGPRs"] == 256 for u in group.values()), group
    gemm = _resource_usage("gemm_rs.hip")
    big = [u for n, u in gemm.items() if "gemm_rs_big_kernel" in n]
    assert len(big) == 1 and big[0]["VGPRs"] + big[0]["AGPRs"] <= 128 and big[0]["LDS Size"] == 128 * 1024, big


@pytest.mark.parametrize("source", [s for s in build.SOURCES if s != "smla_api.hip"])
def test_every_global_to_lds_move_has_its_m0_wait_state(source):
    """The ISA asks for one wait state between a scalar write of M0 and a memory instruction that
    takes its LDS base from M0.  The moves are issued from inline assembly, where the compiler's
    hazard pass does not look, so the s_nop is written out; this checks the compiled code."""
    _, asm = _compile(source)
    lines = [l.strip() for l in asm.splitlines()]
    moves = [i for i, l in enumerate(lines) if l.startswith("global_load_lds")]
    for i in moves:
        assert lines[i - 1].startswith("s_nop") and lines[i - 2].startswith("s_mov_b32 m0"), (source, lines[i - 3:i + 1])


@pytest.mark.parametrize("source", [s for s in build.SOURCES if s != "smla_api.hip"])
def test_agent_scope_stores_from_assembly_keep_their_data_registers(source):
    """A store of more than 8 bytes reads its data registers for two more wait states; the 16-byte
    agent-scope stores are issued from inline assembly, so the s_nop is written out."""
    _, asm = _compile(source)
    lines = [l.strip() for l in asm.splitlines()]
    for i, l in enumerate(lines):
        if l.startswith("global_store_dwordx4") and " sc1" in l and lines[i - 1].startswith(";;#ASMSTART"):
            assert lines[i + 1].startswith("s_nop 1"), (source, lines[i - 1:i + 3])


_LOAD_MNEMONIC = re.compile(r"\b(global_load|buffer_load|flat_load|scratch_load|ds_read|ds_load|s_load|s_buffer_load)")


def _asm_statements(text):
    """(line number, statement text) of every inline-assembly statement in a source file."""
    out = []
    for m in re.finditer(r"\basm\b\s*(?:volatile)?\s*\(", text):
        depth, i = 1, m.end()
        while depth and i < len(text):
            depth += {"(": 1, ")": -1}.get(text[i], 0)
            i += 1
        out.append((text.count("\n", 0, m.start()) + 1, text[m.start():i]))
    return out


@pytest.mark.parametrize("source", sorted(f for f in os.listdir(build.CSRC) if f.endswith((".hip", ".h"))))
def test_no_inline_asm_load_lands_in_a_register(source):
    """Loads from inline assembly may only be direct-to-LDS moves (no register output); everything
    that lands in a register is a load the compiler can see and count.  Every asm statement that
    writes M0 says so in its clobber list."""
    text = open(os.path.join(build.CSRC, source)).read()
    for line, stmt in _asm_statements(text):
        body = stmt.split(":")[0]
        if _LOAD_MNEMONIC.search(body):
            assert "_lds_" in body or " lds" in body, (source, line, "load into registers from inline asm")
            outputs = stmt.split(":")[1] if stmt.count(":") >= 1 else ""
            assert '"=' not in outputs and '"+' not in outputs, (source, line, "asm load with a register output")
        if re.search(r"\bm0\b", body):
            assert '"m0"' in stmt, (source, line, "asm writes m0 without clobbering it")
