"""The kernel sources themselves, run on the CPU emulator (tests/emu) against the oracle.

No GPU is involved: the very .hip files the product compiles for gfx950 are compiled as host
code against a stand-in HIP header and executed lane by lane (fibers), with the cross-lane
operations, matrix-instruction layouts, LDS addressing and global -> LDS moves modelled.  What
this checks is the kernels' logic -- indexing, swizzles, masking, pipelining and waits, split
merge, edge cases -- bit-exact for integer and byte work, and for the attention outputs to bars
several times tighter than the GPU parity tests' (out max-abs 3e-3 against 1e-2, lse 1e-4
against 1e-3; see OUT_TOL / LSE_TOL).  It says nothing about speed, and instruction-level
hazards (registers, spills, cache coherence) are outside its model.

Every forward case runs several times and must give the same bits each time: with the global ->
LDS moves landing as late as the kernel allows (at its waits) and as early as possible (at
issue) -- a missing wait fails the first, a ring slot refilled too soon the second; with a
workgroup's wavefronts advancing in step and one at a time for random stretches -- a missing
barrier fails the second.  Split launches also run with the workgroups in a shuffled order, so
that every split gets to be the one that merges, and with several workgroups sharing the
machine, so that the merging one has to wait for the others."""
import ctypes
import os
import sys

import numpy as np
import pytest
import torch

import oracle
from _util import max_abs, oracle_inputs, run_oracle, to_np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "emu"))
import harness  # noqa: E402

# The contract against the float64 oracle is 1e-2 on out and 1e-3 on the LSE.  The emulator's
# arithmetic is exact where the hardware's is approximate (exp2, log2, rcp), and the kernels'
# own roundings (probabilities and outputs to bf16, scaled fp8 values to bf16) stay far below the
# contract, so these tests hold the kernels to tighter bars: one dropped row of weight 1e-4, which
# the contract would let pass, fails here.  (Worst seen: LSE 4.7e-5, a one-entry list over an fp8
# cache, where the single score carries the bf16 rounding of the scaled values.)
OUT_TOL = 3e-3
LSE_TOL = 1e-4


@pytest.fixture(scope="module", autouse=True)
def _emulator():
    harness.lib()
    yield
    harness.configure()


@pytest.fixture(params=[(0, 0), (3, 0), (5, 4)], ids=["wavefronts_in_step", "wavefronts_skewed", "workgroups_sharing_the_machine"])
def schedule(request):
    """For tests that make a single call: once with a workgroup's wavefronts advancing together,
    once with them running one at a time for random stretches (only barriers keep them in step on
    the hardware), once with that and four workgroups at a time switched every few steps."""
    harness.configure(wave_skew_seed=request.param[0], concurrent_blocks=request.param[1], concurrent_seed=7)
    yield
    harness.configure()


def _check(cfg, out, lse, out_tol=OUT_TOL, lse_tol=LSE_TOL):
    ro, rl = run_oracle(cfg)
    H = cfg["q"].shape[-2]
    eo = max_abs(to_np(out).reshape(-1, H, 512), ro)
    el = max_abs(to_np(lse).reshape(-1, H), rl)
    assert eo <= out_tol, f"out max-abs {eo}"
    assert el <= lse_tol, f"lse max-abs {el}"


def _forward_all_ways(cfg, n_splits, **kw):
    """Forward under every emulator setting -- moves landing late or at once, workgroups in another
    order, one after the other or several sharing the machine, a workgroup's wavefronts advancing
    together or one at a time for random stretches; results must agree bit for bit.  Returns (out, lse)."""
    results = []
    # (skew seeds from 1000 on also hold one wavefront back until no other can move; the last number:
    # how many workgroups share the machine -- with splits, so that the merging one has to wait)
    settings = [(False, 0, 0, 0), (True, 0, 0, 0), (False, 0, 1, 0), (True, 0, 1002, 0)] + (
        [(False, 12345, 5, 4), (True, 777, 1001, 0), (True, 5, 0, 16)] if n_splits > 1 else [])
    for eager, order, skew, together in settings:
        harness.configure(dma_eager=eager, block_order_seed=order, wave_skew_seed=skew, concurrent_blocks=together, concurrent_seed=order)
        out, lse, rc = harness.forward(cfg, n_splits=n_splits, **kw)
        assert rc == 0, rc
        results.append((out, lse))
    harness.configure()
    for out, lse in results[1:]:
        assert torch.equal(out.view(torch.int16) if out.dtype == torch.bfloat16 else out,
                           results[0][0].view(torch.int16) if out.dtype == torch.bfloat16 else results[0][0])
        assert torch.equal(lse, results[0][1])
    return results[0]


def _fp8_cfg(batch, heads, pages_per_seq, topk, seed=1004, pad_frac=0.0):
    """decode_fp8 recipe on the CPU: records written by the emulated cache writer."""
    from flagtree_amd import workloads
    g = torch.Generator().manual_seed(seed)
    n_pages = batch * pages_per_seq
    rows = n_pages * 64
    bt = torch.randperm(n_pages, generator=g).to(torch.int32).view(batch, pages_per_seq)
    latent = (torch.randn((rows, 576), generator=g) * 0.1).to(torch.bfloat16)
    rec = torch.zeros((rows, 656), dtype=torch.uint8)
    rc = harness.lib().smla_kv_quantize_fp8(latent.data_ptr(), None, rec.data_ptr(), rows, rows, None)
    assert rc == 0
    q = (torch.randn((batch, 1, heads, 576), generator=g) * 0.1).to(torch.bfloat16)
    idx = workloads._topk_indices(batch, pages_per_seq * 64, topk, int(pad_frac * topk), g, True)
    return dict(q=q, kv_cache=rec.view(n_pages, 64, 656), indices=idx.view(batch, 1, topk), block_table=bt,
                page_size=64, sm_scale=workloads.SM_SCALE, kv_format="fp8_e4m3_b128", name="decode_fp8"), latent


# ---- forward kernels --------------------------------------------------------------------------

@pytest.mark.parametrize("heads,n_splits", [(128, 1), (128, 2), (64, 3), (96, 1), (40, 2)])
def test_many_heads_kernel_bf16(heads, n_splits):
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16("cpu", batch=2, heads=heads, pages_per_seq=10, topk=390, pad_frac=0.07)
    out, lse = _forward_all_ways(cfg, n_splits)
    _check(cfg, out, lse)


@pytest.mark.parametrize("heads,n_splits", [(16, 1), (16, 2), (8, 1), (32, 2), (24, 1)])
def test_few_heads_kernel_bf16(heads, n_splits):
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16("cpu", batch=2, heads=heads, pages_per_seq=10, topk=330, pad_frac=0.07)
    out, lse = _forward_all_ways(cfg, n_splits)
    _check(cfg, out, lse)


@pytest.mark.parametrize("heads,n_splits", [(16, 1), (16, 2), (128, 1), (128, 2), (8, 1)])
def test_fp8_records(heads, n_splits):
    cfg, _ = _fp8_cfg(2, heads, 6, 300, pad_frac=0.03)
    out, lse = _forward_all_ways(cfg, n_splits)
    _check(cfg, out, lse)


@pytest.mark.parametrize("topk,n_splits", [(1, 1), (31, 1), (32, 1), (33, 1), (64, 2), (65, 1), (96, 1), (97, 1), (128, 1),
                                           (129, 2), (200, 3), (1030, 1), (2100, 2)])
def test_many_heads_fp8_pipeline_at_every_tile_count(topk, n_splits):
    """The raw-record pipeline of the many-heads kernel has a prologue for the first two tiles,
    a steady state from the fourth tile on and a tail for the last three: lists of 1, 2, 3, 4 and 5
    tiles, ragged and full, more than one chunk of 1024 entries, and splits."""
    cfg, _ = _fp8_cfg(1, 40, 40, topk, pad_frac=0.0 if topk < 40 else 0.04)
    out, lse = _forward_all_ways(cfg, n_splits)
    _check(cfg, out, lse)


@pytest.mark.parametrize("topk,n_splits,heads", [(1, 1, 40), (33, 1, 128), (64, 2, 65), (97, 1, 128), (128, 1, 96), (129, 2, 128),
                                                 (200, 3, 128), (1030, 1, 40), (2100, 2, 128)])
def test_head_group_kernel_fp8_pipeline(topk, n_splits, heads, monkeypatch):
    """The same raw-record pipeline inside the wavefront-per-head-group kernel (its own row xor)."""
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1")
    cfg, _ = _fp8_cfg(1, heads, 40, topk, pad_frac=0.0 if topk < 40 else 0.04)
    out, lse = _forward_all_ways(cfg, n_splits)
    _check(cfg, out, lse)
    os.environ.pop("FLAGTREE_SMLA_HEAD_GROUPS")
    out1, lse1, rc = harness.forward(cfg, n_splits=n_splits)             # the first kernel
    assert rc == 0 and max_abs(to_np(out1), to_np(out)) <= 2e-3 and max_abs(to_np(lse1), to_np(lse)) <= 1e-5


@pytest.mark.parametrize("mode", ["first", "wavefront_per_head_group"])
def test_many_heads_fp8_redo_passes(mode, monkeypatch):
    if mode != "first":
        monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1")
    _many_heads_fp8_redo_passes()


def _many_heads_fp8_redo_passes():
    """Scores that outgrow the first tile's reference: the fp8 pipeline runs three times over the list."""
    g = torch.Generator().manual_seed(11)
    latent = (torch.randn((400, 576), generator=g) * 4.0).to(torch.bfloat16)
    latent[:64] *= 0.01
    rec = torch.zeros((400, 656), dtype=torch.uint8)
    assert harness.lib().smla_kv_quantize_fp8(latent.data_ptr(), None, rec.data_ptr(), 400, 400, None) == 0
    q = (torch.randn((2, 64, 576), generator=g) * 4.0).to(torch.bfloat16)
    cfg = dict(q=q, kv_cache=rec, indices=torch.arange(200, dtype=torch.int32).repeat(2, 1), block_table=None, page_size=64,
               sm_scale=576 ** -0.5, kv_format="fp8_e4m3_b128")
    # The kernel multiplies bf16(float(e4m3) * scale).  With scores of +-50 that rounding alone moves
    # a score by a few hundredths and, between two near-equal top scores, the output by percents; so
    # here (and only here) the oracle is fed the rounded products, which pins the pipeline itself.
    qn, kv_small, phys_small, _ = oracle_inputs(cfg)
    kv_small = torch.from_numpy(np.asarray(kv_small, dtype=np.float32)).to(torch.bfloat16).float().numpy()
    ro, rl = oracle.sparse_mla_fwd(qn, kv_small, phys_small, cfg["sm_scale"], 512)
    assert float(np.abs(rl).max()) > 40.0                     # far beyond what the first tile's reference allows for
    for ns in (1, 2):
        out, lse = _forward_all_ways(cfg, ns)
        assert max_abs(to_np(lse).reshape(rl.shape), rl) <= LSE_TOL * max(1.0, float(np.abs(rl).max()))
        assert max_abs(to_np(out).reshape(ro.shape), ro) <= 1.2e-2 * max(1.0, float(np.abs(ro).max()))


@pytest.fixture
def wide_kernel(monkeypatch):
    """Routes many-heads launches to the 128-heads-per-workgroup kernel (opt-in until it is measured)."""
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1")


@pytest.mark.parametrize("heads,n_splits,topk", [(128, 1, 300), (128, 2, 300), (64, 3, 200), (96, 1, 100), (40, 2, 70),
                                                 (200, 2, 130), (128, 4, 1100), (65, 3, 200), (129, 2, 90)])
def test_128_heads_per_workgroup_kernel(wide_kernel, heads, n_splits, topk):
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16("cpu", batch=2, heads=heads, pages_per_seq=20, topk=topk, pad_frac=0.07)
    out, lse = _forward_all_ways(cfg, n_splits)
    _check(cfg, out, lse)
    os.environ.pop("FLAGTREE_SMLA_HEAD_GROUPS")
    out1, lse1, rc = harness.forward(cfg, n_splits=n_splits)             # the first kernel: same results to the bar, not to the bit
    # (it sums in another order, so somewhere a last bit differs: the switch did select another kernel)
    assert rc == 0 and not (torch.equal(out1.view(torch.int16), out.view(torch.int16)) and torch.equal(lse1, lse))
    assert max_abs(to_np(out1), to_np(out)) <= 2e-3 and max_abs(to_np(lse1), to_np(lse)) <= 1e-5


def test_128_heads_kernel_edge_cases_redo_prefill_and_dense(wide_kernel):
    from flagtree_amd import workloads
    g = torch.Generator().manual_seed(7)
    kv = (torch.randn((300, 576), generator=g) * 0.1).to(torch.bfloat16)
    q = (torch.randn((6, 128, 576), generator=g) * 0.1).to(torch.bfloat16)
    idx = torch.full((6, 70), -1, dtype=torch.int32)
    idx[1, 33] = 5
    idx[2, :] = torch.randperm(300, generator=g)[:70].to(torch.int32)
    idx[3, :35] = 17
    idx[4, ::2] = torch.arange(35, dtype=torch.int32)
    idx[5, 0] = 299
    idx[5, 1] = 300
    cfg = dict(q=q, kv_cache=kv, indices=idx, block_table=None, page_size=64, sm_scale=576 ** -0.5, kv_format="bf16")
    for ns in (1, 2):
        out, lse = _forward_all_ways(cfg, ns)
        _check(cfg, out, lse)
        o, l = to_np(out), to_np(lse)
        assert (o[0] == 0).all() and np.isneginf(l[0]).all()
        assert np.array_equal(o[1], np.broadcast_to(to_np(kv)[5, :512], (128, 512)))
    # the exact two-pass path
    kv = (torch.randn((400, 576), generator=g) * 4.0).to(torch.bfloat16)
    kv[:64] *= 0.01
    q = (torch.randn((2, 128, 576), generator=g) * 4.0).to(torch.bfloat16)
    cfg = dict(q=q, kv_cache=kv, indices=torch.arange(200, dtype=torch.int32).repeat(2, 1), block_table=None, page_size=64,
               sm_scale=576 ** -0.5, kv_format="bf16")
    ro, rl = run_oracle(cfg)
    for ns in (1, 2):
        out, lse = _forward_all_ways(cfg, ns)
        assert max_abs(to_np(lse), rl) <= LSE_TOL * max(1.0, float(np.abs(rl).max()))
        assert max_abs(to_np(out), ro) <= 1.2e-2 * max(1.0, float(np.abs(ro).max()))
    # causal prefill, lists longer than a chunk, dense decode with a cap
    cfg = workloads.prefill_causal_bf16("cpu", tokens=40, heads=128, topk=48)
    out, lse = _forward_all_ways(cfg, 1)
    _check(cfg, out, lse)
    cfg = workloads.decode_bf16("cpu", batch=1, heads=128, pages_per_seq=40, topk=2100, pad_frac=0.05)
    out, lse = _forward_all_ways(cfg, 1)
    _check(cfg, out, lse)
    cfg = workloads.decode_bf16("cpu", batch=3, heads=128, pages_per_seq=5, topk=64, pad_frac=0.0)
    lens = torch.tensor([300, 1, 129], dtype=torch.int32)
    didx = torch.full((3, 1, 320), -1, dtype=torch.int32)
    for b, n in enumerate(lens.tolist()):
        didx[b, 0, :n] = torch.arange(n, dtype=torch.int32)
    qn, kv_small, phys_small, _ = oracle_inputs(dict(cfg, indices=didx))
    for cap in (0.0, 0.02):
        wo, wl = oracle.sparse_mla_fwd(qn, kv_small, phys_small, cfg["sm_scale"], 512, logit_cap=cap)
        out, lse = _forward_all_ways(cfg, 2, dense_lens=lens, logit_cap=cap)
        assert max_abs(to_np(lse), wl) <= LSE_TOL and max_abs(to_np(out), wo) <= OUT_TOL


FEW_HEADS_FP8_SWITCHES = {"column_split": "FLAGTREE_SMLA_FEW_FP8", "fp8_mfma": "FLAGTREE_SMLA_FP8_MFMA"}


@pytest.fixture(params=["column_split", "fp8_mfma"])
def few_fp8_kernel(request, monkeypatch):
    """Routes few-heads fp8 launches to one of the two-workgroups-per-CU kernels (opt-in until they are
    measured): the column-split one that converts records to bf16, or the one that contracts the
    records' e4m3 codes on the matrix cores."""
    monkeypatch.setenv(FEW_HEADS_FP8_SWITCHES[request.param], "1")
    return FEW_HEADS_FP8_SWITCHES[request.param]


@pytest.mark.parametrize("heads,n_splits,topk", [(16, 1, 300), (16, 2, 300), (8, 1, 70), (16, 3, 1100), (30, 2, 200), (16, 4, 40)])
def test_fp8_records_column_split_kernel(few_fp8_kernel, heads, n_splits, topk):
    cfg, _ = _fp8_cfg(2, heads, 20, topk, pad_frac=0.05)
    out, lse = _forward_all_ways(cfg, n_splits)
    _check(cfg, out, lse)
    # it is a different kernel: same results to the bar, not to the bit
    os.environ.pop(few_fp8_kernel)
    out1, lse1, rc = harness.forward(cfg, n_splits=n_splits)
    assert rc == 0 and not torch.equal(out1.view(torch.int16), out.view(torch.int16))
    assert max_abs(to_np(out1), to_np(out)) <= 2e-3 and max_abs(to_np(lse1), to_np(lse)) <= 1e-5


def test_column_split_kernel_edge_cases_redo_and_dense(few_fp8_kernel):
    # edge cases: empty list, single entry, duplicates, interleaved padding, out-of-range
    g = torch.Generator().manual_seed(7)
    latent = (torch.randn((300, 576), generator=g) * 0.1).to(torch.bfloat16)
    rec = torch.zeros((300, 656), dtype=torch.uint8)
    assert harness.lib().smla_kv_quantize_fp8(latent.data_ptr(), None, rec.data_ptr(), 300, 300, None) == 0
    q = (torch.randn((6, 16, 576), generator=g) * 0.1).to(torch.bfloat16)
    idx = torch.full((6, 70), -1, dtype=torch.int32)
    idx[1, 33] = 5
    idx[2, :] = torch.randperm(300, generator=g)[:70].to(torch.int32)
    idx[3, :35] = 17
    idx[4, ::2] = torch.arange(35, dtype=torch.int32)
    idx[5, 0] = 299
    idx[5, 1] = 300
    cfg = dict(q=q, kv_cache=rec, indices=idx, block_table=None, page_size=64, sm_scale=576 ** -0.5, kv_format="fp8_e4m3_b128")
    for ns in (1, 2):
        out, lse = _forward_all_ways(cfg, ns)
        _check(cfg, out, lse)
        assert (to_np(out)[0] == 0).all() and np.isneginf(to_np(lse)[0]).all()
    # scores that outgrow the first tile's maximum: the exact two-pass path
    latent = (torch.randn((400, 576), generator=g) * 4.0).to(torch.bfloat16)
    latent[:64] *= 0.01
    rec = torch.zeros((400, 656), dtype=torch.uint8)
    assert harness.lib().smla_kv_quantize_fp8(latent.data_ptr(), None, rec.data_ptr(), 400, 400, None) == 0
    q = (torch.randn((2, 16, 576), generator=g) * 4.0).to(torch.bfloat16)
    cfg = dict(q=q, kv_cache=rec, indices=torch.arange(200, dtype=torch.int32).repeat(2, 1), block_table=None, page_size=64,
               sm_scale=576 ** -0.5, kv_format="fp8_e4m3_b128")
    ro, rl = run_oracle(cfg)
    for ns in (1, 2):
        out, lse = _forward_all_ways(cfg, ns)
        assert max_abs(to_np(lse), rl) <= LSE_TOL * max(1.0, float(np.abs(rl).max()))
        assert max_abs(to_np(out), ro) <= 1.2e-2 * max(1.0, float(np.abs(ro).max()))
    # dense decode with a logit cap
    cfg, _ = _fp8_cfg(3, 16, 5, 64)
    lens = torch.tensor([300, 1, 129], dtype=torch.int32)
    idx = torch.full((3, 1, 320), -1, dtype=torch.int32)
    for b, n in enumerate(lens.tolist()):
        idx[b, 0, :n] = torch.arange(n, dtype=torch.int32)
    qn, kv_small, phys_small, _ = oracle_inputs(dict(cfg, indices=idx))
    for cap in (0.0, 0.02):
        wo, wl = oracle.sparse_mla_fwd(qn, kv_small, phys_small, cfg["sm_scale"], 512, logit_cap=cap)
        out, lse = _forward_all_ways(cfg, 2, dense_lens=lens, logit_cap=cap)
        assert max_abs(to_np(lse), wl) <= LSE_TOL and max_abs(to_np(out), wo) <= OUT_TOL


@pytest.mark.parametrize("kernel", ["many_heads", "wavefront_per_head_group"])
@pytest.mark.parametrize("case", ["prefill", "prefill_200_heads_two_chunks", "decode_many_tokens", "dense"])
def test_persistent_workgroups_give_the_same_bits(case, kernel, monkeypatch):
    """FLAGTREE_SMLA_PERSIST=1: launches of the many-heads kernel that do not split and have at least
    two items per compute unit run one workgroup per compute unit (16 here), which walks its items
    and sends for the next one's indices and Q while the current one's output is on its way out.
    Every item is computed by the same code on the same data: the same bits as one workgroup per
    item, with wavefronts in step, skewed, with moves landing at issue, and with workgroups
    sharing the machine."""
    from flagtree_amd import workloads
    lens = None
    if case == "prefill":
        cfg = workloads.prefill_causal_bf16("cpu", tokens=43, heads=128, topk=48)          # 43 tokens: ids without a token in between
    elif case == "prefill_200_heads_two_chunks":
        cfg = workloads.prefill_causal_bf16("cpu", tokens=40, heads=200, topk=1100)
    elif case == "decode_many_tokens":
        cfg = workloads.decode_bf16("cpu", batch=37, heads=128, pages_per_seq=8, topk=130, pad_frac=0.1)
    else:
        cfg = workloads.decode_bf16("cpu", batch=33, heads=128, pages_per_seq=3, topk=64)
        lens = torch.randint(0, 3 * 64 + 1, (33,), generator=torch.Generator().manual_seed(2), dtype=torch.int32)
    lib = harness.lib()
    monkeypatch.delenv("FLAGTREE_SMLA_PERSIST", raising=False)
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1" if kernel == "wavefront_per_head_group" else "0")
    if kernel == "wavefront_per_head_group" and case == "dense":
        cfg = workloads.decode_bf16("cpu", batch=33, heads=200, pages_per_seq=3, topk=64)       # 128 heads a workgroup: two head blocks an item
    blocks = lib.emu_block_count()
    out0, lse0, rc = harness.forward(cfg, n_splits=1, dense_lens=lens)
    one_per_item = lib.emu_block_count() - blocks
    assert rc == 0 and one_per_item >= 2 * harness.EMU_CUS
    monkeypatch.setenv("FLAGTREE_SMLA_PERSIST", "1")
    for skew, eager, together in ((0, False, 0), (3, True, 0), (5, False, 4)):
        harness.configure(wave_skew_seed=skew, dma_eager=eager, concurrent_blocks=together, concurrent_seed=3)
        blocks = lib.emu_block_count()
        out1, lse1, rc = harness.forward(cfg, n_splits=1, dense_lens=lens)
        assert rc == 0 and lib.emu_block_count() - blocks == harness.EMU_CUS          # it is the persistent launch
        assert torch.equal(out0.view(torch.int16), out1.view(torch.int16)) and torch.equal(lse0, lse1), (skew, eager, together)
    harness.configure()
    if lens is None:
        _check(cfg, out1, lse1)
    # a split launch, or one with fewer than two items per compute unit, is left alone
    blocks = lib.emu_block_count()
    small = workloads.decode_bf16("cpu", batch=3, heads=128, pages_per_seq=8, topk=130, pad_frac=0.1)
    harness.forward(small, n_splits=1)
    assert lib.emu_block_count() - blocks == 8 * (2 if kernel == "many_heads" else 1)


def test_more_than_one_chunk_of_the_list():
    """Lists longer than the 1024 entries the kernels compact at a time, ragged last tile."""
    from flagtree_amd import workloads
    for heads in (128, 16):
        cfg = workloads.decode_bf16("cpu", batch=1, heads=heads, pages_per_seq=40, topk=2100, pad_frac=0.05)
        out, lse = _forward_all_ways(cfg, 1)
        _check(cfg, out, lse)


def test_plumbing_f32_scalar_kernel(schedule):
    from flagtree_amd import workloads
    cfg = workloads.plumbing_f32("cpu", tokens=2, heads=16, s_kv=512, topk=64)
    out, lse, rc = harness.forward(cfg, n_splits=1)
    assert rc == 0
    _check(cfg, out, lse, out_tol=2e-6, lse_tol=2e-5)
    cfg = workloads.decode_bf16("cpu", batch=2, heads=16, pages_per_seq=8, topk=100, pad_frac=0.1)
    out, lse, rc = harness.forward(cfg, scalar=True)
    assert rc == 0
    _check(cfg, out, lse, out_tol=2e-3, lse_tol=1e-5)


def test_causal_prefill_reduced():
    from flagtree_amd import workloads
    cfg = workloads.prefill_causal_bf16("cpu", tokens=40, heads=128, topk=48)
    out, lse = _forward_all_ways(cfg, 1)
    idx = to_np(cfg["indices"]).reshape(40, 48)
    assert (idx[0] >= 0).sum() == 1 and (idx[39] >= 0).sum() == 40
    _check(cfg, out, lse)


@pytest.mark.parametrize("wide", ["0", "1"])
@pytest.mark.parametrize("heads,n_splits", [(128, 1), (128, 2), (16, 1), (16, 3)])
def test_token_bands_only_change_which_workgroup_takes_a_token(heads, n_splits, wide, monkeypatch):
    """FLAGTREE_SMLA_TOKEN_BANDS=1 hands each XCD a contiguous band of tokens instead of every
    eighth one: every token is still computed once, by the same code, so the results are the same
    bits (43 tokens: bands of 6, the last one short, some workgroups without a token)."""
    from flagtree_amd import workloads
    if heads == 16 and wide != "0":
        pytest.skip("the 128-heads kernel does not take 16 heads")
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", wide)
    cfg = workloads.prefill_causal_bf16("cpu", tokens=43, heads=heads, topk=300 if n_splits > 1 else 48)
    out0, lse0, rc = harness.forward(cfg, n_splits=n_splits)
    assert rc == 0
    monkeypatch.setenv("FLAGTREE_SMLA_TOKEN_BANDS", "1")
    out1, lse1, rc = harness.forward(cfg, n_splits=n_splits)
    assert rc == 0
    assert torch.equal(out0.view(torch.int16), out1.view(torch.int16)) and torch.equal(lse0, lse1)
    _check(cfg, out1, lse1)


@pytest.mark.parametrize("heads", [128, 16])
def test_edge_cases(heads):
    g = torch.Generator().manual_seed(7)
    kv = (torch.randn((300, 576), generator=g) * 0.1).to(torch.bfloat16)
    q = (torch.randn((6, heads, 576), generator=g) * 0.1).to(torch.bfloat16)
    idx = torch.full((6, 70), -1, dtype=torch.int32)
    idx[1, 33] = 5                                           # single valid entry
    idx[2, :] = torch.randperm(300, generator=g)[:70].to(torch.int32)   # all valid, ragged top-k (70)
    idx[3, :35] = 17                                         # duplicates count once per occurrence
    idx[4, ::2] = torch.arange(35, dtype=torch.int32)        # interleaved padding
    idx[5, 0] = 299
    idx[5, 1] = 300                                          # out of range -> masked
    cfg = dict(q=q, kv_cache=kv, indices=idx, block_table=None, page_size=64, sm_scale=576 ** -0.5, kv_format="bf16")
    for ns in (1, 2):
        out, lse = _forward_all_ways(cfg, ns)
        _check(cfg, out, lse)
        o, l = to_np(out), to_np(lse)
        assert (o[0] == 0).all() and np.isneginf(l[0]).all()          # token without valid entries
        assert np.array_equal(o[1], np.broadcast_to(to_np(kv)[5, :512], (heads, 512)))   # K = 1: out = v


@pytest.mark.parametrize("heads", [128, 16])
def test_wide_score_range_takes_the_redo_passes(heads):
    """Scores that outgrow the first tile's maximum by more than the slack force the exact
    two-pass path; outputs reach 4, so the bar is relative."""
    g = torch.Generator().manual_seed(11)
    kv = (torch.randn((400, 576), generator=g) * 4.0).to(torch.bfloat16)
    kv[:64] *= 0.01                                          # a first tile with tiny scores
    q = (torch.randn((2, heads, 576), generator=g) * 4.0).to(torch.bfloat16)
    idx = torch.arange(200, dtype=torch.int32).repeat(2, 1)
    cfg = dict(q=q, kv_cache=kv, indices=idx, block_table=None, page_size=64, sm_scale=576 ** -0.5, kv_format="bf16")
    ro, rl = run_oracle(cfg)
    for ns in (1, 2):
        out, lse = _forward_all_ways(cfg, ns)
        assert max_abs(to_np(lse), rl) <= LSE_TOL * max(1.0, float(np.abs(rl).max()))
        assert max_abs(to_np(out), ro) <= 1.2e-2 * max(1.0, float(np.abs(ro).max()))


@pytest.mark.parametrize("heads,fmt", [(128, "bf16"), (16, "bf16"), (16, "fp8")])
def test_dense_decode(heads, fmt):
    from flagtree_amd import workloads
    if fmt == "fp8":
        cfg, _ = _fp8_cfg(3, heads, 5, 64)
    else:
        cfg = workloads.decode_bf16("cpu", batch=3, heads=heads, pages_per_seq=5, topk=64, pad_frac=0.0)
    lens = torch.tensor([300, 1, 129], dtype=torch.int32)
    out, lse = _forward_all_ways(cfg, 2, dense_lens=lens)
    listed = dict(cfg)
    idx = torch.full((3, 1, 320), -1, dtype=torch.int32)
    for b, n in enumerate(lens.tolist()):
        idx[b, 0, :n] = torch.arange(n, dtype=torch.int32)
    listed["indices"] = idx
    _check(listed, out, lse)


@pytest.mark.parametrize("heads,fmt,std,cap,min_diff", [(128, "bf16", 1.5, 2.0, 0.5), (16, "bf16", 1.5, 2.0, 0.5),
                                                        (16, "fp8", 1.5, 2.0, 0.5), (64, "fp8", 0.5, 0.2, 0.01)])
def test_dense_decode_with_logit_cap(heads, fmt, std, cap, min_diff):
    """cap * tanh(score / cap) before the softmax; inputs scaled so that raw scores are several caps.
    (The many-heads kernel rounds dequantised fp8 values to bf16 when it stages them, an error that
    grows with the square of the input scale: its case stays nearer the benchmark's magnitudes.)"""
    g = torch.Generator().manual_seed(31 + heads)
    B, pages = 3, 5
    bt = torch.randperm(B * pages, generator=g).to(torch.int32).view(B, pages)
    latent = (torch.randn((B * pages * 64, 576), generator=g) * std).to(torch.bfloat16)
    q = (torch.randn((B, 1, heads, 576), generator=g) * std).to(torch.bfloat16)
    if fmt == "fp8":
        kv = torch.zeros((latent.shape[0], 656), dtype=torch.uint8)
        assert harness.lib().smla_kv_quantize_fp8(latent.data_ptr(), None, kv.data_ptr(), kv.shape[0], kv.shape[0], None) == 0
        kv, kvf = kv.view(-1, 64, 656), "fp8_e4m3_b128"
    else:
        kv, kvf = latent.view(-1, 64, 576), "bf16"
    lens = torch.tensor([300, 2, 129], dtype=torch.int32)
    cfg = dict(q=q, kv_cache=kv, indices=None, block_table=bt, page_size=64, sm_scale=576 ** -0.5, kv_format=kvf)
    idx = torch.full((B, 1, 320), -1, dtype=torch.int32)
    for b, n in enumerate(lens.tolist()):
        idx[b, 0, :n] = torch.arange(n, dtype=torch.int32)
    listed = dict(cfg, indices=idx)
    qn, kv_small, phys_small, _ = oracle_inputs(listed)
    wo, wl = oracle.sparse_mla_fwd(qn, kv_small, phys_small, cfg["sm_scale"], 512, logit_cap=cap)
    uo, ul = oracle.sparse_mla_fwd(qn, kv_small, phys_small, cfg["sm_scale"], 512)
    assert max_abs(wl, ul) > min_diff
    for ns in (1, 2):
        out, lse = _forward_all_ways(cfg, ns, dense_lens=lens, logit_cap=cap)
        # (fp8: inputs five times the benchmark's and a context of two rows -- the bf16 rounding of the
        # scaled values shows in full, 3e-4; the contract's bar)
        assert max_abs(to_np(lse), wl) <= (1e-3 if fmt == "fp8" else LSE_TOL)
        assert max_abs(to_np(out), wo) <= 5e-3 * max(1.0, float(np.abs(wo).max()))       # (outputs up to 6 here: half a bf16 step of the output alone is 2^-9 of it)


@pytest.mark.parametrize("seed", list(range(12)))
@pytest.mark.parametrize("few_fp8", [False, True, "fp8_mfma", "head_groups"])
def test_random_shapes_against_oracle(seed, few_fp8, monkeypatch):
    """Seeded draws over head counts, list lengths, page sizes, tokens per sequence, split counts,
    padding patterns, page tables with holes and both cache formats (the GPU suite's recipe at sizes
    the emulator handles); each draw also on the opt-in fp8 kernel when it applies."""
    rng = np.random.default_rng(4000 + seed)
    g = torch.Generator().manual_seed(4000 + seed)
    heads = int(rng.choice([1, 7, 16, 17, 32, 33, 64, 65, 127, 128]))
    topk = int(rng.choice([1, 31, 32, 33, 100, 257, 1100]))
    page_size = int(rng.choice([1, 16, 64]))
    tokens_per_seq = int(rng.choice([1, 3]))
    batch = int(rng.choice([1, 2]))
    fmt = "fp8_e4m3_b128" if rng.random() < 0.45 else "bf16"
    n_splits = [1, 2, 3, 5][int(rng.integers(4))]
    paged = rng.random() < 0.7
    ctx = int(rng.choice([64, 300, 1200]))
    if few_fp8 == "head_groups":
        if heads <= 32:
            pytest.skip("the opt-in kernel covers many heads")
        monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1")
    elif few_fp8:
        if fmt != "fp8_e4m3_b128" or heads > 32:
            pytest.skip("the opt-in kernel covers few heads over an fp8 cache")
        monkeypatch.setenv("FLAGTREE_SMLA_FP8_MFMA" if few_fp8 == "fp8_mfma" else "FLAGTREE_SMLA_FEW_FP8", "1")
    if paged:
        pages_per_seq = -(-ctx // page_size)
        n_pages = batch * pages_per_seq + 3
        lat = (torch.randn((n_pages * page_size, 576), generator=g) * 0.1).to(torch.bfloat16)
        bt = torch.randperm(n_pages, generator=g)[:batch * pages_per_seq].to(torch.int32).view(batch, pages_per_seq)
        if pages_per_seq > 2 and rng.random() < 0.5:
            bt[0, 1] = -1
        hi = pages_per_seq * page_size + (3 if rng.random() < 0.3 else 0)
    else:
        lat = (torch.randn((batch * ctx + 128, 576), generator=g) * float(rng.choice([0.05, 0.2]))).to(torch.bfloat16)
        bt = None
        hi = lat.shape[0] + (2 if rng.random() < 0.3 else 0)
    T = batch * tokens_per_seq
    idx = torch.from_numpy(rng.integers(0, hi, size=(T, topk)).astype(np.int32))
    idx[torch.from_numpy(rng.random((T, topk)) < float(rng.choice([0.0, 0.1, 0.6])))] = -1
    if rng.random() < 0.3:
        idx[0, topk // 2:] = -1
    if T > 1 and rng.random() < 0.3:
        idx[1, :] = -1
    q = (torch.randn((batch, tokens_per_seq, heads, 576), generator=g) * 0.1).to(torch.bfloat16)
    if fmt == "bf16":
        kv = lat
    else:
        kv = torch.zeros((lat.shape[0], 656), dtype=torch.uint8)
        assert harness.lib().smla_kv_quantize_fp8(lat.data_ptr(), None, kv.data_ptr(), lat.shape[0], lat.shape[0], None) == 0
    if paged:
        kv = kv.view(-1, page_size, kv.shape[-1])
    n_splits = min(n_splits, max(1, topk // 32))
    cfg = dict(q=q, kv_cache=kv, indices=idx.view(batch, tokens_per_seq, topk), block_table=bt, page_size=page_size,
               sm_scale=576 ** -0.5, kv_format=fmt)
    out, lse = _forward_all_ways(cfg, n_splits)
    _check(cfg, out, lse)


@pytest.mark.parametrize("heads", [16, 128])
@pytest.mark.parametrize("bt_stride", [9001, 8190])
def test_page_tables_that_do_not_fit_or_align(heads, bt_stride):
    """Page-table rows longer than the LDS staging area, or not a multiple of 16 bytes, take the
    global lookup path; long lists span several 1024-entry chunks with an empty one in the middle."""
    g = torch.Generator().manual_seed(77 + heads + bt_stride)
    B, topk = 1, 2300
    n_pages = B * bt_stride + 5
    bt = torch.randperm(n_pages, generator=g)[:B * bt_stride].to(torch.int32).view(B, bt_stride)
    kv = (torch.randn((n_pages, 1, 576), generator=g) * 0.1).to(torch.bfloat16)
    idx = torch.stack([torch.randperm(bt_stride, generator=g)[:topk] for _ in range(B)]).to(torch.int32)
    idx[0, 100:1300] = -1
    q = (torch.randn((B, 1, heads, 576), generator=g) * 0.1).to(torch.bfloat16)
    cfg = dict(q=q, kv_cache=kv, indices=idx.view(B, 1, topk), block_table=bt, page_size=1, sm_scale=576 ** -0.5, kv_format="bf16")
    for ns in (1, 2):
        out, lse = _forward_all_ways(cfg, ns)
        _check(cfg, out, lse)


# ---- split workspace: failure handling --------------------------------------------------------

def _words(ws):
    from flagtree_amd import _lib
    return ws[:_lib.SMLA_WS_HEADER_OFFSET].view(torch.int64)


def _header(ws):
    from flagtree_amd import _lib
    return ws[_lib.SMLA_WS_HEADER_OFFSET:_lib.SMLA_WS_HEADER_OFFSET + 16].view(torch.int32)


@pytest.mark.parametrize("kernel", ["many_heads", "wavefront_per_head_group", "few_heads", "few_heads_fp8_column_split", "few_heads_fp8_mfma"])
def test_merging_workgroup_really_waits_for_the_others(kernel, monkeypatch):
    """With one workgroup at a time the last arrival of a split merge always finds the others'
    partials published.  Here several share the machine and are switched every few steps: the
    merging workgroup polls, the others publish meanwhile (the poll count says it happened), and
    the results are the same bits as without any waiting."""
    from flagtree_amd import workloads
    heads = 128 if kernel in ("many_heads", "wavefront_per_head_group") else 16
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1" if kernel == "wavefront_per_head_group" else "0")
    monkeypatch.setenv("FLAGTREE_SMLA_FEW_FP8", "1" if kernel == "few_heads_fp8_column_split" else "0")
    monkeypatch.setenv("FLAGTREE_SMLA_FP8_MFMA", "1" if kernel == "few_heads_fp8_mfma" else "0")
    if kernel.startswith("few_heads_fp8"):
        cfg, _ = _fp8_cfg(3, heads, 20, 400, pad_frac=0.05)
    else:
        cfg = workloads.decode_bf16("cpu", batch=3, heads=heads, pages_per_seq=20, topk=400, pad_frac=0.05)
    harness.configure()
    out0, lse0, rc = harness.forward(cfg, n_splits=3)
    assert rc == 0
    waited = 0
    for n, seed in enumerate(range(2, 26)):
        if n >= 4 and waited > 0:
            break
        together, skew = ((4, 5), (16, 0), (6, 9), (3, 5))[n % 4]
        harness.configure(dma_eager=bool(seed & 1), wave_skew_seed=skew, concurrent_blocks=together, concurrent_seed=seed, block_order_seed=seed)
        before = harness.lib().emu_poll_count()
        out, lse, rc = harness.forward(cfg, n_splits=3)
        waited += harness.lib().emu_poll_count() - before
        assert rc == 0
        assert torch.equal(out.view(torch.int16), out0.view(torch.int16)) and torch.equal(lse, lse0)
    harness.configure()
    assert waited > 0
    _check(cfg, out0, lse0)


@pytest.mark.parametrize("heads", [128, 16])
@pytest.mark.parametrize("stale", ["one ticket", "own bit", "all ones"])
def test_stale_arrival_word_is_flagged_not_hung(heads, stale, schedule):
    from flagtree_amd import _lib, workloads
    cfg = workloads.decode_bf16("cpu", batch=3, heads=heads, pages_per_seq=6, topk=260, pad_frac=0.05)
    ref_out, ref_lse, rc = harness.forward(cfg, n_splits=1)
    assert rc == 0
    n_hblocks = (heads + 63) // 64 if heads > 32 else (heads + 15) // 16
    ws = harness.make_workspace(harness.lib().smla_workspace_bytes(3, heads, 512, 2))
    _header(ws)[2] = 50
    _words(ws)[1 * n_hblocks] = {"one ticket": 1 << 32, "own bit": 1, "all ones": -1}[stale]
    out, lse, rc = harness.forward(cfg, n_splits=2, workspace=ws)
    assert rc == 0
    rc, status = harness.workspace_status(ws)
    assert rc == _lib.SMLA_EWORKSPACE_STATE and status & (2 | 4)
    per_block = 64 if heads > 32 else 16
    l = to_np(lse)
    assert np.isnan(l[1, :min(per_block, heads)]).all()
    # workgroups that started after the flag went up give up as well (here they run one after the
    # other, on the GPU most start together): every other row is either right or marked, never wrong
    others = l[[0, 2]]
    assert (np.isnan(others) | (np.abs(others - to_np(ref_lse)[[0, 2]]) <= 1e-3)).all()
    marked = np.isnan(l)
    assert not to_np(out).reshape(3, heads, 512)[marked].any()           # marked rows are zero
    assert harness.workspace_status(ws) == (0, 0)
    assert int((_words(ws) != 0).sum()) == 0
    out2, lse2, rc = harness.forward(cfg, n_splits=2, workspace=ws)
    assert rc == 0 and harness.workspace_status(ws) == (0, 0)
    assert max_abs(to_np(lse2), to_np(ref_lse)) <= 1e-3 and max_abs(to_np(out2), to_np(ref_out)) <= 1e-2


@pytest.mark.parametrize("kernel", ["many_heads", "wavefront_per_head_group", "few_heads", "few_heads_fp8_column_split", "few_heads_fp8_mfma"])
def test_flagged_workspace_stays_loud_until_the_host_has_looked(kernel, monkeypatch):
    """A launch that gave up may leave an arrival word in a state the next launch cannot tell from
    a legal one: here one ticket and the OTHER split's published bit, with two splits.  Judged by
    the word alone, this split would draw the last ticket, find the bit set and fold in whatever
    the partial buffer holds.  The status word the first launch left makes every split give up
    instead (NaN LSE, zero output) until smla_workspace_status has run."""
    from flagtree_amd import _lib, workloads
    heads = 128 if kernel in ("many_heads", "wavefront_per_head_group") else 16
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1" if kernel == "wavefront_per_head_group" else "0")
    monkeypatch.setenv("FLAGTREE_SMLA_FEW_FP8", "1" if kernel == "few_heads_fp8_column_split" else "0")
    monkeypatch.setenv("FLAGTREE_SMLA_FP8_MFMA", "1" if kernel == "few_heads_fp8_mfma" else "0")
    if kernel.startswith("few_heads_fp8"):
        cfg, _ = _fp8_cfg(2, heads, 6, 260, pad_frac=0.05)
    else:
        cfg = workloads.decode_bf16("cpu", batch=2, heads=heads, pages_per_seq=6, topk=260, pad_frac=0.05)
    ref_out, ref_lse, rc = harness.forward(cfg, n_splits=1)
    assert rc == 0
    ws = harness.make_workspace(harness.lib().smla_workspace_bytes(2, heads, 512, 2))
    ws[_lib.SMLA_WS_COUNTER_BYTES:] = 0x3C                   # partials nobody wrote: finite garbage
    _header(ws)[1] = 4                                        # what a timed-out merge leaves
    _words(ws)[:] = (1 << 32) | 2                             # ... and a late publisher of split 1
    out, lse, rc = harness.forward(cfg, n_splits=2, workspace=ws)
    assert rc == 0
    assert np.isnan(to_np(lse)).all() and not to_np(out).any()
    assert int((_words(ws) != ((1 << 32) | 2)).sum()) == 0    # nobody took a ticket
    rc, status = harness.workspace_status(ws)
    assert rc == _lib.SMLA_EWORKSPACE_STATE and status == 4
    assert harness.workspace_status(ws) == (0, 0) and int((_words(ws) != 0).sum()) == 0
    out2, lse2, rc = harness.forward(cfg, n_splits=2, workspace=ws)
    assert rc == 0 and harness.workspace_status(ws) == (0, 0)
    assert max_abs(to_np(lse2), to_np(ref_lse)) <= 1e-3 and max_abs(to_np(out2), to_np(ref_out)) <= 1e-2


@pytest.mark.parametrize("how", ["compute units of an unknown layout", "environment"])
@pytest.mark.parametrize("kernel", ["many_heads", "wavefront_per_head_group", "few_heads", "few_heads_fp8_column_split", "few_heads_fp8_mfma"])
def test_splits_merged_by_a_second_launch(kernel, how, monkeypatch, schedule):
    """The merge inside the launch needs all workgroups of a token behind one L2, which the library
    only claims for compute-unit counts it knows the XCD layout of.  Elsewhere (here: 48 compute
    units), or when asked to, every split publishes and the merge kernel runs as a second launch:
    same results to the bar, arrival words never touched, and an uninitialised workspace is fine."""
    from flagtree_amd import workloads
    heads = 128 if kernel in ("many_heads", "wavefront_per_head_group") else 16
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1" if kernel == "wavefront_per_head_group" else "0")
    monkeypatch.setenv("FLAGTREE_SMLA_FEW_FP8", "1" if kernel == "few_heads_fp8_column_split" else "0")
    monkeypatch.setenv("FLAGTREE_SMLA_FP8_MFMA", "1" if kernel == "few_heads_fp8_mfma" else "0")
    if kernel.startswith("few_heads_fp8"):
        cfg, _ = _fp8_cfg(3, heads, 6, 330, pad_frac=0.05)
    else:
        cfg = workloads.decode_bf16("cpu", batch=3, heads=heads, pages_per_seq=6, topk=330, pad_frac=0.05)
    lib = harness.lib()
    assert lib.smla_merge_in_launch() == 1
    out1, lse1, rc = harness.forward(cfg, n_splits=3)
    assert rc == 0
    try:
        if how == "environment":
            monkeypatch.setenv("FLAGTREE_SMLA_SEPARATE_MERGE", "1")
        else:
            lib.emu_set_cu_count(48)
        assert lib.smla_merge_in_launch() == 0
        ws = torch.full((lib.smla_workspace_bytes(3, heads, 512, 3),), 0x3C, dtype=torch.uint8)     # never initialised
        launches = lib.emu_launch_count()
        out, lse, rc = harness.forward(cfg, n_splits=3, workspace=ws)
        assert rc == 0 and lib.emu_launch_count() - launches == 2
        assert int((_words(ws) != 0x3C3C3C3C3C3C3C3C).sum()) == 0 and int((_header(ws) != 0x3C3C3C3C).sum()) == 0
    finally:
        lib.emu_set_cu_count(harness.EMU_CUS)
    _check(cfg, out, lse)
    assert max_abs(to_np(out), to_np(out1)) <= 2e-3 and max_abs(to_np(lse), to_np(lse1)) <= 1e-5


def test_merge_inside_the_launch_only_on_known_compute_unit_counts():
    lib = harness.lib()
    try:
        for n, want in ((16, 1), (32, 1), (64, 1), (128, 1), (256, 1), (20, 1), (48, 0), (96, 0), (240, 0), (304, 0)):
            lib.emu_set_cu_count(n)
            assert lib.smla_merge_in_launch() == want, n
    finally:
        lib.emu_set_cu_count(harness.EMU_CUS)


def test_uninitialised_workspace_is_flagged(schedule):
    from flagtree_amd import _lib, workloads
    cfg = workloads.decode_bf16("cpu", batch=2, heads=128, pages_per_seq=6, topk=260, pad_frac=0.05)
    ws = torch.zeros(harness.lib().smla_workspace_bytes(2, 128, 512, 2), dtype=torch.uint8)
    out, lse, rc = harness.forward(cfg, n_splits=2, workspace=ws)
    assert rc == 0
    rc, status = harness.workspace_status(ws)
    assert rc == _lib.SMLA_EWORKSPACE_STATE and status & 1
    assert np.isnan(to_np(lse)).all()


# ---- integer / byte paths: bit-exact ------------------------------------------------------------

def test_gather_and_translation_bit_exact(schedule):
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16("cpu", batch=5, heads=16, pages_per_seq=8, topk=96, pad_frac=0.2)
    idx = cfg["indices"].clone().view(5, 96)
    idx[0, 0] = -1
    idx[1, 50] = 8 * 64
    idx[2, 95] = 2 ** 31 - 1
    idx[3, :] = -1
    kv = cfg["kv_cache"].view(torch.int16).reshape(-1, 576).contiguous()
    bt = cfg["block_table"].contiguous()
    phys = torch.full((5, 96), -7, dtype=torch.int32)
    rows = torch.full((5, 96, 576), -7, dtype=torch.int16)
    rc = harness.lib().smla_gather_rows(kv.data_ptr(), 1152, idx.data_ptr(), bt.data_ptr(), phys.data_ptr(), rows.data_ptr(),
                                        5, 1, 96, 64, bt.shape[1], 0, kv.shape[0], None)
    assert rc == 0
    want = oracle.translate_indices(to_np(idx), to_np(bt), 64, kv_rows=kv.shape[0])
    assert np.array_equal(to_np(phys).astype(np.int64), want)
    assert np.array_equal(to_np(rows), oracle.gather_rows(to_np(kv), want))


def test_cache_writer_bit_exact(schedule):
    g = torch.Generator().manual_seed(3)
    latent = (torch.randn((200, 576), generator=g) * torch.logspace(-3, 2, 200).view(-1, 1)).to(torch.bfloat16)
    latent[5, 100:228] = 0                                   # an all-zero block
    slots = torch.randperm(260, generator=g)[:200].to(torch.int64) - 20
    for fmt, code, width, dtype in (("fp8_e4m3_b128", 1, 656, torch.uint8), ("bf16", 0, 576, torch.bfloat16)):
        cache = torch.zeros((220, width), dtype=dtype)
        rc = harness.lib().smla_kv_write(code, latent.data_ptr(), slots.data_ptr(), cache.data_ptr(), 200, 220, None)
        assert rc == 0
        want = np.zeros((220, width), dtype=np.uint8 if fmt != "bf16" else np.uint16)
        want = oracle.reshape_and_cache(to_np(latent), want, slots.numpy(), kv_format=fmt)
        got = cache.numpy() if fmt != "bf16" else cache.view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(got, want), fmt


def test_cache_writer_scale_of_every_block_maximum():
    """The writer divides a block's maximum by 448 with a multiplication and a fused correction
    instead of an IEEE division: every positive finite bf16 value is the maximum of one block here
    (with its half and its negative beside it), and scales and codes must be the oracle's bits."""
    bits = np.arange(1, 0x7F80, dtype=np.uint16)                         # every positive finite bf16
    bits = np.concatenate([bits, np.full((-len(bits)) % 4, 0x3F80, np.uint16)])
    blocks = np.zeros((len(bits), 128), dtype=np.uint16)
    blocks[:, 17] = bits
    blocks[:, 90] = bits | 0x8000
    half = np.where((bits >> 7) > 1, bits - 0x80, 0).astype(np.uint16)   # exponent - 1 where that stays normal
    blocks[:, 3] = half
    lat_bits = np.concatenate([blocks.reshape(-1, 512), blocks.reshape(-1, 512)[:, :64]], axis=1)
    lat = torch.from_numpy(lat_bits.view(np.int16).copy()).view(torch.bfloat16)
    n = lat.shape[0]
    cache = torch.zeros((n, 656), dtype=torch.uint8)
    rc = harness.lib().smla_kv_write(1, lat.data_ptr(), None, cache.data_ptr(), n, n, None)
    assert rc == 0
    want = oracle.quantize_kv_records(oracle.bf16_bits_to_f32(lat_bits))
    got = cache.numpy()
    assert np.array_equal(got[:, 512:528], want[:, 512:528]), "scales"
    assert np.array_equal(got, want)


@pytest.mark.parametrize("rows,n,k", [(3, 4096, 2048), (2, 1000, 64), (1, 20000, 300), (2, 70000, 128), (5, 33, 40)])
def test_topk_indices_exact(rows, n, k):
    g = torch.Generator().manual_seed(rows * 131 + n)
    scores = torch.randn((rows, n), generator=g)
    scores[0, : n // 3] = scores[0, 0]                        # ties across the selection boundary
    scores[-1, 5 % n] = float("nan")
    lens = torch.randint(1, n + 1, (rows,), generator=g, dtype=torch.int32)
    want = oracle.topk_indices(to_np(scores), k, to_np(lens))
    for skew in (0, 1, 2):
        harness.configure(wave_skew_seed=skew)
        out = torch.full((rows, k), -9, dtype=torch.int32)
        rc = harness.lib().smla_topk_indices(scores.data_ptr(), lens.data_ptr(), out.data_ptr(), rows, n, n, k, None, 0, None)
        assert rc == 0
        assert np.array_equal(to_np(out), want), skew
    harness.configure()


@pytest.mark.parametrize("n,length,k", [(65537, 300, 64), (65537, 10117, 300), (70001, 70001, 2048), (65536, 1000, 64)])
def test_topk_indices_with_tied_values_in_long_rows(n, length, k):
    """Scores rounded to quarters, so that the k-th place is shared by many entries, in rows above
    and at the length where the launcher changes kernels.  In the kernel for long rows the vote
    that ranks the tied entries is the last thing a lane does: lanes that leave the kernel right
    after it must still count in the vote as the lanes behind them read it (the emulator once
    dropped them)."""
    g = torch.Generator().manual_seed(n + length + k)
    scores = (torch.randn((2, n), generator=g) * 4).round() / 4
    lens = torch.tensor([length, max(1, length // 3)], dtype=torch.int32)
    want = oracle.topk_indices(to_np(scores), k, to_np(lens))
    for skew in (0, 1):
        harness.configure(wave_skew_seed=skew)
        out = torch.full((2, k), -9, dtype=torch.int32)
        rc = harness.lib().smla_topk_indices(scores.data_ptr(), lens.data_ptr(), out.data_ptr(), 2, n, n, k, None, 0, None)
        assert rc == 0
        assert np.array_equal(to_np(out), want), skew
    harness.configure()


@pytest.mark.parametrize("rows,n,k", [(1, 20000, 300), (2, 65536, 2048), (3, 8192, 64), (1, 70001, 2048), (2, 300000, 128), (1, 9000, 9000)])
def test_topk_rows_cut_into_parts_give_the_same_list(rows, n, k):
    """Few long rows with a workspace: every part of a row selects its own k largest, a second
    launch selects the row's from the parts' candidates.  Exact against the oracle and entry for
    entry what one workgroup per row gives: ties (quantised scores) at the k-th value, also across
    part boundaries, NaN, -inf, context lengths that end inside the first part or leave parts empty."""
    lib = harness.lib()
    need = lib.smla_topk_workspace_bytes(rows, n, k)
    assert need > 0
    g = torch.Generator().manual_seed(rows * 1000 + k)
    for case in range(4):
        scores = torch.randn((rows, n), generator=g)
        if case >= 1:
            scores = (scores * 2).round() / 2                           # heavy ties
        if case == 2:
            scores[0, : n // 2] = float("-inf")
            scores[-1, n // 3] = float("nan")
        lens = torch.tensor([n, max(1, n // 5), 3][:rows], dtype=torch.int32)
        if case == 3:
            lens = torch.tensor([n - 1, 4097, 0][:rows], dtype=torch.int32)
        want = oracle.topk_indices(to_np(scores), k, to_np(lens))
        for skew in (0, 3):
            harness.configure(wave_skew_seed=skew, concurrent_blocks=4 if skew else 0, concurrent_seed=5)
            ws = torch.full((need,), 0x5A, dtype=torch.uint8)
            out = torch.full((rows, k), -9, dtype=torch.int32)
            launches = lib.emu_launch_count()
            rc = lib.smla_topk_indices(scores.data_ptr(), lens.data_ptr(), out.data_ptr(), rows, n, n, k, ws.data_ptr(), need, None)
            assert rc == 0 and lib.emu_launch_count() - launches == 2
            assert np.array_equal(to_np(out), want), (case, skew)
    harness.configure()
    # too small a workspace, or none: one workgroup per row, same answer
    out1 = torch.full((rows, k), -9, dtype=torch.int32)
    launches = lib.emu_launch_count()
    assert lib.smla_topk_indices(scores.data_ptr(), lens.data_ptr(), out1.data_ptr(), rows, n, n, k, ws.data_ptr(), need - 1, None) == 0
    assert lib.emu_launch_count() - launches == 1 and np.array_equal(to_np(out1), want)


def test_topk_tie_run_across_a_part_boundary():
    """All entries equal around the boundary between two parts: the k-th place falls inside the run,
    and the entries taken are the ones of lowest index, whichever part they lie in."""
    lib = harness.lib()
    n, k = 16384, 5000
    need = lib.smla_topk_workspace_bytes(1, n, k)
    assert need > 0
    scores = torch.zeros((1, n))
    scores[0, 100:3000] = 1.0                                          # 2900 entries above the run, all in the first part
    scores[0, 12000:12100] = 2.0                                       # 100 more in a later part
    want = oracle.topk_indices(to_np(scores), k, None)
    assert (want[0] >= 0).all() and want[0].max() < 12100
    ws = torch.zeros(need, dtype=torch.uint8)
    out = torch.full((1, k), -9, dtype=torch.int32)
    assert lib.smla_topk_indices(scores.data_ptr(), None, out.data_ptr(), 1, n, n, k, ws.data_ptr(), need, None) == 0
    assert np.array_equal(to_np(out), want)


@pytest.mark.parametrize("rows,n,k,page_size,rows_per_seq", [(4, 3000, 200, 64, 2), (2, 20000, 300, 16, 1), (3, 70001, 128, 128, 1),
                                                             (6, 1000, 1000, 1, 3)])
def test_topk_written_as_physical_rows(rows, n, k, page_size, rows_per_seq):
    """smla_topk_rows = the selection followed by the page translation the attention kernels do
    (oracle.translate_indices), bit for bit: a table that covers only part of the positions, a hole
    (negative page number) and pages past the pool included; one workgroup per row and rows cut
    into parts; and the attention kernel fed with the rows gives the bits it gives when it does
    the look-up itself."""
    lib = harness.lib()
    g = torch.Generator().manual_seed(rows + n)
    scores = torch.randn((rows, n), generator=g)
    lens = torch.randint(1, n + 1, (rows,), generator=g, dtype=torch.int32)
    n_seqs = rows // rows_per_seq
    pages = max(1, (n * 3 // 4) // page_size)                   # the table ends before the longest contexts do
    bt = torch.randperm(n_seqs * pages + 5, generator=g)[:n_seqs * pages].to(torch.int32).view(n_seqs, pages)
    if pages > 2:
        bt[0, 1] = -1
    kv_rows = (n_seqs * pages + 2) * page_size                  # the three highest page numbers lie past the pool
    want = oracle.translate_indices(oracle.topk_indices(to_np(scores), k, to_np(lens)), to_np(bt), page_size, kv_rows=kv_rows,
                                    tokens_per_seq=rows_per_seq)
    assert (want < 0).any() and (want >= 0).any()
    need = lib.smla_topk_workspace_bytes(rows, n, k)
    for ws_bytes in ({0, need}):
        ws = torch.zeros(max(ws_bytes, 1), dtype=torch.uint8)
        out = torch.full((rows, k), -9, dtype=torch.int32)
        rc = lib.smla_topk_rows(scores.data_ptr(), lens.data_ptr(), bt.data_ptr(), out.data_ptr(), rows, n, n, k, rows_per_seq, page_size,
                                pages, kv_rows, ws.data_ptr() if ws_bytes else None, ws_bytes, None)
        assert rc == 0 and np.array_equal(to_np(out), want), ws_bytes


def test_attention_over_physical_rows_from_the_index_producer():
    from flagtree_amd import workloads
    lib = harness.lib()
    cfg = workloads.decode_bf16("cpu", batch=3, heads=128, pages_per_seq=6, topk=200, pad_frac=0.0)
    B, page_size, pages = 3, cfg["page_size"], cfg["block_table"].shape[1]
    n, k = pages * page_size, 200
    g = torch.Generator().manual_seed(3)
    scores = torch.randn((B, n), generator=g)
    lens = torch.tensor([n, n // 2, 150], dtype=torch.int32)
    kv_rows = cfg["kv_cache"].numel() // 576
    logical = torch.full((B, k), -9, dtype=torch.int32)
    rows = torch.full((B, k), -9, dtype=torch.int32)
    assert lib.smla_topk_indices(scores.data_ptr(), lens.data_ptr(), logical.data_ptr(), B, n, n, k, None, 0, None) == 0
    assert lib.smla_topk_rows(scores.data_ptr(), lens.data_ptr(), cfg["block_table"].data_ptr(), rows.data_ptr(), B, n, n, k, 1, page_size,
                              pages, kv_rows, None, 0, None) == 0
    out0, lse0, rc0 = harness.forward(dict(cfg, indices=logical.view(B, 1, k)), n_splits=2)
    out1, lse1, rc1 = harness.forward(dict(cfg, indices=rows.view(B, 1, k), block_table=None, kv_cache=cfg["kv_cache"].reshape(-1, 576)), n_splits=2)
    assert rc0 == 0 and rc1 == 0
    assert torch.equal(out0.view(torch.int16), out1.view(torch.int16)) and torch.equal(lse0, lse1)
    _check(dict(cfg, indices=logical.view(B, 1, k)), out1, lse1)


def test_topk_part_planning():
    lib = harness.lib()
    try:
        lib.emu_set_cu_count(256)
        assert lib.smla_topk_workspace_bytes(64, 65536, 2048) == 64 * 4 * 2048 * 8        # the decode shape: four parts a row
        assert lib.smla_topk_workspace_bytes(4096, 4096, 2048) == 0                       # many short rows: one workgroup a row
        assert lib.smla_topk_workspace_bytes(200, 65536, 2048) == 0                       # rows alone fill most of the device
        assert lib.smla_topk_workspace_bytes(1, 1 << 20, 2048) == 0                       # parts would not fit the registers
        assert lib.smla_topk_workspace_bytes(1, 400000, 2048) == 8 * 2048 * 8             # 8 parts of 50 176 entries
        assert lib.smla_topk_workspace_bytes(1, 33000, 2048) == 7 * 2048 * 8              # 8 parts of 5120 would leave the last one empty: 7
        assert lib.smla_topk_workspace_bytes(8, 65536, 20000) == 8 * 3 * 20000 * 8        # candidates of a row must fit too
    finally:
        lib.emu_set_cu_count(harness.EMU_CUS)


@pytest.mark.parametrize("m,n,k,chunks", [(256, 256, 128, 2), (128, 512, 192, 1), (384, 256, 64, 3), (512, 256, 128, 4),
                                          (2048, 256, 64, 8),      # 8 tiles on 16 units: every tile as two half tiles
                                          (2048, 768, 128, 2)])    # 24 tiles: 16 whole + 8 split into 16 half tiles
def test_local_gemm(m, n, k, chunks):
    g = torch.Generator().manual_seed(m + n + k)
    x = (torch.randn((m, k), generator=g) * 0.1).to(torch.bfloat16)
    w = (torch.randn((k, n), generator=g) * 0.1).to(torch.bfloat16)
    partial = torch.randn((m, n), generator=g)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16)
    for eager, skew in ((False, 0), (True, 0), (False, 1), (True, 2)):
        harness.configure(dma_eager=eager, wave_skew_seed=skew)
        rc = harness.lib().smla_gemm_rs_local(x.data_ptr(), w.data_ptr(), partial.data_ptr(), out.data_ptr(), m, n, k, chunks,
                                              (m // chunks) * n, None)
        assert rc == 0
        want = oracle.gemm_rs_local(to_np(x), to_np(w), to_np(partial), n_chunks=chunks).reshape(m, n)
        assert max_abs(to_np(out), want) <= 1e-2 + 1e-2 * float(np.abs(want).max())
    harness.configure()


@pytest.mark.parametrize("m,n,k,chunks", [(2048, 1280, 128, 2),     # 40 tiles on 16 units: two whole tiles chained per workgroup, then a half tile
                                          (2048, 1280, 192, 8),     # three K-steps: the buffers swap roles from tile to tile
                                          (2048, 1024, 64, 1),      # one K-step a tile, 32 tiles: two chained whole tiles, no halves
                                          (2048, 2048, 64, 4),      # 64 tiles: four chained whole tiles per workgroup
                                          (2048, 768, 128, 2)])     # 24 tiles: one whole tile and one half tile per workgroup
def test_local_gemm_by_persistent_workgroups(m, n, k, chunks, monkeypatch):
    """FLAGTREE_SMLA_GEMM_CHAIN=1: one workgroup per compute unit walks its tiles; the next tile's
    first K-step is sent for during the current tile's last one and lands under the epilogue, which
    stages through the other buffer.  Same bits as one workgroup per tile (every output element is
    the same sum in the same order), under in-step, skewed and eager-move schedules."""
    g = torch.Generator().manual_seed(m + n + k)
    x = (torch.randn((m, k), generator=g) * 0.1).to(torch.bfloat16)
    w = (torch.randn((k, n), generator=g) * 0.1).to(torch.bfloat16)
    partial = torch.randn((m, n), generator=g)
    lib = harness.lib()
    ref = torch.full((m, n), float("nan"), dtype=torch.bfloat16)
    assert lib.smla_gemm_rs_local(x.data_ptr(), w.data_ptr(), partial.data_ptr(), ref.data_ptr(), m, n, k, chunks, (m // chunks) * n, None) == 0
    monkeypatch.setenv("FLAGTREE_SMLA_GEMM_CHAIN", "1")
    for eager, skew, together in ((False, 0, 0), (True, 0, 0), (False, 1, 0), (True, 2, 3)):
        harness.configure(dma_eager=eager, wave_skew_seed=skew, concurrent_blocks=together, concurrent_seed=4)
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16)
        launches, before = lib.emu_launch_count(), harness.work_counts()
        rc = lib.smla_gemm_rs_local(x.data_ptr(), w.data_ptr(), partial.data_ptr(), out.data_ptr(), m, n, k, chunks, (m // chunks) * n, None)
        assert rc == 0 and harness.work_counts()["mfma_flops"] == 2.0 * m * n * k
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), (eager, skew)
    harness.configure()
    want = oracle.gemm_rs_local(to_np(x), to_np(w), to_np(partial), n_chunks=chunks).reshape(m, n)
    assert max_abs(to_np(out), want) <= 1e-2 + 1e-2 * float(np.abs(want).max())


def test_local_gemm_on_a_compute_unit_count_that_is_no_multiple_of_eight():
    """24 tiles on 20 compute units leave a rest of 4 tiles, few enough to be halved; but the half-tile
    mapping needs the whole tiles to come in groups of 8, which 20 does not give: all tiles stay
    whole, every one is computed once."""
    m, n, k = 2048, 768, 128
    g = torch.Generator().manual_seed(99)
    x = (torch.randn((m, k), generator=g) * 0.1).to(torch.bfloat16)
    w = (torch.randn((k, n), generator=g) * 0.1).to(torch.bfloat16)
    partial = torch.randn((m, n), generator=g)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16)
    lib = harness.lib()
    try:
        lib.emu_set_cu_count(20)
        harness.work_counts()
        rc = lib.smla_gemm_rs_local(x.data_ptr(), w.data_ptr(), partial.data_ptr(), out.data_ptr(), m, n, k, 2, (m // 2) * n, None)
        flops = harness.work_counts()["mfma_flops"]
    finally:
        lib.emu_set_cu_count(harness.EMU_CUS)
    assert rc == 0 and flops == 2.0 * m * n * k               # nothing twice, nothing left out
    want = oracle.gemm_rs_local(to_np(x), to_np(w), to_np(partial), n_chunks=2).reshape(m, n)
    assert max_abs(to_np(out), want) <= 1e-2 + 1e-2 * float(np.abs(want).max())


# ---- memory safety: every buffer between inaccessible pages ------------------------------------

def test_no_entry_point_touches_memory_outside_its_buffers():
    """tests/emu/guarded_cases.py runs every entry point with each input, output and workspace
    ending right before (then starting right after) an inaccessible page; an emulated kernel that
    reads or writes outside a buffer ends that process with SIGSEGV."""
    import subprocess
    script = os.path.join(os.path.dirname(os.path.abspath(__file__)), "emu", "guarded_cases.py")
    r = subprocess.run([sys.executable, script], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), (r.returncode, r.stdout[-1500:], r.stderr[-1500:])


def test_guard_pages_do_catch_a_stray_access():
    """Negative control for the test above: the same set-up with a lie about a buffer's size dies."""
    import subprocess
    code = (
        "import sys, torch\n"
        f"sys.path[:0] = [{os.path.dirname(os.path.dirname(os.path.abspath(__file__)))!r}, "
        f"{os.path.dirname(os.path.abspath(__file__))!r}, {os.path.join(os.path.dirname(os.path.abspath(__file__)), 'emu')!r}]\n"
        "import harness\n"
        "kv = harness.Guarded(torch.zeros((8, 576), dtype=torch.int16), True).tensor\n"
        "idx = torch.tensor([[7, 8]], dtype=torch.int32)\n"
        "phys = torch.zeros((1, 2), dtype=torch.int32); rows = torch.zeros((1, 2, 576), dtype=torch.int16)\n"
        "harness.lib().smla_gather_rows(kv.data_ptr(), 1152, idx.data_ptr(), None, phys.data_ptr(), rows.data_ptr(), "
        "1, 1, 2, 64, 0, 0, 16, None)\n"
        "print('survived')\n")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=600)
    assert r.returncode == -11 and "survived" not in r.stdout, (r.returncode, r.stdout, r.stderr[-500:])


# ---- LDS bank accounting ----------------------------------------------------------------------

def _bank_ratio(stats):
    """passes taken / passes a conflict-free access takes, per kind of access that occurred"""
    return {k: v[1] / v[2] for k, v in stats.items() if v[0]}


@pytest.mark.parametrize("mode", ["first", "wavefront_per_head_group", "first_fp8", "wavefront_per_head_group_fp8"])
def test_many_heads_kernels_address_lds_without_bank_conflicts(mode, monkeypatch):
    """The emulator prices every LDS access the kernels make by address (fragment reads, transposing
    reads, probability writes) the way the hardware serves it: 16-byte accesses 16 lanes at a time,
    8-byte ones 32 at a time, 64 banks.  The swizzled tile layouts exist to make these free of
    conflicts; this is the check that they are, on the code as compiled."""
    from flagtree_amd import workloads
    if mode.endswith("_fp8"):
        cfg, _ = _fp8_cfg(1, 128, 8, 300, pad_frac=0.05)
    else:
        cfg = workloads.decode_bf16("cpu", batch=1, heads=128, pages_per_seq=8, topk=300, pad_frac=0.05)
    if mode != "first" and mode != "first_fp8":
        monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1")
    harness.lds_profile_start()
    try:
        out, lse, rc = harness.forward(cfg, n_splits=2)
    finally:
        stats = harness.lds_profile_stop()
    assert rc == 0
    _check(cfg, out, lse)
    assert stats["read"][0] > 1000 and stats["read_tr"][0] > 1000, stats
    assert all(r == 1.0 for r in _bank_ratio(stats).values()), stats


def test_few_heads_kernels_transposing_reads_take_two_passes(monkeypatch):
    """Known and accepted: the few-heads kernels keep rows at a padded stride (1168 bytes), which
    frees the score reads of conflicts but leaves the P.V transposing reads two-way conflicted (a
    stride cannot serve both; the many-heads kernels swizzle instead).  Those reads are a few
    percent of an instruction-bound loop.  The figure is pinned so that a layout change shows up."""
    from flagtree_amd import workloads
    for env, cfg in ((None, workloads.decode_bf16("cpu", batch=1, heads=16, pages_per_seq=8, topk=300, pad_frac=0.05)),
                     (None, _fp8_cfg(1, 16, 8, 300, pad_frac=0.05)[0]),
                     ("FLAGTREE_SMLA_FEW_FP8", _fp8_cfg(1, 16, 8, 300, pad_frac=0.05)[0])):
        if env:
            monkeypatch.setenv(env, "1")
        harness.lds_profile_start()
        try:
            out, lse, rc = harness.forward(cfg, n_splits=2)
        finally:
            stats = harness.lds_profile_stop()
        assert rc == 0 and stats["read_tr"][0] > 100
        assert _bank_ratio(stats)["read_tr"] == 2.0, stats


def test_fp8_mfma_kernel_addresses_lds_without_bank_conflicts(monkeypatch):
    """Records lie in LDS back to back, 656 bytes apart (36 words modulo 64).  The 16-byte score
    reads of 16 consecutive records fall on 16 different bank groups by themselves; the 8-byte
    transposing reads of the V operand take every second record of 16 (the tokens' order inside
    the operands is 0 2 4 6 1 3 5 7 for that reason) and are free of conflicts as well."""
    monkeypatch.setenv("FLAGTREE_SMLA_FP8_MFMA", "1")
    cfg = _fp8_cfg(1, 16, 8, 300, pad_frac=0.05)[0]
    harness.lds_profile_start()
    try:
        out, lse, rc = harness.forward(cfg, n_splits=2)
    finally:
        stats = harness.lds_profile_stop()
    assert rc == 0
    _check(cfg, out, lse)
    assert stats["read"][0] > 500 and stats["read_tr"][0] > 300, stats
    ratio = _bank_ratio(stats)
    assert ratio["read_tr"] == 1.0 and ratio["write"] == 1.0, stats
    # Known and accepted: the eight 4-byte reads of a token's block scale per tile and wavefront
    # (four addresses a wavefront, 16 lanes on each) put token groups 0 and 2, and 1 and 3, on the same
    # bank, two passes instead of one; every 16-byte read is one pass.  Pinned so a change shows.
    assert ratio["read"] == 1.2, stats


def test_gemm_kernels_address_lds_without_bank_conflicts():
    lib = harness.lib()
    for (m, n, k) in ((512, 512, 128), (384, 256, 128)):          # the 256 x 256 kernel, the 128 x 256 kernel
        g = torch.Generator().manual_seed(m)
        x = (torch.randn((m, k), generator=g) * 0.1).to(torch.bfloat16)
        w = (torch.randn((k, n), generator=g) * 0.1).to(torch.bfloat16)
        part = torch.randn((m, n), generator=g)
        out = torch.empty((m, n), dtype=torch.bfloat16)
        harness.lds_profile_start()
        try:
            rc = lib.smla_gemm_rs_local(x.data_ptr(), w.data_ptr(), part.data_ptr(), out.data_ptr(), m, n, k, 1, m * n, None)
        finally:
            stats = harness.lds_profile_stop()
        assert rc == 0
        want = oracle.gemm_rs_local(to_np(x), to_np(w), to_np(part), 1)
        assert max_abs(to_np(out).reshape(want.shape), want) <= 1e-2
        assert stats["read_tr"][0] > 500 and all(r == 1.0 for r in _bank_ratio(stats).values()), stats


def test_work_per_unit_of_the_two_many_heads_kernels(monkeypatch):
    """What each design does per 16 tokens x 128 heads, counted on the code as it runs: the same
    matrix work, and the LDS and global -> LDS traffic the designs were made to differ in."""
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16("cpu", batch=1, heads=128, pages_per_seq=40, topk=1024, pad_frac=0.0)
    units = 1024 * 128 / (16 * 128)
    got = {}
    for name, mode in (("first", None), ("wavefront_per_head_group", "1")):
        if mode:
            monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", mode)
        harness.work_counts()
        out, lse, rc = harness.forward(cfg, n_splits=1)
        assert rc == 0
        got[name] = {k: v / units for k, v in harness.work_counts().items()}
    for w in got.values():
        assert abs(w["mfma_flops"] - 2 * 16 * 128 * (576 + 512)) < 1.0          # 4.456 MFLOP, nothing computed twice
    kb = lambda name, key: round(got[name][key] / 1024, 1)       # (the page-table row's move adds a few bytes per unit)
    assert kb("first", "dma_bytes") == 36.0 and kb("wavefront_per_head_group", "dma_bytes") == 18.0
    assert kb("first", "lds_read_bytes") == 144.0
    assert kb("wavefront_per_head_group", "lds_read_bytes") == 136.0 and got["wavefront_per_head_group"]["lds_write_bytes"] == 0.0
    assert got["wavefront_per_head_group"]["barriers_x_waves"] < got["first"]["barriers_x_waves"]

