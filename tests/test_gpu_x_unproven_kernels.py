"""GPU parity of the kernel paths that have not been timed or run on hardware yet: the many-heads
kernel over an fp8 cache (raw records by global -> LDS moves, converted LDS -> LDS) and the two
opt-in second designs (FLAGTREE_SMLA_FEW_FP8, FLAGTREE_SMLA_HEAD_GROUPS) and the opt-in token order
(FLAGTREE_SMLA_TOKEN_BANDS).  The file sorts after the other
GPU test files on purpose: under `pytest -x` a failure here cannot hide the results of the paths
the defaults rest on.  Same bars: out max-abs <= 1e-2, lse <= 1e-3 against the float64 oracle."""
import numpy as np
import pytest
import torch

import oracle
from _util import check_random_shape, max_abs, oracle_inputs, random_shape_draw, run_oracle, to_np
from test_gpu_sparse_mla import LSE_TOL, OUT_TOL, _check, _fwd, check_logit_cap

pytestmark = pytest.mark.gpu


# ---- many heads over an fp8 cache --------------------------------------------------------------

@pytest.mark.parametrize("heads,n_splits", [(128, 2), (128, 1), (64, 3), (40, 1)])
def test_decode_fp8_many_heads_reduced(dev, heads, n_splits):
    from flagtree_amd import workloads
    cfg = workloads.decode_fp8(dev, batch=3, heads=heads, pages_per_seq=32, topk=512, pad_frac=0.03)
    out, lse = _fwd(cfg, n_splits=n_splits)
    _check(cfg, out, lse)


@pytest.mark.parametrize("topk,n_splits", [(1, 1), (31, 1), (32, 1), (33, 1), (64, 2), (65, 1), (96, 1), (97, 1), (128, 1),
                                           (129, 2), (200, 3), (1030, 1), (2100, 2)])
def test_fp8_many_heads_pipeline_at_every_tile_count(dev, topk, n_splits):
    """Prologue (two tiles), steady state (from the fourth tile on) and tail (last three) of the
    raw-record pipeline: lists of 1..5 tiles, ragged and full, more than one chunk, splits."""
    from flagtree_amd import workloads
    cfg = workloads.decode_fp8(dev, batch=2, heads=40, pages_per_seq=40, topk=topk, pad_frac=0.0 if topk < 40 else 0.04)
    out, lse = _fwd(cfg, n_splits=n_splits)
    _check(cfg, out, lse)


@pytest.mark.parametrize("seed", [1, 4, 7, 12, 18, 27, 34, 36, 38, 44, 52, 69, 72])
def test_random_shapes_many_heads_fp8(dev, seed):
    draw = random_shape_draw(4000 + seed)
    assert draw["kv_format"] != "bf16" and draw["heads"] > 32
    check_random_shape(draw, dev, _fwd, _check)


@pytest.mark.parametrize("splits", [1, 2])
def test_logit_cap_many_heads_fp8(dev, splits):
    """(The kernel rounds dequantised fp8 values to bf16, an error that grows with the square of the
    input scale: this case stays near the benchmark's magnitudes.)"""
    check_logit_cap(dev, 64, "fp8_e4m3_b128", 0.5, 0.2, 0.01, splits)


@pytest.mark.parametrize("topk,n_splits,heads", [(1, 1, 40), (33, 1, 128), (64, 2, 65), (97, 1, 128), (129, 2, 128), (200, 3, 128),
                                                 (1030, 1, 40), (2100, 2, 128), (2048, None, 128)])
def test_head_group_kernel_fp8_pipeline(dev, monkeypatch, topk, n_splits, heads):
    """The raw-record pipeline inside the wavefront-per-head-group kernel (FLAGTREE_SMLA_HEAD_GROUPS=1)."""
    from flagtree_amd import workloads
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1")
    cfg = workloads.decode_fp8(dev, batch=3, heads=heads, pages_per_seq=40, topk=topk, pad_frac=0.0 if topk < 40 else 0.04)
    out, lse = _fwd(cfg, n_splits=n_splits)
    _check(cfg, out, lse)


def test_fp8_many_heads_against_scalar_kernel_at_size(dev):
    """Batch 16 x 128 heads x 2048 records (64 tiles a list, two chunks): against the exact scalar
    kernel on two sequences and against the oracle on one."""
    import flagtree_amd as ft
    from flagtree_amd import workloads
    cfg = workloads.decode_fp8(dev, batch=16, heads=128, pages_per_seq=64, topk=2048, pad_frac=0.05)
    out, lse = _fwd(cfg)
    sub = dict(cfg, q=cfg["q"][:2], indices=cfg["indices"][:2], block_table=cfg["block_table"][:2])
    so, sl = ft.sparse_mla_fwd_scalar(sub["q"], sub["kv_cache"], sub["indices"], sub["sm_scale"], 512,
                                      block_table=sub["block_table"], page_size=64, kv_format="fp8_e4m3_b128")
    assert max_abs(to_np(out[:2]), to_np(so)) <= OUT_TOL and max_abs(to_np(lse[:2]), to_np(sl)) <= LSE_TOL
    _check(dict(sub, q=sub["q"][:1], indices=sub["indices"][:1], block_table=sub["block_table"][:1]), out[:1], lse[:1])


# ---- the two-workgroups-per-CU fp8 kernel (opt-in until it has been measured) -------------------

FEW_HEADS_FP8_SWITCHES = {"column_split": "FLAGTREE_SMLA_FEW_FP8", "fp8_mfma": "FLAGTREE_SMLA_FP8_MFMA"}


@pytest.fixture(params=["column_split", "fp8_mfma"])
def few_fp8_kernel(request, monkeypatch):
    """One of the two opt-in few-heads fp8 kernels: the column-split one that converts records to
    bf16, or the one that contracts the records' e4m3 codes on the matrix cores."""
    monkeypatch.setenv(FEW_HEADS_FP8_SWITCHES[request.param], "1")


@pytest.mark.parametrize("heads,n_splits,topk", [(16, 1, 512), (16, 2, 512), (8, 3, 300), (30, 2, 700), (16, None, 2048)])
def test_column_split_fp8_kernel_against_oracle(dev, few_fp8_kernel, heads, n_splits, topk):
    from flagtree_amd import workloads
    cfg = workloads.decode_fp8(dev, batch=5, heads=heads, pages_per_seq=40, topk=topk, pad_frac=0.03)
    out, lse = _fwd(cfg, n_splits=n_splits)
    _check(cfg, out, lse)


@pytest.mark.parametrize("kernel", ["column_split", "fp8_mfma"])
def test_column_split_fp8_kernel_against_the_first_kernel_at_full_size(dev, monkeypatch, kernel):
    """Full fp8 decode size: the two kernels agree to the bar (they sum in different orders), and a
    slice of the batch agrees with the oracle."""
    from flagtree_amd import workloads
    cfg = workloads.decode_fp8(dev)
    out0, lse0 = _fwd(cfg)
    monkeypatch.setenv(FEW_HEADS_FP8_SWITCHES[kernel], "1")
    out1, lse1 = _fwd(cfg)
    torch.cuda.synchronize()
    assert not torch.equal(out0, out1)                       # it really is the other kernel
    assert max_abs(to_np(out1), to_np(out0)) <= 2e-3 and max_abs(to_np(lse1), to_np(lse0)) <= 1e-4
    sub = dict(cfg, q=cfg["q"][:4], indices=cfg["indices"][:4], block_table=cfg["block_table"][:4])
    ro, rl = run_oracle(sub)
    assert max_abs(to_np(out1[:4]).reshape(4, 16, 512), ro) <= OUT_TOL and max_abs(to_np(lse1[:4]).reshape(4, 16), rl) <= LSE_TOL


def test_column_split_fp8_kernel_edge_cases_and_dense(dev, few_fp8_kernel):
    import flagtree_amd as ft
    g = torch.Generator().manual_seed(7)
    latent = (torch.randn((300, 576), generator=g) * 0.1).to(torch.bfloat16).to(dev)
    rec = ft.quantize_kv_fp8(latent)
    q = (torch.randn((6, 16, 576), generator=g) * 0.1).to(torch.bfloat16).to(dev)
    idx = torch.full((6, 70), -1, dtype=torch.int32)
    idx[1, 33] = 5
    idx[2, :] = torch.randperm(300, generator=g)[:70].to(torch.int32)
    idx[3, :35] = 17
    idx[4, ::2] = torch.arange(35, dtype=torch.int32)
    idx[5, 0] = 299
    idx[5, 1] = 300
    cfg = dict(q=q, kv_cache=rec, indices=idx.to(dev), block_table=None, page_size=64, sm_scale=576 ** -0.5,
               kv_format="fp8_e4m3_b128")
    for ns in (1, 2):
        out, lse = _fwd(cfg, n_splits=ns)
        _check(cfg, out, lse)
        assert (to_np(out)[0] == 0).all() and np.isneginf(to_np(lse)[0]).all()
    # dense decode with a logit cap through the same kernel
    B, L, page_size, cap = 3, 700, 64, 0.02
    lens = torch.tensor([L, 3, 300], dtype=torch.int32)
    n_pages = -(-L // page_size)
    req = torch.randperm(2 * B * n_pages, generator=g)[:B * n_pages].to(torch.int32).view(B, n_pages)
    lat = (torch.randn((2 * B * n_pages * page_size, 576), generator=g) * 0.1).to(torch.bfloat16)
    k_buffer = ft.quantize_kv_fp8(lat.to(dev)).view(-1, page_size, 656)
    qd = (torch.randn((B, 16, 576), generator=g) * 0.1).to(torch.bfloat16)
    o, lse = ft.decode_attention_fwd(qd.to(dev), k_buffer, None, None, req.to(dev), lens.to(dev), None, 2, 576 ** -0.5,
                                     page_size, logit_cap=cap)
    max_len = n_pages * page_size
    idxd = torch.arange(max_len, dtype=torch.int32).repeat(B, 1)
    idxd[idxd >= lens[:, None]] = -1
    cfgd = {"q": qd.view(B, 1, 16, 576), "indices": idxd.view(B, 1, max_len), "kv_cache": k_buffer, "block_table": req,
            "page_size": page_size, "kv_format": "fp8_e4m3_b128", "sm_scale": 576 ** -0.5}
    qn, kv_small, phys_small, _ = oracle_inputs(cfgd)
    wo, wl = oracle.sparse_mla_fwd(qn, kv_small, phys_small, cfgd["sm_scale"], 512, logit_cap=cap)
    assert max_abs(to_np(lse), wl.reshape(B, 16)) <= 1e-3 and max_abs(to_np(o), wo.reshape(B, 16, 512)) <= 1e-2


# ---- the 128-heads-per-workgroup bf16 kernel (opt-in until it has been measured) ----------------

@pytest.fixture
def wide_kernel(monkeypatch):
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1")


@pytest.mark.parametrize("heads,n_splits,topk", [(128, 1, 512), (128, 2, 512), (64, 3, 300), (200, 2, 700), (128, None, 2048),
                                                 (65, 3, 200)])
def test_128_heads_kernel_against_oracle(dev, wide_kernel, heads, n_splits, topk):
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16(dev, batch=5, heads=heads, pages_per_seq=40, topk=topk, pad_frac=0.03)
    out, lse = _fwd(cfg, n_splits=n_splits)
    _check(cfg, out, lse)


def test_128_heads_kernel_against_the_first_kernel_at_full_size(dev, monkeypatch):
    """Headline decode size: the two kernels agree to the bar (they sum in different orders), and a
    slice of the batch agrees with the oracle."""
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16(dev)
    out0, lse0 = _fwd(cfg)
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1")
    out1, lse1 = _fwd(cfg)
    torch.cuda.synchronize()
    assert not torch.equal(out0, out1)                       # it really is the other kernel
    assert max_abs(to_np(out1), to_np(out0)) <= 2e-3 and max_abs(to_np(lse1), to_np(lse0)) <= 1e-4
    sub = dict(cfg, q=cfg["q"][:2], indices=cfg["indices"][:2], block_table=cfg["block_table"][:2])
    ro, rl = run_oracle(sub)
    H = cfg["q"].shape[-2]
    assert max_abs(to_np(out1[:2]).reshape(2, H, 512), ro) <= OUT_TOL and max_abs(to_np(lse1[:2]).reshape(2, H), rl) <= LSE_TOL


def test_128_heads_kernel_prefill_and_redo(dev, wide_kernel):
    from flagtree_amd import workloads
    cfg = workloads.prefill_causal_bf16(dev, tokens=300, heads=128, topk=256)
    out, lse = _fwd(cfg)
    rows = slice(130, 170)                                   # lists of 131..170 entries: more than one chunk of 128
    sub = dict(cfg, q=cfg["q"][:, rows], indices=cfg["indices"][:, rows])
    ro, rl = run_oracle(sub)
    assert max_abs(to_np(out[:, rows]).reshape(ro.shape), ro) <= OUT_TOL
    assert max_abs(to_np(lse[:, rows]).reshape(rl.shape), rl) <= LSE_TOL
    g = torch.Generator().manual_seed(3)
    kv = (torch.randn((400, 576), generator=g) * 4.0).to(torch.bfloat16)
    kv[:64] *= 0.01
    q = (torch.randn((2, 128, 576), generator=g) * 4.0).to(torch.bfloat16)
    cfg = dict(q=q.to(dev), kv_cache=kv.to(dev), indices=torch.arange(200, dtype=torch.int32).repeat(2, 1).to(dev),
               block_table=None, page_size=64, sm_scale=576 ** -0.5, kv_format="bf16")
    ro, rl = run_oracle(cfg)
    for ns in (1, 2):
        out, lse = _fwd(cfg, n_splits=ns)
        assert max_abs(to_np(lse).reshape(rl.shape), rl) <= 1e-3 * max(1.0, float(np.abs(rl).max()))
        assert max_abs(to_np(out).reshape(ro.shape), ro) <= 1.2e-2 * max(1.0, float(np.abs(ro).max()))


# ---- contiguous token bands per XCD (opt-in) ---------------------------------------------------

@pytest.mark.parametrize("heads,n_splits,tokens", [(128, 1, 320), (128, 2, 43), (16, 1, 171), (16, 3, 43)])
def test_token_bands_give_the_same_bits(dev, monkeypatch, heads, n_splits, tokens):
    """FLAGTREE_SMLA_TOKEN_BANDS=1 only changes which workgroup takes which token (an XCD gets a
    contiguous band instead of every eighth token): out and lse must not change by a bit."""
    from flagtree_amd import workloads
    cfg = workloads.prefill_causal_bf16(dev, tokens=tokens, heads=heads, topk=300 if n_splits > 1 else 128)
    out0, lse0 = _fwd(cfg, n_splits=n_splits)
    monkeypatch.setenv("FLAGTREE_SMLA_TOKEN_BANDS", "1")
    out1, lse1 = _fwd(cfg, n_splits=n_splits)
    assert torch.equal(out0.view(torch.int16), out1.view(torch.int16)) and torch.equal(lse0, lse1)
    _check(cfg, out1, lse1)


# ---- persistent workgroups for unsplit many-heads launches (opt-in) ------------------------------

@pytest.mark.parametrize("kernel", ["many_heads", "wavefront_per_head_group"])
@pytest.mark.parametrize("case", ["prefill", "dense"])
def test_persistent_workgroups_give_the_same_bits(dev, monkeypatch, case, kernel):
    """FLAGTREE_SMLA_PERSIST=1: one workgroup per compute unit walks its (token, head block) items and
    sends for the next item's indices and Q under the current item's output stores.  Same code on
    the same data per item: the same bits as one workgroup per item."""
    import flagtree_amd as ft
    from flagtree_amd import workloads
    monkeypatch.delenv("FLAGTREE_SMLA_PERSIST", raising=False)
    monkeypatch.setenv("FLAGTREE_SMLA_HEAD_GROUPS", "1" if kernel == "wavefront_per_head_group" else "0")
    if case == "prefill":
        cfg = workloads.prefill_causal_bf16(dev, tokens=700, heads=128, topk=256)          # 1408 (or 704) items on 256 compute units
        out0, lse0 = _fwd(cfg, n_splits=1)
        monkeypatch.setenv("FLAGTREE_SMLA_PERSIST", "1")
        out1, lse1 = _fwd(cfg, n_splits=1)
        torch.cuda.synchronize()
        rows = slice(300, 340)
        sub = dict(cfg, q=cfg["q"][:, rows], indices=cfg["indices"][:, rows])
        ro, rl = run_oracle(sub)
        assert max_abs(to_np(out1[:, rows]).reshape(ro.shape), ro) <= OUT_TOL and max_abs(to_np(lse1[:, rows]).reshape(rl.shape), rl) <= LSE_TOL
    else:
        B, L, page_size = 600, 400, 64
        g = torch.Generator().manual_seed(21)
        n_pages = -(-L // page_size)
        req = torch.randperm(B * n_pages, generator=g).to(torch.int32).view(B, n_pages).to(dev)
        lens = torch.randint(1, L + 1, (B,), generator=g, dtype=torch.int32).to(dev)
        k_buffer = (torch.randn((B * n_pages * page_size, 576), generator=g) * 0.1).to(torch.bfloat16).to(dev).view(-1, page_size, 576)
        q = (torch.randn((B, 128, 576), generator=g) * 0.1).to(torch.bfloat16).to(dev)
        out0, lse0 = ft.decode_attention_fwd(q, k_buffer, None, None, req, lens, None, 1, 576 ** -0.5, page_size)
        monkeypatch.setenv("FLAGTREE_SMLA_PERSIST", "1")
        out1, lse1 = ft.decode_attention_fwd(q, k_buffer, None, None, req, lens, None, 1, 576 ** -0.5, page_size)
        torch.cuda.synchronize()
    assert torch.equal(out0, out1) and torch.equal(lse0, lse1)
