"""Runs every entry point on the emulator with all of its buffers between inaccessible pages
(tests only; run as a script so that a stray access, which ends the process, fails one test and
not the test session).  ``python tests/emu/guarded_cases.py [case ...]``; no case = all."""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "tests"), HERE):
    if p not in sys.path:
        sys.path.insert(0, p)

import torch  # noqa: E402

import harness  # noqa: E402
from flagtree_amd import workloads  # noqa: E402


def _guard_cfg(cfg, end):
    keep = []
    out = dict(cfg)
    for k in ("q", "kv_cache", "indices", "block_table"):
        if cfg.get(k) is not None:
            g = harness.Guarded(cfg[k], end)
            keep.append(g)
            out[k] = g.tensor
    return out, keep


def forward_case(make, n_splits, dense=False, env=None):
    def run(end):
        for k in ("FLAGTREE_SMLA_FEW_FP8", "FLAGTREE_SMLA_HEAD_GROUPS", "FLAGTREE_SMLA_FP8_MFMA", "FLAGTREE_SMLA_PERSIST"):
            os.environ.pop(k, None)
        os.environ.update(env or {})
        cfg = make()
        gcfg, keep = _guard_cfg(cfg, end)
        T = cfg["q"].numel() // (cfg["q"].shape[-2] * 576)
        H = cfg["q"].shape[-2]
        ws = None
        n = harness.lib().smla_workspace_bytes(T, H, 512, n_splits)
        if n:
            gws = harness.Guarded(harness.make_workspace(n), end)
            keep.append(gws)
            ws = gws.tensor
        lens = None
        if dense:
            glens = harness.Guarded(torch.tensor([70, 1, 129][:T], dtype=torch.int32), end)
            keep.append(glens)
            lens = glens.tensor
        # outputs are allocated inside harness.forward; guard them too by running through the raw ABI
        out, lse, rc = harness.forward(gcfg, n_splits=n_splits, workspace=ws, dense_lens=lens, guard_outputs=end)
        assert rc == 0, rc
        assert not torch.isnan(lse).any()
        for g in keep:
            g.close()
    return run


def fp8_cfg(batch, heads, pages, topk):
    g = torch.Generator().manual_seed(9)
    rows = batch * pages * 64
    latent = (torch.randn((rows, 576), generator=g) * 0.1).to(torch.bfloat16)
    rec = torch.zeros((rows, 656), dtype=torch.uint8)
    assert harness.lib().smla_kv_quantize_fp8(latent.data_ptr(), None, rec.data_ptr(), rows, rows, None) == 0
    bt = torch.randperm(batch * pages, generator=g).to(torch.int32).view(batch, pages)
    q = (torch.randn((batch, 1, heads, 576), generator=g) * 0.1).to(torch.bfloat16)
    idx = workloads._topk_indices(batch, pages * 64, topk, 3, g, True)
    return dict(q=q, kv_cache=rec.view(-1, 64, 656), indices=idx.view(batch, 1, topk), block_table=bt, page_size=64,
                sm_scale=workloads.SM_SCALE, kv_format="fp8_e4m3_b128")


def raw_case(fn):
    def run(end):
        keep = []

        def G(t):
            g = harness.Guarded(t, end)
            keep.append(g)
            return g.tensor
        fn(G)
        for g in keep:
            g.close()
    return run


def _gather(G):
    cfg = workloads.decode_bf16("cpu", batch=3, heads=16, pages_per_seq=4, topk=70, pad_frac=0.1)
    kv = G(cfg["kv_cache"].view(torch.int16).reshape(-1, 576))
    idx, bt = G(cfg["indices"].view(3, 70)), G(cfg["block_table"])
    phys, rows = G(torch.zeros((3, 70), dtype=torch.int32)), G(torch.zeros((3, 70, 576), dtype=torch.int16))
    assert harness.lib().smla_gather_rows(kv.data_ptr(), 1152, idx.data_ptr(), bt.data_ptr(), phys.data_ptr(), rows.data_ptr(),
                                          3, 1, 70, 64, 4, 0, kv.shape[0], None) == 0


def _kv_write(G):
    g = torch.Generator().manual_seed(4)
    latent = G((torch.randn((37, 576), generator=g) * 0.3).to(torch.bfloat16))
    slots = G(torch.randperm(60, generator=g)[:37].to(torch.int64) - 5)
    for code, width, dtype in ((1, 656, torch.uint8), (0, 576, torch.bfloat16)):
        cache = G(torch.zeros((50, width), dtype=dtype))
        assert harness.lib().smla_kv_write(code, latent.data_ptr(), slots.data_ptr(), cache.data_ptr(), 37, 50, None) == 0


def _topk(G):
    g = torch.Generator().manual_seed(5)
    for rows, n, k in ((2, 4099, 300), (1, 20000, 64), (2, 70001, 128), (3, 33, 40)):
        scores = G(torch.randn((rows, n), generator=g))
        lens = G(torch.randint(1, n + 1, (rows,), generator=g, dtype=torch.int32))
        out = G(torch.zeros((rows, k), dtype=torch.int32))
        assert harness.lib().smla_topk_indices(scores.data_ptr(), lens.data_ptr(), out.data_ptr(), rows, n, n, k, None, 0, None) == 0
        need = harness.lib().smla_topk_workspace_bytes(rows, n, k)      # rows cut into parts: the candidate lists in a guarded workspace
        if need:
            ws = G(torch.zeros(need, dtype=torch.uint8))
            out2 = G(torch.zeros((rows, k), dtype=torch.int32))
            assert harness.lib().smla_topk_indices(scores.data_ptr(), lens.data_ptr(), out2.data_ptr(), rows, n, n, k, ws.data_ptr(), need, None) == 0
            assert torch.equal(out, out2)
        pages = -(-n // 64)
        bt = G(torch.randperm(rows * pages, generator=g).to(torch.int32).view(rows, pages))
        out3 = G(torch.zeros((rows, k), dtype=torch.int32))             # the same as physical rows through a guarded page table
        assert harness.lib().smla_topk_rows(scores.data_ptr(), lens.data_ptr(), bt.data_ptr(), out3.data_ptr(), rows, n, n, k, 1, 64, pages,
                                            rows * pages * 64 - 7, None, 0, None) == 0


def _gemm(G):
    g = torch.Generator().manual_seed(6)
    for m, n, k, chunks in ((256, 256, 128, 2), (128, 256, 64, 1), (512, 512, 64, 2)):
        x = G((torch.randn((m, k), generator=g) * 0.1).to(torch.bfloat16))
        w = G((torch.randn((k, n), generator=g) * 0.1).to(torch.bfloat16))
        partial = G(torch.randn((m, n), generator=g))
        out = G(torch.zeros((m, n), dtype=torch.bfloat16))
        assert harness.lib().smla_gemm_rs_local(x.data_ptr(), w.data_ptr(), partial.data_ptr(), out.data_ptr(), m, n, k, chunks,
                                                (m // chunks) * n, None) == 0
    # persistent workgroups chaining two whole tiles each, then a half tile (40 tiles on 16 compute units)
    os.environ["FLAGTREE_SMLA_GEMM_CHAIN"] = "1"
    try:
        m, n, k, chunks = 2048, 1280, 192, 4
        x = G((torch.randn((m, k), generator=g) * 0.1).to(torch.bfloat16))
        w = G((torch.randn((k, n), generator=g) * 0.1).to(torch.bfloat16))
        partial = G(torch.randn((m, n), generator=g))
        out = G(torch.zeros((m, n), dtype=torch.bfloat16))
        assert harness.lib().smla_gemm_rs_local(x.data_ptr(), w.data_ptr(), partial.data_ptr(), out.data_ptr(), m, n, k, chunks,
                                                (m // chunks) * n, None) == 0
    finally:
        os.environ.pop("FLAGTREE_SMLA_GEMM_CHAIN")


def _merge(G):
    g = torch.Generator().manual_seed(8)
    po, pl = G(torch.randn((2, 3, 5, 512), generator=g)), G(torch.randn((2, 3, 5), generator=g))
    out, lse = G(torch.zeros((2, 5, 512), dtype=torch.bfloat16)), G(torch.zeros((2, 5)))
    assert harness.lib().smla_merge_splits(po.data_ptr(), pl.data_ptr(), out.data_ptr(), lse.data_ptr(), 2, 5, 512, 3, None) == 0


CASES = {
    "tall_bf16": forward_case(lambda: workloads.decode_bf16("cpu", batch=2, heads=128, pages_per_seq=5, topk=200, pad_frac=0.06), 1),
    "tall_bf16_split": forward_case(lambda: workloads.decode_bf16("cpu", batch=2, heads=72, pages_per_seq=5, topk=200, pad_frac=0.06), 2),
    # 65 heads: the second head group of the second block lies wholly past the last head
    "tall_bf16_empty_head_group_split": forward_case(lambda: workloads.decode_bf16("cpu", batch=3, heads=65, pages_per_seq=5, topk=200, pad_frac=0.06), 3),
    "tall_fp8_split": forward_case(lambda: fp8_cfg(2, 128, 4, 150), 2),
    "group_fp8_split": forward_case(lambda: fp8_cfg(2, 128, 4, 150), 2, env={"FLAGTREE_SMLA_HEAD_GROUPS": "1"}),
    "group_fp8_short_lists": forward_case(lambda: fp8_cfg(3, 65, 2, 40), 1, env={"FLAGTREE_SMLA_HEAD_GROUPS": "1"}),
    "tall_fp8_short_lists": forward_case(lambda: fp8_cfg(3, 65, 2, 40), 1),
    "short_bf16_split": forward_case(lambda: workloads.decode_bf16("cpu", batch=2, heads=16, pages_per_seq=5, topk=200, pad_frac=0.06), 2),
    "short_bf16_ragged_heads": forward_case(lambda: workloads.decode_bf16("cpu", batch=1, heads=9, pages_per_seq=5, topk=150, pad_frac=0.06), 1),
    "short_fp8_split": forward_case(lambda: fp8_cfg(2, 16, 4, 150), 2),
    "group_bf16_split": forward_case(lambda: workloads.decode_bf16("cpu", batch=2, heads=128, pages_per_seq=5, topk=200, pad_frac=0.06), 2,
                                      env={"FLAGTREE_SMLA_HEAD_GROUPS": "1"}),
    "group_bf16_ragged": forward_case(lambda: workloads.decode_bf16("cpu", batch=3, heads=65, pages_per_seq=5, topk=90, pad_frac=0.06), 3,
                                       env={"FLAGTREE_SMLA_HEAD_GROUPS": "1"}),
    "few_fp8_split": forward_case(lambda: fp8_cfg(2, 16, 4, 150), 2, env={"FLAGTREE_SMLA_FEW_FP8": "1"}),
    "few_fp8_ragged_heads": forward_case(lambda: fp8_cfg(1, 9, 4, 100), 1, env={"FLAGTREE_SMLA_FEW_FP8": "1"}),
    "fp8_mfma_split": forward_case(lambda: fp8_cfg(2, 16, 4, 150), 2, env={"FLAGTREE_SMLA_FP8_MFMA": "1"}),
    "fp8_mfma_ragged_heads": forward_case(lambda: fp8_cfg(1, 9, 4, 100), 1, env={"FLAGTREE_SMLA_FP8_MFMA": "1"}),
    "fp8_mfma_short_lists": forward_case(lambda: fp8_cfg(3, 30, 2, 40), 1, env={"FLAGTREE_SMLA_FP8_MFMA": "1"}),
    "tall_bf16_persistent": forward_case(lambda: workloads.prefill_causal_bf16("cpu", tokens=43, heads=72, topk=48), 1,
                                         env={"FLAGTREE_SMLA_PERSIST": "1"}),
    "dense_tall": forward_case(lambda: workloads.decode_bf16("cpu", batch=3, heads=128, pages_per_seq=3, topk=64), 2, dense=True),
    "dense_short_fp8": forward_case(lambda: fp8_cfg(3, 16, 3, 64), 1, dense=True),
    "scalar_f32": forward_case(lambda: workloads.plumbing_f32("cpu", tokens=2, heads=16, s_kv=256, topk=40), 1),
    "gather": raw_case(_gather), "kv_write": raw_case(_kv_write), "topk": raw_case(_topk), "gemm": raw_case(_gemm),
    "merge": raw_case(_merge),
}


if __name__ == "__main__":
    names = sys.argv[1:] or list(CASES)
    for name in names:
        for end in (True, False):
            print(f"guarded case {name} ({'end' if end else 'start'} of every buffer at a page edge)", flush=True)
            for eager, skew in ((False, 0), (True, 11)):      # (the second pass also with the wavefronts of a workgroup out of step)
                harness.configure(dma_eager=eager, wave_skew_seed=skew)
                CASES[name](end)
    print("ok")
