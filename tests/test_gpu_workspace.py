"""GPU checks of the split workspace's failure handling: a workspace whose arrival words are not in
the state a launch expects must neither hang the launch nor pass for a result.  Every condition is
forced from the host (a word written into the test's own workspace, a tiny poll limit in its
header); every kernel still runs to its normal end."""
import numpy as np
import pytest
import torch

from _util import to_np

pytestmark = pytest.mark.gpu


def _cfg(dev, heads):
    from flagtree_amd import workloads
    if heads <= 32:
        return workloads.decode_fp8(dev, batch=4, heads=heads, pages_per_seq=40, topk=600)
    return workloads.decode_bf16(dev, batch=4, heads=heads, pages_per_seq=48, topk=600, pad_frac=0.05)


def _fwd(cfg, **kw):
    import flagtree_amd as ft
    return ft.sparse_mla_fwd(cfg["q"], cfg["kv_cache"], cfg["indices"], cfg["sm_scale"], 512,
                             block_table=cfg["block_table"], page_size=cfg["page_size"],
                             kv_format=cfg["kv_format"], **kw)


def _header(ws):
    from flagtree_amd import _lib
    return ws[_lib.SMLA_WS_HEADER_OFFSET:_lib.SMLA_WS_HEADER_OFFSET + 16].view(torch.int32)


def _words(ws):
    from flagtree_amd import _lib
    return ws[:_lib.SMLA_WS_HEADER_OFFSET].view(torch.int64)


@pytest.mark.parametrize("heads", [128, 16])
@pytest.mark.parametrize("stale", ["one ticket", "own bit", "all ones"])
def test_stale_arrival_word_is_flagged_and_heals(dev, heads, stale):
    import flagtree_amd as ft
    from flagtree_amd import sparse_mla
    cfg = _cfg(dev, heads)
    ref_out, ref_lse = _fwd(cfg, n_splits=1)
    n_hblocks = (heads + 63) // 64 if heads > 32 else (heads + 15) // 16
    ws = ft.make_workspace(sparse_mla._lib.load().smla_workspace_bytes(4, heads, 512, 2), dev)
    _header(ws)[2] = 2000                                   # poll limit: the give-up path takes milliseconds
    word = {"one ticket": 1 << 32, "own bit": 1, "all ones": -1}[stale]
    token = 2
    _words(ws)[token * n_hblocks] = word                    # head block 0 of token 2
    torch.cuda.synchronize()
    out, lse = _fwd(cfg, n_splits=2, workspace=ws)
    torch.cuda.synchronize()                                # every kernel has ended
    with pytest.raises(RuntimeError, match="flagged"):
        ft.workspace_status(ws)
    assert ft.workspace_status(ws) == 0                     # the workspace was initialised again by the read
    lse_np = to_np(lse).reshape(4, heads)
    per_block = 64 if heads > 32 else 16
    assert np.isnan(lse_np[token, :min(per_block, heads)]).all()      # the rows concerned are marked
    keep = np.ones(4, dtype=bool)
    keep[token] = False
    # (a workgroup that started after the flag went up gives up as well: right or marked, never wrong)
    others, want = lse_np[keep], to_np(ref_lse).reshape(4, heads)[keep]
    assert (np.isnan(others) | (np.abs(others - want) <= 1e-3)).all()
    assert not to_np(out).reshape(4, heads, 512)[np.isnan(lse_np)].any()      # marked rows are zero
    assert int((_words(ws) != 0).sum().item()) == 0          # every arrival word is back to zero
    # the next launch on the same workspace is healthy and right
    out2, lse2 = _fwd(cfg, n_splits=2, workspace=ws)
    torch.cuda.synchronize()
    assert ft.workspace_status(ws) == 0
    assert np.abs(to_np(lse2) - to_np(ref_lse)).max() <= 1e-3
    assert np.abs(to_np(out2) - to_np(ref_out)).max() <= 1e-2


@pytest.mark.parametrize("heads", [128, 16])
def test_workspace_that_was_never_initialised_is_flagged(dev, heads):
    import flagtree_amd as ft
    from flagtree_amd import sparse_mla
    cfg = _cfg(dev, heads)
    n = sparse_mla._lib.load().smla_workspace_bytes(4, heads, 512, 2)
    ws = torch.zeros(n, dtype=torch.uint8, device=dev)
    out, lse = _fwd(cfg, n_splits=2, workspace=ws)
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError, match="never initialised"):
        ft.workspace_status(ws)
    assert np.isnan(to_np(lse)).all()


@pytest.mark.parametrize("heads", [128, 16])
def test_flagged_workspace_stays_loud_until_the_host_has_looked(dev, heads):
    """One ticket and the OTHER split's published bit in every arrival word, as a launch that gave
    up and a late publisher can leave them: judged by the words alone, each split of the next
    launch would draw the last ticket and fold in a stale partial.  The status word makes every
    split give up instead (NaN LSE, zero output) until workspace_status has run."""
    import flagtree_amd as ft
    from flagtree_amd import sparse_mla, _lib
    cfg = _cfg(dev, heads)
    ref_out, ref_lse = _fwd(cfg, n_splits=1)
    ws = ft.make_workspace(sparse_mla._lib.load().smla_workspace_bytes(4, heads, 512, 2), dev)
    ws[_lib.SMLA_WS_COUNTER_BYTES:] = 0x3C                   # partials nobody wrote: finite garbage
    _header(ws)[1] = 4
    _words(ws)[:] = (1 << 32) | 2
    torch.cuda.synchronize()
    out, lse = _fwd(cfg, n_splits=2, workspace=ws)
    torch.cuda.synchronize()
    assert np.isnan(to_np(lse)).all() and not to_np(out).any()
    assert int((_words(ws) != ((1 << 32) | 2)).sum().item()) == 0     # nobody took a ticket
    with pytest.raises(RuntimeError, match="timed out"):
        ft.workspace_status(ws)
    assert ft.workspace_status(ws) == 0
    out2, lse2 = _fwd(cfg, n_splits=2, workspace=ws)
    torch.cuda.synchronize()
    assert ft.workspace_status(ws) == 0
    assert np.abs(to_np(lse2) - to_np(ref_lse)).max() <= 1e-3
    assert np.abs(to_np(out2) - to_np(ref_out)).max() <= 1e-2


@pytest.mark.parametrize("heads", [128, 16])
def test_splits_merged_by_a_second_launch(dev, heads, monkeypatch):
    """FLAGTREE_SMLA_SEPARATE_MERGE=1 (what the library does by itself on a compute-unit count whose
    XCD layout it does not know): every split publishes, the merge kernel runs behind the forward
    kernel on the same stream, the arrival words are never touched."""
    from flagtree_amd import sparse_mla, _lib
    lib = sparse_mla._lib.load()
    cfg = _cfg(dev, heads)
    out1, lse1 = _fwd(cfg, n_splits=3)
    torch.cuda.synchronize()
    monkeypatch.setenv("FLAGTREE_SMLA_SEPARATE_MERGE", "1")
    assert lib.smla_merge_in_launch() == 0
    ws = torch.full((lib.smla_workspace_bytes(4, heads, 512, 3),), 0x3C, dtype=torch.uint8, device=dev)   # never initialised
    out, lse = _fwd(cfg, n_splits=3, workspace=ws)
    torch.cuda.synchronize()
    assert int((ws[:_lib.SMLA_WS_COUNTER_BYTES] != 0x3C).sum().item()) == 0
    assert np.abs(to_np(lse) - to_np(lse1)).max() <= 1e-5
    assert np.abs(to_np(out).astype(np.float64) - to_np(out1).astype(np.float64)).max() <= 2e-3


def test_default_workspace_can_be_checked_without_holding_it(dev):
    import flagtree_amd as ft
    cfg = _cfg(dev, 128)
    _fwd(cfg, n_splits=2)
    assert ft.workspace_status(None, dev) == 0


def test_workspace_argument_is_validated(dev):
    import flagtree_amd as ft
    cfg = _cfg(dev, 128)
    with pytest.raises(ValueError, match="too small"):
        _fwd(cfg, n_splits=2, workspace=torch.zeros(1 << 18, dtype=torch.uint8, device=dev))
    with pytest.raises(ValueError, match="uint8"):
        _fwd(cfg, n_splits=2, workspace=torch.zeros(1 << 22, dtype=torch.float32, device=dev))
    if dev.type == "cuda":                                  # (a rehearsal on the emulator has no second device to tell apart)
        with pytest.raises(ValueError, match="device"):
            _fwd(cfg, n_splits=2, workspace=torch.zeros(1 << 24, dtype=torch.uint8))


def test_each_stream_gets_its_own_default_workspace(dev):
    from flagtree_amd import sparse_mla
    if dev.type != "cuda":
        pytest.skip("needs real streams")
    cfg = _cfg(dev, 128)
    ref_out, ref_lse = _fwd(cfg, n_splits=1)
    streams = [torch.cuda.Stream(device=dev) for _ in range(2)]
    torch.cuda.synchronize()
    results = []
    for s in streams:
        with torch.cuda.stream(s):
            results.append(_fwd(cfg, n_splits=2))
    torch.cuda.synchronize()
    keys = {k for k in sparse_mla._workspaces if k[0] == dev and k[1] in {s.cuda_stream for s in streams}}
    assert len(keys) == 2
    ptrs = {sparse_mla._workspaces[k].data_ptr() for k in keys}
    assert len(ptrs) == 2
    for out, lse in results:
        assert np.abs(to_np(lse) - to_np(ref_lse)).max() <= 1e-3
        assert np.abs(to_np(out) - to_np(ref_out)).max() <= 1e-2
