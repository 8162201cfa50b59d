"""Helpers shared by the parity tests: move a workload's inputs to the host checker."""
import numpy as np
import torch

import oracle


def to_np(t):
    t = t.detach().cpu()
    if t.dtype == torch.bfloat16:
        t = t.float()
    return t.numpy()


def oracle_inputs(cfg):
    """From a workload dict build (q [T,H,D] f32, kv_small [n,576] f32, phys_small [T,K]) where
    kv_small holds only the rows some index selects (so big pools stay on the device)."""
    q = cfg["q"]
    H, D = q.shape[-2], q.shape[-1]
    qn = to_np(q).reshape(-1, H, D)
    T = qn.shape[0]
    idx = to_np(cfg["indices"]).reshape(T, -1)
    kvc = cfg["kv_cache"]
    kv2 = kvc.reshape(-1, kvc.shape[-1])
    bt = cfg.get("block_table")
    B = q.shape[0] if q.dim() == 4 else (bt.shape[0] if bt is not None else 1)
    S = T // B
    stride = 0
    if bt is None and kvc.dim() >= 3 and kvc.shape[0] == B and B > 1:
        stride = kvc[0].numel() // kvc.shape[-1]
    phys = oracle.translate_indices(idx, to_np(bt) if bt is not None else None, cfg.get("page_size", 64),
                                    kv_rows=kv2.shape[0], tokens_per_seq=S, kv_seq_stride=stride)
    uniq = np.unique(phys[phys >= 0])
    if uniq.size == 0:
        uniq = np.zeros(1, dtype=np.int64)
    rows = kv2[torch.from_numpy(uniq).to(kv2.device)]
    if cfg["kv_format"] == "fp8_e4m3_b128":
        kv_small = oracle.dequantize_kv_records(to_np(rows))
    else:
        kv_small = to_np(rows).astype(np.float32)
    phys_small = np.where(phys >= 0, np.searchsorted(uniq, np.where(phys >= 0, phys, uniq[0])), -1)
    return qn, kv_small, phys_small, phys


def run_oracle(cfg, dtype=np.float64):
    qn, kv_small, phys_small, _ = oracle_inputs(cfg)
    return oracle.sparse_mla_fwd(qn, kv_small, phys_small, cfg["sm_scale"], 512, dtype=dtype)


def max_abs(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    both_inf = np.isinf(a) & np.isinf(b) & (np.sign(a) == np.sign(b))
    d = np.abs(np.where(both_inf, 0.0, a - b))
    return float(np.nanmax(d)) if not np.isnan(d).any() else float("nan")


def random_shape_draw(seed):
    """One seeded draw over head counts, list lengths, page sizes, tokens per sequence, split counts,
    padding patterns, page tables with holes and both cache formats (CPU tensors; small enough for
    the host oracle).  `latent` holds bf16 rows; an fp8 cache is made from them by the caller."""
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    heads = int(rng.choice([1, 7, 16, 17, 32, 33, 64, 65, 127, 128]))
    topk = int(rng.choice([1, 31, 32, 33, 100, 257, 1024, 1100, 2300]))
    page_size = int(rng.choice([1, 16, 64]))
    tokens_per_seq = int(rng.choice([1, 3]))
    batch = int(rng.choice([1, 2, 5]))
    fmt = "fp8_e4m3_b128" if rng.random() < 0.35 else "bf16"
    n_splits = [None, 1, 2, 3, 5][int(rng.integers(5))]
    paged = rng.random() < 0.7
    ctx = int(rng.choice([64, 300, 2400]))                             # logical positions per sequence
    lat = (torch.randn((batch * ctx + 128, 576), generator=g) * float(rng.choice([0.05, 0.2]))).to(torch.bfloat16)
    if paged:
        pages_per_seq = -(-ctx // page_size)
        n_pages = batch * pages_per_seq + 3
        kv_rows = n_pages * page_size
        lat = (torch.randn((kv_rows, 576), generator=g) * 0.1).to(torch.bfloat16)
        bt = torch.randperm(n_pages, generator=g)[:batch * pages_per_seq].to(torch.int32).view(batch, pages_per_seq)
        if pages_per_seq > 2 and rng.random() < 0.5:
            bt[0, 1] = -1                                               # a hole: its positions are masked
        hi = pages_per_seq * page_size + (3 if rng.random() < 0.3 else 0)   # a few positions past the table
    else:
        bt = None
        hi = lat.shape[0] + (2 if rng.random() < 0.3 else 0)
    T = batch * tokens_per_seq
    idx = torch.from_numpy(rng.integers(0, hi, size=(T, topk)).astype(np.int32))
    pad = rng.random((T, topk)) < float(rng.choice([0.0, 0.1, 0.6]))
    idx[torch.from_numpy(pad)] = -1
    if rng.random() < 0.3:
        idx[0, topk // 2:] = -1                                        # tail padding
    if T > 1 and rng.random() < 0.3:
        idx[1, :] = -1                                                 # a token with nothing to attend to
    q = (torch.randn((batch, tokens_per_seq, heads, 576), generator=g) * 0.1).to(torch.bfloat16)
    return dict(heads=heads, kv_format=fmt, n_splits=n_splits, page_size=page_size, paged=paged, latent=lat, q=q,
                indices=idx.view(batch, tokens_per_seq, topk), block_table=bt)


def check_random_shape(draw, dev, fwd, check):
    """Runs one draw on the device: MFMA path against the oracle (through `check`) and against the scalar kernel."""
    import flagtree_amd as ft
    fmt, page_size = draw["kv_format"], draw["page_size"]
    kv = draw["latent"].to(dev) if fmt == "bf16" else ft.quantize_kv_fp8(draw["latent"].to(dev))
    if draw["paged"]:
        kv = kv.view(-1, page_size, kv.shape[-1])
    bt = draw["block_table"]
    cfg = dict(q=draw["q"].to(dev), kv_cache=kv, indices=draw["indices"].to(dev),
               block_table=bt.to(dev) if bt is not None else None, page_size=page_size, sm_scale=576 ** -0.5, kv_format=fmt)
    out, lse = fwd(cfg, n_splits=draw["n_splits"])
    check(cfg, out, lse)
    so, sl = ft.sparse_mla_fwd_scalar(cfg["q"], cfg["kv_cache"], cfg["indices"], cfg["sm_scale"], 512,
                                      block_table=cfg["block_table"], page_size=page_size, kv_format=fmt)
    assert max_abs(to_np(out), to_np(so)) <= 1e-2 and max_abs(to_np(lse), to_np(sl)) <= 1e-3
