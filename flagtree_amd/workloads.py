"""Seeded synthetic inputs of the benchmark configurations (no datasets, no checkpoints).

Every generator takes size overrides so tests can run the same recipe at reduced size.
Large pools are generated on the device in slabs; whoever needs the values on the host
copies back the rows it reads, so host checker and device kernel always see the same bits.
"""
import math

import torch

from .sparse_mla import D_QK, D_V, quantize_kv_fp8

SM_SCALE = 1.0 / math.sqrt(D_QK)


def _gen(device, seed):
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def _randn_bf16(shape, device, g, std=0.1, slab_rows=1 << 18):
    """(N(0,1) * std).bf16 generated in slabs along dim 0 to bound the fp32 temporary."""
    out = torch.empty(shape, dtype=torch.bfloat16, device=device)
    flat = out.view(shape[0], -1)
    for r0 in range(0, shape[0], slab_rows):
        r1 = min(shape[0], r0 + slab_rows)
        flat[r0:r1] = (torch.randn((r1 - r0, flat.shape[1]), generator=g, device=device) * std).to(torch.bfloat16)
    return out


def _topk_indices(n_lists, pool, topk, n_pad, g, shuffle_pad):
    """n_lists draws of `topk` distinct positions from [0, pool) (CPU, int32); the last n_pad
    entries become -1, optionally shuffled into random positions."""
    idx = torch.empty((n_lists, topk), dtype=torch.int32)
    for i in range(n_lists):
        row = torch.randperm(pool, generator=g)[:topk].to(torch.int32)
        if n_pad:
            row[topk - n_pad:] = -1
            if shuffle_pad:
                row = row[torch.randperm(topk, generator=g)]
        idx[i] = row
    return idx


def plumbing_f32(device="cuda", seed=1001, tokens=4, heads=16, s_kv=4096, topk=256, pad_frac=0.10):
    """fp32 plumbing case: batch 1, `tokens` query tokens, kv [1, s_kv, 576], tail padding."""
    g = _gen("cpu", seed)
    q = torch.randn((1, tokens, heads, D_QK), generator=g) * 0.1
    kv = torch.randn((1, s_kv, D_QK), generator=g) * 0.1
    idx = _topk_indices(tokens, s_kv, topk, int(pad_frac * topk), g, shuffle_pad=False).view(1, tokens, topk)
    return dict(q=q.to(device), kv_cache=kv.to(device), indices=idx.to(device), block_table=None,
                page_size=64, sm_scale=SM_SCALE, kv_format="f32", name="plumbing_f32")


def decode_bf16(device="cuda", seed=1002, batch=64, heads=128, pages_per_seq=1024, page_size=64,
                topk=2048, pad_frac=0.05, shuffle_pad=True):
    """Paged bf16 decode: one query token per sequence, shuffled block table."""
    g = _gen("cpu", seed)
    gd = _gen(device, seed)
    n_pages = batch * pages_per_seq
    block_table = torch.randperm(n_pages, generator=g).to(torch.int32).view(batch, pages_per_seq)
    kv = _randn_bf16((n_pages, page_size, D_QK), device, gd)
    q = (torch.randn((batch, 1, heads, D_QK), generator=gd, device=device) * 0.1).to(torch.bfloat16)
    idx = _topk_indices(batch, pages_per_seq * page_size, topk, int(pad_frac * topk), g, shuffle_pad)
    return dict(q=q, kv_cache=kv, indices=idx.view(batch, 1, topk).to(device),
                block_table=block_table.to(device), page_size=page_size, sm_scale=SM_SCALE,
                kv_format="bf16", name="decode_bf16")


def prefill_causal_bf16(device="cuda", seed=1003, tokens=8192, heads=128, topk=2048):
    """Causal sparse prefill: query p picks min(topk, p+1) distinct positions of [0, p], rest -1."""
    gd = _gen(device, seed)
    kv = _randn_bf16((tokens, D_QK), device, gd)
    q = _randn_bf16((tokens, heads, D_QK), device, gd)
    idx = torch.empty((tokens, topk), dtype=torch.int32, device=device)
    pos = torch.arange(tokens, device=device)
    for r0 in range(0, tokens, 1024):
        r1 = min(tokens, r0 + 1024)
        key = torch.rand((r1 - r0, tokens), generator=gd, device=device)
        key[pos[None, :] > pos[r0:r1, None]] = 2.0                      # future positions sort last
        k_eff = min(topk, tokens)
        val, sel = torch.topk(key, k_eff, dim=1, largest=False)
        sel = torch.where(val < 1.5, sel, torch.full_like(sel, -1)).to(torch.int32)
        idx[r0:r1, :k_eff] = sel
        idx[r0:r1, k_eff:] = -1
    return dict(q=q.view(1, tokens, heads, D_QK), kv_cache=kv, indices=idx.view(1, tokens, topk),
                block_table=None, page_size=64, sm_scale=SM_SCALE, kv_format="bf16",
                name="prefill_causal_bf16")


def decode_fp8(device="cuda", seed=1004, batch=128, heads=16, pages_per_seq=2048, page_size=64,
               topk=2048, pad_frac=0.0):
    """Paged decode over an fp8 KV cache of 656-byte records (quantised on the device in slabs)."""
    g = _gen("cpu", seed)
    gd = _gen(device, seed)
    n_pages = batch * pages_per_seq
    rows = n_pages * page_size
    block_table = torch.randperm(n_pages, generator=g).to(torch.int32).view(batch, pages_per_seq)
    records = torch.empty((rows, 656), dtype=torch.uint8, device=device)
    slab = 1 << 18
    for r0 in range(0, rows, slab):
        r1 = min(rows, r0 + slab)
        latent = (torch.randn((r1 - r0, D_QK), generator=gd, device=device) * 0.1).to(torch.bfloat16)
        quantize_kv_fp8(latent, records[r0:r1])
    q = (torch.randn((batch, 1, heads, D_QK), generator=gd, device=device) * 0.1).to(torch.bfloat16)
    idx = _topk_indices(batch, pages_per_seq * page_size, topk, int(pad_frac * topk), g, True)
    return dict(q=q, kv_cache=records.view(n_pages, page_size, 656), indices=idx.view(batch, 1, topk).to(device),
                block_table=block_table.to(device), page_size=page_size, sm_scale=SM_SCALE,
                kv_format="fp8_e4m3_b128", name="decode_fp8")


def decode_fp8_h128(device="cuda", seed=1006):
    """The headline decode's shape (batch 64, 128 heads, top-k 2048 with 5 % padding, 65 536-token
    contexts) over an fp8 cache: the many-heads kernel's fp8 path."""
    cfg = decode_fp8(device, seed=seed, batch=64, heads=128, pages_per_seq=1024, topk=2048, pad_frac=0.05)
    cfg["name"] = "decode_fp8_h128"
    return cfg


def gemm_rs_shard(device="cuda", seed=1005, m=8192, k=2048, n=7168, n_chunks=8):
    gd = _gen(device, seed)
    x = (torch.randn((m, k), generator=gd, device=device) * 0.02).to(torch.bfloat16)
    w = (torch.randn((k, n), generator=gd, device=device) * 0.02).to(torch.bfloat16)
    partial = torch.randn((m, n), generator=gd, device=device) * 0.02
    return dict(x=x, w=w, partial=partial, n_chunks=n_chunks, name="gemm_rs_shard")


def attention_work(cfg):
    """Algorithmic work of one forward call: (flops, bytes, n_valid).
    flops = 2 * n_valid * H * (576 + 512); bytes = selected rows + q + out + lse + indices."""
    idx = cfg["indices"]
    n_valid = int((idx >= 0).sum().item())
    q = cfg["q"]
    H = q.shape[-2]
    T = q.numel() // (H * D_QK)
    row_bytes = {"bf16": 1152, "fp8_e4m3_b128": 656, "f32": 2304}[cfg["kv_format"]]
    out_bytes = T * H * D_V * q.element_size()
    flops = 2.0 * n_valid * H * (D_QK + D_V)
    kv_bytes = n_valid * row_bytes
    if cfg["name"] == "prefill_causal_bf16":                 # rows are re-used: count the cache once
        kv_bytes = cfg["kv_cache"].numel() * cfg["kv_cache"].element_size()
    nbytes = kv_bytes + q.numel() * q.element_size() + out_bytes + T * H * 4 + idx.numel() * 4
    return flops, nbytes, n_valid
