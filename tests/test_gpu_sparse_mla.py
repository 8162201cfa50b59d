"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs.

Bars: translation / masking / gather bit-exact; out max-abs <= 1e-2 and lse max-abs <= 1e-3
against the float64 oracle fed the very same (bf16 / dequantised fp8) input values.
"""
import numpy as np
import pytest
import torch

import oracle
from _util import check_random_shape, max_abs, oracle_inputs, random_shape_draw, run_oracle, to_np

pytestmark = pytest.mark.gpu

OUT_TOL = 1e-2
LSE_TOL = 1e-3


def _fwd(cfg, **kw):
    import flagtree_amd as ft
    return ft.sparse_mla_fwd(cfg["q"], cfg["kv_cache"], cfg["indices"], cfg["sm_scale"], 512,
                             block_table=cfg["block_table"], page_size=cfg["page_size"],
                             kv_format=cfg["kv_format"], **kw)


def _check(cfg, out, lse, out_tol=OUT_TOL, lse_tol=LSE_TOL):
    ro, rl = run_oracle(cfg)
    H = cfg["q"].shape[-2]
    o = to_np(out).reshape(-1, H, 512)
    l = to_np(lse).reshape(-1, H)
    eo, el = max_abs(o, ro), max_abs(l, rl)
    assert eo <= out_tol, f"out max-abs {eo}"
    assert el <= lse_tol, f"lse max-abs {el}"
    return eo, el


def test_plumbing_f32_full(dev):
    from flagtree_amd import workloads
    cfg = workloads.plumbing_f32(dev)
    out, lse = _fwd(cfg)
    assert out.shape == (1, 4, 16, 512) and lse.shape == (1, 4, 16) and out.dtype == torch.float32
    _check(cfg, out, lse, out_tol=2e-6, lse_tol=2e-5)


@pytest.mark.parametrize("heads", [128, 64, 16, 96, 8])
@pytest.mark.parametrize("n_splits", [1, 3])
def test_decode_bf16_reduced(dev, heads, n_splits):
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16(dev, batch=3, heads=heads, pages_per_seq=48, topk=520, pad_frac=0.07)
    out, lse = _fwd(cfg, n_splits=n_splits)
    assert out.dtype == torch.bfloat16 and lse.dtype == torch.float32
    _check(cfg, out, lse)


def test_decode_bf16_auto_splits(dev):
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16(dev, batch=4, heads=128, pages_per_seq=64, topk=2048, pad_frac=0.05)
    out, lse = _fwd(cfg)
    _check(cfg, out, lse)


def test_scalar_kernel_matches_oracle(dev):
    import flagtree_amd as ft
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16(dev, batch=2, heads=16, pages_per_seq=16, topk=300, pad_frac=0.1)
    out, lse = ft.sparse_mla_fwd_scalar(cfg["q"], cfg["kv_cache"], cfg["indices"], cfg["sm_scale"], 512,
                                        block_table=cfg["block_table"], page_size=cfg["page_size"])
    _check(cfg, out, lse, out_tol=2e-3, lse_tol=1e-5)      # out is rounded to bf16 once


@pytest.mark.parametrize("heads", [16])               # (128 heads: test_gpu_x_unproven_kernels.py)
def test_decode_fp8_reduced(dev, heads):
    from flagtree_amd import workloads
    cfg = workloads.decode_fp8(dev, batch=3, heads=heads, pages_per_seq=32, topk=512, pad_frac=0.03)
    out, lse = _fwd(cfg, n_splits=2)
    _check(cfg, out, lse)


def test_prefill_causal_reduced(dev):
    from flagtree_amd import workloads
    cfg = workloads.prefill_causal_bf16(dev, tokens=320, heads=128, topk=128)
    out, lse = _fwd(cfg)
    idx = to_np(cfg["indices"]).reshape(320, 128)
    assert (idx[0] >= 0).sum() == 1 and (idx[200] >= 0).sum() == 128
    _check(cfg, out, lse)


def test_gather_and_translation_bit_exact(dev):
    import flagtree_amd as ft
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16(dev, batch=5, heads=16, pages_per_seq=8, topk=256, pad_frac=0.2)
    idx = cfg["indices"].clone().view(5, 256)
    idx[0, 0] = -1
    idx[1, 100] = 8 * 64            # first out-of-range logical position
    idx[2, 255] = 2 ** 31 - 1
    idx[3, :] = -1
    phys, rows = ft.gather_rows(cfg["kv_cache"].view(torch.int16), idx, block_table=cfg["block_table"],
                                page_size=64, tokens_per_seq=1)
    kv2 = to_np(cfg["kv_cache"].view(torch.int16)).reshape(-1, 576)
    want_phys = oracle.translate_indices(to_np(idx), to_np(cfg["block_table"]), 64, kv_rows=kv2.shape[0])
    assert np.array_equal(to_np(phys).astype(np.int64), want_phys)
    assert (want_phys[3] == -1).all() and want_phys[1, 100] == -1 and want_phys[2, 255] == -1
    assert np.array_equal(to_np(rows), oracle.gather_rows(kv2, want_phys))
    # fp8 records: 656-byte rows
    rec = torch.randint(0, 256, (40, 656), dtype=torch.uint8, device=dev)
    idx2 = torch.randint(-1, 40, (3, 64), dtype=torch.int32, device=dev)
    phys2, rows2 = ft.gather_rows(rec, idx2)
    want2 = oracle.translate_indices(to_np(idx2), None, 64, kv_rows=40)
    assert np.array_equal(to_np(phys2), want2)
    assert np.array_equal(to_np(rows2), oracle.gather_rows(to_np(rec), want2))


def test_edge_cases(dev):
    import flagtree_amd as ft
    g = torch.Generator().manual_seed(7)
    kv = (torch.randn((300, 576), generator=g) * 0.1).to(torch.bfloat16).to(dev)
    q = (torch.randn((6, 128, 576), generator=g) * 0.1).to(torch.bfloat16).to(dev)
    idx = torch.full((6, 70), -1, dtype=torch.int32)
    idx[1, 33] = 5                                           # single valid entry
    idx[2, :] = torch.randperm(300, generator=g)[:70].to(torch.int32)   # all valid, ragged top-k (70)
    idx[3, :35] = 17                                         # duplicates count once per occurrence
    idx[4, ::2] = torch.arange(35, dtype=torch.int32)        # interleaved padding
    idx[5, 0] = 299
    idx[5, 1] = 300                                          # out of range -> masked
    cfg = dict(q=q, kv_cache=kv, indices=idx.to(dev), block_table=None, page_size=64,
               sm_scale=576 ** -0.5, kv_format="bf16")
    for ns in (1, 2):
        out, lse = _fwd(cfg, n_splits=ns)
        _check(cfg, out, lse)
        o, l = to_np(out), to_np(lse)
        assert (o[0] == 0).all() and np.isneginf(l[0]).all()          # token without valid entries
        assert np.array_equal(o[1], np.broadcast_to(to_np(kv)[5, :512], (128, 512)))   # K = 1: out = v


def test_merge_splits_kernel(dev):
    import flagtree_amd as ft
    rng = np.random.default_rng(3)
    po = rng.standard_normal((5, 4, 16, 512)).astype(np.float32)
    pl = rng.standard_normal((5, 4, 16)).astype(np.float32) * 3
    pl[0, 1] = -np.inf
    pl[1, :, 3] = -np.inf
    out, lse = ft.merge_splits(torch.from_numpy(po).to(dev), torch.from_numpy(pl).to(dev))
    wo, wl = oracle.merge_splits(po.transpose(1, 0, 2, 3), pl.transpose(1, 0, 2))
    assert max_abs(to_np(lse), wl) <= 1e-5
    assert max_abs(to_np(out), oracle.bf16_round(wo.astype(np.float32))) <= 2e-2   # bf16 ulp at |x|~3
    assert max_abs(to_np(out), wo) <= 2e-2
    assert np.isneginf(to_np(lse)[1, 3]) and (to_np(out)[1, 3] == 0).all()


def test_quantize_fp8_bit_exact(dev):
    import flagtree_amd as ft
    g = torch.Generator().manual_seed(11)
    lat = (torch.randn((257, 576), generator=g) * 0.1).to(torch.bfloat16)
    lat[3, :128] = 0                                         # zero block
    lat[4, 5] = 1000.0
    lat[5, 130] = -3e-6
    rec = ft.quantize_kv_fp8(lat.to(dev))
    want = oracle.quantize_kv_records(lat.float().numpy())
    assert np.array_equal(to_np(rec), want)
    # slot-addressed writes leave other rows alone
    pool = torch.zeros((8, 656), dtype=torch.uint8, device=dev)
    ft.quantize_kv_fp8(lat[:3].to(dev), pool, slot=torch.tensor([6, -1, 2], device=dev))
    p = to_np(pool)
    assert np.array_equal(p[6], want[0]) and np.array_equal(p[2], want[2]) and (p[[0, 1, 3, 4, 5, 7]] == 0).all()


def test_quantize_fp8_bit_exact_special_values(dev):
    """Rounding ties, the saturation edge, subnormal codes and signed zeros: every finite bf16 bit
    pattern appears as an input (NaN / infinity make a block's scale meaningless: not compared)."""
    import flagtree_amd as ft
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)              # all bf16 patterns ...
    bits[(bits & 0x7F80) == 0x7F80] = 0                                      # ... but the non-finite ones
    g = np.random.default_rng(5)
    rows = []
    for rep in range(8):                                                     # 8 x 128 rows x 512 = 8 x 65536 values
        perm = g.permutation(65536)
        rows.append(bits[perm].reshape(128, 512))
    nope = np.concatenate(rows, axis=0)
    lat_bits = np.concatenate([nope, nope[:, :64]], axis=1)
    lat = torch.from_numpy(lat_bits.view(np.int16).copy()).view(torch.bfloat16)
    rec = ft.quantize_kv_fp8(lat.to(dev))
    with np.errstate(all="ignore"):
        want = oracle.quantize_kv_records(oracle.bf16_bits_to_f32(lat_bits))
    assert np.array_equal(to_np(rec), want)
    # small magnitudes only: exercises subnormal e4m3 codes and ties without any NaN in the row
    small = ((g.standard_normal((512, 576)) * 10.0 ** g.uniform(-6, 2, size=(512, 1)))).astype(np.float32)
    small = oracle.bf16_round(small)
    lat2 = torch.from_numpy(small).to(torch.bfloat16)
    assert np.array_equal(to_np(ft.quantize_kv_fp8(lat2.to(dev))), oracle.quantize_kv_records(small))


def test_quantize_fp8_bit_exact_at_midpoints(dev):
    """Quotients that are exactly the midpoint of two fp8 values, and their bf16 neighbours, for block
    scales c * 2^e: the writer multiplies by 1 / scale and must fall back to the division wherever the
    product could land on the other side of a midpoint."""
    import flagtree_amd as ft
    mids = []                                                     # positive fp8 midpoints in [2^-9, 448)
    for e in range(-6, 9):
        for m in range(8):
            mids.append((1 + m / 8 + 1 / 16) * 2.0 ** e)          # normal range: 3 mantissa bits + half a step
    mids += [(2 * j + 1) * 2.0 ** -10 for j in range(8)]          # subnormal range: steps of 2^-9
    mids = np.array([v for v in mids if v < 448], dtype=np.float64)
    rows = []
    for c in (1.0, 1.5, 1.25, 1.75, 1.0078125, 1.9921875):
        for e in (-20, -3, 0, 5, 30):
            scale = c * 2.0 ** e
            base = oracle.bf16_round((mids * scale).astype(np.float32))       # exact where the product fits 8 bits
            b = oracle.f32_to_bf16_bits(base).astype(np.int32)
            vals = np.concatenate([b - 1, b, b + 1, (b - 1) | 0x8000, b | 0x8000, (b + 1) | 0x8000]).astype(np.uint16)
            vals = vals[: 127 * (len(vals) // 127)].reshape(-1, 127)
            amax = oracle.f32_to_bf16_bits(np.full((vals.shape[0], 1), 448.0 * scale, np.float32))
            blocks = np.concatenate([amax, vals], axis=1)                      # one 128-column block per line
            rows.append(blocks)
    blocks = np.concatenate(rows, axis=0)
    blocks = blocks[: 4 * (blocks.shape[0] // 4)]
    nope = blocks.reshape(-1, 512)
    lat_bits = np.concatenate([nope, nope[:, :64]], axis=1)
    lat = torch.from_numpy(lat_bits.view(np.int16).copy()).view(torch.bfloat16)
    want = oracle.quantize_kv_records(oracle.bf16_bits_to_f32(lat_bits))
    assert np.array_equal(to_np(ft.quantize_kv_fp8(lat.to(dev))), want)


def test_quantize_fp8_scale_of_every_block_maximum(dev):
    """Every positive finite bf16 value as the maximum of one block (down to the subnormal ones,
    where the scale is clamped, and just above, where the correction term of the writer's division
    by 448 is itself subnormal)."""
    import flagtree_amd as ft
    bits = np.arange(1, 0x7F80, dtype=np.uint16)
    bits = np.concatenate([bits, np.full((-len(bits)) % 4, 0x3F80, np.uint16)])
    blocks = np.zeros((len(bits), 128), dtype=np.uint16)
    blocks[:, 17] = bits
    blocks[:, 90] = bits | 0x8000
    blocks[:, 3] = np.where((bits >> 7) > 1, bits - 0x80, 0).astype(np.uint16)
    lat_bits = np.concatenate([blocks.reshape(-1, 512), blocks.reshape(-1, 512)[:, :64]], axis=1)
    lat = torch.from_numpy(lat_bits.view(np.int16).copy()).view(torch.bfloat16)
    got = to_np(ft.quantize_kv_fp8(lat.to(dev)))
    want = oracle.quantize_kv_records(oracle.bf16_bits_to_f32(lat_bits))
    assert np.array_equal(got[:, 512:528], want[:, 512:528]), "scales"
    assert np.array_equal(got, want)


def test_quantize_fp8_bit_exact_random_magnitudes(dev):
    """38 million random quotients over forty decades of block scales."""
    import flagtree_amd as ft
    g = np.random.default_rng(77)
    x = g.standard_normal((65536, 576)).astype(np.float32) * (10.0 ** g.uniform(-20, 20, size=(65536, 1))).astype(np.float32)
    x = oracle.bf16_round(x)
    lat = torch.from_numpy(x).to(torch.bfloat16)
    got = to_np(ft.quantize_kv_fp8(lat.to(dev)))
    want = oracle.quantize_kv_records(x)
    assert np.array_equal(got, want), f"{int((got != want).sum())} bytes differ"


def test_reshape_and_cache_both_formats(dev):
    import flagtree_amd as ft
    g = torch.Generator().manual_seed(31)
    n, rows = 300, 4 * 64                                                    # 4 pages of 64
    lat = (torch.randn((n, 576), generator=g) * 0.2).to(torch.bfloat16)
    slots = torch.randperm(rows, generator=g)[:n % rows if n < rows else rows]
    slots = torch.cat([slots, torch.full((n - slots.numel(),), -1, dtype=torch.int64)])[torch.randperm(n, generator=g)]
    slots[7] = rows + 5                                                      # past the pool: skipped
    pool = torch.full((4, 64, 576), 7.0, dtype=torch.bfloat16, device=dev)
    assert ft.reshape_and_cache(lat.to(dev), pool, slots.to(dev), "bf16") is None
    want = oracle.reshape_and_cache(lat.float().numpy(), oracle.f32_to_bf16_bits(np.full((rows, 576), 7.0, np.float32)),
                                    slots.numpy(), "bf16")
    assert np.array_equal(to_np(pool.view(torch.int16)).view(np.uint16).reshape(rows, 576), want)
    pool8 = torch.full((4, 64, 656), 0x5A, dtype=torch.uint8, device=dev)
    ft.reshape_and_cache(lat.to(dev), pool8, slots.to(dev), "fp8_e4m3_b128")
    want8 = oracle.reshape_and_cache(lat.float().numpy(), np.full((rows, 656), 0x5A, np.uint8), slots.numpy(), "fp8_e4m3_b128")
    assert np.array_equal(to_np(pool8).reshape(rows, 656), want8)
    with pytest.raises(ValueError):
        ft.reshape_and_cache(lat.to(dev), pool8, slots.to(dev), "bf16")


@pytest.mark.parametrize("n,k,quant", [(1, 1, 0), (37, 64, 0), (1024, 1024, 0), (1500, 256, 0), (4096, 2048, 8),
                                       (65536, 2048, 0), (65536, 2048, 64), (10000, 2048, 2)])
def test_topk_indices_exact(dev, n, k, quant):
    """(The rows of 10 000 and 65 536 entries are cut into parts when the wrapper may allocate a
    workspace; both ways must give the oracle's list.)"""
    import flagtree_amd as ft
    g = np.random.default_rng(1000 + n + k)
    x = g.standard_normal((5, n)).astype(np.float32)
    if quant:
        x = (np.round(x * quant) / quant).astype(np.float32)      # heavy ties at the threshold
    if n > 8:
        x[0, 3] = np.nan; x[0, 5] = np.inf; x[1, 7] = -np.inf; x[2, :n // 2] = 0.25; x[3, 0] = -0.0; x[3, 1] = 0.0
    lens = np.array([n, n // 2, n, max(1, n - 1), 0], dtype=np.int32)
    got = ft.topk_indices(torch.from_numpy(x).to(dev), k, torch.from_numpy(lens).to(dev))
    assert np.array_equal(to_np(got), oracle.topk_indices(x, k, lens))
    got2 = ft.topk_indices(torch.from_numpy(x).to(dev), k)
    assert np.array_equal(to_np(got2), oracle.topk_indices(x, k))
    got3 = ft.topk_indices(torch.from_numpy(x).to(dev), k, torch.from_numpy(lens).to(dev), workspace=False)
    assert np.array_equal(to_np(got3), oracle.topk_indices(x, k, lens))


@pytest.mark.parametrize("rows,n,k,quant", [(1100, 4096, 300, 0),      # many short rows
                                             (1030, 5000, 512, 4),      # many rows, four rounds a wavefront, the last ones partial
                                             (1024, 6000, 5500, 0),     # list too long for the LDS staging
                                             (3, 16384, 9000, 16), (2, 40000, 30000, 0), (2, 70000, 100, 2),
                                             (6, 65537, 64, 4)])        # the first length of the kernel for long rows, tied values
def test_topk_indices_shapes(dev, rows, n, k, quant):
    """Every kernel variant the launcher picks (by row count and length), with context lengths that
    leave wavefronts without entries, rounds partly filled and rows empty."""
    import flagtree_amd as ft
    g = np.random.default_rng(rows + n + k)
    x = g.standard_normal((rows, n)).astype(np.float32)
    if quant:
        x = (np.round(x * quant) / quant).astype(np.float32)
    lens = g.integers(0, n + 1, size=rows).astype(np.int32)
    lens[:3] = [n, 1, 0][:min(3, rows)]
    got = ft.topk_indices(torch.from_numpy(x).to(dev), k, torch.from_numpy(lens).to(dev))
    assert np.array_equal(to_np(got), oracle.topk_indices(x, k, lens))
    if ft.topk_workspace_bytes(rows, n, k):                        # cut into parts above: also one workgroup per row
        got = ft.topk_indices(torch.from_numpy(x).to(dev), k, torch.from_numpy(lens).to(dev), workspace=False)
        assert np.array_equal(to_np(got), oracle.topk_indices(x, k, lens))


@pytest.mark.parametrize("n", [1000, 4099, 20000])
def test_topk_indices_unaligned_rows(dev, n):
    """Rows that start off a 16-byte boundary and lie a non-multiple of 4 apart (a column slice of a
    wider matrix): the kernel reads them 4 bytes at a time."""
    import flagtree_amd as ft
    g = np.random.default_rng(n)
    big = g.standard_normal((6, n + 7)).astype(np.float32)
    view = torch.from_numpy(big).to(dev)[:, 1:n + 1]
    assert view.stride(0) == n + 7 and view.data_ptr() % 16 != 0
    got = ft.topk_indices(view, 128)
    assert np.array_equal(to_np(got), oracle.topk_indices(np.ascontiguousarray(big[:, 1:n + 1]), 128))


@pytest.mark.parametrize("n,k", [(4096, 2048), (16384, 100), (65536, 2048), (70000, 64)])
def test_topk_indices_degenerate_rows(dev, n, k):
    """Rows where every pass of the selection sees a single bin: all entries equal, all NaN, all
    -inf; sorted rows; a row whose candidates for the last place are a run of 500 equal values."""
    import flagtree_amd as ft
    g = np.random.default_rng(n + k)
    rows = [np.zeros(n), np.full(n, np.nan), np.full(n, -np.inf), np.full(n, 3.5),
            np.arange(n, dtype=np.float64), -np.arange(n, dtype=np.float64),
            np.where(np.arange(n) % 2 == 0, 1.0, -1.0)]
    tied = g.standard_normal(n)
    order = np.argsort(-tied)
    tied[order[max(0, k - 250):k + 250]] = tied[order[k]]          # 500 equal values straddle the k-th place
    rows.append(tied)
    x = np.stack(rows).astype(np.float32)
    got = ft.topk_indices(torch.from_numpy(x).to(dev), k)
    got1 = ft.topk_indices(torch.from_numpy(x).to(dev), k, workspace=False)
    with np.errstate(all="ignore"):
        assert np.array_equal(to_np(got), oracle.topk_indices(x, k))
        assert np.array_equal(to_np(got1), oracle.topk_indices(x, k))


@pytest.mark.parametrize("rows,n,k,page_size,rows_per_seq", [(4, 3000, 200, 64, 2), (8, 65536, 2048, 64, 1), (6, 1000, 1000, 1, 3)])
def test_topk_written_as_physical_rows(dev, rows, n, k, page_size, rows_per_seq):
    """The index producer's list as physical rows of the paged cache = its list of positions put
    through the translation of the attention kernels (oracle.translate_indices), bit for bit, with a
    table shorter than the contexts, a hole and pages past the pool."""
    import flagtree_amd as ft
    g = torch.Generator().manual_seed(rows + n)
    scores = torch.randn((rows, n), generator=g)
    lens = torch.randint(1, n + 1, (rows,), generator=g, dtype=torch.int32)
    n_seqs = rows // rows_per_seq
    pages = max(1, (n * 3 // 4) // page_size)
    bt = torch.randperm(n_seqs * pages + 5, generator=g)[:n_seqs * pages].to(torch.int32).view(n_seqs, pages)
    if pages > 2:
        bt[0, 1] = -1
    kv_rows = (n_seqs * pages + 2) * page_size
    want = oracle.translate_indices(oracle.topk_indices(scores.numpy(), k, lens.numpy()), bt.numpy(), page_size, kv_rows=kv_rows,
                                    tokens_per_seq=rows_per_seq)
    for ws in (None, False):
        got = ft.topk_indices(scores.to(dev), k, lens.to(dev), workspace=ws, block_table=bt.to(dev), page_size=page_size,
                              kv_rows=kv_rows, rows_per_seq=rows_per_seq)
        assert np.array_equal(to_np(got), want)


def test_attention_over_physical_rows_from_the_index_producer(dev):
    """Rows from the index producer, no page table for the attention kernel: the same bits as
    positions plus page table."""
    import flagtree_amd as ft
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16(dev, batch=6, heads=128, pages_per_seq=24, topk=512, pad_frac=0.0)
    B, page_size, pages = 6, cfg["page_size"], cfg["block_table"].shape[1]
    n, k = pages * page_size, 512
    g = torch.Generator().manual_seed(3)
    scores = torch.randn((B, n), generator=g).to(dev)
    lens = torch.tensor([n, n // 2, 150, n, 700, n - 1], dtype=torch.int32).to(dev)
    kv_rows = cfg["kv_cache"].numel() // 576
    logical = ft.topk_indices(scores, k, lens)
    rows = ft.topk_indices(scores, k, lens, block_table=cfg["block_table"], page_size=page_size, kv_rows=kv_rows)
    out0, lse0 = _fwd(dict(cfg, indices=logical.view(B, 1, k)), n_splits=2)
    out1, lse1 = ft.sparse_mla_fwd(cfg["q"], cfg["kv_cache"].reshape(-1, 576), rows.view(B, 1, k), cfg["sm_scale"], 512,
                                   kv_format="bf16", n_splits=2, per_sequence=False)
    torch.cuda.synchronize()
    assert torch.equal(out0, out1) and torch.equal(lse0, lse1)
    _check(dict(cfg, indices=logical.view(B, 1, k)), out1, lse1)


def test_topk_feeds_sparse_mla(dev):
    """Indexer scores -> top-k indices -> sparse attention: same result as handing the oracle's
    index list to the attention kernel."""
    import flagtree_amd as ft
    g = torch.Generator().manual_seed(9)
    n_ctx, k = 640, 128
    q = (torch.randn((2, 1, 16, 576), generator=g) * 0.1).to(torch.bfloat16)
    kv = (torch.randn((2, n_ctx, 576), generator=g) * 0.1).to(torch.bfloat16)
    scores = torch.randn((2, 1, n_ctx), generator=g)
    idx = ft.topk_indices(scores.to(dev), k)
    want_idx = oracle.topk_indices(scores.numpy(), k)
    assert np.array_equal(to_np(idx), want_idx)
    out, lse = ft.sparse_mla_fwd(q.to(dev), kv.to(dev), idx, 576 ** -0.5, 512)
    out2, lse2 = ft.sparse_mla_fwd(q.to(dev), kv.to(dev), torch.from_numpy(want_idx).to(dev), 576 ** -0.5, 512)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)


@pytest.mark.parametrize("H,page_size,fmt", [(16, 16, "bf16"), (128, 64, "bf16"), (16, 64, "fp8_e4m3_b128"), (64, 1, "bf16")])
def test_decode_attention_fwd_dense(dev, H, page_size, fmt):
    """Dense decode = sparse forward handed the index list 0 .. len-1 (shapes follow the reference's
    test_decode_attention: B in (3, 5), L = 1027: not a multiple of anything)."""
    import flagtree_amd as ft
    g = torch.Generator().manual_seed(123 + H + page_size)
    B, L = 3, 1027
    lens = torch.tensor([L, 1, 517], dtype=torch.int32)
    n_pages = -(-L // page_size)
    cache_pages = 4 * B * n_pages
    req_to_token = torch.randperm(cache_pages, generator=g)[:B * n_pages].to(torch.int32).view(B, n_pages)
    lat = (torch.randn((cache_pages * page_size, 576), generator=g) * 0.1).to(torch.bfloat16)
    q = (torch.randn((B, H, 576), generator=g) * 0.1).to(torch.bfloat16)
    if fmt == "bf16":
        k_buffer = lat.to(dev).view(cache_pages, page_size, 576)
        v_buffer = k_buffer[..., :512]
    else:
        k_buffer = ft.quantize_kv_fp8(lat.to(dev)).view(cache_pages, page_size, 656)
        v_buffer = None
    o = torch.zeros((B, H, 512), dtype=torch.bfloat16, device=dev)
    o2, lse = ft.decode_attention_fwd(q.to(dev), k_buffer, v_buffer, o, req_to_token.to(dev), lens.to(dev), None, 2,
                                      576 ** -0.5, page_size)
    assert o2 is o
    # the same through the sparse entry point with an explicit list
    max_len = n_pages * page_size
    idx = torch.arange(max_len, dtype=torch.int32).repeat(B, 1)
    idx[idx >= lens[:, None]] = -1
    want, want_lse = ft.sparse_mla_fwd(q.to(dev).view(B, 1, H, 576), k_buffer, idx.view(B, 1, max_len).to(dev), 576 ** -0.5, 512,
                                       block_table=req_to_token.to(dev), page_size=page_size, n_splits=2)
    assert torch.equal(o, want.view(B, H, 512)) and torch.equal(lse, want_lse.view(B, H))
    o3, lse3 = ft.decode_attention_fwd(q.to(dev), k_buffer, v_buffer, None, req_to_token.to(dev), lens.to(dev), None, None,
                                       576 ** -0.5, page_size)          # the library's own split count
    assert max_abs(to_np(o3), to_np(o)) <= 1e-3 and max_abs(to_np(lse3), to_np(lse)) <= 1e-5
    # and against the host oracle
    cfg = {"q": q.view(B, 1, H, 576), "indices": idx.view(B, 1, max_len), "kv_cache": k_buffer, "block_table": req_to_token,
           "page_size": page_size, "kv_format": fmt, "sm_scale": 576 ** -0.5}
    wo, wl = run_oracle(cfg)
    assert max_abs(to_np(o), wo.reshape(B, H, 512)) <= 1e-2 and max_abs(to_np(lse), wl.reshape(B, H)) <= 1e-3
    with pytest.raises(ValueError):
        ft.decode_attention_fwd(q.to(dev), k_buffer, v_buffer, o, req_to_token.to(dev), lens.to(dev), None, None,
                                576 ** -0.5, page_size, logit_cap=-1.0)


@pytest.mark.parametrize("H,fmt,std,cap,min_diff", [(128, "bf16", 1.5, 2.0, 0.5), (16, "bf16", 1.5, 2.0, 0.5),
                                                    (16, "fp8_e4m3_b128", 1.5, 2.0, 0.5)])
@pytest.mark.parametrize("splits", [1, 2])
def test_decode_attention_fwd_logit_cap(dev, H, fmt, std, cap, min_diff, splits):
    check_logit_cap(dev, H, fmt, std, cap, min_diff, splits)


def check_logit_cap(dev, H, fmt, std, cap, min_diff, splits):
    """logit_cap * tanh(score / logit_cap) before the softmax (reference test_accuracy_musa_vllm_mla.py:299-302);
    inputs scaled so that raw scores reach several times the cap.  (The many-heads kernel rounds
    dequantised fp8 values to bf16 when it stages them, an error that grows with the square of the
    input scale: its case stays nearer the benchmark's magnitudes.)"""
    import flagtree_amd as ft
    g = torch.Generator().manual_seed(77 + H)
    B, L, page_size = 3, 700, 64
    lens = torch.tensor([L, 3, 300], dtype=torch.int32)
    n_pages = -(-L // page_size)
    req_to_token = torch.randperm(2 * B * n_pages, generator=g)[:B * n_pages].to(torch.int32).view(B, n_pages)
    lat = (torch.randn((2 * B * n_pages * page_size, 576), generator=g) * std).to(torch.bfloat16)
    q = (torch.randn((B, H, 576), generator=g) * std).to(torch.bfloat16)
    if fmt == "bf16":
        k_buffer = lat.to(dev).view(-1, page_size, 576)
    else:
        k_buffer = ft.quantize_kv_fp8(lat.to(dev)).view(-1, page_size, 656)
    o, lse = ft.decode_attention_fwd(q.to(dev), k_buffer, None, None, req_to_token.to(dev), lens.to(dev), None, splits,
                                     576 ** -0.5, page_size, logit_cap=cap)
    max_len = n_pages * page_size
    idx = torch.arange(max_len, dtype=torch.int32).repeat(B, 1)
    idx[idx >= lens[:, None]] = -1
    cfg = {"q": q.view(B, 1, H, 576), "indices": idx.view(B, 1, max_len), "kv_cache": k_buffer, "block_table": req_to_token,
           "page_size": page_size, "kv_format": fmt, "sm_scale": 576 ** -0.5}
    qn, kv_small, phys_small, _ = oracle_inputs(cfg)
    wo, wl = oracle.sparse_mla_fwd(qn, kv_small, phys_small, cfg["sm_scale"], 512, logit_cap=cap)
    uo, ul = oracle.sparse_mla_fwd(qn, kv_small, phys_small, cfg["sm_scale"], 512)
    assert max_abs(wl, ul) > min_diff                                   # the cap matters on these inputs
    assert max_abs(to_np(lse), wl.reshape(B, H)) <= 1e-3
    assert max_abs(to_np(o), wo.reshape(B, H, 512)) <= 1e-2 * max(1.0, float(np.abs(wo).max()))


@pytest.mark.parametrize("heads,ns", [(128, 2), (128, 4), (16, 2), (16, 8)])
def test_split_merge_does_not_depend_on_arrival_order(dev, heads, ns):
    """Which split arrives last differs from launch to launch; the merged result must not."""
    import flagtree_amd as ft
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16(dev, batch=16, heads=heads, pages_per_seq=64)
    outs = []
    for rep in range(6):
        out, lse = ft.sparse_mla_fwd(cfg["q"], cfg["kv_cache"], cfg["indices"], cfg["sm_scale"], 512,
                                     block_table=cfg["block_table"], page_size=cfg["page_size"], n_splits=ns)
        outs.append((out.clone(), lse.clone()))
        torch.empty(1 << 24, device=dev).normal_()                  # unrelated work between the launches
    for out, lse in outs[1:]:
        assert torch.equal(out, outs[0][0]) and torch.equal(lse, outs[0][1])
    wo, wl = run_oracle(cfg)
    assert max_abs(to_np(outs[0][0]).reshape(wo.shape), wo) <= 1e-2 and max_abs(to_np(outs[0][1]).reshape(wl.shape), wl) <= 1e-3


def test_forward_replays_from_a_hip_graph(dev):
    """The forward (split merge included) is one kernel launch with no memset or allocation, so it
    can be captured; every replay, with eager work and synchronisations in between, must give the
    eager result (the arrival counters are left ready by the kernel itself)."""
    import flagtree_amd as ft
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16(dev, batch=8, pages_per_seq=64)
    T, H, K = 8, cfg["q"].shape[2], cfg["indices"].shape[-1]
    ws = ft.make_workspace(ft._lib.load().smla_workspace_bytes(T, H, 512, 2), dev)
    def fwd():
        return ft.sparse_mla_fwd(cfg["q"], cfg["kv_cache"], cfg["indices"], cfg["sm_scale"], 512,
                                 block_table=cfg["block_table"], page_size=cfg["page_size"], n_splits=2, workspace=ws)
    want_out, want_lse = fwd()
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        fwd()                                                        # warm-up on the capture stream
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            g_out, g_lse = fwd()
    for rep in range(3):
        g_out.zero_(); g_lse.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_out, want_out) and torch.equal(g_lse, want_lse), rep
        e_out, e_lse = fwd()                                         # eager call between replays, same workspace
        torch.cuda.synchronize()
        assert torch.equal(e_out, want_out) and torch.equal(e_lse, want_lse)


@pytest.mark.parametrize("seed", list(range(24)))
def test_random_shapes_against_oracle(dev, seed):
    """Seeded draws over head counts, list lengths, page sizes, tokens per sequence, split counts,
    padding patterns, page tables with holes and both cache formats (small enough for the host oracle)."""
    draw = random_shape_draw(4000 + seed)
    if draw["kv_format"] != "bf16" and draw["heads"] > 32:
        pytest.skip("many heads over an fp8 cache: runs in test_gpu_x_unproven_kernels.py")
    check_random_shape(draw, dev, _fwd, _check)


@pytest.mark.parametrize("heads", [16, 128])
@pytest.mark.parametrize("bt_stride", [9001, 8190])
def test_page_tables_that_do_not_fit_or_align(dev, heads, bt_stride):
    """Page-table rows longer than the LDS staging area, or not a multiple of 16 bytes, take the
    global lookup path; long lists span several 1024-entry chunks (only the first chunk's indices
    are loaded ahead)."""
    import flagtree_amd as ft
    g = torch.Generator().manual_seed(77 + heads + bt_stride)
    B, topk = 2, 2600
    n_pages = B * bt_stride + 5
    bt = torch.randperm(n_pages, generator=g)[:B * bt_stride].to(torch.int32).view(B, bt_stride)
    kv = (torch.randn((n_pages, 1, 576), generator=g) * 0.1).to(torch.bfloat16)       # page_size 1
    idx = torch.stack([torch.randperm(bt_stride, generator=g)[:topk] for _ in range(B)]).to(torch.int32)
    idx[0, 100:1300] = -1                                                           # a whole chunk without valid entries in the middle
    q = (torch.randn((B, 1, heads, 576), generator=g) * 0.1).to(torch.bfloat16)
    cfg = dict(q=q.to(dev), kv_cache=kv.to(dev), indices=idx.view(B, 1, topk).to(dev), block_table=bt.to(dev),
               page_size=1, sm_scale=576 ** -0.5, kv_format="bf16")
    for ns in (1, 2):
        out, lse = _fwd(cfg, n_splits=ns)
        _check(cfg, out, lse)


def test_mfma_vs_scalar_device_kernels_large(dev):
    """Full decode geometry (B=64, h=128, topk=2048, 65536-token paged contexts) is too big for the
    host checker; the two independent device implementations must agree there, and the host
    oracle checks a sample of the batch."""
    import flagtree_amd as ft
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16(dev, batch=16, pages_per_seq=1024)
    out, lse = _fwd(cfg)
    so, sl = ft.sparse_mla_fwd_scalar(cfg["q"], cfg["kv_cache"], cfg["indices"], cfg["sm_scale"], 512,
                                      block_table=cfg["block_table"], page_size=64)
    assert (out.float() - so.float()).abs().max().item() <= OUT_TOL
    assert (lse - sl).abs().max().item() <= LSE_TOL
    sub = dict(cfg)
    sub["q"], sub["indices"], sub["block_table"] = cfg["q"][:2], cfg["indices"][:2], cfg["block_table"][:2]
    _check(sub, out[:2], lse[:2])


@pytest.mark.parametrize("q_std", [0.3, 1.0, 4.0])
@pytest.mark.parametrize("n_splits", [1, 2])
def test_wide_score_range_redo_path(dev, q_std, n_splits):
    """Scores spread over tens to hundreds of nats: later tiles exceed the first tile's maximum by
    more than the fast pass tolerates, which forces the exact-maximum redo passes."""
    import flagtree_amd as ft
    g = torch.Generator().manual_seed(23)
    kv = torch.randn((4096, 576), generator=g).to(torch.bfloat16).to(dev)
    q = (torch.randn((3, 128, 576), generator=g) * q_std).to(torch.bfloat16).to(dev)
    idx = torch.stack([torch.randperm(4096, generator=g)[:1024] for _ in range(3)]).to(torch.int32)
    # put the weakest keys first so the reference of the fast pass starts low
    qn, kvn = q.float().cpu().numpy(), kv.float().cpu().numpy()
    for t in range(3):
        s = kvn[idx[t].numpy()] @ qn[t, 0]
        idx[t] = idx[t][torch.from_numpy(np.argsort(s).copy())]
    cfg = dict(q=q, kv_cache=kv, indices=idx.to(dev), block_table=None, page_size=64, sm_scale=1.0,
               kv_format="bf16")
    out, lse = _fwd(cfg, n_splits=n_splits)
    ro, rl = run_oracle(cfg)
    # |v| ~ N(0,1) here, so outputs reach ~4: half a bf16 ulp of the output alone is 1.6e-2 there;
    # the bar scales with the magnitude (1.2e-2 relative = bf16 rounding of out + of the probabilities)
    err = np.abs(to_np(out).astype(np.float64) - ro)
    assert np.all(err <= 1.2e-2 * np.maximum(1.0, np.abs(ro))), float(err.max())
    assert np.max(np.abs(to_np(lse) - rl) / np.maximum(1.0, np.abs(rl))) <= 1e-3


@pytest.mark.parametrize("n_splits", [1, 2])
def test_golden_fixture(dev, n_splits):
    """Committed vectors made from library routines only (tests/golden/make_golden.py)."""
    import os
    import flagtree_amd as ft
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "sparse_mla_small.npz"))
    q = torch.from_numpy(z["q_bf16_bits"].view(np.int16)).view(torch.bfloat16).to(dev)
    kv = torch.from_numpy(z["kv_bf16_bits"].view(np.int16)).view(torch.bfloat16).to(dev)
    out, lse = ft.sparse_mla_fwd(q.view(2, 1, 16, 576), kv.view(4, 16, 576), torch.from_numpy(z["indices"]).view(2, 1, 48).to(dev),
                                 float(z["sm_scale"]), 512, block_table=torch.from_numpy(z["block_table"]).to(dev),
                                 page_size=int(z["page_size"]), n_splits=n_splits)
    # inputs here are N(0, 0.5): outputs reach ~1, where half a bf16 ulp is 2e-3
    assert max_abs(to_np(out).reshape(2, 16, 512), z["out"]) <= OUT_TOL
    assert max_abs(to_np(lse).reshape(2, 16), z["lse"]) <= LSE_TOL
    so, sl = ft.sparse_mla_fwd_scalar(q.view(2, 1, 16, 576), kv.view(4, 16, 576), torch.from_numpy(z["indices"]).view(2, 1, 48).to(dev),
                                      float(z["sm_scale"]), 512, block_table=torch.from_numpy(z["block_table"]).to(dev),
                                      page_size=int(z["page_size"]))
    assert max_abs(to_np(so).reshape(2, 16, 512), z["out"]) <= 4e-3 and max_abs(to_np(sl).reshape(2, 16), z["lse"]) <= 1e-5


def test_properties_at_full_decode_size(dev):
    """B=64, h=128, topk=2048 over 65536-token paged contexts: size-independent properties.
    Appending padding, permuting the list and changing the split count must not change the result
    beyond rounding, and probabilities sum to one (a cache whose value columns are all 1 gives 1)."""
    import flagtree_amd as ft
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16(dev)
    out, lse = _fwd(cfg)
    assert out.shape == (64, 1, 128, 512) and torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    g = torch.Generator().manual_seed(5)
    idx = cfg["indices"]
    perm = torch.randperm(2048, generator=g).to(dev)
    cfg_p = dict(cfg, indices=idx[:, :, perm].contiguous())
    out_p, lse_p = _fwd(cfg_p, n_splits=3)
    assert (out.float() - out_p.float()).abs().max().item() <= 2e-3       # bf16 rounding of |out| <~ 0.1
    assert (lse - lse_p).abs().max().item() <= 1e-4
    pad = torch.full((64, 1, 100), -1, dtype=torch.int32, device=dev)
    out_q, lse_q = _fwd(dict(cfg, indices=torch.cat([pad, idx], dim=2).contiguous()), n_splits=1)
    assert (out.float() - out_q.float()).abs().max().item() <= 2e-3
    assert (lse - lse_q).abs().max().item() <= 1e-4
    ones = cfg["kv_cache"].clone()
    ones[..., :512] = 1.0
    out_1, _ = _fwd(dict(cfg, kv_cache=ones))
    assert (out_1.float() - 1.0).abs().max().item() <= 4e-3               # one bf16 ulp below 1


def test_properties_at_full_prefill_size(dev):
    """8192 causal query tokens, h=128, topk=2048: size-independent properties.  Token 0 sees only
    row 0 (its output is that row's value part, bit for bit); rewriting the rows of the second
    half of the sequence leaves the first half's results bit-identical (causality of the lists);
    a few tokens spread over the sequence agree with the oracle."""
    from flagtree_amd import workloads
    cfg = workloads.prefill_causal_bf16(dev)
    out, lse = _fwd(cfg)
    assert out.shape == (1, 8192, 128, 512) and torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    kv = cfg["kv_cache"]
    assert torch.equal(out[0, 0].view(torch.int16), kv[0, :512].view(torch.int16).expand(128, 512))
    kv2 = kv.clone()
    kv2[4096:] = kv2[4096:] * -2.0
    out2, lse2 = _fwd(dict(cfg, kv_cache=kv2))
    assert torch.equal(out[0, :4096].view(torch.int16), out2[0, :4096].view(torch.int16))
    assert torch.equal(lse[0, :4096], lse2[0, :4096])
    assert not torch.equal(out[0, 4097:].view(torch.int16), out2[0, 4097:].view(torch.int16))
    for t in (1, 31, 2047, 2048, 8191):
        sub = dict(cfg, q=cfg["q"][:, t:t + 1].contiguous(), indices=cfg["indices"][:, t:t + 1].contiguous())
        _check(sub, out[:, t:t + 1], lse[:, t:t + 1])


def test_properties_at_full_fp8_decode_size(dev):
    """B=128, h=16, topk=2048 over 131072-token paged fp8 contexts (11 GB of records): the MFMA and
    the scalar device kernels agree on a slice of the batch, and the split count does not matter."""
    import flagtree_amd as ft
    from flagtree_amd import workloads
    cfg = workloads.decode_fp8(dev)
    out, lse = _fwd(cfg)
    assert out.shape == (128, 1, 16, 512) and torch.isfinite(out.float()).all()
    out2, lse2 = _fwd(cfg, n_splits=1)
    assert (out.float() - out2.float()).abs().max().item() <= 2e-3 and (lse - lse2).abs().max().item() <= 1e-4
    sub = dict(cfg, q=cfg["q"][:8], indices=cfg["indices"][:8], block_table=cfg["block_table"][:8])
    so, sl = ft.sparse_mla_fwd_scalar(sub["q"], sub["kv_cache"], sub["indices"], sub["sm_scale"], 512,
                                      block_table=sub["block_table"], page_size=64)
    assert (out[:8].float() - so.float()).abs().max().item() <= OUT_TOL
    assert (lse[:8] - sl).abs().max().item() <= LSE_TOL
    _check(dict(sub, q=sub["q"][:2], indices=sub["indices"][:2], block_table=sub["block_table"][:2]), out[:2], lse[:2])
