"""Seeded random cases through the emulator build of the kernels, every buffer between inaccessible
pages (test infrastructure; run by tests/test_emu_fuzz.py in a process of its own, because a stray
access ends the process):

    python tests/emu/fuzz_cases.py forward LO HI     sparse / dense attention, all kernels and switches
    python tests/emu/fuzz_cases.py other LO HI       index producer, local GEMM, cache writer, gather

Each seed draws a shape, a cache format, the kernel switches, where the buffers sit against their
guard pages and how the emulator schedules wavefronts and workgroups; the result is held against
the numpy oracle (attention: out 3e-3, LSE 1e-4; integer and byte paths: exact).  Prints one line
per case and "done, failures: N" at the end; the exit status is 1 when N > 0."""
import os
import sys
import traceback

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [os.path.dirname(os.path.dirname(HERE)), os.path.dirname(HERE), HERE]

import numpy as np      # noqa: E402
import torch            # noqa: E402

import harness          # noqa: E402
import oracle           # noqa: E402
from _util import max_abs, oracle_inputs, to_np   # noqa: E402

G = harness.Guarded
SWITCHES = ("FLAGTREE_SMLA_FEW_FP8", "FLAGTREE_SMLA_FP8_MFMA", "FLAGTREE_SMLA_HEAD_GROUPS", "FLAGTREE_SMLA_TOKEN_BANDS",
            "FLAGTREE_SMLA_SEPARATE_MERGE", "FLAGTREE_SMLA_PERSIST")


def random_schedule(rng):
    harness.configure(dma_eager=bool(rng.random() < 0.5), block_order_seed=int(rng.integers(0, 3)),
                      wave_skew_seed=int(rng.integers(0, 2000)) if rng.random() < 0.8 else 0,
                      concurrent_blocks=int(rng.choice([0, 0, 3, 8, 20])), concurrent_seed=int(rng.integers(0, 1000)))


def forward_case(seed):
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    heads = int(rng.choice([1, 2, 7, 15, 16, 17, 31, 32, 33, 47, 48, 63, 64, 65, 80, 96, 97, 127, 128, 129, 160, 192, 200]))
    topk = int(rng.choice([1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 257, 512, 1023, 1024, 1025, 1100]))
    page_size = int(rng.choice([1, 2, 16, 64, 128]))
    tps, batch = int(rng.choice([1, 2, 3])), int(rng.choice([1, 2, 3]))
    while batch * tps > 1 and batch * tps * max(heads, 64) * topk > 100_000:      # keeps a case to a few seconds of emulation
        if tps > 1:
            tps -= 1
        else:
            batch -= 1
    fmt = "fp8_e4m3_b128" if rng.random() < 0.5 else "bf16"
    ns = min(int(rng.choice([1, 2, 3, 4, 5, 8])), max(1, topk // 32))
    paged = rng.random() < 0.7
    ctx = int(rng.choice([1, 33, 64, 300, 1200]))
    dense = rng.random() < 0.2 and paged
    for k in SWITCHES:
        os.environ.pop(k, None)
    if rng.random() < 0.5:                                  # the opt-in kernels (each applies to its own head counts)
        os.environ["FLAGTREE_SMLA_FP8_MFMA" if rng.random() < 0.5 else "FLAGTREE_SMLA_FEW_FP8"] = "1"
        os.environ["FLAGTREE_SMLA_HEAD_GROUPS"] = "1"
    if rng.random() < 0.5:
        os.environ["FLAGTREE_SMLA_TOKEN_BANDS"] = "1"
    if rng.random() < 0.25:
        os.environ["FLAGTREE_SMLA_SEPARATE_MERGE"] = "1"
    if rng.random() < 0.5:
        os.environ["FLAGTREE_SMLA_PERSIST"] = "1"           # (takes effect on unsplit many-heads launches with enough items)
    cap = float(rng.choice([0.0, 0.0, 0.05])) if dense else 0.0
    if paged:
        pps = -(-ctx // page_size)
        n_pages = batch * pps + 3
        lat = (torch.randn((n_pages * page_size, 576), generator=g) * 0.1).to(torch.bfloat16)
        bt = torch.randperm(n_pages, generator=g)[:batch * pps].to(torch.int32).view(batch, pps)
        if pps > 2 and rng.random() < 0.5:
            bt[0, 1] = -1                                   # a hole in the page table
        hi = pps * page_size + (3 if rng.random() < 0.3 else 0)
    else:
        lat = (torch.randn((batch * ctx + 128, 576), generator=g) * 0.1).to(torch.bfloat16)
        bt = None
        hi = lat.shape[0] + (2 if rng.random() < 0.3 else 0)
    T = batch * tps
    idx = torch.from_numpy(rng.integers(0, hi, size=(T, topk)).astype(np.int32))
    idx[torch.from_numpy(rng.random((T, topk)) < float(rng.choice([0.0, 0.1, 0.6])))] = -1
    if rng.random() < 0.3:
        idx[0, topk // 2:] = -1
    if T > 1 and rng.random() < 0.3:
        idx[1, :] = -1                                      # a token without a valid entry
    q = (torch.randn((batch, tps, heads, 576), generator=g) * 0.1).to(torch.bfloat16)
    if fmt == "bf16":
        kv = lat
    else:
        kv = torch.zeros((lat.shape[0], 656), dtype=torch.uint8)
        assert harness.lib().smla_kv_quantize_fp8(lat.data_ptr(), None, kv.data_ptr(), lat.shape[0], lat.shape[0], None) == 0
    if paged:
        kv = kv.view(-1, page_size, kv.shape[-1])
    end = bool(rng.random() < 0.5)                          # buffers end right before / start right after the guard page
    cfg = dict(q=G(q, end).tensor, kv_cache=G(kv, end).tensor, indices=G(idx.view(batch, tps, topk), end).tensor,
               block_table=G(bt, end).tensor if bt is not None else None, page_size=page_size, sm_scale=576 ** -0.5, kv_format=fmt)
    lens, ref_cfg = None, cfg
    if dense:
        lens_t = torch.from_numpy(rng.integers(0, pps * page_size + 1, size=(batch,)).astype(np.int32))
        lens = G(lens_t, end).tensor
        didx = torch.arange(pps * page_size, dtype=torch.int32).repeat(batch, 1)
        didx[didx >= lens_t[:, None]] = -1
        ref_cfg = dict(cfg, indices=didx.view(batch, 1, -1).repeat(1, tps, 1))
    wsb = harness.lib().smla_workspace_bytes(T, heads, 512, ns)
    ws = G(harness.make_workspace(wsb), end).tensor if wsb else None
    random_schedule(rng)
    print(f"seed {seed}: H={heads} K={topk} P={page_size} tps={tps} B={batch} {fmt} ns={ns} paged={paged} ctx={ctx} dense={dense} "
          f"cap={cap} switches={[k[14:] for k in SWITCHES if k in os.environ]}", flush=True)
    out, lse, rc = harness.forward(cfg, n_splits=ns, workspace=ws, dense_lens=lens, logit_cap=cap, guard_outputs=end)
    assert rc == 0, rc
    if ws is not None:
        assert harness.workspace_status(ws) == (0, 0)
    qn, kv_small, phys_small, _ = oracle_inputs(ref_cfg)
    ro, rl = oracle.sparse_mla_fwd(qn, kv_small, phys_small, cfg["sm_scale"], 512, logit_cap=cap)
    eo, el = max_abs(to_np(out), ro), max_abs(to_np(lse), rl)
    assert eo <= 3e-3 and el <= 1e-4, f"out {eo} lse {el}"


def topk_case(seed, rng, g, end):
    lib = harness.lib()
    rows = int(rng.choice([1, 2, 5]))
    n = int(rng.choice([1, 17, 255, 256, 1023, 1024, 1025, 4096, 4099, 16384, 20000, 65536, 70001]))
    k = int(rng.choice([1, 2, 64, 300, 2048]))
    stride = n + int(rng.choice([0, 0, 3, 8]))
    buf = torch.randn((rows, stride), generator=g)
    if rng.random() < 0.5:
        buf = (buf * 4).round() / 4                         # many ties
    if rng.random() < 0.3:
        buf[0, : n // 2] = float("-inf")
    if rng.random() < 0.3:
        buf[-1, n // 3] = float("nan")
    sc = G(buf, end).tensor
    lens_t = torch.from_numpy(rng.integers(0, n + 1, size=(rows,)).astype(np.int32))
    lens = G(lens_t, end).tensor if rng.random() < 0.7 else None
    out = G(torch.full((rows, k), -9, dtype=torch.int32), end).tensor
    print(f"seed {seed} topk rows={rows} n={n} k={k} stride={stride} lens={lens is not None}", flush=True)
    random_schedule(rng)
    need = lib.smla_topk_workspace_bytes(rows, n, k)
    ws = G(torch.full((need,), 0x5A, dtype=torch.uint8), end).tensor if need and rng.random() < 0.7 else None      # rows cut into parts
    rc = lib.smla_topk_indices(sc.data_ptr(), lens.data_ptr() if lens is not None else None, out.data_ptr(), rows, n, stride, k,
                               ws.data_ptr() if ws is not None else None, need if ws is not None else 0, None)
    assert rc == 0, rc
    want = oracle.topk_indices(to_np(buf)[:, :n], k, to_np(lens_t) if lens is not None else None)
    assert np.array_equal(to_np(out), want)


def gemm_case(seed, rng, g, end):
    lib = harness.lib()
    m = int(rng.choice([128, 256, 384, 512, 2048]))
    n = int(rng.choice([256, 512, 768, 1280]))
    k = int(rng.choice([64, 128, 192]))
    chunks = int(rng.choice([c for c in (1, 2, 4, 8) if m % c == 0]))
    extra = int(rng.choice([0, 8, 64]))
    stride = (m // chunks) * n + extra
    x = G((torch.randn((m, k), generator=g) * 0.1).to(torch.bfloat16), end).tensor
    w = G((torch.randn((k, n), generator=g) * 0.1).to(torch.bfloat16), end).tensor
    use_p = rng.random() < 0.8
    pt = torch.randn((m, n), generator=g)
    part = G(pt, end).tensor if use_p else None
    out = G(torch.full((chunks * stride,), float("nan"), dtype=torch.bfloat16), end).tensor
    cus = int(rng.choice([16, 16, 20, 256]))                # 20: no multiple of 8, so no half tiles
    os.environ.pop("FLAGTREE_SMLA_GEMM_CHAIN", None)
    if rng.random() < 0.5:
        os.environ["FLAGTREE_SMLA_GEMM_CHAIN"] = "1"        # persistent workgroups (where the shape has more tiles than units)
    print(f"seed {seed} gemm m={m} n={n} k={k} chunks={chunks} stride_extra={extra} partial={use_p} cus={cus} "
          f"chain={'FLAGTREE_SMLA_GEMM_CHAIN' in os.environ}", flush=True)
    random_schedule(rng)
    try:
        lib.emu_set_cu_count(cus)
        rc = lib.smla_gemm_rs_local(x.data_ptr(), w.data_ptr(), part.data_ptr() if use_p else None, out.data_ptr(), m, n, k, chunks, stride, None)
    finally:
        lib.emu_set_cu_count(harness.EMU_CUS)
    assert rc == 0, rc
    want = oracle.gemm_rs_local(to_np(x), to_np(w), to_np(pt) if use_p else np.zeros((m, n), np.float32), n_chunks=chunks)
    got = to_np(out).reshape(chunks, stride)[:, :(m // chunks) * n].reshape(chunks, m // chunks, n)
    e = max_abs(got, want)
    assert e <= 1e-2 + 1e-2 * float(np.abs(want).max()), e
    assert not extra or np.isnan(to_np(out).reshape(chunks, stride)[:, (m // chunks) * n:]).all(), "wrote into the gap between chunks"


def kv_write_case(seed, rng, g, end):
    lib = harness.lib()
    ntok = int(rng.choice([1, 3, 4, 5, 63, 64, 65, 300]))
    rows = int(rng.choice([1, 7, 64, 257]))
    lat_t = (torch.randn((ntok, 576), generator=g) * float(rng.choice([1e-3, 0.1, 30.0]))).to(torch.bfloat16)
    if rng.random() < 0.3:
        lat_t[0, :200] = 0
    lat = G(lat_t, end).tensor
    slots_t = torch.from_numpy(rng.integers(-3, rows + 3, size=(ntok,)).astype(np.int64))
    seen = set()            # two tokens with the same slot race, as in the reference: valid slots stay distinct
    for i in range(ntok):
        v = int(slots_t[i])
        if 0 <= v < rows and v in seen:
            slots_t[i] = -1
        seen.add(v)
    slots = G(slots_t, end).tensor
    code, width, dt = ((1, 656, torch.uint8), (0, 576, torch.bfloat16))[int(rng.integers(2))]
    cache = G(torch.zeros((rows, width), dtype=dt), end).tensor
    print(f"seed {seed} kv_write ntok={ntok} rows={rows} fmt={code}", flush=True)
    random_schedule(rng)
    rc = lib.smla_kv_write(code, lat.data_ptr(), slots.data_ptr(), cache.data_ptr(), ntok, rows, None)
    assert rc == 0, rc
    want = np.zeros((rows, width), dtype=np.uint8 if code == 1 else np.uint16)
    want = oracle.reshape_and_cache(to_np(lat_t), want, slots_t.numpy(), kv_format="fp8_e4m3_b128" if code == 1 else "bf16")
    got = cache.numpy() if code == 1 else cache.view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)


def gather_case(seed, rng, g, end):
    lib = harness.lib()
    T, K = int(rng.choice([1, 3])), int(rng.choice([1, 5, 64, 130]))
    rows, rb = int(rng.choice([8, 100])), int(rng.choice([16, 656, 1152]))
    kv_t = torch.randint(0, 256, (rows, rb), generator=g, dtype=torch.uint8)
    idx_t = torch.from_numpy(rng.integers(-2, rows + 2, size=(T, K)).astype(np.int32))
    kv, idx = G(kv_t, end).tensor, G(idx_t, end).tensor
    phys = G(torch.zeros((T, K), dtype=torch.int32), end).tensor
    ro = G(torch.zeros((T, K, rb), dtype=torch.uint8), end).tensor
    print(f"seed {seed} gather T={T} K={K} rows={rows} row_bytes={rb}", flush=True)
    random_schedule(rng)
    rc = lib.smla_gather_rows(kv.data_ptr(), rb, idx.data_ptr(), None, phys.data_ptr(), ro.data_ptr(), T, 1, K, 64, 0, 0, rows, None)
    assert rc == 0, rc
    want = oracle.translate_indices(to_np(idx_t), None, 64, kv_rows=rows)
    assert np.array_equal(to_np(phys), want) and np.array_equal(to_np(ro), oracle.gather_rows(to_np(kv_t), want))


def other_case(seed):
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    end = bool(rng.random() < 0.5)
    (topk_case, gemm_case, kv_write_case, gather_case)[seed % 4](seed, rng, g, end)


def main(argv):
    kind, lo, hi = argv[1], int(argv[2]), int(argv[3])
    case = {"forward": forward_case, "other": other_case}[kind]
    bad = 0
    for seed in range(lo, hi):
        try:
            case(seed)
        except Exception as e:
            bad += 1
            print(f"  FAILED seed {seed}: {e!r}", flush=True)
            traceback.print_exc()
    print("done, failures:", bad)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
