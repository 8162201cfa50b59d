#!/usr/bin/env python3
"""Benchmark of the sparse-MLA forward hot path on one MI355X.

A step is one `sparse_mla_fwd` call over the decode workload BASELINE.json quotes its metric
on: batch 64, one query token per sequence, 128 heads, top-k 2048 (5 % padding), 65 536-token
paged bf16 contexts, inputs resident in HBM.  Consecutive steps rotate over several
independent (q, indices) sets so the selected rows of one step are not cache-resident from
the previous one (the selected rows of a single set would fit the 256 MB Infinity Cache).

Prints ONE JSON line: throughput in TFLOP/s (algorithmic flops = 2 * n_valid * H * (576+512)),
plus `roofline` for the dominant kernel (HIP-event time of the single forward launch) and
`cpu_baseline` (the numpy oracle timed on a bounded sample of the same workload).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E
TRAFFIC_NOTE = ("replayed from profiles/hbm_traffic.json (separate rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of the "
                "same command, see profiles/*.md for the build they were taken on); not counted in this run")
TIMING_NOTE = ("value and ms_per_step: wall clock over the timed steps, Python launch overhead included; "
               "roofline.achieved and kernel_ms: one HIP event pair on the launch stream around the same steps; "
               "steps rotate over independent input sets instead of flushing the caches between launches")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="decode_bf16",
                    choices=["decode_bf16", "decode_fp8", "decode_fp8_h128", "prefill_causal_bf16", "gemm_rs_shard", "kv_write_fp8", "kv_write_bf16", "topk_decode", "topk_prefill", "decode_dense_bf16"])
    ap.add_argument("--sets", type=int, default=8, help="independent (q, indices) sets rotated over steps")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--n-splits", type=int, default=0, help="override the split count (0 = library's choice)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run three plain 1 GiB device copies (known HBM traffic) so a rocprofv3 --pmc "
                         "run of this command holds a reference kernel to scale FETCH_SIZE / WRITE_SIZE by")
    ap.add_argument("--cpu-sample", type=int, default=0, help="sequences in the CPU sample (0 = auto)")
    ap.add_argument("--head-groups", action="store_true",
                    help="many-heads workloads on the 128-heads-per-workgroup kernel, a wavefront per 32 heads (sets "
                         "FLAGTREE_SMLA_HEAD_GROUPS=1; opt-in until measured)")
    ap.add_argument("--few-fp8", action="store_true",
                    help="decode_fp8 on the two-workgroups-per-CU kernel (sets FLAGTREE_SMLA_FEW_FP8=1; opt-in until measured)")
    ap.add_argument("--fp8-mfma", action="store_true",
                    help="decode_fp8 on the kernel that contracts the records' e4m3 codes with fp8 MFMAs (sets "
                         "FLAGTREE_SMLA_FP8_MFMA=1; opt-in until measured)")
    ap.add_argument("--persist", action="store_true",
                    help="unsplit many-heads launches (prefill_causal_bf16, decode_dense_bf16) by one persistent workgroup per "
                         "compute unit (sets FLAGTREE_SMLA_PERSIST=1; opt-in until measured)")
    ap.add_argument("--topk-one-workgroup", action="store_true",
                    help="topk_* workloads: one workgroup per row even where the rows would be cut into parts")
    ap.add_argument("--token-bands", action="store_true",
                    help="each XCD takes a contiguous band of tokens instead of every eighth one (sets "
                         "FLAGTREE_SMLA_TOKEN_BANDS=1; for prefill_causal_bf16; opt-in until measured)")
    return ap.parse_args()


def cpu_threads():
    """Threads the CPU baseline really runs on: those of the BLAS pool numpy's matrix products use
    (the environment caps it below what os.cpu_count() shows on a shared box)."""
    try:
        import numpy  # noqa: F401  (loads the BLAS library the pool belongs to)
        from threadpoolctl import threadpool_info
        n = max((p.get("num_threads", 0) for p in threadpool_info() if p.get("user_api") == "blas"), default=0)
        if n:
            return int(n)
    except Exception:
        pass
    return int(os.environ.get("OMP_NUM_THREADS") or os.cpu_count())


def many_heads_kernel(a, fmt):
    """Name of the kernel a launch with more than 32 heads goes to under this run's switches."""
    return "fwd_group_kernel" if a.head_groups else "fwd_tall_kernel"


def measured_traffic(workload):
    """HBM bytes per launch of the workload's kernel as counted by rocprofv3 (FETCH_SIZE and
    WRITE_SIZE, each scaled by what the same counter reads for a plain copy of known size);
    the counter runs are separate commands, their result is kept in profiles/hbm_traffic.json."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            return float(json.load(f)[workload]["hbm_bytes_per_launch"])
    except (OSError, KeyError, ValueError, TypeError):
        return None


def _time_oracle(qn, kv_small, phys_small, sm_scale):
    """Median time of the numpy oracle (fp32, BLAS threads = host cores) on the given sample: at
    least 3 runs, then more until about 10 s of CPU time are spent.  Returns (TFLOP/s, runs)."""
    import numpy as np
    import oracle
    n_valid = int((phys_small >= 0).sum())
    flops = 2.0 * n_valid * qn.shape[1] * (576 + 512)
    oracle.sparse_mla_fwd(qn[:1], kv_small, phys_small[:1], sm_scale, 512, dtype=np.float32)
    reps, t_used, times = 0, 0.0, []
    while reps < 3 or (t_used < 10.0 and reps < 50):
        t0 = time.perf_counter()
        oracle.sparse_mla_fwd(qn, kv_small, phys_small, sm_scale, 512, dtype=np.float32)
        dt = time.perf_counter() - t0
        times.append(dt)
        t_used += dt
        reps += 1
    times.sort()
    return flops / times[len(times) // 2] / 1e12, reps


def cpu_baseline(cfg, n_seq):
    """The oracle on the first n_seq sequences of a decode workload."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from _util import oracle_inputs
    sub = dict(cfg)
    sub["q"], sub["indices"] = cfg["q"][:n_seq], cfg["indices"][:n_seq]
    if cfg["block_table"] is not None:
        sub["block_table"] = cfg["block_table"][:n_seq]
    qn, kv_small, phys_small, _ = oracle_inputs(sub)
    return _time_oracle(qn, kv_small, phys_small, cfg["sm_scale"])


def cpu_baseline_prefill(cfg, n_rows=256):
    """The oracle on every (tokens / n_rows)-th query token of the causal prefill (a stratified
    sample: short and long index lists in the workload's own proportion)."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from _util import oracle_inputs
    T = cfg["q"].shape[1]
    pick = list(range(T // n_rows - 1, T, T // n_rows))
    sub = dict(cfg)
    sub["q"] = cfg["q"][0, pick]                                   # [n_rows, H, 576]
    sub["indices"] = cfg["indices"][0, pick]
    qn, kv_small, phys_small, _ = oracle_inputs(sub)
    return _time_oracle(qn, kv_small, phys_small, cfg["sm_scale"]) + (len(pick),)


def main():
    a = parse()
    if a.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {a.gpus} is not supported in this build "
              "(no collective path exists: work units are independent per token).", file=sys.stderr)
        sys.exit(2)
    if a.few_fp8:
        os.environ["FLAGTREE_SMLA_FEW_FP8"] = "1"
    if a.fp8_mfma:
        os.environ["FLAGTREE_SMLA_FP8_MFMA"] = "1"
    if a.persist:
        os.environ["FLAGTREE_SMLA_PERSIST"] = "1"
    if a.head_groups:
        os.environ["FLAGTREE_SMLA_HEAD_GROUPS"] = "1"
    if a.token_bands:
        os.environ["FLAGTREE_SMLA_TOKEN_BANDS"] = "1"
    import torch
    import flagtree_amd as ft
    from flagtree_amd import workloads

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if a.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if a.workload == "gemm_rs_shard":
        return bench_gemm(a, torch, ft, workloads, dev)
    if a.workload.startswith("kv_write_"):
        return bench_kv_write(a, torch, ft, dev)
    if a.workload.startswith("topk_"):
        return bench_topk(a, torch, ft, dev)
    if a.workload == "decode_dense_bf16":
        return bench_dense(a, torch, ft, workloads, dev)

    make = getattr(workloads, a.workload)
    cfg = make(dev)
    fmt = cfg["kv_format"]
    flops, nbytes, n_valid = workloads.attention_work(cfg)
    sets = [cfg]
    for i in range(1, max(1, a.sets)):
        if a.workload == "prefill_causal_bf16":
            break
        g = torch.Generator().manual_seed(5000 + i)
        B, _, K = cfg["indices"].shape
        H = cfg["q"].shape[2]
        pad = int((cfg["indices"][0, 0] < 0).sum().item())
        idx = workloads._topk_indices(B, cfg["block_table"].shape[1] * cfg["page_size"], K, pad, g, True)
        gd = torch.Generator(device=dev).manual_seed(5000 + i)
        q = (torch.randn(cfg["q"].shape, generator=gd, device=dev) * 0.1).to(torch.bfloat16)
        s = dict(cfg)
        s["q"], s["indices"] = q, idx.view(B, 1, K).to(dev)
        sets.append(s)

    # the same index sets with their padding moved to the end of every list (the benchmark
    # shuffles padding through the list; both orders are reported for the bf16 decode)
    tail_sets = []
    if a.workload == "decode_bf16":
        for c in sets:
            idx = c["indices"]
            order = torch.argsort((idx < 0).to(torch.int8), dim=-1, stable=True)
            t = dict(c)
            t["indices"] = torch.gather(idx, -1, order).contiguous()
            tail_sets.append(t)

    T = cfg["q"].shape[0] * cfg["q"].shape[1]
    H = cfg["q"].shape[2]
    K = cfg["indices"].shape[-1]
    n_splits = a.n_splits or ft.plan_splits(T, H, K, fmt)
    lib = ft._lib.load()
    ws_bytes = lib.smla_workspace_bytes(T, H, 512, n_splits)
    ws = ft.make_workspace(ws_bytes, dev) if ws_bytes else None

    def step(i, which=None):
        which = which or sets
        c = which[i % len(which)]
        return ft.sparse_mla_fwd(c["q"], c["kv_cache"], c["indices"], c["sm_scale"], 512,
                                 block_table=c["block_table"], page_size=c["page_size"], kv_format=fmt,
                                 n_splits=n_splits, workspace=ws)

    def run_timed():
        for i in range(a.warmup):
            step(i)
        torch.cuda.synchronize()
        # The forward is a single kernel launch (the split merge happens inside it; on a device whose
        # XCD layout the library does not know, a merge launch follows it), issued on torch's current
        # stream.  One HIP event pair on that stream brackets the K launches: the
        # span divided by K is the average launch duration including the gap between back-to-back
        # launches; a second pass with one event pair per launch gives the per-launch distribution.
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for i in range(a.steps):
            step(i)
        e1.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ms_per_step = wall * 1e3 / a.steps
        kern_ms = e0.elapsed_time(e1) / a.steps
        n_dist = min(a.steps, 50)
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_dist)]
        for i in range(n_dist):
            ev[i][0].record()
            step(i)
            ev[i][1].record()
        torch.cuda.synchronize()
        op_ms = sorted(x.elapsed_time(y) for x, y in ev)
        op_ms_avg = sum(op_ms) / len(op_ms)
        tail_ms = None
        if tail_sets:
            for i in range(min(a.warmup, 10)):
                step(i, tail_sets)
            torch.cuda.synchronize()
            f0, f1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            f0.record()
            for i in range(a.steps):
                step(i, tail_sets)
            f1.record()
            torch.cuda.synchronize()
            tail_ms = f0.elapsed_time(f1) / a.steps
        # A split merge that gave up marks its rows with a NaN LSE and flags the workspace, and every
        # later launch on that workspace gives up too: no figure is printed for such a run.
        if ws is not None:
            ft.workspace_status(ws)                       # raises when any launch above flagged it
        last_lse = step(0)[1]
        torch.cuda.synchronize()
        if not bool(torch.isfinite(last_lse).all().item()):
            raise RuntimeError("non-finite LSE after the timed loop: the run measured a launch that did not compute")
        if ws is not None:
            ft.workspace_status(ws)

        return ms_per_step, kern_ms, op_ms, op_ms_avg, tail_ms

    # A merge inside the launch that gives up (a workspace flagged, NaN rows) means this device does
    # not do what the in-launch merge relies on.  The run is then repeated once with the merge as a
    # second launch, which relies on nothing but the kernel boundary, and the line says so.
    merge_note = None
    try:
        ms_per_step, kern_ms, op_ms, op_ms_avg, tail_ms = run_timed()
    except RuntimeError as e:
        if ws is None or os.environ.get("FLAGTREE_SMLA_SEPARATE_MERGE") == "1":
            raise
        merge_note = f"second launch (the merge inside the launch failed on this device: {e})"
        print("bench.py: " + merge_note, file=sys.stderr)
        os.environ["FLAGTREE_SMLA_SEPARATE_MERGE"] = "1"
        ws = ft.make_workspace(ws_bytes, dev)
        ms_per_step, kern_ms, op_ms, op_ms_avg, tail_ms = run_timed()

    tflops = flops / (ms_per_step * 1e-3) / 1e12
    gbs = nbytes / (ms_per_step * 1e-3) / 1e9
    # the few-heads fp8 decode is priced against HBM; with 128 heads the same records feed 8 x the
    # matrix work and the MFMA floor (13.9 us) lies above the HBM floor (12.5 us)
    hbm_bound = fmt == "fp8_e4m3_b128" and H <= 32
    if hbm_bound:
        roof = dict(bound="hbm", achieved=nbytes / (kern_ms * 1e-3) / 1e9, peak=PEAK_HBM_GBS, unit="GB/s")
    else:
        roof = dict(bound="mfma", achieved=flops / (kern_ms * 1e-3) / 1e12, peak=PEAK_BF16_TFLOPS, unit="TFLOP/s")
    roof["frac"] = roof["achieved"] / roof["peak"]
    # (the stored counter figures were taken on the default kernels: none for a kernel behind a switch)
    roof["traffic"] = None if (a.head_groups or a.few_fp8 or a.fp8_mfma or a.token_bands or a.persist) else measured_traffic(a.workload)
    roof["traffic_source"] = TRAFFIC_NOTE
    roof["kernel"] = many_heads_kernel(a, fmt) if H > 32 else ("fwd_few_f8_kernel" if a.fp8_mfma and hbm_bound else "fwd_few_fp8_kernel" if a.few_fp8 and hbm_bound else "fwd_short_kernel")
    roof["kernel_ms"] = kern_ms
    roof["other_bound"] = (dict(bound="hbm", achieved=nbytes / (kern_ms * 1e-3) / 1e9, peak=PEAK_HBM_GBS, unit="GB/s")
                           if not hbm_bound else
                           dict(bound="mfma", achieved=flops / (kern_ms * 1e-3) / 1e12, peak=PEAK_BF16_TFLOPS, unit="TFLOP/s"))
    roof["other_bound"]["frac"] = roof["other_bound"]["achieved"] / roof["other_bound"]["peak"]

    res = {
        # BASELINE.json's metric is quoted on the bf16 decode configuration; the other workloads of
        # the same operator say which configuration their figure is for
        "metric": "sparse-MLA fwd TFLOP/s + HBM GB/s (% roofline), " + {
            "decode_bf16": "decode B=64 h=128 topk=2048",
            "decode_fp8": "decode B=128 h=16 topk=2048, fp8 KV",
            "decode_fp8_h128": "decode B=64 h=128 topk=2048, fp8 KV",
            "prefill_causal_bf16": "causal prefill S=8192 h=128 topk=2048"}[a.workload],
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3" if (a.fp8_mfma and hbm_bound) else "bf16", "data": "synthetic",
        "config": {"workload": a.workload, "batch": cfg["q"].shape[0], "heads": H, "topk": K,
                   "n_valid": n_valid, "kv_format": fmt, "page_size": cfg["page_size"],
                   "n_splits": n_splits, "input_sets": len(sets), "token_bands": bool(a.token_bands),
                   "flops_per_step": flops, "bytes_per_step": nbytes},
        "hbm_gbs": gbs, "pct_mfma_peak": 100.0 * tflops / PEAK_BF16_TFLOPS,
        "pct_hbm_peak": 100.0 * gbs / PEAK_HBM_GBS,
        "event_ms_per_launch": {"avg": op_ms_avg, "p50": op_ms[len(op_ms) // 2], "p20": op_ms[len(op_ms) // 5],
                              "p80": op_ms[(4 * len(op_ms)) // 5]},
        "roofline": roof,
        "timing": TIMING_NOTE,
    }
    res["config"]["split_merge"] = ("none" if n_splits == 1 else merge_note if merge_note else
                                    "inside the launch" if lib.smla_merge_in_launch() else "second launch")
    if tail_ms is not None:
        res["padding_order"] = {"shuffled_kernel_ms": kern_ms, "tail_kernel_ms": tail_ms,
                                "note": "same index sets, -1 entries spread through the list (the headline) / moved to its end"}
    if not a.no_cpu_baseline and a.workload == "prefill_causal_bf16":
        try:
            v, reps, n_rows = cpu_baseline_prefill(cfg)
            res["cpu_baseline"] = {"value": v, "unit": "TFLOP/s", "cores": cpu_threads(), "kind": "port",
                                   "sample": f"numpy fp32 oracle on a stratified sample of {n_rows} of the {cfg['q'].shape[1]} query "
                                             f"tokens (every {cfg['q'].shape[1] // n_rows}th), median of {reps} runs; a rate, not extrapolated"}
        except Exception as e:
            res["cpu_baseline"] = {"value": None, "unit": "TFLOP/s", "cores": cpu_threads(), "kind": "port",
                                   "sample": f"failed: {e}"}
    if not a.no_cpu_baseline and a.workload != "prefill_causal_bf16":
        n_seq = a.cpu_sample or min(cfg["q"].shape[0], 8)
        try:
            import numpy  # noqa: F401
            v, reps = cpu_baseline(cfg, n_seq)
            res["cpu_baseline"] = {"value": v, "unit": "TFLOP/s", "cores": cpu_threads(), "kind": "port",
                                   "sample": f"numpy fp32 oracle on the first {n_seq} of {cfg['q'].shape[0]} sequences "
                                             f"of the same workload, median of {reps} runs"}
        except Exception as e:   # the baseline is a reported extra; never lose the GPU number over it
            res["cpu_baseline"] = {"value": None, "unit": "TFLOP/s", "cores": cpu_threads(), "kind": "port",
                                   "sample": f"failed: {e}"}
    print(json.dumps(res))


def bench_gemm(a, torch, ft, workloads, dev):
    cfg = workloads.gemm_rs_shard(dev)
    M, Kd = cfg["x"].shape
    N = cfg["w"].shape[1]
    flops = 2.0 * M * N * Kd
    out = torch.empty((cfg["n_chunks"], M // cfg["n_chunks"], N), dtype=torch.bfloat16, device=dev)
    for _ in range(a.warmup):
        ft.gemm_rs_local(cfg["x"], cfg["w"], cfg["partial"], cfg["n_chunks"], out=out)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(a.steps):
        ft.gemm_rs_local(cfg["x"], cfg["w"], cfg["partial"], cfg["n_chunks"], out=out)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = wall * 1e3 / a.steps
    kern_ms = e0.elapsed_time(e1) / a.steps
    tf = flops / (ms * 1e-3) / 1e12
    ach = flops / (kern_ms * 1e-3) / 1e12
    res = {
        "metric": "local GEMM of GEMM+reduce-scatter TFLOP/s", "value": tf, "unit": "TFLOP/s", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "gemm_rs_shard", "m": M, "n": N, "k": Kd, "n_chunks": cfg["n_chunks"]},
        "roofline": {"bound": "mfma", "achieved": ach, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": ach / PEAK_BF16_TFLOPS, "traffic": measured_traffic("gemm_rs_shard"),
                     "traffic_source": TRAFFIC_NOTE, "kernel": "gemm_rs_big_kernel",
                     "kernel_ms": kern_ms}}
    if not a.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        import oracle
        rows = 2048                                          # two of the eight output chunks
        xs = cfg["x"][:rows].float().cpu().numpy()
        ws = cfg["w"].float().cpu().numpy()
        ps = cfg["partial"][:rows].cpu().numpy()
        t0 = time.perf_counter()
        oracle.gemm_rs_local(xs, ws, ps, n_chunks=2)
        dt = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": 2.0 * rows * N * Kd / dt / 1e12, "unit": "TFLOP/s", "cores": cpu_threads(), "kind": "port",
                               "sample": f"numpy oracle (float64, BLAS threads) on the first {rows} of the {M} rows"}
    print(json.dumps(res))


def bench_kv_write(a, torch, ft, dev):
    """KV-cache writer: 131 072 latent rows scattered into a paged pool of twice as many rows."""
    fmt = "fp8_e4m3_b128" if a.workload == "kv_write_fp8" else "bf16"
    n, pool_rows = 131072, 262144
    g = torch.Generator(device=dev).manual_seed(77)
    lat = (torch.randn((n, 576), generator=g, device=dev) * 0.1).to(torch.bfloat16)
    slots = torch.randperm(pool_rows, generator=g, device=dev)[:n].contiguous()
    if fmt == "bf16":
        pool = torch.zeros((pool_rows // 64, 64, 576), dtype=torch.bfloat16, device=dev)
        row_out = 1152
    else:
        pool = torch.zeros((pool_rows // 64, 64, 656), dtype=torch.uint8, device=dev)
        row_out = 656
    nbytes = n * (1152 + row_out + 8)                   # latent row in, cache row out, slot
    for _ in range(a.warmup):
        ft.reshape_and_cache(lat, pool, slots, fmt)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(a.steps):
        ft.reshape_and_cache(lat, pool, slots, fmt)
    e1.record()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / a.steps
    kern_ms = e0.elapsed_time(e1) / a.steps
    ach = nbytes / (kern_ms * 1e-3) / 1e9
    res = {
        "metric": "KV-cache writer GB/s", "value": nbytes / (ms * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8" if fmt != "bf16" else "bf16", "data": "synthetic",
        "config": {"workload": a.workload, "rows": n, "pool_rows": pool_rows, "kv_format": fmt, "bytes_per_step": nbytes},
        "roofline": {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": ach / PEAK_HBM_GBS,
                     "traffic": measured_traffic(a.workload), "traffic_source": TRAFFIC_NOTE,
                     "kernel": "quantize_kernel" if fmt != "bf16" else "kv_copy_kernel", "kernel_ms": kern_ms}}
    if not a.no_cpu_baseline:
        import numpy as np
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        import oracle
        m = 8192
        lat_h = lat[:m].float().cpu().numpy()
        slot_h = np.arange(m, dtype=np.int64)
        pool_h = np.zeros((m, 576), np.uint16) if fmt == "bf16" else np.zeros((m, 656), np.uint8)
        t0 = time.perf_counter()
        oracle.reshape_and_cache(lat_h, pool_h, slot_h, fmt)
        dt = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": m * (1152 + row_out + 8) / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"numpy oracle on the first {m} rows of the same workload"}
    print(json.dumps(res))


def bench_dense(a, torch, ft, workloads, dev):
    """Dense MLA decode: 64 sequences x 128 heads over 8192-token paged contexts (no index list)."""
    cfg = workloads.decode_bf16(dev)
    B, H, ctx = cfg["q"].shape[0], cfg["q"].shape[2], 8192
    q = cfg["q"].view(B, H, 576)
    bt = cfg["block_table"][:, :ctx // cfg["page_size"]].contiguous()
    lens = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    o = torch.empty((B, H, 512), dtype=torch.bfloat16, device=dev)
    flops = 2.0 * (576 + 512) * H * B * ctx
    nbytes = B * ctx * 1152 + q.numel() * 2 + o.numel() * 2 + B * H * 4
    def step():
        ft.decode_attention_fwd(q, cfg["kv_cache"], None, o, bt, lens, None, None, cfg["sm_scale"], cfg["page_size"])
    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(a.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / a.steps
    kern_ms = e0.elapsed_time(e1) / a.steps
    ach = flops / (kern_ms * 1e-3) / 1e12
    res = {
        "metric": "dense MLA decode TFLOP/s", "value": flops / (ms * 1e-3) / 1e12, "unit": "TFLOP/s", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "decode_dense_bf16", "batch": B, "heads": H, "context": ctx, "page_size": cfg["page_size"],
                   "flops_per_step": flops, "bytes_per_step": nbytes},
        "roofline": {"bound": "mfma", "achieved": ach, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": ach / PEAK_BF16_TFLOPS, "traffic": None if (a.head_groups or a.persist) else measured_traffic("decode_dense_bf16"),
                     "traffic_source": TRAFFIC_NOTE, "kernel": many_heads_kernel(a, "bf16"), "kernel_ms": kern_ms,
                     "other_bound": {"bound": "hbm", "achieved": nbytes / (kern_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                                     "unit": "GB/s", "frac": nbytes / (kern_ms * 1e-3) / 1e9 / PEAK_HBM_GBS}},
        "timing": TIMING_NOTE}
    if not a.no_cpu_baseline:
        n_seq = a.cpu_sample or 4
        try:
            idx = torch.arange(ctx, dtype=torch.int32, device=dev).repeat(n_seq, 1).view(n_seq, 1, ctx)
            sub = dict(cfg, q=cfg["q"][:n_seq], indices=idx, block_table=bt[:n_seq])
            sys.path.insert(0, os.path.join(ROOT, "tests"))
            from _util import oracle_inputs
            qn, kv_small, phys_small, _ = oracle_inputs(sub)
            v, reps = _time_oracle(qn, kv_small, phys_small, cfg["sm_scale"])
            res["cpu_baseline"] = {"value": v, "unit": "TFLOP/s", "cores": cpu_threads(), "kind": "port",
                                   "sample": f"numpy fp32 oracle on the first {n_seq} of {B} sequences of the same workload, "
                                             f"median of {reps} runs"}
        except Exception as e:
            res["cpu_baseline"] = {"value": None, "unit": "TFLOP/s", "cores": cpu_threads(), "kind": "port",
                                   "sample": f"failed: {e}"}
    print(json.dumps(res))


def bench_topk(a, torch, ft, dev):
    """Top-k index producer: decode = 64 rows of 65 536 scores, prefill = 4096 rows of 4096; k = 2048."""
    rows, n = (64, 65536) if a.workload == "topk_decode" else (4096, 4096)
    k = 2048
    g = torch.Generator(device=dev).manual_seed(78)
    sets = [torch.randn((rows, n), generator=g, device=dev) for _ in range(4)]
    nbytes = rows * n * 4 + rows * k * 4                 # every score read once, every index written once
    # few long rows are cut into parts (two launches on the stream: the parts' selections, then the
    # rows'); the scratch for the candidates is allocated once, outside the timed loop
    need = ft.topk_workspace_bytes(rows, n, k)
    ws = torch.empty(need, dtype=torch.uint8, device=dev) if need and not a.topk_one_workgroup else False
    for i in range(a.warmup):
        ft.topk_indices(sets[i % 4], k, workspace=ws)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(a.steps):
        ft.topk_indices(sets[i % 4], k, workspace=ws)
    e1.record()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / a.steps
    kern_ms = e0.elapsed_time(e1) / a.steps
    ach = nbytes / (kern_ms * 1e-3) / 1e9
    res = {
        "metric": "top-k index producer GB/s", "value": nbytes / (ms * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": a.workload, "rows": rows, "cols": n, "k": k, "bytes_per_step": nbytes,
                   "rows_cut_into_parts": ws is not False},
        "roofline": {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": ach / PEAK_HBM_GBS,
                     "traffic": None if ws is not False else measured_traffic(a.workload), "traffic_source": TRAFFIC_NOTE,
                     "kernel": "topk_part_kernel + topk_merge_kernel" if ws is not False else "topk_resident_kernel",
                     "kernel_ms": kern_ms}}
    if not a.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        import oracle
        m = min(rows, 64)
        x = sets[0][:m].cpu().numpy()
        t0 = time.perf_counter()
        oracle.topk_indices(x, k)
        dt = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": (m * n * 4 + m * k * 4) / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"numpy oracle on the first {m} rows of the same workload"}
    print(json.dumps(res))


if __name__ == "__main__":
    main()
