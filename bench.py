#!/usr/bin/env python3
"""Benchmark of the sparse-embedding hot path on one MI355X.

Workload (the configuration the headline metric is quoted on, "C2 DLRM-style"): 26 fp32 tables of dim 128 with about 60 M rows in total
(+ Adam m and v), batch 65536 with one key per field (N = 1 703 936 lookups per step), keys Zipf(1.05) over each
table's rows hashed to 64-bit ids that the device hash table resolves.  One step =
    dedup (unique + inverse) -> key -> slot (insert new keys) -> row gather [N,128] -> gradient segment-reduce
    -> sparse Adam on the touched rows.
All inputs are resident in HBM before the timed region.  Prints ONE JSON line.
"""
import argparse
import ctypes
import json
import os
import sys
import time
from ctypes import c_void_p

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # bytes/s, MI355X HBM3E
# kernels the library launches on its own side streams, beside kernels of the caller's stream
SIDE_STREAM_KERNELS = {"sort_positions_by_rank", "k_lists_bounds", "k_dedup_classify", "k_lists_finish",
                       "k_long_meta", "k_apply_long_chunks"}
T, DIM, BATCH = 26, 128, 65536
# the other configurations' legs: (--config of recsdk_amd.config_bench, timed steps, warm-up steps, further arguments)
OTHER_CONFIG_PLAN = [("c1", 100, 10, []), ("c3", 20, 3, []), ("c4", 100, 3, []), ("c5", 20, 150, [])]
ALPHA = 1.05
LR, B1, B2, EPS = 1e-3, 0.9, 0.999, 1e-8


def make_key_batches(rows, nbatches, seed=2):
    """nbatches arrays of int64 [T*BATCH], feature-major (table t at [t*BATCH, (t+1)*BATCH))."""
    from recsdk_amd import synth
    rng = np.random.default_rng(seed)
    samplers = [synth.ZipfSampler(ALPHA, int(r)) for r in rows]
    out = []
    for _ in range(nbatches):
        out.append(np.concatenate([synth.ranks_to_keys(samplers[t].ranks(rng, BATCH), t) for t in range(T)]))
    return out


def cpu_baseline(key_batches, rows, steps, threads=1):
    """The CPU oracle (the restated reference algorithms) on the first `steps` batches of the same key stream:
    hash-map dedup, serial slot assignment, row-copy gather, sequential segment sum, scalar Adam.  threads > 1: the
    tables of a step are spread over that many threads, one table's whole pipeline per task, as the reference's
    key-process threads take whole batches (the oracle's C functions run without the interpreter lock)."""
    from concurrent.futures import ThreadPoolExecutor

    import oracle
    # tables of the configuration's own row counts; slots are handed out in first-seen order, so only the rows the
    # sample touches are ever paged in (the arrays are zero pages until then)
    tabs = [oracle.Table(int(r)) for r in rows]
    w = [np.zeros((int(r), DIM), np.float32) for r in rows]
    m = [np.zeros((int(r), DIM), np.float32) for r in rows]
    v = [np.zeros((int(r), DIM), np.float32) for r in rows]
    grad = np.random.default_rng(0).normal(0, 1e-3, (BATCH, DIM)).astype(np.float32)
    oracle.lib()

    def table_step(s, t, lr_t):
        keys = key_batches[s % len(key_batches)][t * BATCH:(t + 1) * BATCH]
        split, _, restore, _ = oracle.hash_split(keys, 1, with_counts=False)
        slots, _ = tabs[t].key2offset(split, 0)
        oracle.gather_rows(w[t], DIM, slots[restore], DIM)
        g = oracle.segment_sum(grad, restore, split.size)
        oracle.byaddr_apply(2, g, slots, w[t], m[t], v[t], DIM, float(lr_t), B1, B2, EPS, 0.0, delta_form=False)

    pool = ThreadPoolExecutor(threads) if threads > 1 else None
    t0 = time.perf_counter()
    for s in range(steps):
        lr_t = LR * np.sqrt(1 - B2 ** (s + 1)) / (1 - B1 ** (s + 1))
        if pool is None:
            for t in range(T):
                table_step(s, t, lr_t)
        else:
            list(pool.map(lambda t: table_step(s, t, lr_t), range(T)))
    dt = time.perf_counter() - t0
    if pool is not None:
        pool.shutdown()
    return {"value": T * BATCH * steps / dt, "unit": "keys/s", "cores": threads, "kind": "port",
            "sample": f"{steps} steps of the same key stream, all {T} tables, batch {BATCH}; "
                      f"{dt:.1f} s of wall time"}


def boundaries(torch, capi, host, synth):
    """The drop-in boundaries called with host vectors (recsdk_amd.config_bench.run_bounds) and, beside each, the CPU
    oracle's restatement of the same reference function on the same input, one core."""
    import oracle
    from recsdk_amd import config_bench as cb
    cb.PRINT_LINES = False
    ids, batches = cb.bounds_inputs(synth)
    first = len(cb.RESULTS)
    cb.run_bounds(cb.default_args(), torch, capi, host, synth, inputs=(ids, batches))
    lines = [dict(d) for d in cb.RESULTS[first:]]
    T, B = 26, 65536

    def med(v):
        return sorted(v)[len(v) // 2]

    cpu = {}
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        for t in range(T):
            oracle.unique_sharded(ids[t * B:(t + 1) * B], 8)
        ts.append(time.perf_counter() - t0)
    cpu["DoEnhancedUnique"] = med(ts) * 1e6
    om = oracle.OffsetMapper(cb.BOUNDS_CACHE_SLOTS)
    ts = []
    for b in batches:
        t0 = time.perf_counter()
        om.get_swap_pairs_and_key2offset(b)
        ts.append(time.perf_counter() - t0)
    cpu["GetSwapPairsAndKey2Offset"] = med(ts[-8:]) * 1e6
    del om
    sw = oracle.Swap(cb.BOUNDS_CACHE_SLOTS)
    ts = []
    for b in batches:
        t0 = time.perf_counter()
        sw.compute_swap_info(b[:cb.BOUNDS_SWAP_KEYS])
        ts.append(time.perf_counter() - t0)
    cpu["ComputeSwapInfo"] = med(ts[-8:]) * 1e6
    out = []
    for d in lines:
        us = d.get("us_per_batch", d.get("us_per_call"))
        e = {"call": d["call"], "workload": d["workload"], "us": us,
             "cpu_restatement_us": round(cpu[d["call"]], 1), "cpu_cores": 1}
        if "error" in d:
            e["error"] = d["error"]
        if us is None:
            e["note"] = "library not built here (it compiles against the reference's headers)"
        out.append(e)
    return out


def calibrate(torch, capi, L, dev, tables):
    """What the memory system of this device sustains, measured after the timed region with the library's own plain
    kernels and HIP events: a streaming copy of 2 GiB, and a copy of 1.7 M random 512-byte rows of the largest table
    (the by-address lookup: one row address per output row, nothing else to do)."""
    out = {}
    n_bytes = 2 << 30
    src = torch.empty(n_bytes // 4, device=dev)
    dst = torch.empty(n_bytes // 4, device=dev)
    sp = c_void_p(torch.cuda.current_stream().cuda_stream)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def timed(fn, reps=5):
        fn()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) / reps * 1e-3

    t = timed(lambda: capi.check(L.recsdk_calib_copy(c_void_p(dst.data_ptr()), c_void_p(src.data_ptr()), n_bytes, sp)))
    out["stream_copy_GBps"] = round(2 * n_bytes / t / 1e9, 1)
    del src, dst
    big = max(tables, key=lambda x: x.shape[0])
    n = T * BATCH
    rows = torch.randint(0, big.shape[0], (n,), device=dev, dtype=torch.int64)
    addr = big.data_ptr() + rows * (big.shape[1] * 4)       # first DIM floats of the row
    y = torch.empty((n, DIM), device=dev)
    t = timed(lambda: capi.check(L.recsdk_lookup_by_addr(c_void_p(addr.data_ptr()), n, DIM, capi.DT_F32,
                                                         c_void_p(y.data_ptr()), sp)))
    out["random_row_copy_GBps"] = round(2 * n * DIM * 4 / t / 1e9, 1)
    out["note"] = "bytes read + written per second; the row kernels' rates are to be set beside these, not beside 8000"
    return out


TRAFFIC_SUMMARY = "profiles/c2_dlrm_step_hbm_traffic_pmc.txt"


def recorded_traffic(kernel):
    """HBM bytes per launch of `kernel` as the committed counter summary of this workload states them (its line
    `roofline_traffic_bytes_per_launch <kernel> <bytes>`), or None."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), TRAFFIC_SUMMARY)
    try:
        with open(path) as f:
            for ln in f:
                w = ln.split()
                if len(w) == 3 and w[0] == "roofline_traffic_bytes_per_launch" and w[1] == kernel:
                    return int(w[2])
    except OSError:
        pass
    return None


def other_configs():
    """C1, C3, C4 and C5 for a few steps each: keys/s, algorithmic GB/s and what is specific to each (C4: hash probes
    per second, C5: rows over the host link against its 64 GB/s).  Each leg is `python -m recsdk_amd.config_bench
    --config cN` in a process of its own, started when this process has released its tables: a leg then meets the
    device as a caller of its own would (which streams share a hardware queue depends on every stream the process has
    created before, and legs run one after the other in this process were up to 15 % slower than alone), and the
    command line is the only interface between the two files."""
    import subprocess
    out = []
    here = os.path.dirname(os.path.abspath(__file__))
    for name, steps, warmup, extra in OTHER_CONFIG_PLAN:
        cmd = [sys.executable, "-m", "recsdk_amd.config_bench", "--config", name, "--steps", str(steps), "--warmup",
               str(warmup)] + list(extra)
        t0 = time.perf_counter()
        lines = []
        try:
            r = subprocess.run(cmd, cwd=here, capture_output=True, text=True, timeout=600)
            lines = [json.loads(ln) for ln in r.stdout.splitlines() if ln.startswith("{")]
            if r.returncode != 0 or not lines:
                # a configuration that does not fit this box is reported, not fatal
                out.append({"config": name.upper(), "error": (r.stderr.strip() or "no result line")[-300:]})
        except subprocess.TimeoutExpired:
            out.append({"config": name.upper(), "error": "no result within 600 s"})
        for d in lines:
            d["value"] = round(d["value"], 1)
            d["wall_s"] = round(time.perf_counter() - t0, 1)
            out.append(d)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--cpu-steps", type=int, default=30,
                    help="steps of the CPU baseline leg, about 10 s on one core (0 = skip); the batches repeat after warmup + steps")
    ap.add_argument("--total-rows", type=int, default=60_000_000)
    ap.add_argument("--pipeline", action="store_true",
                    help="resolve the next batches' keys on a second stream while the current batch's rows are read "
                         "and updated (about 9 %% more keys/s on one MI355X; per-kernel times then overlap, so the "
                         "default keeps every step on one stream)")
    ap.add_argument("--ext-rows", action="store_true",
                    help="tables as extended rows [w | m | v] of 3 x dim floats (the by-address layout) instead of three "
                         "arrays per table")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the short runs of the other configurations (C1, C3, C4, C5) after the headline one")
    ap.add_argument("--one-stream-only", action="store_true",
                    help="skip the two-stream schedule that is reported beside the one-stream figure (for kernel traces "
                         "whose per-kernel averages should cover one-stream steps only)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="after the timed region copy one 1 GiB tensor (a kernel of known traffic for counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from recsdk_amd import capi, host, synth

    L = capi.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    rows = synth.dlrm_table_rows(T, args.total_rows)
    N = T * BATCH
    nb = args.warmup + args.steps
    t_gen = time.perf_counter()
    # the timed steps, the median loop and the graph replay each get batches of their own: a batch that was
    # looked up before finds all its keys in the tables
    batches = make_key_batches(rows, nb + 2 * args.steps)
    d_keys = [torch.from_numpy(b).to(dev) for b in batches]
    offsets = np.arange(T + 1, dtype=np.int64) * BATCH
    d_off = torch.from_numpy(offsets).to(dev)
    if args.ext_rows:
        # one extended row [w | m | v] per key, as the reference's by-address tables hold them
        ext = [torch.zeros((int(r), 3 * DIM), device=dev) for r in rows]
        for e in ext:
            e[:, :DIM].normal_(0, 0.01)
        w = ext
        flat = [e.view(-1) for e in ext]
        rows_h = host.Rows(DIM, ext, [f[DIM:] for f in flat], [f[2 * DIM:] for f in flat], [3 * DIM] * T)
    else:
        w = [torch.randn((int(r), DIM), device=dev) * 0.01 for r in rows]
        m = [torch.zeros((int(r), DIM), device=dev) for r in rows]
        v = [torch.zeros((int(r), DIM), device=dev) for r in rows]
        rows_h = host.Rows(DIM, w, m, v)
    grad = torch.randn((N, DIM), device=dev) * 1e-3
    out = torch.empty((N, DIM), device=dev)
    # Three dedup workspaces: the keys of the next batches are deduplicated and resolved to slots (index stream)
    # while the rows of batch i are gathered and updated (row stream), as the reference's key-process threads run
    # ahead of the device step.  Every step still does all of its work; table state only changes on the index stream.
    NBUF = 3
    # plain HashSplit: no per-key counts are asked for before the gradient reduce (key_process.cpp:1134-1156)
    uqs = [host.Unique(N, T, early_counts=False, max_table_keys=BATCH) for _ in range(NBUF)]
    tg = host.EmbeddingTables([int(r) for r in rows], N)
    p_uk, p_uo = [c_void_p() for _ in range(NBUF)], [c_void_p() for _ in range(NBUF)]
    for b in range(NBUF):
        capi.check(L.recsdk_unique_results(uqs[b].h, ctypes.byref(p_uk[b]), ctypes.byref(p_uo[b]), None, None))
    s_index, s_rows = torch.cuda.Stream(), torch.cuda.Stream()
    ev_index = [torch.cuda.Event() for _ in range(NBUF)]
    ev_rows = [torch.cuda.Event() for _ in range(NBUF)]
    torch.cuda.synchronize()
    print(f"[bench] setup {time.perf_counter() - t_gen:.1f}s, rows total {int(rows.sum())}, "
          f"HBM in use {torch.cuda.memory_allocated() / 2**30:.1f} GiB (torch)", file=sys.stderr, flush=True)

    step_no = [0]

    def index_part(i, stream_obj):
        """dedup + key -> slot of batch i into workspace i % NBUF"""
        b = i % NBUF
        sp = c_void_p(stream_obj.cuda_stream)
        with torch.cuda.stream(stream_obj):
            uqs[b].run(d_keys[i], d_off)
        # distinct keys -> slots, in place in the handle's buffer (as the reference overwrites lookupKeys)
        capi.check(L.recsdk_tables_key2offset(tg.h, p_uk[b], p_uo[b], T, N, capi.CHANNEL_TRAIN, sp))

    def rows_part(i, stream_obj):
        """forward gather + segment-reduce + Adam of batch i"""
        b = i % NBUF
        sp = c_void_p(stream_obj.cuda_stream)
        step_no[0] += 1
        lr_t = LR * np.sqrt(1 - B2 ** step_no[0]) / (1 - B1 ** step_no[0])
        capi.check(L.recsdk_gather_unique(rows_h.h, uqs[b].h, p_uk[b], c_void_p(out.data_ptr()), sp))
        capi.check(L.recsdk_sparse_apply(rows_h.h, uqs[b].h, p_uk[b], c_void_p(grad.data_ptr()), capi.OPT_ADAM,
                                         float(lr_t), B1, B2, EPS, 0.0, sp))

    def step(i):
        cur = torch.cuda.current_stream()
        index_part(i, cur)
        rows_part(i, cur)

    def run_steps(first, last, pipeline=None):
        """steps first..last-1; on two streams with --pipeline"""
        if not (args.pipeline if pipeline is None else pipeline):
            for i in range(first, last):
                step(i)
            return
        cur = torch.cuda.current_stream()
        s_index.wait_stream(cur)
        s_rows.wait_stream(cur)
        ahead = NBUF - 1                      # batches the index stream may run ahead of the row stream
        issued = first
        for i in range(first, last):
            while issued < last and issued <= i + ahead - 1:
                if issued - NBUF >= first:
                    s_index.wait_event(ev_rows[issued % NBUF])   # the workspace was last read by step issued - NBUF
                index_part(issued, s_index)
                ev_index[issued % NBUF].record(s_index)
                issued += 1
            s_rows.wait_event(ev_index[i % NBUF])
            rows_part(i, s_rows)
            ev_rows[i % NBUF].record(s_rows)
        cur.wait_stream(s_index)
        cur.wait_stream(s_rows)

    run_steps(0, args.warmup)
    torch.cuda.synchronize()

    # which kernel dominates: one extra pass over the last warm-up batch with every kernel timed (untimed region)
    dominant = "k_apply_short"
    per_kernel = {}
    if args.warmup > 0:
        capi.profile_start("")
        step(args.warmup - 1)
        torch.cuda.synchronize()
        per_kernel = capi.profile_stop()
        if per_kernel:
            # kernels that run on a side stream beside others (the position lists beside the key -> slot kernels and
            # the gather, the chunk sums beside the short-list update) are stretched by the overlap: not candidates
            on_caller_stream = {k: v for k, v in per_kernel.items() if k not in SIDE_STREAM_KERNELS}
            dominant = max(on_caller_stream, key=lambda k: on_caller_stream[k][1])

    # timed region: K steps, only the dominant kernel bracketed by HIP events
    u_counts = []
    capi.profile_start(dominant)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run_steps(args.warmup, nb)
    host_issue = time.perf_counter() - t0
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    prof = capi.profile_stop()
    # as many steps again, over new batches, with an event between them: the median step time (outside the timed region)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    saved_step = step_no[0]
    marks[0].record()
    for k, i in enumerate(range(nb, nb + args.steps)):
        step(i)
        marks[k + 1].record()
    torch.cuda.synchronize()
    step_no[0] = saved_step
    per_step_ms = sorted(marks[k].elapsed_time(marks[k + 1]) for k in range(args.steps))
    median_ms = per_step_ms[len(per_step_ms) // 2]
    ms_per_step = elapsed / args.steps * 1e3
    value = N * args.steps / elapsed

    # distinct keys per step (measured on the last batch) for the algorithmic byte counts
    uk, uo, inv, cnt = uqs[(nb - 1) % NBUF].fetch()
    U = int(uk.numel())
    cnt_h = cnt.cpu().numpy().astype(np.int64)
    short = cnt_h <= 64
    u_short, n_short = int(short.sum()), int(cnt_h[short].sum())
    R = DIM * 4
    step_bytes = 1036 * N + 3616 * U  # keys 8N + inverse 4N + out R*N + grad R*N; per distinct key 32 + R + 6R
    kernel_bytes = {
        "k_apply_short": R * n_short + 6 * R * u_short,          # grad rows in + (w,m,v) read and written
        "k_apply_long": R * (N - n_short) + 6 * R * (U - u_short),
        "k_gather_rows": R * U + R * N,                          # distinct rows in + per-lookup rows out
    }
    roofline = None
    if dominant in prof and prof[dominant][0] > 0:
        launches, tot_ms = prof[dominant]
        avg_s = tot_ms / launches * 1e-3
        kb = kernel_bytes.get(dominant)
        if kb is not None:
            ach = kb / avg_s / 1e9
            roofline = {"bound": "hbm", "kernel": dominant, "achieved": round(ach, 1), "peak": HBM_PEAK / 1e9,
                        "unit": "GB/s", "frac": round(ach * 1e9 / HBM_PEAK, 4),
                        "traffic": None, "avg_kernel_us": round(avg_s * 1e6, 1), "algorithmic_bytes": kb}
            # HBM bytes per launch come from a pair of counter runs of this same workload, not from this run: the
            # figure recorded with their summary is reported when the workload is the one they ran
            if args.total_rows == 60_000_000 and not args.ext_rows:
                rec = recorded_traffic(dominant)
                if rec is not None:
                    roofline["traffic"] = rec
                    roofline["traffic_source"] = ("FETCH_SIZE / WRITE_SIZE runs of this workload under rocprofv3, "
                                                  "summary in " + TRAFFIC_SUMMARY)
    result = {
        "metric": "lookup+update keys/sec at batch 65536 (dedup + hash-slot resolve + gather + segment-reduce + Adam)",
        "value": round(value, 1), "unit": "keys/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "ms_per_step_median": round(median_ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "C2 DLRM-style: 26 fp32 tables dim 128, batch 65536 one key per field, Zipf(1.05) "
                               "64-bit keys resolved by the device hash table, lookup + dedup + Adam",
                   "tables": T, "dim": DIM, "batch": BATCH, "total_rows": int(rows.sum()), "lookups_per_step": N,
                   "distinct_keys_last_step": U,
                   "schedule": "one stream" if not args.pipeline else
                               "two streams: keys of step i+1 resolved while rows of step i are read and updated"},
        "host_issue_ms_per_step": round(host_issue / args.steps * 1e3, 4),
        "step_algorithmic_bytes": step_bytes,
        "step_achieved_GBps": round(step_bytes / (elapsed / args.steps) / 1e9, 1),
        "step_hbm_frac": round(step_bytes / (elapsed / args.steps) / HBM_PEAK, 4),
        "roofline": roofline,
        "kernel_ms_one_step": {k: round(vv[1], 4) for k, vv in sorted(per_kernel.items(), key=lambda kv: -kv[1][1])},
    }
    if not args.pipeline and not args.one_stream_only:
        # The same batches once more on two streams (keys of the next batches resolved while the rows of the current one
        # are read and updated, as the reference's key-process threads run ahead of the device step); reported beside
        # `value`, which stays the one-stream figure with its clean per-kernel times.
        run_steps(args.warmup, nb, pipeline=True)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        run_steps(args.warmup, nb, pipeline=True)
        torch.cuda.synchronize()
        el2 = time.perf_counter() - t1
        result["two_stream_schedule"] = {"ms_per_step": round(el2 / args.steps * 1e3, 4),
                                         "value": round(N * args.steps / el2, 1), "unit": "keys/s",
                                         "note": "over the batches of the timed steps again: their keys are in the "
                                                 "tables by now"}
    if not args.pipeline and not args.one_stream_only:
        # The same step once more as a HIP graph: captured once on a key buffer of its own (the keys of every batch are
        # copied into it before a replay) and replayed over batches of its own; Adam's bias-corrected rate, which changes
        # every step, is read by the update from a device word that is rewritten before every replay
        # (recsdk_sparse_apply_lr_dev).  Outside the timed region and reported beside `value`.
        try:
            kbuf = d_keys[args.warmup].clone()
            lr_dev = torch.zeros(1, dtype=torch.float32, device=dev)

            def graph_step():
                b = args.warmup % NBUF
                cur = torch.cuda.current_stream()
                sp = c_void_p(cur.cuda_stream)
                uqs[b].run(kbuf, d_off)
                capi.check(L.recsdk_tables_key2offset(tg.h, p_uk[b], p_uo[b], T, N, capi.CHANNEL_TRAIN, sp))
                capi.check(L.recsdk_gather_unique(rows_h.h, uqs[b].h, p_uk[b], c_void_p(out.data_ptr()), sp))
                capi.check(L.recsdk_sparse_apply_lr_dev(rows_h.h, uqs[b].h, p_uk[b], c_void_p(grad.data_ptr()),
                                                        capi.OPT_ADAM, c_void_p(lr_dev.data_ptr()), B1, B2, EPS, 0.0,
                                                        sp))

            def replay(i, g):
                step_no[0] += 1
                kbuf.copy_(d_keys[i])
                lr_dev.fill_(float(LR * np.sqrt(1 - B2 ** step_no[0]) / (1 - B1 ** step_no[0])))
                g.replay()

            gs = torch.cuda.Stream()
            gs.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(gs):
                graph_step()                            # every buffer the step grows on demand has its size
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=gs):
                    graph_step()
                for i in range(args.warmup, min(args.warmup + 3, nb)):
                    replay(i, g)
                torch.cuda.synchronize()
                t1 = time.perf_counter()
                for i in range(nb + args.steps, nb + 2 * args.steps):
                    replay(i, g)
                torch.cuda.synchronize()
                el3 = time.perf_counter() - t1
            torch.cuda.current_stream().wait_stream(gs)
            result["graph_replay"] = {"ms_per_step": round(el3 / args.steps * 1e3, 4),
                                      "value": round(N * args.steps / el3, 1), "unit": "keys/s",
                                      "note": "the step captured once; before every replay the batch's keys are copied "
                                              "into the captured buffer and Adam's rate of the step is written to the "
                                              "device word the update reads it from"}
            del g
        except Exception as e:  # the headline above does not depend on this line
            result["graph_replay"] = {"error": str(e)[:200]}
    if args.calib_copy:
        a = torch.empty(1 << 28, device=dev)
        b = torch.empty(1 << 28, device=dev)
        b.copy_(a)
        torch.cuda.synchronize()
        del a, b
    result["calibration"] = calibrate(torch, capi, L, dev, w)
    if not args.no_other_configs:
        # the other configurations, each for a few steps, after this one's tables have been released
        del rows_h, tg, uqs, grad, out, w
        if not args.ext_rows:
            del m, v
        torch.cuda.empty_cache()
        result["other_configs"] = other_configs()
        try:
            result["boundaries"] = boundaries(torch, capi, host, synth)
        except Exception as e:  # the headline does not depend on this leg
            result["boundaries"] = {"error": str(e)[:200]}
    if args.cpu_steps > 0:
        k = args.cpu_steps
        result["cpu_baseline"] = cpu_baseline(batches, rows, k)
        # the same with the reference's default of 6 key-process threads and with all the host cores of one GPU's share
        share = min(16, os.cpu_count() or 16)
        result["cpu_baseline_threads"] = [cpu_baseline(batches, rows, k, threads=n) for n in (6, share)]
        result["nproc"] = os.cpu_count()
        result["host_cores_share"] = share
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
