"""Throughput of the hot path on the synthetic configurations other than the headline one (which bench.py measures):
keys/s and algorithmic GB/s, as a fraction of the 8 TB/s HBM peak.  One JSON line per configuration.

    python -m recsdk_amd.config_bench --config c1|c3|c4|c5|ops|keys|bounds|all [--steps K] [--warmup W]

  c1  one fp32 table 1M x 16, batch 4096 uniform keys, forward gather + sparse Adagrad
  c3  26 bf16 tables 2M x 64, batch 16384, bag lengths U[1,50], Zipf(1.1): sum-pooled forward + exact backward + Adam
  c4  dynamic expansion: dim 32, 200M-slot table, batches of 131072 keys (70 % Zipf(1.2) hot set of 10M, 30 % fresh),
      admission at count >= 2, eviction of keys idle > 20 steps, gather + Adam on the admitted keys
  ops the by-address lookup / update operators and the fused LazyAdam / Sgd operators one by one, 512-byte rows
  keys batch ingestion, padding mask, sharded unique, sorted unique and hot-key split on 26 x 65536 Zipf(1.05) keys
  bounds the drop-in libraries (AccCTR plugin, Embcache classes) called with host vectors, beside the CPU restatement
  c5  host-backed cache: dim 64 rows in pinned host DRAM behind a 20M-row HBM cache, batch 65536 x 26 keys Zipf(1.05):
      unique, cache plan, swap-out / swap-in, gather + Adagrad.  --host-rows scales the host table (default 100M rows
      of weights + accumulator = 51 GB of pinned memory; 400M rows would be 205 GB); new rows take constants by default,
      with --normal-init N(0, 0.01) weights from the reference's host stream (then the host's generation of ~8 M normal
      values per step, spread over its cores, is most of what is measured).
Inputs are synthetic and resident in HBM before timing; every step does all of its work; results are checked against
the oracle at small sizes by the tests, not here.
"""
import argparse
import ctypes
import json
import sys
import time
from ctypes import c_int64, c_void_p

import numpy as np

PEAK_GBS = 8000.0
HOST_LINK_GBS = 64.0   # PCIe Gen5 x16, one direction
RESULTS = []           # every line of this process, for callers that run the configurations in-process
PRINT_LINES = True


def _line(config, workload, keys_per_step, bytes_per_step, steps, elapsed, extra=None):
    ms = elapsed / steps * 1e3
    gbs = bytes_per_step / (ms * 1e-3) / 1e9
    d = {"config": config, "workload": workload, "metric": "lookup+update keys/s", "value": keys_per_step / (ms * 1e-3),
         "unit": "keys/s", "ms_per_step": round(ms, 4), "algorithmic_GB_per_step": round(bytes_per_step / 1e9, 4),
         "achieved_GBs": round(gbs, 1), "frac_of_hbm_peak": round(gbs / PEAK_GBS, 4), "steps": steps,
         "data": "synthetic",
         # the whole step against the HBM peak: algorithmic bytes of the step / the step's wall time
         "roofline": {"bound": "hbm", "scope": "whole step, every kernel and the gaps between them",
                      "achieved": round(gbs, 1), "peak": PEAK_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_GBS, 4),
                      "traffic": None}}
    if extra:
        d.update(extra)
    rec = recorded_step_traffic(config) if workload_is_the_profiled_one(config, workload) else None
    if rec is not None and d["roofline"]["bound"] == "hbm":
        d["roofline"]["traffic"] = rec[0]
        d["roofline"]["traffic_source"] = "FETCH_SIZE / WRITE_SIZE runs of this workload under rocprofv3, summary in " + rec[1]
    RESULTS.append(d)
    if PRINT_LINES:
        print(json.dumps(d), flush=True)
    return d


def workload_is_the_profiled_one(config, workload):
    """The counter summaries cover the first line of a configuration (its step proper), not its variants."""
    return config == "C3" and workload.startswith("26 bf16 tables 2M x 64, batch 16384")


def recorded_step_traffic(config):
    """HBM bytes per step of `config` as the committed counter summary of that configuration states them (its line
    `step_traffic_bytes <config> <bytes>`), or None: counter runs cannot be part of a timed run."""
    import glob
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for path in sorted(glob.glob(os.path.join(root, "profiles", "*_pmc.txt"))):
        try:
            with open(path) as f:
                for ln in f:
                    w = ln.split()
                    if len(w) == 3 and w[0] == "step_traffic_bytes" and w[1] == config:
                        return int(w[2]), os.path.relpath(path, root)
        except OSError:
            pass
    return None


def _timed(torch, fn, warmup, steps):
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(warmup, warmup + steps):
        fn(i)
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def run_c1(args, torch, capi, host, synth):
    dev = "cuda:0"
    rows, dim, batch = 1_000_000, 16, 4096
    rng = np.random.default_rng(0)
    nb = args.warmup + args.steps
    # fresh batches for the graph replay as well: a batch seen before finds all its keys in the table
    keys = [torch.from_numpy(rng.integers(0, rows, batch).astype(np.int64)).to(dev) for _ in range(2 * nb)]
    off = torch.tensor([0, batch], dtype=torch.int64, device=dev)
    w = torch.randn((rows, dim), device=dev) * 0.01
    acc = torch.full((rows, dim), 0.1, device=dev)
    grad = torch.randn((batch, dim), device=dev) * 1e-3
    out = torch.empty((batch, dim), device=dev)
    rows_h = host.Rows(dim, [w], [acc], None)
    uq = host.Unique(batch, 1)
    tg = host.EmbeddingTables([rows], batch)
    p_uk, p_uo = c_void_p(), c_void_p()
    capi.check(capi.lib().recsdk_unique_results(uq.h, ctypes.byref(p_uk), ctypes.byref(p_uo), None, None))

    def step(i):
        sp = c_void_p(torch.cuda.current_stream().cuda_stream)
        uq.run(keys[i], off)
        capi.check(capi.lib().recsdk_tables_key2offset(tg.h, p_uk, p_uo, 1, batch, capi.CHANNEL_TRAIN, sp))
        capi.check(capi.lib().recsdk_gather_unique(rows_h.h, uq.h, p_uk, c_void_p(out.data_ptr()), sp))
        capi.check(capi.lib().recsdk_sparse_apply(rows_h.h, uq.h, p_uk, c_void_p(grad.data_ptr()), capi.OPT_ADAGRAD,
                                                  0.01, 0.9, 0.999, 1e-8, 0.0, sp))

    elapsed = _timed(torch, step, args.warmup, args.steps)
    U = uq.total()
    R = dim * 4
    nbytes = 12 * batch + 2 * R * batch + 5 * R * U
    _line("C1", "1 fp32 table 1M x 16, batch 4096 uniform, gather + Adagrad", batch, nbytes, args.steps, elapsed,
          {"note": "four launches (one-block dedup, one-block key -> slot, gather, scan-based reduce + update), each a "
                   "chain of a few dependent memory round trips; issued one by one from the host"})
    # the same step recorded once into a HIP graph and replayed on new keys (copied into the captured key buffer)
    kbuf = keys[0].clone()
    saved, keys[0] = keys[0], kbuf
    g = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        step(0)
    keys[0] = saved

    def replay(i):
        kbuf.copy_(keys[nb + i])
        g.replay()

    elapsed = _timed(torch, replay, args.warmup, args.steps)
    _line("C1", "the same step as a HIP graph replay", batch, nbytes, args.steps, elapsed,
          {"note": "bound by the device's launch-to-launch latency"})


def run_ops(args, torch, capi, host, synth):
    """The by-address operators and the fused optimizer operators one by one, at the DLRM-style shape: 65536 x 26
    lookups of 512-byte rows, 430 k distinct rows per step (what the reference's TF graph issues around its own
    dedup).  One line per operator; bytes = the tensors each must read and write once."""
    dev = "cuda:0"
    n, u, dim, rows = 26 * 65536, 430_000, 128, 8_000_000
    R = dim * 4
    g = torch.Generator(device=dev).manual_seed(0)
    table = torch.randn((rows, dim), device=dev, generator=g) * 0.01
    m = torch.zeros((rows, dim), device=dev)
    v = torch.zeros((rows, dim), device=dev)
    look = torch.randint(0, rows, (n,), device=dev, generator=g)
    addr = table.data_ptr() + look * R
    distinct = torch.randperm(rows, device=dev, generator=g)[:u]
    uaddr = table.data_ptr() + distinct * R
    idx32 = distinct.to(torch.int32)
    delta = torch.randn((u, dim), device=dev, generator=g) * 1e-4
    grad = torch.randn((u, dim), device=dev, generator=g) * 1e-3
    y = torch.empty((n, dim), device=dev)
    L = capi.lib()

    def timed(fn):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(max(args.warmup, 1)):
            fn()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) * 1e-3

    sp = lambda: c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: c_void_p(t.data_ptr())
    cases = [
        ("EmbeddingLookupByAddress", n, 8 * n + 2 * R * n,
         lambda: capi.check(L.recsdk_lookup_by_addr(p(addr), n, dim, capi.DT_F32, p(y), sp()))),
        ("EmbeddingUpdateByAddress (atomic add)", u, 8 * u + 3 * R * u,
         lambda: capi.check(L.recsdk_update_by_addr(p(uaddr), u, dim, capi.DT_F32, p(delta), 0, sp()))),
        ("EmbeddingUpdateByAddress (overwrite)", u, 8 * u + 2 * R * u,
         lambda: capi.check(L.recsdk_update_by_addr(p(uaddr), u, dim, capi.DT_F32, p(delta), 1, sp()))),
        ("LazyAdam", u, 4 * u + 7 * R * u,
         lambda: capi.check(L.recsdk_lazy_adam(p(grad), p(idx32), u, dim, p(m), p(v), p(table), 1e-3, 0.9, 0.999, 1e-8,
                                               sp()))),
        ("Sgd", u, 4 * u + 3 * R * u,
         lambda: capi.check(L.recsdk_sgd(p(grad), p(idx32), u, dim, p(table), 1e-3, 0.0, sp()))),
    ]
    for name, keys, nbytes, fn in cases:
        _line("ops", f"{name}: {keys} rows of {R} bytes", keys, nbytes, args.steps, timed(fn))


def run_keys(args, torch, capi, host, synth):
    """The key-side entry points that the five configurations do not time, one by one, on the keys of one DLRM-style
    batch (26 tables x 65536 Zipf(1.05) keys): batch ingestion, padding mask, sharded unique with id counts, sorted
    unique, hot-key split.  Each line is the host call as a caller makes it (its own result fetches included);
    bytes = the key and index arrays each must read and write once."""
    dev = "cuda:0"
    T, B = 26, 65536
    n = T * B
    rng = np.random.default_rng(0)
    rows = synth.dlrm_table_rows(T)
    per_table = [synth.zipf_keys(rng, 1.05, int(rows[t]), B, table=t) for t in range(T)]
    keys_h = np.concatenate(per_table).astype(np.int64)
    keys = torch.from_numpy(keys_h).to(dev)
    offs = torch.arange(T + 1, device=dev, dtype=torch.int64) * B
    raw_ids = torch.from_numpy(np.unique(keys_h, return_inverse=True)[1].astype(np.int64)).to(dev)   # same pattern
    u = int(sum(np.unique(k).size for k in per_table))
    splits = np.full(T, B, dtype=np.int64)
    pad_keys = keys_h[rng.integers(0, n, 16)]
    sharded = host.ShardedUnique(n, sharding_num=8, use_sharding=True, use_id_count=True)
    uq = host.Unique(n, 1, position_lists=False)
    rg = c_void_p()
    capi.check(capi.lib().recsdk_regroup_create(n, ctypes.byref(rg)))
    kp = host.KeyProcess(n, T)
    kp.enable_hot_keys([2048] * T)          # the hot sets are chosen from batch 0 (an untimed step), then every 1000th
    cases = [
        ("ReadEmbKeyV2 (int64 sample -> keys + offsets)", 16 * n, lambda i: host.read_emb_key(keys, splits)),
        ("PushPaddingKeysTensors (16 padding keys)", 12 * n, lambda i: host.padding_keys_mask(keys, pad_keys)),
        ("Unique, 8 shards + id counts (one id stream)", 8 * n + 4 * n + 12 * u,
         lambda i: sharded.do_enhanced_unique(keys)),
        ("UniqueParallel (sorted distinct ids + inverse), hashed 64-bit ids", 8 * n + 8 * n + 8 * u,
         lambda i: host.unique_parallel(keys, uq, rg)),
        ("UniqueParallel, the same pattern of ids renumbered below 2^19", 8 * n + 8 * n + 8 * u,
         lambda i: host.unique_parallel(raw_ids, uq, rg)),
        ("HotHashSplit (26 tables, 2048 hot keys each, hot sets from the first batch)", 8 * n + 4 * n + 12 * u,
         lambda i: kp.hot_hash_split(keys, i, offs)),
    ]
    for name, nbytes, fn in cases:
        elapsed = _timed(torch, fn, max(args.warmup, 1), args.steps)
        _line("keys", f"{name}: {n} keys, {u} distinct", n, nbytes, args.steps, elapsed)
    torch.cuda.synchronize()
    capi.lib().recsdk_regroup_destroy(rg)
    sharded.close()
    uq.close()
    kp.close()


def run_c3(args, torch, capi, host, synth):
    dev = "cuda:0"
    T, D, B, rows = 26, 64, 16384, 2_000_000
    rng = np.random.default_rng(0)
    nb = 3
    batches = []
    for _ in range(nb):
        lens = rng.integers(1, 51, T * B)
        offsets = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        idx = synth.zipf_ranks(rng, 1.1, rows, int(offsets[-1])).astype(np.int64)
        batches.append((torch.from_numpy(idx).to(dev), torch.from_numpy(offsets).to(dev)))
    max_nnz = max(int(b[0].numel()) for b in batches)
    w = (torch.randn(T * rows * D, device=dev) * 0.01).to(torch.bfloat16)
    m1 = torch.zeros(T * rows * D, device=dev)
    m2 = torch.zeros(T * rows * D, device=dev)
    woff = torch.arange(T, device=dev, dtype=torch.int64) * rows * D
    doff = torch.arange(T + 1, device=dev, dtype=torch.int32) * D
    cumsum = torch.arange(T + 1, device=dev, dtype=torch.int64) * rows
    gout = torch.randn((B, T * D), device=dev) * 1e-3
    bwd = host.SplitEmbeddingBackward(T, max_nnz)

    def step(i):
        idx, offs = batches[i % nb]
        host.split_embedding_codegen_forward_unweighted(w, woff, doff, T * D, D, idx, offs, capi.POOL_SUM)
        bwd(capi.OPT_ADAM, gout, w, woff, doff, T * D, D, cumsum, idx, offs, capi.POOL_SUM, m1, m2,
            learning_rate=1e-3, iter=i + 1)

    elapsed = _timed(torch, step, args.warmup, args.steps)
    nnz = float(np.mean([int(b[0].numel()) for b in batches]))
    uniq = float(np.mean([len(np.unique(b[0].cpu().numpy() + np.repeat(np.arange(T), B)[
        np.searchsorted(b[1].cpu().numpy(), np.arange(b[0].numel()), side="right") - 1] * rows)) for b in batches[:1]]))
    # Algorithmic bytes, every logically required tensor touched once.  Forward: indices 8 nnz, offsets 8 TB, each
    # distinct bf16 row once 128 U, pooled fp32 output 256 TB.  Backward: grad_output 256 TB, indices 8 nnz + bag of
    # every index 4 nnz, per distinct row the bf16 weights and two fp32 moments read and written (128 + 2 * 256) * 2 U.
    TB = T * B
    nbytes = 20 * nnz + (2 * D * 4 + 16) * TB + (2 * D * 2 + 2 * D * 4 * 2 + D * 2) * uniq
    # What the compute units pull through the caches instead: a row per INDEX in the forward and a gradient row per
    # index in the backward (served by L2 / Infinity Cache when a bag or a row repeats); reported beside, never as the
    # roofline figure.
    cache_side = nnz * (D * 2 + D * 4 + 16) + TB * D * 4 + uniq * (2 * D * 2 + 4 * D * 4)
    c3_extra = {"nnz_per_step": int(nnz), "distinct_rows_per_step": int(uniq), "bags_per_step": TB,
                "cache_side_GB_per_step": round(cache_side / 1e9, 4)}
    _line("C3", "26 bf16 tables 2M x 64, batch 16384, bags U[1,50], Zipf(1.1): pooled forward + backward + Adam",
          nnz, nbytes, args.steps, elapsed, dict(c3_extra))
    # The reference's unique variant: the caller (the ids mapper in front of the operator) hands over the distinct rows
    # of every table and, per index, which of them it is, so the backward groups by that instead of sorting by row.
    uniq_in = []
    for idx, offs in batches:
        idx_h, offs_h = idx.cpu().numpy(), offs.cpu().numpy()
        ids, inv, uoff = [], [], [0]
        for t in range(T):
            u, i = np.unique(idx_h[offs_h[t * B]:offs_h[(t + 1) * B]], return_inverse=True)
            ids.append(u)
            inv.append(i.astype(np.int64))
            uoff.append(uoff[-1] + u.size)
        uniq_in.append(tuple(torch.from_numpy(x).to(dev) for x in (
            np.concatenate(ids).astype(np.int64), np.asarray(uoff, dtype=np.int64), np.concatenate(inv))))

    def step_unique(i):
        idx, offs = batches[i % nb]
        u_ids, u_off, u_inv = uniq_in[i % nb]
        host.split_embedding_codegen_forward_unweighted(w, woff, doff, T * D, D, idx, offs, capi.POOL_SUM)
        bwd(capi.OPT_ADAM, gout, w, woff, doff, T * D, D, cumsum, idx, offs, capi.POOL_SUM, m1, m2,
            learning_rate=1e-3, iter=i + 1, unique_ids=u_ids, unique_offsets=u_off, unique_inverse=u_inv)

    elapsed = _timed(torch, step_unique, args.warmup, args.steps)
    _line("C3", "the same step with unique_ids / unique_offsets / unique_inverse given (the reference's unique backward)",
          nnz, nbytes + nnz * 8 + uniq * 8, args.steps, elapsed, dict(c3_extra))


def run_c4(args, torch, capi, host, synth):
    dev = "cuda:0"
    dim, slots, batch, hot = 32, 200_000_000, 131072, 10_000_000
    ext = 3 * dim
    rng = np.random.default_rng(0)
    nb = args.warmup + args.steps
    fresh = 1 << 40
    keys = []
    hot_sampler = synth.ZipfSampler(1.2, hot)
    for i in range(nb):
        is_hot = rng.random(batch) < 0.7
        k = np.where(is_hot, synth.splitmix64(hot_sampler.ranks(rng, batch).astype(np.uint64)),
                     synth.splitmix64(np.arange(fresh, fresh + batch, dtype=np.uint64))).astype(np.int64)
        fresh += batch
        keys.append(torch.from_numpy(k).to(dev))
    off = torch.tensor([0, batch], dtype=torch.int64, device=dev)
    arena = torch.zeros((slots, ext), device=dev)          # [w | m | v] rows, 76.8 GB
    flat = arena.view(-1)
    rows_h = host.Rows(dim, [arena], [flat[dim:]], [flat[2 * dim:]], [ext])
    grad = torch.randn((batch, dim), device=dev) * 1e-3
    out = torch.empty((batch, dim), device=dev)
    uq = host.Unique(batch, 1)
    tg = host.EmbeddingTables([slots], 1 << 20)            # also takes the evicted keys of a step in one call
    faae = host.FeatureAdmitAndEvict([4_000_000], [2], [20], max_keys=batch)   # ~1.3 M live records
    L = capi.lib()
    p_uk, p_uo, p_cnt = c_void_p(), c_void_p(), c_void_p()
    capi.check(L.recsdk_unique_results(uq.h, ctypes.byref(p_uk), ctypes.byref(p_uo), None, ctypes.byref(p_cnt)))
    ev_cap = 1 << 20
    ev_keys = torch.empty(ev_cap, dtype=torch.int64, device=dev)
    ev_off = torch.zeros(2, dtype=torch.int64, device=dev)
    ts = torch.zeros(1, dtype=torch.int64, device=dev)
    kbuf = keys[0].clone()

    # The eviction of a step touches the admission history and the key -> slot table, not the rows: by default it is
    # issued on a second stream beside the step's gather and update (the keys it evicts have been idle for 20 steps,
    # so none of them is in the batch) and joins the step's stream at the end.
    beside = not args.evict_in_line
    s_evict = torch.cuda.Stream() if beside else None
    ev_fork, ev_join = torch.cuda.Event(), torch.cuda.Event()

    def evict(sp):
        # eviction of keys idle for more than 20 steps, every step
        capi.check(L.recsdk_faae_evict_dev(faae.h, 1, c_void_p(ev_keys.data_ptr()), ev_cap, c_void_p(ev_off.data_ptr()),
                                           sp))
        capi.check(L.recsdk_tables_evict(tg.h, c_void_p(ev_keys.data_ptr()), c_void_p(ev_off.data_ptr()), 1, ev_cap, sp))

    def step(i, beside=beside):
        """nothing returns to the host: the timestamp is read from device memory, the evicted keys and their count
        stay on the device and the key -> slot table consumes them there"""
        cur = torch.cuda.current_stream()
        sp = c_void_p(cur.cuda_stream)
        uq.run(kbuf, off)
        capi.check(L.recsdk_faae_admit_distinct_dev(faae.h, capi.CHANNEL_TRAIN, p_uk, p_cnt, p_uo, 1, batch,
                                                    c_void_p(ts.data_ptr()), sp))
        capi.check(L.recsdk_tables_key2offset(tg.h, p_uk, p_uo, 1, batch, capi.CHANNEL_TRAIN, sp))
        if beside:
            ev_fork.record(cur)
            s_evict.wait_event(ev_fork)
            evict(c_void_p(s_evict.cuda_stream))
            ev_join.record(s_evict)
        capi.check(L.recsdk_gather_unique(rows_h.h, uq.h, p_uk, c_void_p(out.data_ptr()), sp))
        capi.check(L.recsdk_sparse_apply(rows_h.h, uq.h, p_uk, c_void_p(grad.data_ptr()), capi.OPT_ADAM, 1e-3, 0.9,
                                         0.999, 1e-8, 0.0, sp))
        if beside:
            cur.wait_event(ev_join)
        else:
            evict(sp)

    def eager(i):
        kbuf.copy_(keys[i])
        ts.fill_(i)
        step(i)

    R = dim * 4
    if args.steps < 6:
        raise ValueError("c4 needs at least 6 steps: half of them issued eagerly, two untimed replays, the rest replayed")
    half = args.steps // 2
    elapsed = _timed(torch, eager, args.warmup, half)
    U = uq.total()
    nbytes = 12 * batch + 2 * R * batch + 48 * U + 7 * R * U
    workload = ("dynamic expansion: dim 32, 200M slots, batch 131072 (70 % Zipf(1.2) of 10M + 30 % fresh), admit >= 2, "
                "evict idle > 20, gather + Adam")
    # hash probes: one into the dedup scratch per key, one into the admission history and at most one into the
    # key -> slot table per distinct key (a 200M-slot table is probe-latency bound, not bandwidth bound)
    _line("C4", workload, batch, nbytes, half, elapsed,
          {"distinct_keys_last_step": U, "probes_per_s": round((batch + 2 * U) / (elapsed / half), 1),
           "schedule": "eviction beside gather + update on a second stream" if beside else "one stream",
           "note": "issued call by call from the host; eviction every step, its keys and count stay on the device"})
    # the same step recorded once into a HIP graph and replayed on the following batches
    g = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        # in one line: as a second branch of the graph the eviction made the replay slower (0.225 against 0.209 ms)
        step(0, beside=False)

    def replay(i):
        kbuf.copy_(keys[i])
        ts.fill_(i)
        g.replay()

    first = args.warmup + half
    for i in range(first, first + 2):
        replay(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(first + 2, nb):
        replay(i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    n_rep = nb - first - 2
    U = uq.total()
    _line("C4", "the same step as a HIP graph replay", batch, 12 * batch + 2 * R * batch + 48 * U + 7 * R * U, n_rep,
          elapsed, {"distinct_keys_last_step": U, "probes_per_s": round((batch + 2 * U) / (elapsed / n_rep), 1),
                    "schedule": "one stream"})


def run_c5(args, torch, capi, host, synth):
    dev = "cuda:0"
    T, batch, dim, cache_rows = 26, 65536, 64, 20_000_000
    ext = 2 * dim                                           # [w | Adagrad accumulator]
    host_rows = args.host_rows
    n = T * batch
    rng = np.random.default_rng(0)
    # two batches more than are gathered and updated: the stages that run ahead keep running ahead to the end of the
    # timed region, which then holds as many passes of every stage as it has steps
    nb = args.warmup + args.steps + 2
    sampler = synth.ZipfSampler(1.05, host_rows)            # one cumulative table for all batches
    keys = [torch.from_numpy(synth.splitmix64(sampler.ranks(rng, n).astype(np.uint64)).astype(np.int64)).to(dev)
            for _ in range(nb)]
    del sampler
    off = torch.tensor([0, n], dtype=torch.int64, device=dev)
    cache = torch.zeros((cache_rows, ext), device=dev)
    flat = cache.view(-1)
    rows_h = host.Rows(dim, [cache], [flat[dim:]], None, [ext])
    grad = torch.randn((n, dim), device=dev) * 1e-3
    out = torch.empty((n, dim), device=dev)
    t0 = time.perf_counter()
    # weights N(0, 0.01) with --normal-init: the reference's initializer is ONE sequential stream per initializer object
    # (std::normal_distribution over std::default_random_engine); the library produces that very stream in pieces on
    # the host's cores, which then bounds the step: some 130 k rows are created per batch
    w_init = ((capi.INIT_RANDOM_NORMAL, 0, dim, 0.0, 0.01, 0, 1.0) if args.normal_init else
              (capi.INIT_CONSTANT, 0, dim, 0.01, 0.0, 0, 1.0))
    store = host.EmbLocalTable(host_rows, ext, [w_init, (capi.INIT_CONSTANT, dim, dim, 0.1, 0.0, 0, 1.0)])
    print(f"[c5] pinned host arena of {host_rows * ext * 4 / 2**30:.1f} GiB in {time.perf_counter() - t0:.1f} s",
          file=sys.stderr, flush=True)
    # batch i uses set i % 3 of the dedup handles and lists: three batches are in flight in the default schedule
    # multiplicities come with the position lists: collecting them in the insert kernel costs one device atomic per
    # block and key, and on ONE table whose hottest keys are in every block those pile up on a few entries (insert
    # 402 -> 131 us)
    uqs = [host.Unique(n, 1, early_counts=False) for _ in range(3)]
    om = host.OffsetMapper(cache_rows, max_keys=n)
    swapped = [0, 0]
    lists = [None] * 3

    L = capi.lib()
    p_uk = [c_void_p() for _ in range(3)]
    for b in range(3):
        capi.check(L.recsdk_unique_results(uqs[b].h, ctypes.byref(p_uk[b]), None, None, None))
    plan_bufs = [[torch.empty(n, dtype=torch.int64, device=dev) for _ in range(4)] for _ in range(3)]

    def index(i):
        """dedup and cache plan of batch i: distinct keys -> slots IN PLACE in the dedup handle's own array (no copy of
        keys, inverse or counts, and no wait for the position lists, which only the update reads), and the lists of rows
        to move.  Two values return to the host: the number of distinct keys and the lengths of the lists."""
        b = i % 3
        uqs[b].run(keys[i], off)
        u = uqs[b].total()
        sp = c_void_p(torch.cuda.current_stream().cuda_stream)
        bufs = plan_bufs[b]
        capi.check(L.recsdk_om_compute(om.h, p_uk[b], u, *[c_void_p(x.data_ptr()) for x in bufs], sp))
        si, so, _, _ = om.counts()
        lists[b] = (bufs[0][:si], bufs[1][:si], bufs[2][:so], bufs[3][:so])     # the key lists stay on the device
        if args.warmup <= i < args.warmup + args.steps:          # the timed batches only
            swapped[0] += si
            swapped[1] += so

    def move(i):
        """rows of batch i's victims to the host, rows of its missing keys into their slots"""
        swapin_keys, swapin_pos, swapout_keys, swapout_pos = lists[i % 3]
        if args.swaps_in_turn:
            if swapout_keys.numel():
                store.swap_out(swapout_keys, swapout_pos, cache)
            if swapin_keys.numel():
                store.swap_in(swapin_keys, swapin_pos, cache)
        else:
            store.swap(swapout_keys, swapout_pos, swapin_keys, swapin_pos, cache)   # both ways over the link at once

    def rows(i):
        """forward gather and Adagrad update of batch i"""
        b = i % 3
        sp = c_void_p(torch.cuda.current_stream().cuda_stream)
        capi.check(L.recsdk_gather_unique(rows_h.h, uqs[b].h, p_uk[b], c_void_p(out.data_ptr()), sp))
        capi.check(L.recsdk_sparse_apply(rows_h.h, uqs[b].h, p_uk[b], c_void_p(grad.data_ptr()), capi.OPT_ADAGRAD, 0.01,
                                         0.9, 0.999, 1e-8, 0.0, sp))

    last = nb
    if args.serial:
        def step(i):
            index(i)
            move(i)
            rows(i)
        schedule = "one stream"
    else:
        # Three stages on three streams: while batch i is gathered and updated, the rows of batch i + 1 cross the host
        # link and batch i + 2 is deduplicated and planned.  What makes that legal: the planner never hands out a slot
        # that the call before it needed, so the rows that move for batch i + 1 are not rows batch i touches; a slot
        # batch i - 1 used may be a victim of batch i + 1, so its move waits for the rows stage of batch i - 1; the
        # planner itself reads no rows.  --two-stages keeps the index stage on the stream of the move stage.
        s_index = torch.cuda.Stream()
        s_move = s_index if args.two_stages else torch.cuda.Stream()
        s_rows = torch.cuda.Stream()
        ev_index = [torch.cuda.Event() for _ in range(3)]
        ev_move = [torch.cuda.Event() for _ in range(3)]
        ev_rows = [torch.cuda.Event() for _ in range(3)]

        def do_index(i):
            with torch.cuda.stream(s_index):
                if i >= 3:
                    s_index.wait_event(ev_rows[i % 3])    # rows(i - 3) is done with this set of dedup buffers
                index(i)
                ev_index[i % 3].record(s_index)

        def do_move(i):
            with torch.cuda.stream(s_move):
                s_move.wait_event(ev_index[i % 3])
                if i >= 2:
                    s_move.wait_event(ev_rows[(i - 2) % 3])   # the updates of this batch's victims are complete
                move(i)
                ev_move[i % 3].record(s_move)

        ahead = 1 if args.two_stages else 2                # batches the index stage runs ahead of the rows stage

        # The rows stage of batch i starts when the link kernel of batch i + 1 starts, not when the move of batch i
        # ends: in between run the short kernels that prepare the move of batch i + 1 (host rows of its keys, the copy
        # aside of its victims' rows), during which the link is idle, and beside the gather and the update they took
        # twice as long.  --rows-beside-prep keeps the old order.
        ev_link = None
        if ahead == 2 and not args.rows_beside_prep and not args.swaps_in_turn:
            ev_link = torch.cuda.Event()
            ev_link.record(s_move)
            store.on_link_start(ev_link)

        def do_rows(i):
            with torch.cuda.stream(s_rows):
                s_rows.wait_event(ev_move[i % 3])
                if ev_link is not None:
                    s_rows.wait_event(ev_link)
                rows(i)
                ev_rows[i % 3].record(s_rows)

        def step(i):
            if i == 0:
                do_index(0)
                do_move(0)
                if ahead == 2 and last > 1:
                    do_index(1)
            if ahead == 1:
                do_rows(i)
                if i + 1 < last:
                    do_index(i + 1)
                    do_move(i + 1)
            else:
                if ev_link is None:
                    do_rows(i)
                if i + 1 < last:
                    do_move(i + 1)
                if ev_link is not None:
                    do_rows(i)
                if i + 2 < last:
                    do_index(i + 2)
        schedule = ("index and move of the next batch on a second stream" if args.two_stages else
                    "three stages on three streams: rows of batch i, host link of batch i + 1, dedup and plan of batch i + 2")
    elapsed = _timed(torch, step, args.warmup, args.steps)
    U = uqs[(args.warmup + args.steps - 1) % 3].total()
    R = dim * 4
    per_step_swaps = (swapped[0] + swapped[1]) / args.steps
    _line("C5", f"host-backed cache: {host_rows / 1e6:.0f}M x 64 host rows "
          f"({'weights N(0, 0.01) from the host stream' if args.normal_init else 'constant initializer'}), 20M-row HBM cache, "
          "batch 65536 x 26, Zipf(1.05): unique, plan, swap, gather + Adagrad", n,
          12 * n + 2 * R * n + 5 * R * U + per_step_swaps * 2 * ext * 4, args.steps, elapsed,
          {"distinct_keys_last_step": U, "rows_swapped_per_step": int(per_step_swaps),
           "host_link_GBs_each_way": round(per_step_swaps / 2 * ext * 4 / (elapsed / args.steps) / 1e9, 1),
           "host_link_frac_of_64GBs": round(per_step_swaps / 2 * ext * 4 / (elapsed / args.steps) / 1e9 / HOST_LINK_GBS, 3),
           # this step is bound by the host link, not by HBM: rows moved each way against the link's 64 GB/s
           "roofline": {"bound": "host link", "scope": "whole step: rows moved each way over the host link",
                        "achieved": round(per_step_swaps / 2 * ext * 4 / (elapsed / args.steps) / 1e9, 1),
                        "peak": HOST_LINK_GBS, "unit": "GB/s",
                        "frac": round(per_step_swaps / 2 * ext * 4 / (elapsed / args.steps) / 1e9 / HOST_LINK_GBS, 4),
                        "traffic": None},
           "rows_in_per_step": swapped[0] // args.steps, "rows_out_per_step": swapped[1] // args.steps,
           "schedule": schedule,
           "note": "the planner's key lists stay on the device, the rows cross the host link once each way"})


def bounds_inputs(synth):
    """The inputs of the boundary timings: the ids of one DLRM-style batch (26 tables x 65536, Zipf(1.05)) and the
    distinct keys of 20 host-backed-cache batches (65536 x 26 keys each, Zipf(1.05) over 100 M rows)."""
    T, B = 26, 65536
    rng = np.random.default_rng(0)
    rows = synth.dlrm_table_rows(T)
    ids = np.concatenate([synth.zipf_keys(rng, 1.05, int(rows[t]), B, table=t) for t in range(T)]).astype(np.int64)
    sampler = synth.ZipfSampler(1.05, 100_000_000)
    batches = [np.unique(synth.splitmix64(sampler.ranks(rng, T * B).astype(np.uint64)).astype(np.int64))
               for _ in range(20)]
    return ids, batches


BOUNDS_CACHE_SLOTS = 4_000_000
BOUNDS_SWAP_KEYS = 1_000_000


def run_bounds(args, torch, capi, host, synth, inputs=None):
    """What the drop-in boundaries cost a reference caller, host vectors in and out (every call uploads its input, runs
    the kernels, waits and downloads the results):
      DoEnhancedUnique            lib_ock_ctr_common.so, one call per table of a DLRM-style batch (26 x 65536 ids),
                                  as KeyProcess calls it (key_process.cpp:205-251)
      GetSwapPairsAndKey2Offset   the same library, the distinct keys of a host-backed-cache batch against a full
                                  4 M-slot cache, as HybridMgmt calls it (hybrid_mgmt.cpp:545-560)
      ComputeSwapInfo             libembcache_hip.so, Embcache::SwapManager on a 1 M-key batch against a full 4 M-slot
                                  cache, as EmbcacheManager calls it (embcache_manager.cpp:89-282)
    The libraries are built against the reference's headers where a reference checkout is present; without them a
    measurement is reported as missing.  bench.py times the CPU restatement on the same inputs beside these."""
    import os
    import subprocess
    import tempfile

    from recsdk_amd.embcache import build as embcache_build
    from recsdk_amd.plugin import build as plugin_build
    T, B = 26, 65536
    ids, batches = inputs if inputs is not None else bounds_inputs(synth)
    K = len(batches)

    def med(v):
        return sorted(v)[len(v) // 2]

    # ---- the AccCTR plugin through the reference's factory
    plugin = {"DoEnhancedUnique": None, "GetSwapPairsAndKey2Offset": None}
    if os.path.isfile(plugin_build.DRIVER) and os.path.isfile(plugin_build.PLUGIN):
        with tempfile.NamedTemporaryFile(suffix=".bin", delete=False) as f:
            path = f.name
            np.asarray([T, B, K], dtype=np.int64).tofile(f)
            ids.tofile(f)
            for b in batches:
                np.asarray([b.size], dtype=np.int64).tofile(f)
                b.tofile(f)
        env = dict(os.environ)
        env["LD_LIBRARY_PATH"] = plugin_build.OUT + os.pathsep + env.get("LD_LIBRARY_PATH", "")
        try:
            run = subprocess.run([plugin_build.DRIVER, "--bench", path], env=env, capture_output=True, text=True,
                                 timeout=600)
        finally:
            os.unlink(path)
        for ln in run.stdout.splitlines():
            w = ln.split()
            if len(w) >= 5 and w[0] == "bench":
                plugin[w[1]] = float(w[3])
        if run.returncode != 0:
            plugin["error"] = (run.stdout[-300:] + run.stderr[-300:]).strip()
    extra = {"error": plugin["error"]} if "error" in plugin else {}
    _line("bounds", "DoEnhancedUnique (lib_ock_ctr_common.so), 26 calls of 65536 ids, 8 shards, id counts; host vectors "
          "in and out", T * B, 8 * T * B + 4 * T * B, 1,
          (plugin["DoEnhancedUnique"] or float("nan")) * 1e-6,
          dict(extra, call="DoEnhancedUnique", us_per_batch=plugin["DoEnhancedUnique"]))
    _line("bounds", "GetSwapPairsAndKey2Offset (lib_ock_ctr_common.so), the distinct keys of one host-backed-cache batch, "
          "4 M-slot cache full; host vectors in and out", int(batches[-1].size), 16 * int(batches[-1].size), 1,
          (plugin["GetSwapPairsAndKey2Offset"] or float("nan")) * 1e-6,
          dict(extra, call="GetSwapPairsAndKey2Offset", us_per_call=plugin["GetSwapPairsAndKey2Offset"]))

    # ---- Embcache::SwapManager through the class compiled against the reference's header
    swap_us = None
    if os.path.isfile(embcache_build.SHIM):
        os.environ.setdefault("RECSDK_EMBCACHE_MAX_KEYS", str(1 << 20))
        lib = ctypes.CDLL(embcache_build.SHIM)
        P, I64 = ctypes.c_void_p, ctypes.c_int64
        lib.dropin_swap_create.restype, lib.dropin_swap_create.argtypes = P, [I64, I64]
        lib.dropin_swap_destroy.argtypes = [P]
        lib.dropin_swap_compute.restype, lib.dropin_swap_compute.argtypes = ctypes.c_int32, [P, P, I64]
        h = lib.dropin_swap_create(BOUNDS_CACHE_SLOTS, 0)
        t_gpu = []
        for k in range(K):
            b = np.ascontiguousarray(batches[k][:BOUNDS_SWAP_KEYS])
            t0 = time.perf_counter()
            rc = lib.dropin_swap_compute(h, b.ctypes.data_as(P), b.size)
            t_gpu.append(time.perf_counter() - t0)
            if rc != 0:
                t_gpu = None
                break
        lib.dropin_swap_destroy(h)
        if t_gpu:
            swap_us = med(t_gpu[-8:]) * 1e6
    _line("bounds", "Embcache::SwapManager::ComputeSwapInfo (libembcache_hip.so), 1 M distinct keys, 4 M-slot cache full; "
          "host vectors in and out", BOUNDS_SWAP_KEYS, 16 * BOUNDS_SWAP_KEYS, 1, (swap_us or float("nan")) * 1e-6,
          {"call": "ComputeSwapInfo", "us_per_call": None if swap_us is None else round(swap_us, 1)})


def make_parser():
    """The command line of this module; `default_args` hands its defaults to callers that run a configuration
    in-process, so the two never drift apart."""
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", default="all", choices=["c1", "c3", "c4", "c5", "ops", "keys", "bounds", "all"])
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default 20; c4: 100, as the configuration says)")
    ap.add_argument("--two-stages", action="store_true",
                    help="c5: dedup, plan and move of the next batch on ONE second stream (default: three stages)")
    ap.add_argument("--swaps-in-turn", action="store_true",
                    help="c5: swap rows out, then in, as two calls (default: one call that moves both ways at once)")
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps first (default 3; c5: 150, so that the HBM cache is full and every step swaps rows "
                         "out as well as in)")
    ap.add_argument("--host-rows", type=int, default=100_000_000,
                    help="c5: rows of the pinned host table (512 B each with the Adagrad accumulator)")
    ap.add_argument("--serial", action="store_true", help="c5: plan, swaps and row kernels of a batch on one stream")
    ap.add_argument("--normal-init", action="store_true",
                    help="c5: new rows take N(0, 0.01) weights from the initializer stream (default: constants)")
    ap.add_argument("--rows-beside-prep", action="store_true",
                    help="c5: start the rows stage of a batch when its move ends (default: when the link kernel of the "
                         "next batch starts)")
    ap.add_argument("--evict-in-line", action="store_true",
                    help="c4: the eviction of a step after its update on the same stream (default: on a second stream "
                         "beside the gather and the update)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="end with one device-to-device copy of 1 GiB: the known traffic a counter run scales its "
                         "FETCH_SIZE / WRITE_SIZE readings by")
    return ap


def default_args(**overrides):
    """A namespace with every option at its default (what `run_c1` … `run_c5` read), with `overrides` applied; an
    override that names no option of the parser is an error."""
    args = make_parser().parse_args([])
    for k, v in overrides.items():
        if not hasattr(args, k):
            raise AttributeError(f"config_bench has no option {k!r}")
        setattr(args, k, v)
    return args


def main():
    ap = make_parser()
    args = ap.parse_args()
    import torch

    from . import capi, host, synth

    capi.lib()
    torch.cuda.set_device(0)
    runs = {"c1": run_c1, "c3": run_c3, "c4": run_c4, "c5": run_c5, "ops": run_ops, "keys": run_keys,
            "bounds": run_bounds}
    steps = args.steps
    warmup = args.warmup
    for name in (runs if args.config == "all" else [args.config]):
        args.steps = steps if steps is not None else (100 if name == "c4" else 20)
        args.warmup = warmup if warmup is not None else (150 if name == "c5" else 3)
        runs[name](args, torch, capi, host, synth)
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
    if args.calib_copy:
        a = torch.empty(1 << 28, device="cuda:0")
        b = torch.empty(1 << 28, device="cuda:0")
        b.copy_(a)
        torch.cuda.synchronize()


if __name__ == "__main__":
    main()
