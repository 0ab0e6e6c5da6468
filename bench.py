#!/usr/bin/env python3
"""Benchmark of the embedding hot path on one MI355X.

One "step" = preprocess(batch t) + push_pull(grad of batch t-1, dst of batch t) on synthetic keys that are
already resident in HBM, in steady state (every timed step both pushes and pulls).  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg2] [--no-cpu]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="cfg2")
    ap.add_argument("--batches", type=int, default=4, help="distinct key batches cycled through")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink rows and samples (debugging only)")
    ap.add_argument("--samples", type=int, default=0,
                    help="samples per batch instead of the config's (the reference's script defaults to 2048, "
                         "tests/benchmark.py:74); the table keeps its size")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-steps", type=int, default=10,
                    help="full-size steps of the CPU baseline leg (about 12 core-seconds at the default)")
    ap.add_argument("--no-stage-timing", action="store_true")
    ap.add_argument("--no-variants", action="store_true",
                    help="skip the extra passes (literal call protocol, permuted ids): for profiles of the headline alone")
    ap.add_argument("--no-others", action="store_true",
                    help="skip the short passes over the other configurations that the default cfg2 run appends as "
                         "`other_configs`")
    ap.add_argument("--other-steps", type=int, default=10, help="timed steps of each `other_configs` pass")
    ap.add_argument("--host-keys", action="store_true",
                    help="hand the ids over as pageable host buffers (adds their transfer to the step)")
    ap.add_argument("--pooled", action="store_true",
                    help="multi-hot configs: sum-pool every bag of `hot` ids (hctr_push_pull_pooled): one gradient row "
                         "and one output row per bag instead of per id")
    ap.add_argument("--bag", type=int, default=0, help="--pooled: bag size (default: the config's ids per field)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="only run the library's plain 1 GiB copy kernel (scale factor of the HBM byte counters)")
    ap.add_argument("--active-peers", action="store_true",
                    help="sharded configs: every rank caches hot rows and feeds batches (default: rank 0 only)")
    ap.add_argument("--pull-bound", type=int, default=0, help="sharded configs: staleness bound of pulls")
    ap.add_argument("--push-bound", type=int, default=0, help="sharded configs: staleness bound of pushes")
    ap.add_argument("--layout", choices=("random", "partitioned"), default="random",
                    help="sharded configs: owners drawn uniformly and the hottest rows cached (random), or owners, "
                         "cache contents and per-rank batches from the offline partitioner run on a click log")
    ap.add_argument("--partition", action="store_true",
                    help="time the offline partitioner on a click log over the cfg2 table instead of the training step")
    ap.add_argument("--part-samples", type=int, default=1_000_000, help="--partition: samples of the click log")
    ap.add_argument("--part-rounds", type=int, default=2, help="--partition: rounds of both sweeps")
    ap.add_argument("--part-cache-frac", type=float, default=0.10,
                    help="--partition: cache candidates kept per part, as a fraction of the table")
    return ap.parse_args()


def cpu_baseline(cfg, ks, batches, width, lr, steps):
    """Times the CPU restatement of the same step (the parity oracle, all host threads it is given) on a
    bounded sample of the same workload: same table size, same batches, Zero-initialised table."""
    from oracle import oracle as orc
    rows = ks.rows
    root = np.zeros(rows, np.uint8)
    o = orc.Oracle(1, rows, width, 0, 0, root, [np.arange(rows, dtype=np.int64)], init=("Zero", 0.0, 0.0),
                   learning_rate=lr)
    o.set_parallel(True)
    n = batches[0].shape[0]
    rng = np.random.default_rng(7)
    grad = rng.normal(0, 1e-3, size=(n, width)).astype(np.float32)
    dst = np.empty((n, width), np.float32)
    o.preprocess_raw([batches[0]])
    o.push_pull_into([None], [dst])                       # warm-up: first pull, nothing to push yet
    for b in range(1, len(batches) + 2):                  # ... then every batch once: the rows they reach are paged in
        o.preprocess_raw([batches[b % len(batches)]])
        o.push_pull_into([grad], [dst])
    t0 = time.perf_counter()
    for s in range(steps):
        o.preprocess_raw([batches[(s + 2) % len(batches)]])
        o.push_pull_into([grad], [dst])
    dt = time.perf_counter() - t0
    cores = o.num_threads()
    o.set_parallel(False)                                 # the same steps on one host thread
    one = max(1, steps // 5)
    t0 = time.perf_counter()
    for s in range(one):
        o.preprocess_raw([batches[(s + 2) % len(batches)]])
        o.push_pull_into([grad], [dst])
    dt1 = time.perf_counter() - t0
    o.close()
    return dict(value=n * steps / dt, unit="IDs/s", cores=cores, kind="port",
                ms_per_step=1e3 * dt / steps,
                single_thread={"value": n * one / dt1, "ms_per_step": 1e3 * dt1 / one, "steps": one},
                sample="%d full-size steps (%d keys each, %d-row x %d table, zero-initialised) of the same batches, "
                       "OpenMP oracle, warm" % (steps, n, rows, width))


def cpu_baseline_sharded(ks, R, width, lr, bounds, root, storage, batches, active, steps):
    """Times the CPU oracle with the same R logical ranks on the same batches (bounded number of steps, table
    zero-initialised so that only the rows the batches reach cost memory)."""
    from oracle import oracle as orc
    o = orc.Oracle(R, ks.rows, width, bounds[0], bounds[1], root, storage, init=("Zero", 0.0, 0.0), learning_rate=lr)
    o.set_parallel(True)
    nb = len(batches[active[0]])
    n = batches[active[0]][0].shape[0]
    empty = np.zeros(0, np.int64)
    rng = np.random.default_rng(7)
    grad = rng.normal(0, 1e-3, size=(n, width)).astype(np.float32)

    def step(i, with_grad=True):
        o.preprocess([batches[r][i % nb] if r in batches else empty for r in range(R)])
        o.push_pull([grad if (r in batches and with_grad) else None for r in range(R)])

    step(0, False)
    for i in range(1, nb + 1):                            # warm: every batch's rows have been touched once
        step(i)
    t0 = time.perf_counter()
    for i in range(steps):
        step(nb + 1 + i)
    dt = time.perf_counter() - t0
    cores = o.num_threads()
    o.close()
    keys = n * len(active)
    return dict(value=keys * steps / dt, unit="IDs/s", cores=cores, kind="port", ms_per_step=1e3 * dt / steps,
                sample="%d full-size steps of the same batches (%d keys per step over %d feeding ranks, %d logical "
                       "ranks, %d-row x %d table, zero-initialised), OpenMP oracle, warm" %
                       (steps, keys, len(active), R, ks.rows, width))


def reference_partitioner():
    """The reference's partitioner built from its own sources WITH OpenMP (as shipped), or None."""
    import importlib.util
    d = os.path.join(ROOT, "oracle", "_ref", "partition_omp")
    so = [f for f in os.listdir(d) if f.startswith("hetuCTR_partition")] if os.path.isdir(d) else []
    if not so:
        return None
    spec = importlib.util.spec_from_file_location("hetuCTR_partition", os.path.join(d, so[0]))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def click_log(workloads, samples, scale=1.0):
    """samples x 26 ids over the cfg2 table (per-field Zipf), as int32."""
    cfg = dict(workloads.CONFIGS["cfg2"])
    cfg["samples"] = samples
    ks = workloads.KeyStream(cfg, seed=0, scale=scale)
    data = ks.batch().reshape(-1, ks.fields * ks.hot).astype(np.int32)
    ks.release_tables()
    return data, ks.rows


def main_partition(a):
    """Offline partitioner: construction, `rounds` x (sample sweep, embedding sweep, communication cost) on the host,
    then the cache candidates of every part on the GPU.  The CPU leg runs the reference's own sources (OpenMP build)
    through the same steps of its driver script on a quarter-size sample of the same log."""
    import torch
    from hetuctr_amd import workloads
    import hetuctr_amd.partition as hp
    P, B = 8, 8192
    data, rows = click_log(workloads, a.part_samples, a.scale)
    nd = data.shape[0]
    mat = hp.get_comm_mat(P, P)
    t0 = time.perf_counter()
    p = hp.partition(data, mat, P, B)
    create_s = time.perf_counter() - t0
    cost0 = float((p.get_communication() * mat).sum())
    rounds, costs = [], []
    for r in range(a.part_rounds):
        t0 = time.perf_counter()
        p.refine_data()
        t1 = time.perf_counter()
        p.refine_embed()
        t2 = time.perf_counter()
        c = p.get_communication()
        t3 = time.perf_counter()
        rounds.append({"sample_sweep_s": t1 - t0, "embedding_sweep_s": t2 - t1, "communication_s": t3 - t2})
        costs.append(float((c * mat).sum()))
    refine_s = sum(sum(r.values()) for r in rounds)
    keep = int(a.part_cache_frac * p.n_embed)
    torch.cuda.synchronize()
    p.cache_lists(1024)                                           # warm-up: kernels loaded
    t0 = time.perf_counter()
    lists, kernel_ms = p.cache_lists(keep)
    lists_s = time.perf_counter() - t0
    list_bytes = workloads.cache_list_bytes(p.n_embed, P, keep)
    gbs = list_bytes / (kernel_ms * 1e-3) / 1e9
    # measured HBM bytes of the same kernels at the default size (rocprofv3 --pmc runs summarised under profiles/)
    measured = None
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath) and a.scale == 1.0 and a.part_samples == 1_000_000 and a.part_cache_frac == 0.10:
        measured = json.load(open(tpath)).get("partition", {}).get("cache_lists")
    out = {
        "metric": "partitioner: samples refined per second (one round = sample sweep + embedding sweep + cost)",
        "value": nd * a.part_rounds / refine_s, "unit": "samples/s", "n_gpus": 1, "steps": a.part_rounds, "warmup": 0,
        "ms_per_step": 1e3 * refine_s / a.part_rounds, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "click log of %d samples x %d slots over the %d-id cfg2 table (per-field Zipf 1.05), "
                               "%d parts, batch %d, cost 0.1 between all parts" % (nd, data.shape[1], rows, P, B),
                   "n_embed": p.n_embed},
        "construction_s": create_s, "rounds": rounds, "cost_initial": cost0, "cost_after_round": costs,
        "cache_lists": {"kept_per_part": keep, "wall_s_with_upload_and_download": lists_s, "kernel_ms": kernel_ms},
        "roofline": {"bound": "hbm", "kernel": "priority keys + %d radix sorts + list emit" % P, "achieved": gbs,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "traffic": measured,
                     "algorithmic_bytes": int(list_bytes)},
    }
    p.close()
    del lists
    if not a.no_cpu:
        ref = reference_partitioner()
        if ref is None:
            out["cpu_baseline"] = {"value": None, "error": "oracle/_ref/partition_omp is not built"}
        else:
            sdata, srows = click_log(workloads, a.part_samples, a.scale * 0.25)
            t0 = time.perf_counter()
            rp = ref.partition(sdata, mat, P, B)
            t1 = time.perf_counter()
            rp.refine_data()
            rp.refine_embed()
            rp.get_communication()
            t2 = time.perf_counter()
            pr = rp.get_priority()
            owner = rp.get_result()[1]
            for i in range(P):                                    # experimental/partition.py:53-57
                idxs = np.where(owner == i)[0]
                pr[i][idxs] = -1
                np.argsort(pr[i])[len(idxs):][::-1]
            t3 = time.perf_counter()
            out["cpu_baseline"] = dict(
                value=sdata.shape[0] / (t2 - t1), unit="samples/s", cores=min(16, os.cpu_count() or 1),
                kind="reference", construction_s=t1 - t0, round_s=t2 - t1, priority_and_sort_s=t3 - t2,
                sample="the reference's partition.cc + pybind.cc compiled with -O3 -fopenmp, one round and the "
                       "script's priority sort on a quarter-size log (%d samples, %d ids)" % (sdata.shape[0], srows))
    print(json.dumps(out), flush=True)


def run_sharded(a, cfg, steps, warmup, with_cpu, stage_timing=True, name=None):
    """cfg3: the shards of an 8-way partition live on this one GPU behind the loopback.  By default only rank 0 feeds
    batches and holds the hot-row cache; the seven peers own their rows and serve rank 0's pushes and queries with
    the real owner-side kernels (in a deployment that work runs on the other GPUs, here it is inside the step
    time).  With --active-peers every rank has a cache and feeds its own batches, so rows do go stale and get
    refreshed; the GPU then does the work of all eight ranks in turn and `value` counts all their keys."""
    import torch
    from hetuctr_amd import capi, workloads
    name = name or name
    R, width, lr = cfg["nrank"], cfg["width"], cfg["lr"]
    active = list(range(R)) if a.active_peers else [0]
    ks = workloads.KeyStream(cfg, seed=0, scale=a.scale)
    nb = max(2, a.batches)
    layout_info = None
    if a.layout == "partitioned":
        say = lambda m: print("[bench] " + m, file=sys.stderr, flush=True)
        root, storage, per_rank, layout_info = workloads.partitioned_layout(
            ks, R, cfg["cache_frac"], R * ks.samples * (nb + 1), ks.samples, rounds=3, cached_ranks=active, log=say)
        nb = min(nb, min(len(per_rank[r]) for r in active))
        assert nb >= 2, "the click log leaves a rank fewer than two full batches"
        batches = {r: per_rank[r][:nb] for r in active}
        del per_rank
    else:
        batches = {r: [ks.batch() for _ in range(nb)] for r in active}
        root, storage = workloads.shard_layout(ks, R, cfg["cache_frac"], cached_ranks=active)
    ks.release_tables()
    n = batches[0][0].shape[0]
    print("[bench] %s: %d rows x %d over %d shards, rank 0 owns %d and caches %d rows, %d keys/batch, ranks with "
          "batches: %s" % (name, ks.rows, width, R, int((root == 0).sum()),
                           storage[0].shape[0] - int((root == 0).sum()), n, active), file=sys.stderr, flush=True)
    torch.cuda.set_device(0)
    capi.seed(0)
    bounds = (a.pull_bound, a.push_bound)
    tables = [capi.Table(r, R, 0, "127.0.0.1", 23456, ks.rows, width, bounds[0], bounds[1], root, storage[r],
                         cfg["init"], lr, 0) for r in range(R)]
    dkeys = {r: [torch.from_numpy(b).cuda() for b in batches[r]] for r in active}
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    grad = torch.randn((n, width), device="cuda", generator=gen) * 1e-3
    dsts = {r: torch.empty((n, width), device="cuda") for r in active}
    torch.cuda.synchronize()
    counts = [n if r in dkeys else 0 for r in range(R)]
    gptr = [grad.data_ptr() if r in dkeys else 0 for r in range(R)]
    dptr = [dsts[r].data_ptr() if r in dkeys else 0 for r in range(R)]

    # the argument arrays of the two calls, one set per batch, built outside the loop
    calls = [capi.GroupStep(tables, [dkeys[r][b].data_ptr() if r in dkeys else 0 for r in range(R)], counts, gptr, dptr)
             for b in range(nb)]

    def step(i):
        c = calls[i % nb]
        c.preprocess()
        c.push_pull()

    w0 = max(warmup, 2) + nb
    for i in range(w0):
        step(i)
    # the timed pass: nothing but the two calls of every step
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(w0 + i)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    # the library's own device times of the two calls (a pass of its own: their events cost host time)
    pre_ms = pp_ms = 0.0
    tables[0].call_timing(True)
    for i in range(steps):
        step(w0 + i)
        p, q = tables[0].last_times()
        pre_ms += p
        pp_ms += q
    tables[0].call_timing(False)
    # how long each of the two calls holds the host (a pass of its own: the clock reads cost time)
    call_s = [0.0, 0.0]
    for i in range(steps):
        c = calls[(w0 + i) % nb]
        t1 = time.perf_counter()
        c.preprocess()
        t2 = time.perf_counter()
        c.push_pull()
        t3 = time.perf_counter()
        call_s[0] += t2 - t1
        call_s[1] += t3 - t2
    stages = None
    if stage_timing and not a.no_stage_timing:
        tables[0].stage_timing(True)
        for i in range(steps):
            step(w0 + steps + i)
        stages = {k: {"ms_per_step": v[0] / steps, "intervals_per_step": v[1] / steps}
                  for k, v in tables[0].stage_times().items() if v[1]}
        tables[0].stage_timing(False)
    k = min(steps, nb)                     # counters of a few more steps, outside the timed region
    acc = np.zeros(6)                        # per step, summed over the ranks: hit, miss, refreshed, pushed, returned, received
    us = 0.0
    for i in range(k):
        step(w0 + 2 * steps + i)
        for t in tables:
            acc += np.asarray(t.fetch(capi.STATS)[:6], dtype=np.float64) / k
        us += sum(float(tables[r].fetch(capi.SIZES)[1]) for r in active) / k
    hit, miss, refresh, pushed, served, received = acc
    ms_step = 1e3 * dt / steps
    keys_step = n * len(active)
    bytes_step = workloads.algorithmic_bytes(keys_step, us, width) + workloads.sharded_extra_bytes(
        width, hit + refresh, pushed, received, us, served, refresh)
    gbs = bytes_step / (ms_step * 1e-3) / 1e9
    out = {
        "metric": "sparse IDs/sec per train step (pull+push)", "value": keys_step * steps / dt, "unit": "IDs/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": ms_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: %d shards of a %d-row x %d fp32 table (%s) on one GPU behind the "
                               "loopback, ranks %s feed batches of %d keys (per-field Zipf %.2f) and cache %.0f%% of "
                               "their remote rows (%s), bounds pull/push %d/%d; the other ranks only serve" %
                               (name, R, ks.rows, width,
                                "uniform owners" if a.layout == "random" else "owners from the offline partitioner",
                                active, n, cfg["alpha"], 100 * cfg["cache_frac"],
                                "the hottest" if a.layout == "random" else "the partitioner's first candidates; "
                                "each rank's batches are the samples assigned to it", bounds[0], bounds[1]),
                   "layout": a.layout, "partitioner": layout_info,
                   "keys_per_step": keys_step, "unique_keys_per_step": us, "width": width, "rows": ks.rows},
        "cache_per_step_all_ranks": {"remote_unique_keys_hit": hit, "missed_not_cached": miss, "refreshed": refresh,
                                     "rows_pushed_to_owners": pushed, "rows_returned_by_owners": served},
        "device_ms_per_step": {"preprocess": pre_ms / steps, "push_pull": pp_ms / steps},
        "host_ms_per_call": {"preprocess": 1e3 * call_s[0] / steps, "push_pull": 1e3 * call_s[1] / steps},
        "step_hbm": {"algorithmic_bytes": int(bytes_step), "achieved_GBps": gbs, "frac": gbs / HBM_PEAK_GBS},
        "roofline": {"bound": "hbm", "kernel": "whole step (all shards' kernels)", "achieved": gbs, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "traffic": None, "avg_ms": ms_step,
                     "algorithmic_bytes": int(bytes_step)},
        "stages_all_shards": stages,
        "cpu_baseline": None,
    }
    for t in tables:
        t.close()
    # measured HBM bytes per launch of the dominant kernels (rocprofv3 --pmc runs of this same command, summarised
    # under profiles/), valid for the default invocation only
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath) and a.scale == 1.0 and not a.active_peers and a.layout == "random" and bounds == (0, 0):
        measured = json.load(open(tpath)).get(name)
        if measured:
            out["roofline"]["traffic"] = measured.get("whole_step")
            out["kernels"] = {k: v for k, v in measured.items() if k != "whole_step"}
    del dkeys, grad, dsts
    torch.cuda.empty_cache()
    if with_cpu:
        try:
            out["cpu_baseline"] = cpu_baseline_sharded(ks, R, width, lr, bounds, root, storage, batches, active,
                                                       a.cpu_steps)
        except Exception as e:  # the GPU line stands without it
            out["cpu_baseline"] = {"value": None, "error": str(e)}
    return out


def quick_single(name, cfg, steps, warmup, host_keys=False, stage_timing=True):
    """A short pass over one single-shard configuration: `warmup` untimed steps, `steps` timed ones (nothing but the
    two calls in the loop), then the same steps with stage events for the push and gather kernels alone.  The table
    and every buffer are released before it returns."""
    import torch
    from hetuctr_amd import capi, workloads
    width, lr = cfg["width"], cfg["lr"]
    ks = workloads.KeyStream(cfg, seed=0)
    batches = [ks.batch() for _ in range(3)]
    ks.release_tables()
    n = batches[0].shape[0]
    capi.seed(0)
    table = capi.Table(0, 1, 0, "127.0.0.1", 23456, ks.rows, width, 0, 0, np.zeros(ks.rows, np.uint8),
                       np.arange(ks.rows, dtype=np.int64), cfg["init"], lr, 0)
    dkeys = [torch.from_numpy(b).cuda() for b in batches]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    grad = torch.randn((n, width), device="cuda", generator=gen) * 1e-3
    dst = torch.empty((n, width), device="cuda")
    torch.cuda.synchronize()
    ptrs = [b.ctypes.data for b in batches] if host_keys else [d.data_ptr() for d in dkeys]

    def step(i):
        table.preprocess(ptrs[i % len(ptrs)], n)
        table.push_pull(grad.data_ptr(), dst.data_ptr())

    us = []
    for i in range(max(warmup, len(ptrs) + 1)):
        step(i)
        us.append(int(table.fetch(capi.SIZES)[1]))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    ms = 1e3 * (time.perf_counter() - t0) / steps
    u = float(np.mean(us[-len(ptrs):]))
    res = {"workload": "%s: %d-row x %d fp32 table, %d samples x %d fields x %d ids = %d keys per batch, %s, ids handed "
                       "over in %s" % (name, ks.rows, width, ks.samples, ks.fields, ks.hot, n,
                                       "uniform ids" if cfg["alpha"] is None else "per-field Zipf %.2f" % cfg["alpha"],
                                       "pageable host memory" if host_keys else "HBM"),
           "steps": steps, "warmup": warmup, "ms_per_step": ms, "value": n / (ms * 1e-3), "keys_per_step": n,
           "unique_keys_per_step": u,
           "step_hbm_frac": workloads.algorithmic_bytes(n, u, width) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    if stage_timing:
        table.stage_timing(True)
        for i in range(steps):
            step(i)
        st = table.stage_times()
        table.stage_timing(False)
        res["stage_ms"] = {k: v[0] / max(v[1], 1) for k, v in st.items() if v[1]}
        for k, kern in (("segment_sum_apply", "push_fused"), ("gather", "gather")):
            if k in res["stage_ms"]:
                res[kern + "_frac"] = (workloads.stage_bytes(k, n, u, n, u, width) / (res["stage_ms"][k] * 1e-3) / 1e9 /
                                       HBM_PEAK_GBS)
    table.close()
    del dkeys, grad, dst
    torch.cuda.empty_cache()
    return res


def other_configs(a):
    """Short passes (no CPU leg) over every other configuration the headline is not quoted on, the reference's own
    default batch (tests/benchmark.py:74-75: 2048 samples x 26 fields) and cfg2 with the ids in pageable host memory,
    as every script of the reference hands them over (tests/benchmark.py:63)."""
    from hetuctr_amd import workloads
    out = {}
    K, W = a.other_steps, 5

    def run(name, f):
        t0 = time.perf_counter()
        try:
            out[name] = f()
        except Exception as e:  # the headline stands without it
            out[name] = {"error": "%s: %s" % (type(e).__name__, e)}
        print("[bench] other_configs.%s done in %.1fs" % (name, time.perf_counter() - t0), file=sys.stderr, flush=True)

    small = dict(workloads.CONFIGS["cfg2"])
    small["samples"] = 2048
    run("samples_2048", lambda: quick_single("cfg2 table, 2048-sample batches", small, 5 * K, 2 * W))
    run("cfg2_host_ids", lambda: quick_single("cfg2", workloads.CONFIGS["cfg2"], K, W, host_keys=True, stage_timing=False))
    run("cfg1", lambda: quick_single("cfg1", workloads.CONFIGS["cfg1"], 5 * K, 2 * W))

    def cfg3():
        r = run_sharded(a, dict(workloads.CONFIGS["cfg3"]), K, W, with_cpu=False, name="cfg3")
        keep = ("ms_per_step", "value", "steps", "warmup", "cache_per_step_all_ranks", "device_ms_per_step",
                "host_ms_per_call")
        res = {k: r[k] for k in keep}
        res["workload"] = r["config"]["workload"]
        res["keys_per_step"] = r["config"]["keys_per_step"]
        res["unique_keys_per_step"] = r["config"]["unique_keys_per_step"]
        res["step_hbm_frac"] = r["step_hbm"]["frac"]
        if r.get("stages_all_shards"):
            res["stage_ms"] = {k: v["ms_per_step"] for k, v in r["stages_all_shards"].items()}
        return res

    run("cfg3", cfg3)
    run("cfg4", lambda: quick_single("cfg4", workloads.CONFIGS["cfg4"], K, W))
    run("cfg5_zipf", lambda: quick_single("cfg5_zipf", workloads.CONFIGS["cfg5_zipf"], K, W))
    run("cfg5_uniform", lambda: quick_single("cfg5_uniform", workloads.CONFIGS["cfg5_uniform"], K, W))
    return out


def main_sharded(a, cfg):
    print(json.dumps(run_sharded(a, cfg, a.steps, a.warmup, not a.no_cpu)), flush=True)


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no collectives, no second device); --gpus %d is not supported"
              % a.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    from hetuctr_amd import capi, workloads

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    if a.copy_probe:
        # yardstick for hardware byte counters and for the memory system itself: 1 GiB read + 1 GiB written per launch
        nbytes = 1 << 30
        src = torch.ones(nbytes // 4, device="cuda")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        ms = capi.copy_probe(dst.data_ptr(), src.data_ptr(), nbytes, 5)
        assert bool((dst[:: 1 << 16] == 1).all())
        print(json.dumps({"probe": "plain_copy", "bytes_read": nbytes, "bytes_written": nbytes, "avg_ms": ms,
                          "GBps": 2 * nbytes / (ms * 1e-3) / 1e9}), flush=True)
        return
    if a.partition:
        return main_partition(a)
    cfg = dict(workloads.CONFIGS[a.config])
    if a.samples:
        cfg["samples"] = a.samples
    if cfg.get("nrank", 1) > 1:
        return main_sharded(a, cfg)
    width, lr = cfg["width"], cfg["lr"]
    t_gen = time.perf_counter()
    ks = workloads.KeyStream(cfg, seed=0, scale=a.scale)
    batches = [ks.batch() for _ in range(max(2, a.batches))]
    ks.release_tables()
    n = batches[0].shape[0]
    print("[bench] %s: %d rows x %d, %d keys/batch, %d batches generated in %.1fs" %
          (a.config, ks.rows, width, n, len(batches), time.perf_counter() - t_gen), file=sys.stderr, flush=True)

    torch.cuda.set_device(0)
    t_init = time.perf_counter()
    root = np.zeros(ks.rows, np.uint8)
    storage = np.arange(ks.rows, dtype=np.int64)
    capi.seed(0)
    table = capi.Table(0, 1, 0, "127.0.0.1", 23456, ks.rows, width, 0, 0, root, storage, cfg["init"], lr, 0)
    del root, storage
    dkeys = [torch.from_numpy(b).cuda() for b in batches]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    bag = (a.bag or ks.hot) if a.pooled else 1       # sum-pooled bags: one gradient / output row per bag
    grad = torch.randn((n // bag, width), device="cuda", generator=gen) * 1e-3
    dst = torch.empty((n // bag, width), device="cuda")
    torch.cuda.synchronize()
    print("[bench] table + inputs resident in HBM after %.1fs" % (time.perf_counter() - t_init), file=sys.stderr, flush=True)

    # --host-keys: the ids are handed over as pageable host buffers, like the reference's own tests do; the step then
    # includes their transfer (never the reported headline: `value` is quoted with the ids resident in HBM)
    key_ptr = [b.ctypes.data for b in batches] if a.host_keys else [d.data_ptr() for d in dkeys]

    if bag > 1:
        def step(i):
            table.preprocess(key_ptr[i % len(dkeys)], n)
            table.push_pull_pooled(grad.data_ptr(), dst.data_ptr(), bag)
    else:
        def step(i):
            table.preprocess(key_ptr[i % len(dkeys)], n)
            table.push_pull(grad.data_ptr(), dst.data_ptr())

    uniq = {}
    for i in range(max(a.warmup, 1)):
        step(i)
        uniq[i % len(dkeys)] = int(table.fetch(capi.SIZES)[1])
    for i in range(len(dkeys)):                      # make sure U of every batch is known
        if i not in uniq:
            table.preprocess(dkeys[i].data_ptr(), n)
            uniq[i] = int(table.fetch(capi.SIZES)[1])
            table.push_pull_pooled(grad.data_ptr(), dst.data_ptr(), bag)
    w0 = max(a.warmup, 1) + len(dkeys)
    # ---- timed region: K full steps, nothing else on the GPU and nothing but the two calls on the host
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(w0 + i)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    # ---- device time of the two calls (HIP events inside the library, switched on for this pass only): a pass of
    # its own, because the events cost host time in every call
    pre_ms = pp_ms = push_ms = 0.0
    table.call_timing(True)
    for i in range(a.steps):
        step(w0 + i)
        p, q = table.last_times()
        pre_ms += p
        pp_ms += q
        push_ms += table.last_push_ms()
    table.call_timing(False)
    # ---- same K steps again with every stage bracketed by HIP events on the table's stream (the events cost a
    # few microseconds per stage, so the throughput above is taken without them)
    stages = {}
    ms_step_ev = None
    if not a.no_stage_timing:
        table.stage_timing(True)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for i in range(a.steps):
            step(w0 + a.steps + i)
        torch.cuda.synchronize()
        ms_step_ev = 1e3 * (time.perf_counter() - t1) / a.steps
        stages = table.stage_times()
        table.stage_timing(False)

    ms_step = 1e3 * dt / a.steps
    # distinct keys of the batches the timed steps used (current batch = pulled, previous = pushed)
    u_cur = np.mean([uniq[(w0 + i) % len(dkeys)] for i in range(a.steps)])
    u_prev = np.mean([uniq[(w0 + i - 1) % len(dkeys)] for i in range(a.steps)])
    bytes_step = workloads.algorithmic_bytes(n, 0.5 * (u_cur + u_prev), width, bag)
    step_gbs = bytes_step / (ms_step * 1e-3) / 1e9

    # HBM traffic per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this same command (committed
    # under profiles/, scaled by what the counters read for a plain copy of known size)
    traffic = {}
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath) and a.scale == 1.0:
        traffic = json.load(open(tpath)).get(a.config, {})
    kernel_names = {"segment_sum_apply": "push_fused", "gather": "gather"}
    roof_all = {}
    for k, (tot, cnt) in stages.items():
        if k in kernel_names and cnt > 0:
            avg_ms = tot / cnt
            b = workloads.stage_bytes(k, n, u_cur, n, u_prev, width, bag)
            gbs = b / (avg_ms * 1e-3) / 1e9
            roof_all[k] = dict(bound="hbm", kernel=kernel_names[k], achieved=gbs, peak=HBM_PEAK_GBS, unit="GB/s",
                               frac=gbs / HBM_PEAK_GBS, traffic=traffic.get(k), avg_ms=avg_ms, algorithmic_bytes=int(b))
    roof = roof_all[max(roof_all, key=lambda k: roof_all[k]["avg_ms"])] if roof_all else None
    if roof is not None:
        roof = dict(roof)
        roof["measured"] = ("HIP events around the kernel's launches on the table's stream, in the pass with stage "
                            "events, where the stages run one after the other (as under rocprofv3)")
        if "segment_sum_apply" in roof_all:
            # in the timed pass the index kernels of the next batch run beside the push on a second stream
            b = roof_all["segment_sum_apply"]["algorithmic_bytes"]
            co = push_ms / a.steps
            roof["push_in_timed_pass"] = {"avg_ms": co, "achieved": b / (co * 1e-3) / 1e9,
                                          "frac": b / (co * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                          "note": "start of push_pull to end of the push kernel while the sort/unique "
                                                  "kernels of the current batch share the GPU with it"}

    def variant(ptrs, timing=True):
        """The same table stepped with other key batches or another call protocol: ms per step, and the push / gather
        kernels alone (pass with stage events)."""
        def vstep(i):
            table.preprocess(ptrs[i % len(ptrs)], n)
            table.push_pull_pooled(grad.data_ptr(), dst.data_ptr(), bag)
        us = []
        for i in range(len(ptrs) + 2):
            vstep(i)
            us.append(int(table.fetch(capi.SIZES)[1]))
        torch.cuda.synchronize()
        tv0 = time.perf_counter()
        for i in range(a.steps):
            vstep(i)
        torch.cuda.synchronize()
        ms = 1e3 * (time.perf_counter() - tv0) / a.steps
        u = float(np.mean(us[2:]))
        res = {"ms_per_step": ms, "value": n / (ms * 1e-3), "unique_keys_per_step": u,
               "step_hbm_frac": workloads.algorithmic_bytes(n, u, width, bag) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
        if timing and not a.no_stage_timing:
            table.stage_timing(True)
            for i in range(a.steps):
                vstep(i)
            st = table.stage_times()
            table.stage_timing(False)
            res["stage_ms"] = {k: v[0] / max(v[1], 1) for k, v in st.items() if v[1]}
            for k in kernel_names:
                if k in res["stage_ms"]:
                    res[kernel_names[k] + "_frac"] = (workloads.stage_bytes(k, n, u, n, u, width, bag) /
                                                      (res["stage_ms"][k] * 1e-3) / 1e9 / HBM_PEAK_GBS)
        return res

    # the reference's literal call protocol: preprocess returns when all its work is done (hetu_gpu_table.cu:64), so
    # nothing of the batch's index runs beside the push
    literal = None
    if not a.host_keys and not a.no_variants:
        table.defer_index(False)
        literal = variant(key_ptr, timing=False)
        table.defer_index(True)
    # the same workload with the hot rows of every field scattered over the field instead of lying side by side
    permuted = None
    if a.config == "cfg2" and a.scale == 1.0 and not a.host_keys and not a.no_variants and not a.samples:
        pcfg = workloads.CONFIGS["cfg2_permuted"]
        pks = workloads.KeyStream(pcfg, seed=0, scale=a.scale)
        pkeys = [torch.from_numpy(pks.batch()).cuda() for _ in range(len(dkeys))]
        pks.release_tables()
        torch.cuda.synchronize()
        permuted = variant([k.data_ptr() for k in pkeys])
        permuted["note"] = ("rank -> id through a seeded permutation per field (cfg2_permuted); the headline keeps "
                            "the Zipf rank as the local id, i.e. every field's hot rows are its first rows")
        del pkeys

    out = {
        "metric": "sparse IDs/sec per train step (pull+push)", "value": n * a.steps / dt, "unit": "IDs/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: %d-row x %d fp32 table, batch %d samples x %d fields x %d ids = %d keys, %s, "
                               "SGD lr %g, one shard (all rows local)%s" %
                               (a.config, ks.rows, width, ks.samples, ks.fields, ks.hot, n,
                                "uniform ids" if cfg["alpha"] is None else "per-field Zipf %.2f (%s)" %
                                (cfg["alpha"], "rank -> id permuted per field" if cfg.get("permute") else "rank = local id"),
                                lr, "" if bag == 1 else ", bags of %d ids sum-pooled" % bag),
                   "keys_per_step": n, "unique_keys_per_step": float(u_cur), "width": width, "rows": ks.rows,
                   "ids_handed_over_in": "pageable host memory" if a.host_keys else "HBM"},
        "unique_rows_per_sec": u_cur * a.steps / dt,
        "device_ms_per_step": {"preprocess_until_ids_are_read": pre_ms / a.steps, "push_pull": pp_ms / a.steps},
        "step_hbm": {"algorithmic_bytes": int(bytes_step), "achieved_GBps": step_gbs, "frac": step_gbs / HBM_PEAK_GBS},
        "stage_ms": {k: v[0] / max(v[1], 1) for k, v in stages.items() if v[1]},
        "pooling": None if bag == 1 else {
            "bag": bag, "gradient_rows_per_step": n // bag, "output_rows_per_step": n // bag,
            "unpooled_output_bytes": 4 * width * n, "pooled_output_bytes": 4 * width * (n // bag),
            "bytes_saved_per_step": 2 * 4 * width * (n - n // bag),
            "note": "the reference hands one row per id both ways (its API has no pooling); pooled, the gradient and "
                    "the output shrink by the bag size, the table rows read per id stay"},
        "ms_per_step_with_stage_events": ms_step_ev,
        "roofline": roof,
        "roofline_stages": roof_all,
        "literal_contract": literal,
        "permuted_ids": permuted,
    }
    if not a.no_cpu:
        dst = None
        torch.cuda.empty_cache()
        try:
            out["cpu_baseline"] = cpu_baseline(cfg, ks, batches, width, lr, a.cpu_steps)
        except MemoryError as e:  # pragma: no cover
            out["cpu_baseline"] = {"value": None, "error": str(e)}
    table.close()
    # every other configuration in the same record: the headline keys above stay as they are
    default_run = (a.config == "cfg2" and a.scale == 1.0 and not a.samples and not a.host_keys and not a.pooled and
                   not a.no_variants and not a.no_others)
    if default_run:
        dkeys = grad = dst = None
        torch.cuda.empty_cache()
        out["other_configs"] = other_configs(a)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
