#!/usr/bin/env python3
"""Benchmark of the sampling-server hot path on one MI355X.

A "step" is one mini-batch: seed ids in -> multi-hop sampled blocks + gathered
feature rows resident in HBM.  Inputs (CSR graph, feature table, cache, train
set) are synthetic, generated on the GPU from a fixed seed, and resident before
the timed region starts.  One JSON line is printed on stdout.

    python bench.py [--gpus 1] [--steps 50] [--warmup 5] [--workload paper100m]

Workloads: paper100m (default, the configuration the
metric is quoted on), products, paper100m-lru, mag240m-int8 (down-scaled node
count, stated in the output), cora.  `--scale` shrinks node counts for quick runs.
"""
import argparse
import importlib.util
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
HOST_LINK_PEAK_GBS = 64.0  # PCIe Gen5 x16 per direction, nominal


def load_package():
    path = os.path.join(ROOT, "legion-ibp_amd", "__init__.py")
    spec = importlib.util.spec_from_file_location("legion_ibp_amd", path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules["legion_ibp_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


WORKLOADS = {
    # name: nodes, mean degree, alpha, d_max, dim, dtype, batch, fanout, train, cache
    "paper100m": dict(nodes=111_059_956, mean_deg=14.548, alpha=2.0, d_max=100_000, dim=128, dtype="f32",
                      batch=8000, fanout=[25, 10], train=1_200_000, cache=("static", 38e9),
                      # groups of 8: the seeds' and the first hop's misses leave over the host link while the second
                      # hop is still sampled (two host-link gathers per group), 6 blocks for each of the 8 batches
                      tune={"miss_blocks": 48, "split_lookup": 2}),
    "products": dict(nodes=2_449_029, mean_deg=25.27, alpha=2.1, d_max=17_000, dim=100, dtype="f32",
                     batch=800, fanout=[25, 10], train=196_615, cache=("static_frac", 0.30)),
    "paper100m-lru": dict(nodes=111_059_956, mean_deg=14.548, alpha=2.0, d_max=100_000, dim=128, dtype="f32",
                          batch=4096, fanout=[15, 10, 5], train=1_200_000, cache=("lru", 20e9),
                          locality=(0.8, 10)),   # 80 % of a batch's seeds come from the last 10 batches' frontiers
    "mag240m-int8": dict(nodes=244_160_499, mean_deg=7.08, alpha=2.0, d_max=100_000, dim=768, dtype="f16",
                         batch=1024, fanout=[25, 15], train=1_112_392, cache=("int8", 80e9),
                         # the host link paces these batches (3.5 k rows of 1 536 B each): a wider host-link
                         # gather (55 instead of 49 GB/s) is worth more than what it costs the kernels beside it
                         tune={"miss_blocks": 64}),
    "cora": dict(nodes=2_708, mean_deg=7.8, alpha=None, d_max=40, dim=1433, dtype="f32",
                 batch=64, fanout=[25, 10], train=2_708, cache=("static_frac", 1.0)),
}


def recorded_traffic(workload):
    """HBM bytes per launch of the hit gather, from the committed rocprofv3 --pmc summary
    (FETCH_SIZE + WRITE_SIZE, calibrated on the copy kernel); None when no summary exists."""
    path = os.path.join(ROOT, "profiles", "%s_hit_gather_hbm_traffic.txt" % workload)
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch="):
                return int(line.split("=")[1])
    except OSError:
        pass
    return None


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


def mem_available_gb():
    """MemAvailable of the box in GB (0 when /proc/meminfo cannot be read)."""
    try:
        for line in open("/proc/meminfo"):
            if line.startswith("MemAvailable:"):
                return int(line.split()[1]) * 1024 / 1e9
    except OSError:
        pass
    return 0.0


def pinned_table(lmi, w, host_budget_gb):
    """The feature table in pinned host memory, as large as this box allows: the full node count
    when it fits, otherwise the largest node count whose table (a) stays under the budget -- by
    default 70 % of the box's available RAM, the rest being for the host copy of the graph the
    CPU baseline needs -- and (b) hipHostMalloc actually grants (the driver's limit on pinned
    memory can be far below the RAM).  Returns (HostBuffer, n_nodes, note)."""
    np_dtype = np.float16 if w["dtype"] == "f16" else np.float32
    row_bytes = w["dim"] * np.dtype(np_dtype).itemsize
    ram_gb = mem_available_gb()
    budget_gb = host_budget_gb if host_budget_gb > 0 else (0.70 * ram_gb if ram_gb > 0 else 64.0)
    full_gb = w["nodes"] * row_bytes / 1e9
    n_nodes, refused = w["nodes"], 0
    if full_gb > budget_gb:
        n_nodes = int(w["nodes"] * budget_gb / full_gb)
    while True:
        try:
            feats = lmi.HostBuffer((n_nodes, w["dim"]), np_dtype)
            break
        except lmi.LegionError:
            refused += 1
            if n_nodes < 1000 or refused > 200:
                raise
            n_nodes = int(n_nodes * 0.95)   # a refusal costs nothing: step down until one is granted
    note = None
    if n_nodes != w["nodes"]:
        note = ("box: %.0f GB RAM available, hipHostMalloc grants a %.1f GB table%s; the full table is %.0f GB, so node "
                "count and cache budget are down-scaled x%.3f" % (
                    ram_gb, n_nodes * row_bytes / 1e9,
                    " (%d larger requests refused)" % refused if refused else "", full_gb, n_nodes / w["nodes"]))
        log(note)
    return feats, n_nodes, note


def build_inputs(lmi, w, seed, host_budget_gb, neighbours="degree"):
    """Graph (HBM), feature table (pinned host memory) and train set of a workload."""
    feats, n_nodes, note = pinned_table(lmi, w, host_budget_gb)
    t0 = time.time()
    if w["alpha"] is None:   # Erdos-Renyi-like: Poisson degrees, uniform neighbours
        from math import exp
        lam = w["mean_deg"]
        pmf = [exp(-lam)]
        for d in range(1, w["d_max"] + 1):
            pmf.append(pmf[-1] * lam / d)
        cdf = np.cumsum(pmf) / np.sum(pmf)
        t = np.minimum(np.floor(cdf * 4294967296.0), 4294967295.0).astype(np.uint64)
        t[-1] = 4294967295
        cdf_u32, mode = t.astype(np.uint32), 0
    else:
        cdf_u32, mode = lmi.zipf_cdf(w["alpha"], w["d_max"], w["mean_deg"]), (0 if neighbours == "uniform" else 1)
    d_indptr, d_indices, n_edges = lmi.synth_graph(seed, cdf_u32, n_nodes, mode)
    log("graph: %d nodes, %d edges in HBM (%.1f s)" % (n_nodes, n_edges, time.time() - t0))
    t0 = time.time()
    lmi.synth_features(seed + 1, feats)
    log("features: %.2f GB in pinned host memory (%.1f s)" % (feats.nbytes / 1e9, time.time() - t0))
    n_train = min(w["train"], n_nodes)
    train = lmi.synth_trainset(seed + 2, n_nodes, n_train)
    return dict(n_nodes=n_nodes, n_edges=n_edges, n_train=n_train, note=note, feats=feats, d_indptr=d_indptr,
                d_indices=d_indices, train=train, scale=n_nodes / w["nodes"],
                graph="%s degrees%s, %s neighbours" % (
                    "Poisson" if w["alpha"] is None else "Zipf-Mandelbrot", "" if w["alpha"] is None else " alpha=%s" % w["alpha"],
                    "uniform" if mode == 0 else "degree-proportional"))


def free_inputs(lmi, inputs):
    inputs["feats"].free()
    for k in ("d_indptr", "d_indices"):
        lmi.check(lmi.lib().lmi_device_free(inputs[k]))


def build_server(lmi, w, inputs, seed, pipes, table=2, policy="degree"):
    """A server over prepared inputs, with the workload's cache; returns (server, info)."""
    np_dtype = np.float16 if w["dtype"] == "f16" else np.float32
    esz = np.dtype(np_dtype).itemsize
    n_nodes, n_train, scale = inputs["n_nodes"], inputs["n_train"], inputs["scale"]
    srv = lmi.Server(w["batch"], w["fanout"], w["dim"], feat_dtype=lmi.F16 if w["dtype"] == "f16" else lmi.F32,
                     pipes=pipes, seed=seed)
    srv.attach_graph_device(inputs["d_indptr"], inputs["d_indices"], n_nodes, inputs["n_edges"])
    srv.attach_features(inputs["feats"])
    srv.load_idset(lmi.MODE_TRAIN, inputs["train"])
    if policy == "presampled":
        # the reference's policy: one presampling pass over the training set, rank by sampled frequency
        t0 = time.time()
        srv.presample(-(-n_train // w["batch"]))
        srv.cache_policy(lmi.POLICY_PRESAMPLED)
        lmi.check(lmi.lib().lmi_device_sync())
        log("presampled one epoch (%.2f s)" % (time.time() - t0))
    t0 = time.time()
    kind, amount = w["cache"]
    if kind in ("static", "lru", "int8"):
        amount = amount * scale   # a down-scaled table keeps its cached fraction
    row_bytes = w["dim"] * esz
    if kind == "static":
        rows = min(n_nodes, int(amount // row_bytes))
        srv.build_static_cache(rows, table)
    elif kind == "static_frac":
        rows = max(1, int(n_nodes * amount))
        srv.build_static_cache(rows, table)
    elif kind == "lru":
        ways = 8
        rows = min(n_nodes, int(amount // row_bytes))
        srv.build_lru_cache(max(1, rows // ways), ways)
    elif kind == "int8":
        rows = min(n_nodes, int(amount // (w["dim"] + 4)))
        srv.build_int8_cache(rows, table)
    ci = srv.cache_info()
    log("cache: kind=%d rows=%d (%.2f GB) table %.2f GB (%.1f s)" % (
        ci.kind, ci.capacity_rows, ci.capacity_rows * ci.row_bytes / 1e9, ci.table_bytes / 1e9, time.time() - t0))
    info = dict(inputs, row_bytes=row_bytes, cache_rows=int(ci.capacity_rows), cache_kind=kind)
    return srv, info


def build_workload(lmi, w, seed, pipes, host_budget_gb, table=2, policy="degree", neighbours="degree"):
    """Generate the graph, features, train set and cache; returns (server, info)."""
    inputs = build_inputs(lmi, w, seed, host_budget_gb, neighbours)
    return build_server(lmi, w, inputs, seed, pipes, table, policy)


def record_seed_plan(lmi, srv, w, info, n_batches, seed):
    """Seed batches with temporal locality: a fraction of every batch is drawn from the frontiers
    (all node ids) of the previous batches, the rest uniformly from the train set.  The frontiers
    depend on the sampled batches, so the sequence is recorded in one untimed pass; the caller
    resets the cache afterwards and replays the recorded seeds (same RNG seeds, same batches)."""
    frac, depth = w["locality"]
    rng = np.random.default_rng(seed + 7)
    B, train = w["batch"], info["train"]
    recent, plan = [], []
    for t in range(n_batches):
        n_loc = int(frac * B) if recent else 0
        parts = [train[rng.integers(0, len(train), B - n_loc)]]
        if n_loc:
            pool = np.concatenate(recent[-depth:])
            parts.insert(0, pool[rng.integers(0, len(pool), n_loc)])
        seeds = np.array(list(dict.fromkeys(np.concatenate(parts).tolist())), np.int32)   # distinct, order kept
        srv.run_once(seeds, rng_seed=seed + t)
        recent.append(srv.fetch_ids())
        recent = recent[-depth:]
        plan.append(seeds)
    return plan


def cpu_baseline(lmi, srv, w, info, seed, budget_s, issue):
    """The CPU oracle on the same workload and host cores; also checks the GPU output of the same
    batches bit for bit.  `issue` = dict(pipes, group, first_sizes, steps_per_epoch, plan): the GPU side
    issues the checked batches the way the timed region does -- lmi_run_group with the same group sizes
    (first the split the timed region used, e.g. 7, 7, 6 for 20 steps, then full groups), batch i into
    pipe i % pipes, same tuning, two groups in flight before anything is read back -- so that what is
    compared with the oracle is the path that was timed."""
    from oracle import binding as orc
    from concurrent.futures import ThreadPoolExecutor
    cores = len(os.sched_getaffinity(0))
    box_share = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
    threads = min(cores, box_share) if box_share > 0 else cores
    n_nodes, n_edges = info["n_nodes"], info["n_edges"]
    t0 = time.time()
    indptr = lmi.to_host(info["d_indptr"], n_nodes + 1, np.int64)
    indices = lmi.to_host(info["d_indices"], n_edges, np.int32)
    log("cpu baseline: CSR copied to host (%.1f s), %d threads" % (time.time() - t0, threads))
    feats = info["feats"].array
    B = w["batch"]
    done, spent, parity_ok, rows, at_a_time = 0, 0.0, True, 0, 1
    pipes, group, spe, plan = issue["pipes"], issue["group"], issue["steps_per_epoch"], issue["plan"]
    max_batches = min(256, len(plan) if plan else len(info["train"]) // B)
    stream = lmi.stream_create()

    def same_as_oracle(g, o, out):
        same = (np.array_equal(g.ids, o.ids) and np.array_equal(g.agg_src_off, o.agg_src_off) and
                np.array_equal(g.agg_dst_off, o.agg_dst_off) and np.array_equal(g.agg_src_ids, o.agg_src_ids) and
                list(g.node_counter) == list(o.node_counter) and list(g.edge_counter) == list(o.edge_counter) and
                all(np.array_equal(a, b) for a, b in zip(g.blk_indptr, o.blk_indptr)))
        if info["cache_kind"] != "int8":
            same = same and g.features.tobytes() == out.tobytes()
        else:
            # misses are the host rows; hits are the oracle's codec applied to the host rows of the ids
            # that hit (the codec works row by row, so quantising just these rows is the cached content)
            hit = g.cache_index >= 0
            same = same and g.features[~hit].tobytes() == out[~hit].tobytes()
            if hit.any():
                q, sc = orc.quantize_rows(out[hit])
                same = same and g.features[hit].tobytes() == orc.dequant_rows(q, sc, out.dtype).tobytes()
        # threshold property of the degree-ordered static cache
        if info["cache_kind"] in ("static", "static_frac", "int8") and len(o.ids):
            deg = indptr[o.ids + 1] - indptr[o.ids]
            hit = g.cache_index >= 0
            if hit.any() and (~hit).any():
                same = same and deg[hit].min() >= deg[~hit].max()
        return same

    sizes = list(issue["first_sizes"])   # the timed region's own split first, then full groups
    checked_sizes = []
    nxt = 0                              # next batch to issue
    while done < max_batches and spent < budget_s:
        in_flight = []                   # (batch, pipe), issued and not yet read back
        while nxt < max_batches and len(in_flight) < 2 * group:
            n = min(sizes.pop(0) if sizes else group, max_batches - nxt)
            ks = list(range(nxt, nxt + n))
            if {k % pipes for k in ks} & {p for _, p in in_flight}:
                sizes.insert(0, n)       # would overwrite a batch not yet compared: read those back first
                break
            if group == 1:
                srv.run_once(plan[nxt] if plan else None, batch_counter=nxt % spe, rng_seed=seed + nxt, pipe=nxt % pipes,
                             stream=stream)
            else:
                srv.run_group([k % pipes for k in ks], [k % spe for k in ks], seeds=[plan[k] for k in ks] if plan else None,
                              rng_seeds=[seed + k for k in ks], stream=stream)
            checked_sizes.append(n)
            in_flight += [(k, k % pipes) for k in ks]
            nxt += n
        # the CPU side of the same batches: independent batches on independent cores, `threads` at a time, one
        # thread each (1.5x the rate of one batch at a time with all threads inside it on the box's 16 threads, 3.5x on
        # 8 cores of a desktop: the dedup / relabel pass of a batch is one thread's loop); ctypes releases the
        # interpreter lock for the duration of a call
        # (with fewer batches in flight than threads -- one batch per launch on two pipes -- each takes its share
        # of them: faster than one batch after the other with every thread inside it)
        together = max(1, min(threads, len(in_flight)))
        per_batch = max(1, threads // together)

        def cpu_batch(b):
            seeds = plan[b] if plan else info["train"][(b % spe) * B:(b % spe + 1) * B]
            o = orc.sample_batch(indptr, indices, seeds, w["fanout"], seed + b, threads=per_batch)
            return o, orc.gather_rows(o.ids, np.full(len(o.ids), -1, np.int32), None, feats, threads=per_batch)
        t0 = time.time()
        if together > 1:
            with ThreadPoolExecutor(min(threads, together)) as pool:
                cpu = list(pool.map(cpu_batch, [b for b, _ in in_flight]))
        else:
            cpu = [cpu_batch(b) for b, _ in in_flight]
        spent += time.time() - t0
        at_a_time = max(at_a_time, min(threads, together))
        for (b, pipe), (o, out) in zip(in_flight, cpu):
            rows += len(o.ids)
            parity_ok = same_as_oracle(srv.fetch(pipe=pipe, stream=stream), o, out) and parity_ok
            done += 1
        del cpu
        if not in_flight:
            break
    how = ("lmi_run_group, groups of %s, batch i in pipe i %% %d, two groups in flight" % (
        ", ".join(str(n) for n in checked_sizes[:6]) + (", ..." if len(checked_sizes) > 6 else ""), pipes)
           if group > 1 else "lmi_run_once on %d pipes" % pipes)
    return dict(value=done / spent, unit="batches/s", cores=threads, kind="port",
                sample="%d batches of the same workload (oracle sample_batch + gather; up to %d batches at a time, the %d host "
                       "threads shared out between them); "
                       "GPU output of the same batches, issued as the timed region issues them (%s), %s" % (
                           done, at_a_time, threads, how, "bit-exact" if parity_ok else "MISMATCH"),
                gather_rows_per_s=rows / spent, checked_batches=done, checked_group_sizes=checked_sizes), parity_ok


def gather_variants(lmi, srv, info, w):
    """Sweeps the memory-access choices of the feature gather on the loaded workload -- bytes per
    lane access, lanes per row (thread per row .. wavefront per row), rows in flight per lane,
    store policy, grid of the host-link gather -- one batch per launch on two pipes, timed by HIP
    events inside the library.  Every variant is a tuning key; each is a different
    move_rows_kernel<V, LPR, U, NT, HOSTLINK> instantiation, so the same run under
    `rocprofv3 --kernel-trace --stats` (or --pmc) lists them one by one."""
    stream = lmi.stream_create()
    spe = -(-info["n_train"] // w["batch"])
    rb = info["row_bytes"]
    hit_bytes = (w["dim"] + 4 + rb + 8) if info["cache_kind"] == "int8" else 2 * rb + 8
    own = dict(w.get("tune", {}))        # the workload's own settings are what "default" means here
    for k, v in own.items():
        srv.tune(k, int(v))

    def run(label, steps=60):
        for i in range(3):
            srv.run_once(None, batch_counter=i % spe, rng_seed=100 + i, pipe=i % 2, stream=stream)
        lmi.check(lmi.lib().lmi_device_sync())
        srv.profile_read(True)
        srv.profile_enable(1)
        t0 = time.perf_counter()
        for i in range(steps):
            srv.run_once(None, batch_counter=i % spe, rng_seed=100 + i, pipe=i % 2, stream=stream)
        lmi.check(lmi.lib().lmi_device_sync())
        t1 = time.perf_counter()
        srv.profile_enable(0)
        p = srv.profile_read(True)
        hit_ms = p.gather_hit_ms / max(p.gather_hit_launches, 1)
        rows = p.gather_hit_rows / max(p.gather_hit_launches, 1)
        miss_ms = p.gather_miss_ms / max(p.gather_miss_launches, 1)
        mrows = p.gather_miss_rows / max(p.gather_miss_launches, 1)
        gbs = rows * hit_bytes / (hit_ms * 1e-3) / 1e9 if hit_ms else 0.0
        print("%-68s hit %6.1f us %5.0f GB/s (%4.1f%% of 8 TB/s) | miss %6.1f us %5.1f GB/s | sample %6.1f us | %6.1f us/batch" % (
            label, hit_ms * 1e3, gbs, gbs / 80, miss_ms * 1e3, mrows * rb / (miss_ms * 1e-3) / 1e9 if miss_ms else 0.0,
            p.sample_ms / max(p.sample_launches, 1) * 1e3, (t1 - t0) * 1e6 / steps), flush=True)

    print("feature-gather access variants, %d-byte rows, %d algorithmic bytes per hit row" % (rb, hit_bytes), flush=True)
    run("default")
    if info["cache_kind"] != "int8":
        for vb in (4, 8):
            srv.tune("gather_vector_bytes", vb)
            run("vector %2d B per lane (lanes per row auto)" % vb)
        srv.tune("gather_vector_bytes", 0)
    for lpr in (1, 4, 8, 16, 32, 64):
        srv.tune("gather_lanes_per_row", lpr)
        run("lanes per row %2d%s" % (lpr, "  = thread per row" if lpr == 1 else "  = wavefront per row" if lpr == 64 else ""))
    srv.tune("gather_lanes_per_row", 0)
    for u in (2, 4, 8):
        srv.tune("gather_unroll", u)
        run("rows in flight per lane %d" % u)
    srv.tune("gather_unroll", 0)         # back to each mover's own choice
    srv.tune("gather_nontemporal", 0)
    run("plain (temporal) output stores")
    srv.tune("gather_nontemporal", 1)
    for mb in (8, 16, 64, 256):
        srv.tune("miss_blocks", mb)
        run("host-link gather on %3d blocks" % mb)
    srv.tune("miss_blocks", int(own.get("miss_blocks", 32)))
    srv.tune("split_miss", 0)
    run("host-link gather on the caller's stream (no overlap)")
    srv.tune("split_miss", 1)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--workload", default="paper100m", choices=sorted(WORKLOADS))
    ap.add_argument("--scale", type=float, default=1.0, help="shrink node/train counts (testing only)")
    ap.add_argument("--pipes", type=int, default=16, help="output buffer sets in flight")
    ap.add_argument("--streams", type=int, default=1, help="caller streams the pipes are spread over")
    ap.add_argument("--group", type=int, default=8,
                    help="at most this many mini-batches are issued together with lmi_run_group (their sampling "
                         "kernels share launches)")
    ap.add_argument("--group-sizes", default="",
                    help="comma-separated sizes of the groups the timed region is issued in (must add up to --steps), "
                         "instead of the fewest groups of at most --group, sized evenly")
    ap.add_argument("--seed", type=int, default=20260101)
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU baseline budget (0 = skip)")
    ap.add_argument("--host-gb", type=float, default=0.0,
                    help="pinned host memory budget for the feature table; 0 = 70 %% of the box's available RAM, "
                         "stepping down to what hipHostMalloc grants")
    ap.add_argument("--neighbours", default="degree", choices=["degree", "uniform"],
                    help="how the synthetic graph draws neighbours: degree-proportional (in-degree follows the "
                         "out-degree law, default) or uniform over the nodes")
    ap.add_argument("--steady-steps", type=int, default=200,
                    help="when --steps is smaller, an extra untimed-for-`value` leg of this many steps gives "
                         "steady_state_batches_s (0 = skip)")
    ap.add_argument("--issue", default="group", choices=["group", "runner"],
                    help="how batches are issued in the timed region: 'group' = lmi_run_group on --pipes pipes (what the "
                         "reference-shaped Server::Run does when nothing takes the batches one by one); 'runner' = one "
                         "lmi_run_once per batch on two pipes with a host wait per batch (GPURunner::RunOnce with a trainer "
                         "attached).  The default line carries the runner figure too (runner_issue_batches_s)")
    ap.add_argument("--runner-steps", type=int, default=100, help="steps of the extra runner-issue leg (0 = skip)")
    ap.add_argument("--companion-steps", type=int, default=96,
                    help="steps of the extra leg on the same workload with uniform neighbours (0 = skip)")
    ap.add_argument("--shape-study", action="store_true",
                    help="after the run, sweep the row-streaming kernel of this workload's gather shape (scattered rows, "
                         "computed places, no index) over rows per block visit, idle blocks in the grid and idle lanes "
                         "that load anyway, and print one line per setting instead of the benchmark line")
    ap.add_argument("--gather-variants", action="store_true",
                    help="instead of the benchmark line, sweep the feature gather's access patterns on this "
                         "workload and print one line per variant")
    ap.add_argument("--table", default="rank", choices=["hash", "direct", "rank"], help="id->slot table layout")
    ap.add_argument("--policy", default="degree", choices=["degree", "presampled"],
                    help="ranking of the static hot set: out-degree (the configs' choice) or presampled frequency")
    ap.add_argument("--tune", action="append", default=[], help="key=value passed to lmi_tune")
    ap.add_argument("--profile-every", type=int, default=4,
                    help="gather kernels of one batch in this many carry timing events in the timed region")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; there is no multi-GPU path (got --gpus %d)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    lmi = load_package()
    w = dict(WORKLOADS[args.workload])
    if args.scale != 1.0:
        w["nodes"] = max(1000, int(w["nodes"] * args.scale))
        w["train"] = max(w["batch"], int(w["train"] * args.scale))
        if w["cache"][0] in ("static", "lru", "int8"):
            w["cache"] = (w["cache"][0], w["cache"][1] * args.scale)
    if w["cache"][0] == "lru":
        args.group = 1                      # the LRU cache takes one batch at a time
        args.pipes = min(args.pipes, 2)
    if args.gather_variants:
        args.pipes = 2
    srv, info = build_workload(lmi, w, args.seed, args.pipes, args.host_gb,
                               {"hash": 0, "direct": 1, "rank": 2}[args.table], args.policy, args.neighbours)
    if args.gather_variants:
        gather_variants(lmi, srv, info, w)
        srv.close()
        return
    tunes = {k: str(v) for k, v in w.get("tune", {}).items()}   # the workload's own settings, then --tune
    tunes.update(kv.split("=") for kv in args.tune)
    # paper100m-shaped in groups of 8 on 16 pipes (the host-link grid is shared out evenly, so it counts in
    # eights), 20-step run / 200-step run, batches/s: one lookup per group and 40 blocks 7.2 k / 8.4 k; split
    # lookups and 40 blocks 7.6 k / 8.3 k; split lookups and 48 blocks 7.6 k / 8.4 k (the HBM gather 0.69, 0.69
    # and 0.67 of peak: what more host-link reads beside it cost)
    for k, v in tunes.items():
        srv.tune(k, int(v))
    steps_per_epoch = -(-info["n_train"] // w["batch"])
    streams = [lmi.stream_create() for _ in range(max(1, args.streams))]
    plan = None
    if w.get("locality"):
        t0 = time.time()
        extra = args.steady_steps if args.steps < args.steady_steps else 0
        plan = record_seed_plan(lmi, srv, w, info, args.warmup + args.steps + extra + args.runner_steps + min(args.steps, 20) + 2,
                                args.seed)
        ci = srv.cache_info()
        srv.build_lru_cache(int(ci.n_sets), int(ci.ways))   # start the replay from an empty cache again
        log("recorded %d seed batches with temporal locality (%.1f s)" % (len(plan), time.time() - t0))

    group = max(1, args.group)
    if group > 1 and (args.pipes < group or info["cache_kind"] == "lru"):
        print("bench.py: --group needs at least as many pipes (twice as many keep two groups in flight), and no "
              "LRU cache", file=sys.stderr)
        sys.exit(2)

    def step(i, n=None):
        # consecutive batches alternate output buffer sets (pipes), so the host-link part of batch i
        # (on the server's side stream) overlaps the sampling of batch i+1; a pipe always uses the
        # same caller stream.  With --group g, batches i .. i+g-1 are issued together (step is then
        # called with i a multiple of g) and consecutive groups alternate sets of g pipes.
        p = i % args.pipes
        if group == 1:
            srv.run_once(plan[i] if plan else None, batch_counter=i % steps_per_epoch, rng_seed=args.seed + i, pipe=p,
                         stream=streams[p % len(streams)])
        else:
            ks = range(i, i + (n or group))   # the timed region's last group may be a partial one
            srv.run_group([k % args.pipes for k in ks], [k % steps_per_epoch for k in ks],
                          seeds=[plan[k] for k in ks] if plan else None, rng_seeds=[args.seed + k for k in ks],
                          stream=streams[(p // group) % len(streams)])

    def group_sizes(count):
        """`count` batches as the fewest groups of at most `group`, sized evenly (20 in groups of up to
        8: 7, 7, 6): the side stream's last, exposed, host-link gather is then no longer than the others."""
        if args.group_sizes and count == args.steps:
            sizes = [int(x) for x in args.group_sizes.split(",")]
            if sum(sizes) != count or max(sizes) > min(group, lmi.MAX_GROUP) or min(sizes) < 1:
                raise SystemExit("--group-sizes must add up to --steps, each 1..%d" % min(group, lmi.MAX_GROUP))
            return sizes
        n_groups = -(-count // group)
        base, extra = divmod(count, n_groups) if n_groups else (0, 0)
        return [base + 1] * extra + [base] * (n_groups - extra)

    def run_steps(first, count):
        """Batches first .. first+count-1, group by group."""
        i = first
        for n in group_sizes(count):
            step(i, n)
            i += n

    def leg(first, count):
        """`count` batches from batch `first`, timed from the first call to an idle device; the gather kernels
        of one group in --profile-every carry HIP start / stop events of their own (level 2: nothing is
        queued between kernels; an event pair costs its group about 10 us)."""
        srv.profile_read(reset=True)
        srv.tune("profile_every", args.profile_every)
        srv.profile_enable(2)
        t0 = time.perf_counter()
        if args.issue == "runner":
            runner_steps(first, count)
        else:
            run_steps(first, count)
        for st in streams:
            lmi.check(lmi.lib().lmi_stream_sync(st))   # the caller's own kernels are done ...
        t_caller = time.perf_counter()
        lmi.check(lmi.lib().lmi_device_sync())          # ... and now the server's side stream is too
        t1 = time.perf_counter()
        srv.status()   # a batch a kernel flagged (bad seed id, scan that gave up) voids the measurement
        srv.profile_enable(0)
        return dict(sec=t1 - t0, drain_ms=(t1 - t_caller) * 1e3, prof=srv.profile_read(reset=True), steps=count)

    post_stream = lmi.stream_create()

    def runner_steps(first, count):
        """The reference-shaped runner's issue pattern with a trainer attached (GPURunner::RunOnce of the
        host shim, hand-off on): one batch per call on TWO output buffer sets, and before batch i + 1 is
        issued the host waits until batch i - 1 is complete (that is when the runner posts it to the
        trainer).  No semaphores and no trainer here, so this is the rate the sampler side sustains."""
        for i in range(first, first + count):
            srv.run_once(plan[i] if plan else None, batch_counter=i % steps_per_epoch, rng_seed=args.seed + i,
                         pipe=i % 2, stream=streams[0])
            if i > first:
                srv.batch_wait((i - 1) % 2, post_stream)
                lmi.check(lmi.lib().lmi_stream_sync(post_stream))
        srv.batch_wait((first + count - 1) % 2, post_stream)
        lmi.check(lmi.lib().lmi_stream_sync(post_stream))

    if args.issue == "runner":
        for i in range(args.warmup):
            srv.run_once(plan[i] if plan else None, batch_counter=i % steps_per_epoch, rng_seed=args.seed + i,
                         pipe=i % 2, stream=streams[0])
    else:
        run_steps(0, args.warmup)
    lmi.check(lmi.lib().lmi_device_sync())
    timed = leg(args.warmup, args.steps)   # exactly --steps batches
    t1_minus_t0 = timed["sec"]
    ms_per_step = t1_minus_t0 * 1e3 / args.steps
    # the tail nothing overlaps: how long the side stream (host-link gathers, LRU insertion) of the last
    # batches kept running after the caller's stream had finished
    drain_ms = timed["drain_ms"]
    done = args.warmup + args.steps
    # Short runs are dominated by their ends: the first group's sampling and the last group's host-link gather
    # have nothing to overlap with.  A longer leg of the same loop gives the rate a serving loop sustains, and
    # its launches are the ones the roofline figures below are taken from.
    if args.steps >= args.steady_steps or args.steady_steps <= 0:
        steady_leg, steady = timed, dict(batches_s=round(args.steps / timed["sec"], 2), steps=args.steps,
                                         drain_ms=round(drain_ms, 3), same_run_as="value")
    else:
        steady_leg = leg(done, args.steady_steps)
        steady = dict(batches_s=round(args.steady_steps / steady_leg["sec"], 2), steps=args.steady_steps,
                      drain_ms=round(steady_leg["drain_ms"], 3), same_run_as=None)
        done += args.steady_steps
    prof = steady_leg["prof"]
    # what a drop-in user of the reference-shaped runner gets with a trainer attached: see runner_steps
    runner = None
    if args.issue != "runner" and args.runner_steps > 0:
        lmi.check(lmi.lib().lmi_device_sync())
        if "miss_blocks" not in dict(kv.split("=") for kv in args.tune):
            srv.tune("miss_blocks", 32)   # the runner of the host shim sets no knobs: the library's own host-link grid
        r0 = time.perf_counter()
        runner_steps(done, args.runner_steps)
        lmi.check(lmi.lib().lmi_device_sync())
        r1 = time.perf_counter()
        srv.status()
        srv.tune("miss_blocks", int(tunes.get("miss_blocks", 32)))
        runner = dict(batches_s=round(args.runner_steps / (r1 - r0), 2), steps=args.runner_steps,
                      what="one lmi_run_once per batch on 2 pipes, the library's default host-link grid; before batch i+1 "
                           "is issued the host waits for batch i-1 to be complete (GPURunner::RunOnce with the hand-off "
                           "on, without a trainer's own time)")
        done += args.runner_steps
    # untimed extra leg with every phase of every batch bracketed (level 1), for the per-phase breakdown only
    srv.tune("profile_every", 1)
    srv.profile_enable(1)
    run_steps(done, -(-min(args.steps, 20) // group) * group)
    srv.profile_enable(0)
    phases = srv.profile_read(reset=True)

    # algorithmic bytes per gathered row: row read + row written + 4 (id) + 4 (slot)
    rb = info["row_bytes"]
    if info["cache_kind"] == "int8":
        hit_bytes = w["dim"] + 4 + rb + 8
    else:
        hit_bytes = 2 * rb + 8
    # a group's hit gathers are one launch (on the caller's stream) and so are its host-link
    # gathers (on the side stream)
    split = int(tunes.get("split_miss", 1)) == 1
    # batches per launch of the profiled groups (the library counts the batches of the calls it profiles)
    timed_group = prof.batches / max(prof.gather_hit_launches, 1) if group > 1 else 1
    hit_batches = timed_group if split else 1
    miss_batches = timed_group if (split and int(tunes.get("group_miss", 1))) else 1
    hit_ms = prof.gather_hit_ms / max(prof.gather_hit_launches, 1)
    hit_rows = prof.gather_hit_rows / max(prof.gather_hit_launches, 1)
    miss_ms = prof.gather_miss_ms / max(prof.gather_miss_launches, 1)
    miss_rows = prof.gather_miss_rows / max(prof.gather_miss_launches, 1)
    # host-link launches per group: two with split lookups (the per-launch figures above are of one of them)
    lpg = (max(prof.gather_miss_launches / max(prof.gather_hit_launches, 1) * miss_batches / max(hit_batches, 1), 1.0)
           if split else 1.0)
    achieved = hit_rows * hit_bytes / (hit_ms * 1e-3) / 1e9 if hit_ms > 0 else 0.0
    copy_ms = lmi.bench_copy(1 << 30, 10)
    copy_gbs = 2 * (1 << 30) / (copy_ms * 1e-3) / 1e9
    # the plain copy kernel moving as many bytes as one launch of the hit gather does: what a launch of
    # this size can reach at all (a launch of a few hundred MB is over before the device is warm)
    launch_bytes = int(hit_rows * hit_bytes) // 32 * 16
    same_copy_gbs = same_launch_gbs = None
    if launch_bytes >= 1 << 16:
        same_ms = lmi.bench_copy(launch_bytes, 20)                 # back to back: launches overlap their ramps
        same_copy_gbs = 2 * launch_bytes / (same_ms * 1e-3) / 1e9
        same_ms = lmi.bench_copy_launch(launch_bytes, 20)          # launch by launch, timed as the gather is
        same_launch_gbs = 2 * launch_bytes / (same_ms * 1e-3) / 1e9
    # the streaming kernel of the gather's own read : write shape (no indirection): an int8 -> fp16 gather
    # writes twice what it reads and HBM takes writes more slowly than reads, rows of 16 k + 12 bytes put
    # every 16-byte access 4 bytes off its natural boundary -- a 1 : 1 aligned copy is the wrong yardstick for both
    shape_gbs = shape_launch_gbs = shape = rows_gbs = rows_launch_gbs = None
    if hit_rows * rb >= 1 << 16:
        if info["cache_kind"] == "int8":
            rd = 8 if w["dtype"] == "f16" else 4                 # int8 bytes a lane reads per 16-byte store
            units, wr, mis = int(hit_rows) * w["dim"] // rd, 16, 0
        else:
            rd, wr, mis = 16, 16, 4 if rb % 16 else 0
            units = int(hit_rows) * (rb // 16)
        shape = "%d:%d bytes per lane and step%s" % (rd, wr, ", 4 bytes off a 16-byte boundary" if mis else "")
        ms = lmi.bench_stream(units, rd, wr, mis, 20, False)
        shape_gbs = units * (rd + wr) / (ms * 1e-3) / 1e9
        ms = lmi.bench_stream(units, rd, wr, mis, 20, True)
        shape_launch_gbs = units * (rd + wr) / (ms * 1e-3) / 1e9
        # ... and with the rows taken from all over a table as large as the cache (computed places: no index
        # to wait for): what HBM gives a gather of this shape before the gather's own costs
        src_pitch = w["dim"] if info["cache_kind"] == "int8" else rb
        upr = src_pitch // rd
        moved = int(hit_rows) * upr * (rd + wr)
        ms = lmi.bench_row_stream(int(hit_rows), src_pitch, rd, wr, max(2, info["cache_rows"]), 20, False)
        rows_gbs = moved / (ms * 1e-3) / 1e9
        ms = lmi.bench_row_stream(int(hit_rows), src_pitch, rd, wr, max(2, info["cache_rows"]), 20, True)
        rows_launch_gbs = moved / (ms * 1e-3) / 1e9

    if args.shape_study:
        src_pitch = w["dim"] if info["cache_kind"] == "int8" else rb
        upr = src_pitch // rd
        rows_n, table = int(hit_rows), max(2, info["cache_rows"])
        moved = rows_n * upr * (rd + wr)
        print("row-streaming kernel in the shape of the %s hit gather: %d rows of %d B from hashed places of a table of %d rows,"
              " %d:%d bytes per lane and step, one launch at a time on an idle device, timed by the launch's own events;"
              " the gather itself: %.1f us per launch, %.3f of the 8 TB/s peak" % (
                  args.workload, rows_n, src_pitch, table, rd, wr, hit_ms * 1e3, achieved / HBM_PEAK_GBS))
        auto_rpb = max(1, min(64, 32768 // max(1, (src_pitch if src_pitch % 16 else upr * wr))))
        print("%-16s %-26s %-18s %10s %10s" % ("rows per visit", "grid", "idle lanes", "us", "of peak"))
        for rpb in sorted({1, 2, 4, 8, 16, 32, 64, auto_rpb}):
            tiles = -(-rows_n // rpb)
            for label, grid in (("one block per visit", tiles), ("2x: half the blocks idle", 2 * tiles),
                                ("4x: three in four idle", 4 * tiles), ("half: two visits a block", max(1, tiles // 2))):
                for every in (False, True):
                    if every and grid != tiles:
                        continue
                    ms = lmi.bench_row_stream_shape(rows_n, src_pitch, rd, wr, table, rpb, grid, every, 20, True)
                    print("%-16d %-26s %-18s %10.1f %10.3f" % (rpb, label, "load anyway" if every else "issue nothing", ms * 1e3,
                                                             moved / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS), flush=True)
        srv.close()
        return

    def mover(host_link):
        # the instantiation the library picks for this row size (launch_move_rows): a power-of-two lane
        # group when the row is 8, 16, 32 or 64 aligned 16-byte chunks, the tiled mover otherwise
        flat = int(tunes.get("miss_flat" if host_link else "gather_flat", 0))
        knobs = int(tunes.get("gather_vector_bytes", 0)) != 0 or (not host_link and int(tunes.get("gather_lanes_per_row", 0)) != 0)
        exact = rb % 16 == 0 and rb // 16 in (8, 16, 32, 64)
        hl = "true" if host_link else "false"
        if not host_link and rb >= 16 and not knobs and flat in (0, 3):   # the hits: the flat gather
            unroll = int(tunes.get("gather_unroll", 0)) or 2
            return "gather_rows_flat_kernel<%s,%d,true>" % ("u32x4" if rb % 16 == 0 else "u32x4 at 4-byte alignment",
                                                            4 if unroll >= 4 else 2 if unroll >= 2 else 1)
        if rb >= 16 and (flat == 1 or (flat == 0 and not exact and not knobs)):
            unroll = int(tunes.get("miss_unroll", 1)) if host_link else (int(tunes.get("gather_unroll", 0)) or 2)
            unroll = 4 if unroll >= 4 else 2 if unroll >= 2 else 1
            return "move_rows_tiled_kernel<%s,%d,%d,true,%s>" % ("u32x4" if rb % 16 == 0 else "u32x4 at 4-byte alignment",
                                                                 256 if rb < 128 else 64, unroll, hl)
        vec = 16 if rb % 16 == 0 else 8 if rb % 8 == 0 else 4
        narrower = int(tunes.get("gather_vector_bytes", 0))
        if narrower == 4 or (narrower == 8 and vec == 16):
            vec = narrower
        lanes = 0 if host_link else int(tunes.get("gather_lanes_per_row", 0))
        if lanes not in (1, 4, 8, 16, 32, 64):
            lanes = 8
            while lanes < rb // vec and lanes < 64:
                lanes *= 2
        unroll = int(tunes.get("miss_unroll", 1)) if host_link else (int(tunes.get("gather_unroll", 0)) or 1)
        return "move_rows_kernel<%s,%d,%d,true,%s>" % ({16: "u32x4", 8: "u32x2", 4: "u32"}[vec], lanes, unroll, hl)
    if info["cache_kind"] == "int8":
        half = w["dtype"] == "f16"
        if w["dim"] % 16 == 0 and int(tunes.get("gather_flat", 0)) != 2:
            epl = int(tunes.get("int8_elements_per_lane", 0))
            if epl not in (4, 8, 16) or (half and epl == 4):
                epl = 8 if half else 4
            unroll = int(tunes.get("gather_unroll", 0))
            hit_kernel = "gather_int8_tiled_kernel<%s,%d,%d>" % ("__half" if half else "float", epl,
                                                                 4 if unroll >= 4 else 1 if unroll == 1 else 2)
        else:
            hit_kernel = "gather_int8_kernel<%s,%d>" % ("__half" if half else "float", 16 if w["dim"] // 16 <= 16 else 32)
        hit_kernel += " (HBM gather of cache hits, dequantisation fused)"
    else:
        hit_kernel = mover(False) + " (HBM gather of cache hits)"
    # HBM bytes per launch as the counters saw them: not collected by this run (rocprofv3 --pmc needs runs of
    # its own), but recorded from the same command in the file named beside it
    traffic = recorded_traffic(args.workload) if (args.scale == 1.0 and info["scale"] == 1.0 and
                                                  args.neighbours == "degree") else None
    traffic_source = ("recorded: profiles/%s_hit_gather_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE of "
                      "this command, calibrated on the copy kernel; not counted during this run)" % args.workload
                      ) if traffic is not None else None
    # the same figure from the launches profiled inside the timed region itself, when that is a leg of its own
    # (a short run: few launches, the first of them beside an idle side stream)
    tp = timed["prof"]
    t_ms = tp.gather_hit_ms / max(tp.gather_hit_launches, 1)
    t_rows = tp.gather_hit_rows / max(tp.gather_hit_launches, 1)
    timed_sample = dict(launches=int(tp.gather_hit_launches), batches=int(tp.batches), rows_per_launch=round(t_rows, 1),
                        avg_launch_ms=round(t_ms, 4),
                        frac=round(t_rows * hit_bytes / (t_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4) if t_ms > 0 else None)
    roofline = dict(bound="hbm", kernel=hit_kernel, achieved=round(achieved, 1),
                    peak=HBM_PEAK_GBS, unit="GB/s", frac=round(achieved / HBM_PEAK_GBS, 4),
                    traffic=traffic, traffic_source=traffic_source,
                    rows_per_launch=round(hit_rows, 1), batches_per_launch=round(hit_batches, 2), bytes_per_row=hit_bytes,
                    avg_launch_ms=round(hit_ms, 4), launches=int(prof.gather_hit_launches),
                    measured_over=("the timed region" if steady_leg is timed else
                                   "the %d-step steady leg of the same loop (the timed region's own sample: timed_region)"
                                   % steady_leg["steps"]),
                    timed_region=timed_sample,
                    measured_copy_gbs=round(copy_gbs, 1),
                    same_bytes_copy_gbs=round(same_copy_gbs, 1) if same_copy_gbs else None,
                    same_bytes_copy_single_launch_gbs=round(same_launch_gbs, 1) if same_launch_gbs else None,
                    same_shape_stream=shape,
                    same_shape_stream_gbs=round(shape_gbs, 1) if shape_gbs else None,
                    same_shape_stream_single_launch_gbs=round(shape_launch_gbs, 1) if shape_launch_gbs else None,
                    same_shape_scattered_rows_gbs=round(rows_gbs, 1) if rows_gbs else None,
                    same_shape_scattered_rows_single_launch_gbs=round(rows_launch_gbs, 1) if rows_launch_gbs else None)
    link_bytes = min(1 << 28, info["feats"].nbytes)
    link_ms = lmi.bench_host_read(info["feats"], link_bytes)
    host_link = dict(bound="host-link", kernel=mover(True) + " (host-link gather of misses)",
                     measured_stream_read_gbs=round(link_bytes // 16 * 16 / (link_ms * 1e-3) / 1e9, 2),
                     achieved=round(miss_rows * rb / (miss_ms * 1e-3) / 1e9, 2) if miss_ms > 0 else 0.0,
                     peak=HOST_LINK_PEAK_GBS, unit="GB/s", rows_per_launch=round(miss_rows, 1),
                     batches_per_launch=round(miss_batches, 2),
                     launches_per_group=round(lpg, 2),
                     avg_launch_ms=round(miss_ms, 4))
    # the sampling kernels are bound by cold random reads: what the device sustains on the neighbour array
    rr_reads = 1 << 24
    rr_ms = lmi.bench_random_read(info["d_indices"], info["n_edges"] * 4, rr_reads)
    total_rows = prof.gather_hit_rows + prof.gather_miss_rows
    profiled_batches = int(prof.batches)
    out = {
        "metric": "sampled mini-batches/sec", "value": round(args.steps / timed["sec"], 2), "unit": "batches/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "drain_ms": round(drain_ms, 3),
        "steady_state_batches_s": steady["batches_s"] if steady else None, "steady_state": steady,
        "runner_issue_batches_s": runner["batches_s"] if runner else None, "runner_issue": runner,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int32", "feature_dtype": "fp16" if w["dtype"] == "f16" else "fp32",
        "data": "synthetic",
        "config": {"workload": args.workload, "nodes": info["n_nodes"], "edges": info["n_edges"],
                   "feat_dim": w["dim"], "batch": w["batch"], "fanout": w["fanout"],
                   "cache": "%s, %d rows, %s id->slot table" % (info["cache_kind"], info["cache_rows"], args.table),
                   "pipes": args.pipes, "streams": args.streams, "group": group, "issue": args.issue,
                   "group_sizes": group_sizes(args.steps) if (group > 1 and args.issue == "group") else None, "tune": tunes,
                   "cache_policy": args.policy,
                   "graph": info["graph"],
                   "seeds": ("%d %% of a batch from the frontiers of the previous %d batches, the rest uniform from the "
                             "train set" % (w["locality"][0] * 100, w["locality"][1])) if w.get("locality")
                   else "consecutive slices of the train set",
                   "note": info["note"]},
        "feature_gather_gbs": round(achieved, 1),
        "feature_gather_frac_hbm_peak": round(achieved / HBM_PEAK_GBS, 4),
        # hits and misses together: all bytes moved into the output rows over the time of both kernels
        # (they run on different streams, so this is a lower bound on what the batch sees)
        "feature_gather_blended_gbs": round((hit_rows / hit_batches * hit_bytes + lpg * miss_rows / miss_batches * (2 * rb + 8)) /
                                            ((hit_ms / hit_batches + lpg * miss_ms / miss_batches) * 1e-3) / 1e9, 1)
        if hit_ms + miss_ms > 0 else None,
        "cache_hit_rate": round(prof.gather_hit_rows / total_rows, 4) if total_rows else None,
        "rows_per_batch": round(total_rows / max(profiled_batches, 1), 1),
        "profiled_batches": profiled_batches,
        "phase_ms_per_batch": {"sample_dedup_lookup": round(phases.sample_ms / max(phases.sample_launches, 1) / group, 4),
                               "gather_hit": round(hit_ms / hit_batches, 4),
                               # all of a group's host-link launches (two with split lookups), per batch
                               "gather_miss_side_stream": round(lpg * miss_ms / miss_batches, 4)},
        "roofline": roofline, "host_link": host_link,
        "random_read": {"measured_g_reads_per_s": round(rr_reads / (rr_ms * 1e-3) / 1e9, 1),
                        "what": "independent 4-byte reads at random places of the neighbour array"},
    }
    if args.cpu_seconds > 0:
        issue = dict(pipes=2 if args.issue == "runner" else args.pipes, group=1 if args.issue == "runner" else group,
                     first_sizes=group_sizes(args.steps) if (group > 1 and args.issue == "group") else [],
                     steps_per_epoch=steps_per_epoch, plan=plan)
        if plan:   # the replayed LRU sequence is only the recorded one from an empty cache again
            ci = srv.cache_info()
            srv.build_lru_cache(int(ci.n_sets), int(ci.ways))
        cb, ok = cpu_baseline(lmi, srv, w, info, args.seed, args.cpu_seconds, issue)
        out["cpu_baseline"] = cb
        out["parity_at_bench_scale"] = "bit-exact" if ok else "MISMATCH"
        out["parity_issue"] = cb["sample"].split("issued as the timed region issues them (")[1].rsplit(")", 1)[0]
    else:
        out["cpu_baseline"] = None
    srv.close()
    # The headline rests on a graph whose in-degrees follow the out-degree law (degree-proportional
    # neighbours: 96 % of the rows of a batch hit a degree-ordered cache).  The same workload on a graph
    # with uniform neighbours is the other end: the cache hits at exactly capacity / nodes and the batch rate
    # is the host link's.  A short leg of it keeps that visible wherever the headline goes.
    out["uniform_neighbours_companion"] = None
    if (args.companion_steps > 0 and args.neighbours == "degree" and w["alpha"] is not None and group > 1
            and args.issue == "group"):
        try:
            out["uniform_neighbours_companion"] = companion(lmi, w, info, args, tunes, group)
        except Exception as e:   # the companion must never cost the run its line
            out["uniform_neighbours_companion"] = {"error": str(e)[:300]}
    print(json.dumps(out), flush=True)


def companion(lmi, w, info, args, tunes, group):
    """The same workload, features, train set and cache budget on a graph with uniform neighbours."""
    t0 = time.time()
    lmi.check(lmi.lib().lmi_device_free(info["d_indptr"]))
    lmi.check(lmi.lib().lmi_device_free(info["d_indices"]))
    cdf = lmi.zipf_cdf(w["alpha"], w["d_max"], w["mean_deg"])
    d_indptr, d_indices, n_edges = lmi.synth_graph(args.seed, cdf, info["n_nodes"], 0)
    inputs = dict(info, d_indptr=d_indptr, d_indices=d_indices, n_edges=n_edges)
    info["d_indptr"], info["d_indices"] = d_indptr, d_indices    # main()'s caller frees what is current
    srv, cinfo = build_server(lmi, w, inputs, args.seed, args.pipes, {"hash": 0, "direct": 1, "rank": 2}[args.table])
    try:
        for k, v in tunes.items():
            srv.tune(k, int(v))
        stream = lmi.stream_create()
        spe = -(-cinfo["n_train"] // w["batch"])

        def run(first, count):
            i = first
            while i < first + count:
                n = min(group, first + count - i)
                ks = range(i, i + n)
                srv.run_group([k % args.pipes for k in ks], [k % spe for k in ks], rng_seeds=[args.seed + k for k in ks],
                              stream=stream)
                i += n
        run(0, 2 * group)
        lmi.check(lmi.lib().lmi_device_sync())
        srv.profile_read(reset=True)
        srv.tune("profile_every", 2)
        srv.profile_enable(2)
        c0 = time.perf_counter()
        run(2 * group, args.companion_steps)
        lmi.check(lmi.lib().lmi_device_sync())
        c1 = time.perf_counter()
        srv.status()
        srv.profile_enable(0)
        p = srv.profile_read(reset=True)
        rb = cinfo["row_bytes"]
        hit_bytes = (w["dim"] + 4 + rb + 8) if cinfo["cache_kind"] == "int8" else 2 * rb + 8
        hit_ms = p.gather_hit_ms / max(p.gather_hit_launches, 1)
        miss_ms = p.gather_miss_ms / max(p.gather_miss_launches, 1)
        total = p.gather_hit_rows + p.gather_miss_rows
        return dict(graph="the same degrees, uniform neighbours", steps=args.companion_steps,
                    batches_s=round(args.companion_steps / (c1 - c0), 2),
                    cache_hit_rate=round(p.gather_hit_rows / total, 4) if total else None,
                    rows_per_batch=round(total / max(int(p.batches), 1), 1),
                    hit_gather_frac_hbm_peak=round(p.gather_hit_rows / max(p.gather_hit_launches, 1) * hit_bytes /
                                                   (hit_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4) if hit_ms > 0 else None,
                    host_link_gbs=round(p.gather_miss_rows / max(p.gather_miss_launches, 1) * rb / (miss_ms * 1e-3) / 1e9, 2)
                    if miss_ms > 0 else None,
                    setup_s=round(time.time() - t0 - (c1 - c0), 1))
    finally:
        srv.close()


if __name__ == "__main__":
    main()
