#!/usr/bin/env python3
"""Measures the feature-gather memory-access variants on the paper100m-shaped workload:
bytes per lane access, lanes per row (thread-per-row ... wavefront-per-row), rows in flight
per lane, temporal / non-temporal stores, and how many blocks the host-link gather gets.
Every variant is a tuning key of lmi_tune; times are HIP events inside the library.  Run it
under `rocprofv3 --kernel-trace --stats` to get the per-instantiation kernel durations too
(each variant is a different move_rows_kernel<V, LPR, U, NT> instantiation).

    python legion-ibp_amd/gather_variants.py
"""
import sys, os, time, json
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))  # repo root (bench.py)
import bench
lmi = bench.load_package()
w = dict(bench.WORKLOADS["paper100m"])
srv, info = bench.build_workload(lmi, w, 20260101, 2, 64.0)
stream = lmi.stream_create()
spe = -(-info["n_train"] // w["batch"])
def run(steps=60):
    for i in range(3): srv.run_once(None, batch_counter=i % spe, rng_seed=100+i, pipe=i%2, stream=stream)
    lmi.check(lmi.lib().lmi_device_sync()); srv.profile_read(True); srv.profile_enable(True)
    t0=time.perf_counter()
    for i in range(steps): srv.run_once(None, batch_counter=i % spe, rng_seed=100+i, pipe=i%2, stream=stream)
    lmi.check(lmi.lib().lmi_device_sync()); t1=time.perf_counter()
    srv.profile_enable(False); p = srv.profile_read(True)
    hit_ms = p.gather_hit_ms/max(p.gather_hit_launches,1); rows = p.gather_hit_rows/max(p.gather_hit_launches,1)
    miss_ms = p.gather_miss_ms/max(p.gather_miss_launches,1); mrows = p.gather_miss_rows/max(p.gather_miss_launches,1)
    return "hit %.1f us %.0f GB/s (%.1f%% of 8 TB/s) | miss %.1f us %.1f GB/s | sample %.1f us | %.1f us/batch" % (
        hit_ms*1e3, rows*1032/(hit_ms*1e-3)/1e9, rows*1032/(hit_ms*1e-3)/1e9/80, miss_ms*1e3, mrows*512/(miss_ms*1e-3)/1e9 if miss_ms else 0,
        p.sample_ms/max(p.sample_launches,1)*1e3, (t1-t0)*1e6/steps)
print("default (16 B lanes, 32 lanes/row, 1 row in flight, nt stores)       ", run(), flush=True)
for vb in (4, 8):
    srv.tune("gather_vector_bytes", vb); print("vector %2d B per lane (lanes/row auto)                               " % vb, run(), flush=True)
srv.tune("gather_vector_bytes", 0)
for lpr in (1, 4, 8, 16, 64):
    srv.tune("gather_lanes_per_row", lpr); print("lanes per row %2d (16 B lanes)%s" % (lpr, "  = thread per row                  " if lpr == 1 else "  = wavefront per row               " if lpr == 64 else "                                    "), run(), flush=True)
srv.tune("gather_lanes_per_row", 0)
for u in (2, 4, 8):
    srv.tune("gather_unroll", u); print("rows in flight per lane %d                                          " % u, run(), flush=True)
srv.tune("gather_unroll", 1)
srv.tune("gather_nontemporal", 0); print("plain (temporal) output stores                                      ", run(), flush=True)
srv.tune("gather_nontemporal", 1)
for mb in (8, 16, 64, 256):
    srv.tune("miss_blocks", mb); print("host-link gather on %3d blocks                                      " % mb, run(), flush=True)
srv.tune("miss_blocks", 32)
srv.tune("split_miss", 0); print("host-link gather on the caller's stream (no overlap)                ", run(), flush=True)
srv.close()
