#!/usr/bin/env python3
"""Writes tests/golden/spec_v1.npz: small fixed inputs (graph, seeds, features) together
with the outputs the CPU oracle gives for them today -- sampled batches for three fan-out
shapes, the degree-ordered static cache, an LRU trace and the int8 codec.

The fixture freezes the sampling specification: tests/test_golden.py checks the oracle
(CPU) and the HIP path (GPU) against it, so a change that moved both in step would still
be seen.  Inputs are stored in the file, not regenerated, so the fixture does not depend
on a random-number library's version.  Run from the repository root:

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import binding as orc  # noqa: E402

CASES = [("a", [25, 10], 48), ("b", [3, 2, 2], 40), ("c", [64], 16)]


def main():
    rng = np.random.default_rng(20240607)
    n = 400
    deg = rng.poisson(9, n).astype(np.int64)
    deg[rng.random(n) < 0.1] = 0
    deg[[7, 123, 301]] = [150, 90, 260]                      # hubs: rows longer than any fan-out
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    indices = rng.integers(0, n, int(indptr[-1])).astype(np.int32)
    feats = rng.standard_normal((n, 16)).astype(np.float32)
    out = dict(indptr=indptr, indices=indices, feats=feats)
    for tag, fanout, batch in CASES:
        seeds = rng.choice(n, batch, replace=False).astype(np.int32)
        seeds[3] = seeds[1]                                  # a repeated seed
        rs = 1234 + len(fanout)
        b = orc.sample_batch(indptr, indices, seeds, fanout, rs)
        out.update({tag + "_seeds": seeds, tag + "_fanout": np.array(fanout, np.int32), tag + "_rng": np.int64(rs),
                    tag + "_ids": b.ids, tag + "_src_ids": b.agg_src_ids, tag + "_src": b.agg_src_off,
                    tag + "_dst": b.agg_dst_off, tag + "_nc": b.node_counter, tag + "_ec": b.edge_counter,
                    tag + "_indptr": np.concatenate(b.blk_indptr)})
    out["static_cap"] = np.int64(120)
    out["static_slots"] = orc.static_cache_build(indptr, 120)
    # LRU: 16 sets x 4 ways, three batches of case a's shape (fan-out [25, 10], 48 seeds, RNG seeds 1236 + k)
    lru = orc.Lru(16, 4, 64)
    rows = feats.view(np.uint8).reshape(n, 64)
    for k in range(3):
        seeds = out["a_seeds"] if k == 0 else rng.choice(n, 48, replace=False).astype(np.int32)
        b = orc.sample_batch(indptr, indices, seeds, [25, 10], 1236 + k)
        hit, fill, got = lru.access(b.ids, rows)
        out["lru_seeds_%d" % k], out["lru_hit_%d" % k], out["lru_fill_%d" % k] = seeds, hit, fill
        assert got.tobytes() == rows[b.ids].tobytes()
    out["lru_keys"], out["lru_use"] = lru.state()
    # int8 codec on the first 64 rows, fp32 and fp16
    q, sc = orc.quantize_rows(feats[:64])
    out["q32"], out["scale32"], out["deq32"] = q, sc, orc.dequant_rows(q, sc, np.float32)
    h = feats[:64].astype(np.float16)
    q, sc = orc.quantize_rows(h)
    out["q16"], out["scale16"], out["deq16"] = q, sc, orc.dequant_rows(q, sc, np.float16)
    path = os.path.join(HERE, "spec_v1.npz")
    np.savez_compressed(path, **out)
    print("wrote %s (%d bytes)" % (path, os.path.getsize(path)))


if __name__ == "__main__":
    main()
