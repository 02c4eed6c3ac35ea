"""A trainer that only takes the batches: attaches to a running `sampling_server`, receives every
batch of the schedule through the semaphore handshake (the headers are read, nothing else is), and
releases it at once.  Prints the rate, which is then the sampler side's own (run by
test_gpu_server_binary.py as a subprocess).
usage: handoff_drain.py <batches>
"""
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from conftest import load_ipc_service  # noqa: E402


def main():
    total = int(sys.argv[1])
    ipc = load_ipc_service()
    ipc.initialize()
    rows = 0
    ipc._next(120.0)            # the first batch also carries the server's start-up
    ipc.synchronize()
    t0 = time.perf_counter()
    for _ in range(total - 1):
        b = ipc._next(120.0)
        rows += int(b.n_ids)
        ipc.synchronize()
    t1 = time.perf_counter()
    ipc.finalize()
    print("DRAIN_OK %d batches, %.1f batches/s, %.0f rows per batch" % (total, (total - 1) / (t1 - t0), rows / max(total - 1, 1)),
          flush=True)


if __name__ == "__main__":
    main()
