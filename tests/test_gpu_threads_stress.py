"""Many blocking collectives in a row from one host thread per rank, and two worlds running side by side: the
rendezvous must pair the k-th call of every rank whatever the interleaving of the threads."""
import threading

import numpy as np
import pytest

import hccl_amd
from hccl_amd import HcclDataType as DT, HcclReduceOp as OP

from gpu_util import require_library_on_gpu

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


def rank_main(n, info, rank, iters, count, failures, tag):
    import torch
    try:
        comm = hccl_amd.comm_init_root_info(n, info, rank)
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            x = torch.full((count,), float(rank + 1), dtype=torch.float32, device="cuda")
            y = torch.zeros(count, dtype=torch.float32, device="cuda")
            g = torch.zeros(n * count, dtype=torch.float32, device="cuda")
            s = torch.zeros(count // n, dtype=torch.float32, device="cuda")
        stream.synchronize()
        total = n * (n + 1) / 2
        for it in range(iters):
            kind = it % 4
            if kind == 0:
                hccl_amd.all_reduce(comm, x, y, count, DT.FP32, OP.SUM, stream)
            elif kind == 1:
                hccl_amd.all_gather(comm, x, g, count, DT.FP32, stream)
            elif kind == 2:
                hccl_amd.reduce_scatter(comm, x, s, count // n, DT.FP32, OP.SUM, stream)
            else:
                hccl_amd.broadcast(comm, y, count, DT.FP32, it % n, stream)
            if it % 37 == 0 or it >= iters - 4:
                stream.synchronize()
                if kind == 0 and not bool((y == total).all()):
                    failures.append((tag, rank, it, "all_reduce"))
                if kind == 1 and not all(bool((g[r * count:(r + 1) * count] == r + 1).all()) for r in range(n)):
                    failures.append((tag, rank, it, "all_gather"))
                if kind == 2 and not bool((s == total).all()):
                    failures.append((tag, rank, it, "reduce_scatter"))
                if kind == 3 and not bool((y == total).all()):      # every y already holds the AllReduce result
                    failures.append((tag, rank, it, "broadcast"))
        stream.synchronize()
        hccl_amd.comm_destroy(comm)
    except Exception as e:   # noqa: BLE001 - reported by the caller
        failures.append((tag, rank, -1, repr(e)))


def test_three_hundred_blocking_collectives_per_rank_in_two_worlds_at_once():
    failures = []
    threads = []
    for tag, n, count in (("a", 8, 8 * 1024), ("b", 3, 3 * 5000)):
        info = hccl_amd.get_root_info()
        threads += [threading.Thread(target=rank_main, args=(n, info, r, 300, count, failures, tag)) for r in range(n)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(110)
    assert not any(t.is_alive() for t in threads), "a rank is stuck"
    assert not failures, failures[:5]
