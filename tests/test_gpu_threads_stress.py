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


def test_three_hundred_blocking_collectives_per_rank_in_two_worlds_at_once(monkeypatch):
    # A stuck rank gives up after a minute (the variable is read when a world is created) and, being a daemon
    # thread, cannot keep the interpreter from exiting after the assertion below has failed.
    monkeypatch.setenv("HCCL_EXEC_TIMEOUT", "60")
    failures = []
    threads = []
    for tag, n, count in (("a", 8, 8 * 1024), ("b", 3, 3 * 5000)):
        info = hccl_amd.get_root_info()
        threads += [threading.Thread(target=rank_main, args=(n, info, r, 300, count, failures, tag), daemon=True)
                    for r in range(n)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(110)
    assert not any(t.is_alive() for t in threads), "a rank is stuck"
    assert not failures, failures[:5]


def test_two_threads_each_grouping_half_of_the_ranks():
    """Each thread queues the calls of four of the eight ranks inside a group on its own stream; whichever
    thread completes a set launches it.  After HcclGroupEnd every rank's stream of the calling thread is ordered
    behind the collective, so a stream synchronisation followed by a read sees the result."""
    import torch
    n, count, iters = 8, 4096 + 8, 40
    comms = hccl_amd.comm_init_all(n)
    failures = []
    xs = [torch.full((count,), float(r + 1), dtype=torch.float32, device="cuda") for r in range(n)]
    ys = [torch.zeros(count, dtype=torch.float32, device="cuda") for _ in range(n)]
    torch.cuda.synchronize()
    total = n * (n + 1) / 2

    def half(k):
        try:
            stream = torch.cuda.Stream()
            mine = range(4 * k, 4 * k + 4)
            for it in range(iters):
                for r in mine:
                    ys[r].zero_()
                torch.cuda.current_stream().synchronize()
                with hccl_amd.group():
                    for r in mine:
                        hccl_amd.all_reduce(comms[r], xs[r], ys[r], count, DT.FP32, OP.SUM, stream)
                stream.synchronize()
                for r in mine:
                    if not bool((ys[r] == total).all()):
                        failures.append((k, it, r))
        except Exception as e:   # noqa: BLE001 - reported by the caller
            failures.append((k, -1, repr(e)))

    threads = [threading.Thread(target=half, args=(k,), daemon=True) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(100)
    assert not any(t.is_alive() for t in threads), "a thread is stuck"
    assert not failures, failures[:5]
    for c in comms:
        hccl_amd.comm_destroy(c)
