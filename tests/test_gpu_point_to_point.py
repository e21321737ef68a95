"""Send / Recv / BatchSendRecv on the GPU against the oracle's pairing rule, through the Python mirror of
hccl4py.ops (reference experimental/eco_system/python/tests/run_dtype_suite.py:333-380: one element per
neighbour travels round the ring)."""
import threading

import numpy as np
import pytest

import hccl_amd
import oracle
from hccl_amd import HcclDataType as DT, HcclSendRecvType as T

from gpu_util import World, dev_zeros, require_library_on_gpu, to_dev, to_host

pytestmark = pytest.mark.gpu
NP = {DT.INT8: np.int8, DT.FP16: np.float16, DT.FP32: np.float32, DT.INT64: np.int64, DT.UINT8: np.uint8}


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


def payload(rng, dtype, count):
    return rng.integers(0, 255, count * np.dtype(NP[dtype]).itemsize, dtype=np.uint8).view(NP[dtype])


@pytest.mark.parametrize("n", [2, 5, 8])
@pytest.mark.parametrize("dtype,count", [(DT.FP32, 1), (DT.FP32, 100_003), (DT.INT8, 77_777), (DT.INT64, 4_097)])
def test_ring_of_sends_and_receives_inside_a_group(n, dtype, count):
    w = World(n)
    try:
        rng = np.random.default_rng(n * 11 + count)
        ins = [payload(rng, dtype, count) for _ in range(n)]
        want = [np.zeros(count, dtype=NP[dtype]) for _ in range(n)]
        assert oracle.batch_send_recv([[(0, ins[r], count, int(dtype), (r + 1) % n),
                                        (1, want[r], count, int(dtype), (r - 1) % n)] for r in range(n)]) == 0
        sends = [to_dev(x, 2 * (r % 3)) for r, x in enumerate(ins)]
        recvs = [dev_zeros(x.nbytes, 4 * (r % 2)) for r, x in enumerate(ins)]
        w.inputs_ready()
        with hccl_amd.group():
            for r in range(n):
                hccl_amd.send(w.comms[r], sends[r], count, dtype, (r + 1) % n, w.stream)
                hccl_amd.recv(w.comms[r], recvs[r], count, dtype, (r - 1) % n, w.stream)
        w.sync()
        for r in range(n):
            assert np.array_equal(to_host(recvs[r], NP[dtype]).view(np.uint8), want[r].view(np.uint8)), r
    finally:
        w.close()


def test_blocking_calls_from_one_thread_per_rank_on_streams_of_their_own():
    """Even ranks send first, odd ranks receive first; every rank works on its own stream, produces its payload
    there just before sending and consumes what it received right after: the streams must be ordered by the
    library."""
    import torch
    n, count = 4, 1 << 20
    info = hccl_amd.get_root_info()
    got = [None] * n
    errors = []
    all_through = threading.Barrier(n)   # destroying one rank ends the world: wait until every rank has made its calls

    def main(rank):
        try:
            comm = hccl_amd.comm_init_root_info(n, info, rank)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                mine = torch.full((count,), float(rank + 1), dtype=torch.float32, device="cuda")
                inbox = torch.zeros(count, dtype=torch.float32, device="cuda")
                for _ in range(20):                 # keep the stream busy so that ordering matters
                    mine = mine * 1.0
            nxt, prv = (rank + 1) % n, (rank - 1) % n
            if rank % 2 == 0:
                hccl_amd.send(comm, mine, count, DT.FP32, nxt, stream)
                hccl_amd.recv(comm, inbox, count, DT.FP32, prv, stream)
            else:
                hccl_amd.recv(comm, inbox, count, DT.FP32, prv, stream)
                hccl_amd.send(comm, mine, count, DT.FP32, nxt, stream)
            with torch.cuda.stream(stream):
                total = (inbox * 2.0).sum()
            stream.synchronize()
            got[rank] = float(total.item())
            all_through.wait(90)
            hccl_amd.comm_destroy(comm)
        except Exception as e:   # noqa: BLE001 - reported below
            errors.append((rank, repr(e)))

    threads = [threading.Thread(target=main, args=(r,)) for r in range(n)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(100)
    assert not errors, errors
    for rank in range(n):
        assert got[rank] == 2.0 * count * (((rank - 1) % n) + 1), (rank, got[rank])


@pytest.mark.parametrize("n", [2, 4, 7])
def test_batches_pair_repeated_transfers_by_size_then_type(n):
    """Every ordered pair exchanges three transfers listed in different orders on the two sides, one rank also
    sends to itself, some items are empty."""
    w = World(n)
    try:
        rng = np.random.default_rng(500 + n)
        shapes = [(DT.FP32, 4_000), (DT.FP16, 4_000), (DT.UINT8, 65_537)]      # two equal counts: the type decides
        host_items = [[] for _ in range(n)]
        dev_items = [[] for _ in range(n)]
        checks = []
        keep = []                     # the items hold raw addresses: keep the tensors alive
        for a in range(n):
            for b in range(n):
                if a == b and a != 1:
                    continue
                order_s = rng.permutation(3)
                order_r = rng.permutation(3)
                for k in order_s:
                    dtype, count = shapes[k]
                    x = payload(rng, dtype, count)
                    host_items[a].append((0, x, count, int(dtype), b))
                    keep.append(to_dev(x))
                    dev_items[a].append(hccl_amd.make_send_recv_item(T.SEND, keep[-1], count, dtype, b))
                for k in order_r:
                    dtype, count = shapes[k]
                    y = np.zeros(count, dtype=NP[dtype])
                    d = dev_zeros(y.nbytes)
                    host_items[b].append((1, y, count, int(dtype), a))
                    dev_items[b].append(hccl_amd.make_send_recv_item(T.RECV, d, count, dtype, a))
                    checks.append((d, y, NP[dtype]))
            host_items[a].append((0, None, 0, int(DT.FP32), (a + 1) % n))
            dev_items[a].append(hccl_amd.make_send_recv_item(T.SEND, None, 0, DT.FP32, (a + 1) % n))
        assert oracle.batch_send_recv(host_items) == 0
        w.inputs_ready()
        with hccl_amd.group():
            for r in range(n):
                hccl_amd.batch_send_recv(w.comms[r], dev_items[r], w.stream)
        w.sync()
        for d, y, npdt in checks:
            assert np.array_equal(to_host(d, npdt).view(np.uint8), y.view(np.uint8))
    finally:
        w.close()


def test_unequal_counts_on_the_two_sides_are_reported_to_both():
    w = World(2)
    try:
        a, b = dev_zeros(64), dev_zeros(64)
        codes = []
        hccl_amd.group_start()
        for fn, args in ((hccl_amd.send, (w.comms[0], a, 8, DT.FP32, 1, w.stream)),
                         (hccl_amd.recv, (w.comms[1], b, 4, DT.FP32, 0, w.stream))):
            try:
                codes.append(fn(*args))
            except hccl_amd.HcclError as e:
                codes.append(e.code)
        with pytest.raises(hccl_amd.HcclError) as ended:
            hccl_amd.group_end()
        assert ended.value.code == 1                                 # the group's end reports it for the queued side
        assert codes[-1] == 1                                        # HCCL_E_PARA at the call that completes the pair
        w.sync()
        assert np.all(to_host(b, np.uint8) == 0xAB)                  # nothing was copied
    finally:
        w.close()


def test_barrier_orders_the_streams_of_all_ranks():
    """Every rank fills its buffer on its own stream, all meet at the barrier, then every rank reads its
    neighbour's buffer on its own stream: without the barrier's ordering the read could overtake the fill."""
    import torch
    n, count = 4, 1 << 22
    comms = hccl_amd.comm_init_all(n)
    try:
        streams = [torch.cuda.Stream() for _ in range(n)]
        bufs = [torch.zeros(count, dtype=torch.float32, device="cuda") for _ in range(n)]
        sums = [None] * n
        torch.cuda.synchronize()
        for r in range(n):
            with torch.cuda.stream(streams[r]):
                for _ in range(10):
                    bufs[r].add_(0.1 * (r + 1))
        with hccl_amd.group():
            for r in range(n):
                hccl_amd.barrier(comms[r], streams[r])
        for r in range(n):
            with torch.cuda.stream(streams[r]):
                sums[r] = bufs[(r + 1) % n].sum(dtype=torch.float64)
        torch.cuda.synchronize()
        for r in range(n):
            acc = torch.zeros(1, dtype=torch.float32)
            for _ in range(10):
                acc.add_(0.1 * (((r + 1) % n) + 1))
            assert abs(float(sums[r].item()) - float(acc.item()) * count) < 1e-3 * count, r
    finally:
        for c in comms:
            hccl_amd.comm_destroy(c)
