"""HcclAmdAlltoAllVNoAlloc, the AlltoAllV entry point that allocates nothing: its results must equal those
of HcclAlltoAllV bit for bit (and the CPU oracle's), also on a second call with a smaller input that reuses
the library's device-resident table array, across worlds of different size, and with ranks on different
streams.  Collected last so that a failure here cannot hide another test."""
import numpy as np
import pytest

import hccl_amd
import oracle
from hccl_amd import HcclDataType as DT

from gpu_util import World, a2a_case, dev_zeros, rand_bytes, require_library_on_gpu, to_dev, to_host

pytestmark = pytest.mark.gpu
FILL = 0xAB


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


def run_both(w, rng, n, esz, max_count, aligned, streams=None):
    """One AlltoAllV case through both entry points; returns nothing, asserts equality with each other and the oracle."""
    sc, sd, rc, rd, in_sz, out_sz = a2a_case(rng, n, esz, max_count, aligned)
    ins = [rand_bytes(rng, in_sz * esz) for _ in range(n)]
    want = [np.full(out_sz * esz, FILL, dtype=np.uint8) for _ in range(n)]
    assert oracle.all_to_all_v(ins, want, sc, sd, rc, rd, int(DT.BFP16)) == 0
    sends = [to_dev(x) for x in ins]
    ref = [dev_zeros(out_sz * esz, fill=FILL) for _ in range(n)]
    got = [dev_zeros(out_sz * esz, fill=FILL) for _ in range(n)]
    w.all_to_all_v(sends, sc, sd, ref, rc, rd, DT.BFP16)
    w.inputs_ready()
    with hccl_amd.group():
        for r in range(n):
            s = w.stream if streams is None else streams[r % len(streams)]
            hccl_amd.all_to_all_v_no_alloc(w.comms[r], sends[r], sc[r], sd[r], DT.BFP16, got[r], rc[r], rd[r], DT.BFP16, s)
    w.sync()
    if streams is not None:
        for s in streams:
            s.synchronize()
    for r in range(n):
        g = to_host(got[r], np.uint8)
        assert np.array_equal(g, to_host(ref[r], np.uint8)), (n, aligned, max_count, r, "vs HcclAlltoAllV")
        assert np.array_equal(g, want[r]), (n, aligned, max_count, r, "vs oracle")


@pytest.mark.parametrize("aligned", [True, False])
def test_two_calls_in_a_row_the_second_smaller(aligned):
    n = 8
    w = World(n)
    try:
        rng = np.random.default_rng(7 + aligned)
        run_both(w, rng, n, 2, 40_000, aligned)
        run_both(w, rng, n, 2, 300, aligned)     # smaller: the tables of the first call are still in the array
        run_both(w, rng, n, 2, 9, aligned)       # many empty segments
    finally:
        w.close()


def test_worlds_of_different_size_share_the_array():
    rng = np.random.default_rng(11)
    big = World(64)
    small = World(3)
    single = World(1)
    try:
        run_both(big, rng, 64, 2, 6_000, False)     # thousands of segments: the tables take dozens of writer launches
        run_both(small, rng, 3, 2, 5_000, False)
        run_both(big, rng, 64, 2, 700, True)
        run_both(single, rng, 1, 2, 1_000, True)
    finally:
        big.close()
        small.close()
        single.close()


def test_ranks_on_their_own_streams():
    import torch
    n = 4
    w = World(n)
    try:
        rng = np.random.default_rng(13)
        streams = [torch.cuda.Stream() for _ in range(n)]
        run_both(w, rng, n, 2, 20_000, False, streams)
        run_both(w, rng, n, 2, 100, True, streams)
    finally:
        w.close()


def test_two_worlds_on_unordered_streams_take_turns_at_the_array():
    """Two worlds, each on a stream of its own and nothing between the streams: the second world's call is made while
    the first world's copy kernel may still be reading its tables from the GPU's one array.  The library orders the
    array's users itself (the table writes of a call wait for the copy kernel of the call before it), so both get
    the oracle's bytes, several times over and in both orders."""
    rng = np.random.default_rng(17)
    first, second = World(8), World(5)          # a stream each (World creates its own)
    try:
        cases = []
        for w, max_count in ((first, 1_500_000), (second, 4_000)):
            n = w.n
            sc, sd, rc, rd, in_sz, out_sz = a2a_case(rng, n, 2, max_count, False)
            ins = [rand_bytes(rng, in_sz * 2) for _ in range(n)]
            want = [np.full(out_sz * 2, FILL, dtype=np.uint8) for _ in range(n)]
            assert oracle.all_to_all_v(ins, want, sc, sd, rc, rd, int(DT.BFP16)) == 0
            cases.append((w, sc, sd, rc, rd, [to_dev(x) for x in ins], want, out_sz))
        for order in ((0, 1), (1, 0), (0, 1)):
            outs = {}
            for k in (0, 1):
                w, _, _, _, _, _, _, out_sz = cases[k]
                outs[k] = [dev_zeros(out_sz * 2, fill=FILL) for _ in range(w.n)]
            first.inputs_ready()
            for k in order:                     # back to back, no synchronisation in between
                w, sc, sd, rc, rd, sends, _, _ = cases[k]
                with hccl_amd.group():
                    for r in range(w.n):
                        hccl_amd.all_to_all_v_no_alloc(w.comms[r], sends[r], sc[r], sd[r], DT.BFP16, outs[k][r], rc[r],
                                                       rd[r], DT.BFP16, w.stream)
            first.sync()
            second.sync()
            for k in (0, 1):
                w, want = cases[k][0], cases[k][6]
                for r in range(w.n):
                    assert np.array_equal(to_host(outs[k][r], np.uint8), want[r]), (order, k, r)
    finally:
        first.close()
        second.close()


def test_mixing_the_two_entry_points_in_one_collective_is_rejected():
    n = 2
    w = World(n)
    try:
        rng = np.random.default_rng(17)
        sc, sd, rc, rd, in_sz, out_sz = a2a_case(rng, n, 2, 64, True)
        sends = [to_dev(rand_bytes(rng, in_sz * 2)) for _ in range(n)]
        recvs = [dev_zeros(out_sz * 2) for _ in range(n)]
        w.inputs_ready()
        codes = []
        hccl_amd.group_start()
        for r, fn in enumerate((hccl_amd.all_to_all_v, hccl_amd.all_to_all_v_no_alloc)):
            try:
                fn(w.comms[r], sends[r], sc[r], sd[r], DT.BFP16, recvs[r], rc[r], rd[r], DT.BFP16, w.stream)
                codes.append(0)
            except hccl_amd.HcclError as e:
                codes.append(e.code)
        with pytest.raises(hccl_amd.HcclError) as ended:
            hccl_amd.group_end()
        assert ended.value.code == hccl_amd.HcclResult.E_PARA
        assert codes[-1] == hccl_amd.HcclResult.E_PARA
        for r in range(n):
            assert np.all(to_host(recvs[r], np.uint8) == FILL)
    finally:
        w.close()


def test_it_can_be_captured_into_a_graph_and_replayed():
    """After one eager call (set-up) the entry point is kernel launches only, the tables travelling in their
    arguments: a captured graph reproduces the eager result on every replay, with eager work between the replays,
    and reads the buffers as they are at replay time."""
    import torch
    n = 8
    w = World(n)
    try:
        rng = np.random.default_rng(23)
        sc, sd, rc, rd, in_sz, out_sz = a2a_case(rng, n, 2, 9_000, False)
        ins = [rand_bytes(rng, in_sz * 2) for _ in range(n)]
        want = [np.full(out_sz * 2, FILL, dtype=np.uint8) for _ in range(n)]
        assert oracle.all_to_all_v(ins, want, sc, sd, rc, rd, int(DT.BFP16)) == 0
        sends = [to_dev(x) for x in ins]
        recvs = [dev_zeros(out_sz * 2, fill=FILL) for _ in range(n)]

        def step():
            with hccl_amd.group():
                for r in range(n):
                    hccl_amd.all_to_all_v_no_alloc(w.comms[r], sends[r], sc[r], sd[r], DT.BFP16, recvs[r], rc[r], rd[r],
                                                   DT.BFP16, w.stream)

        w.inputs_ready()
        step()
        w.sync()
        for r in range(n):
            assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), ("eager", r)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=w.stream):
            step()
        for replay in range(3):
            for t in recvs:
                t.fill_(FILL)                                   # eager work between the replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for r in range(n):
                assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), (replay, r)
        # new payload through the same graph
        ins2 = [rand_bytes(rng, in_sz * 2) for _ in range(n)]
        want2 = [np.full(out_sz * 2, FILL, dtype=np.uint8) for _ in range(n)]
        assert oracle.all_to_all_v(ins2, want2, sc, sd, rc, rd, int(DT.BFP16)) == 0
        for r in range(n):
            sends[r].copy_(torch.from_numpy(ins2[r]))
            recvs[r].fill_(FILL)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for r in range(n):
            assert np.array_equal(to_host(recvs[r], np.uint8), want2[r]), ("new payload", r)
    finally:
        w.close()
