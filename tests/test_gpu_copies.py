"""GPU parity of the slice-copy (AllGather / AllGatherV) and pack / unpack (AlltoAllV) kernels
against the CPU oracle: bit-exact, including bytes the collective must not touch."""
import threading

import numpy as np
import pytest

import hccl_amd
import oracle
from hccl_amd import HcclDataType as DT, HcclReduceOp as OP

from gpu_util import World, a2a_case, dev_zeros, rand_bytes, require_library_on_gpu, to_dev, to_host

pytestmark = pytest.mark.gpu
FILL = 0xAB


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


FORMS = ["by_size", "two_kernels"]


def world_with_form(monkeypatch, n, form):
    """A world whose one-to-many copies take the launcher's choice, or the two-kernel form (segments into the
    first destination, then a fan-out of that range) with windows of 4 KiB whatever the size."""
    if form == "two_kernels":
        monkeypatch.setenv("HCCL_AMD_COPY_TWO_KERNELS", "1")
        monkeypatch.setenv("HCCL_AMD_ALLREDUCE_PIECE_BYTES", "4096")
    w = World(n)
    monkeypatch.delenv("HCCL_AMD_COPY_TWO_KERNELS", raising=False)
    monkeypatch.delenv("HCCL_AMD_ALLREDUCE_PIECE_BYTES", raising=False)
    return w


@pytest.mark.parametrize("n", [1, 2, 3, 8, 64])
@pytest.mark.parametrize("dtype,esz", [(DT.UINT8, 1), (DT.BFP16, 2), (DT.FP32, 4), (DT.INT64, 8)])
def test_all_gather(n, dtype, esz):
    w = World(n)
    try:
        rng = np.random.default_rng(n * 10 + esz)
        for count in (1, 7, 4096, 70_001):
            ins = [rand_bytes(rng, count * esz) for _ in range(n)]
            want = [np.zeros(n * count * esz, dtype=np.uint8) for _ in range(n)]
            assert oracle.all_gather(ins, want, count, int(dtype)) == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(n * count * esz) for _ in range(n)]
            w.all_gather(sends, recvs, count, dtype)
            for r in range(n):
                assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), (n, count, r)
    finally:
        w.close()


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("n", [2, 6, 8, 64])
def test_all_gather_v_unordered_holes_and_odd_offsets(monkeypatch, n, form):
    w = world_with_form(monkeypatch, n, form)
    try:
        rng = np.random.default_rng(n)
        esz = 2
        for trial in range(3):
            counts = rng.integers(0, 5000, n).astype(np.uint64)
            counts[rng.integers(0, n)] = 0                      # an empty contribution
            if trial == 2:
                counts = (counts // 8) * 8                      # all 16-byte multiples: vector path
            order = rng.permutation(n)
            displs = np.zeros(n, dtype=np.uint64)
            off = int(rng.integers(0, 4))
            for j in order:                                     # shuffled layout with gaps
                displs[j] = off
                off += int(counts[j]) + (0 if trial == 2 else int(rng.integers(0, 5)))
            total = off + 3
            ins = [rand_bytes(rng, max(int(c), 1) * esz) for c in counts]
            want = [np.full(total * esz, FILL, dtype=np.uint8) for _ in range(n)]
            assert oracle.all_gather_v(ins, want, counts, displs, int(DT.FP16)) == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(total * esz, fill=FILL) for _ in range(n)]
            w.all_gather_v(sends, recvs, counts, displs, DT.FP16)
            for r in range(n):
                assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), (n, trial, r)
    finally:
        w.close()


@pytest.mark.parametrize("n", [2, 3, 8, 64])
@pytest.mark.parametrize("aligned", [True, False])
def test_all_to_all_v(n, aligned):
    w = World(n)
    try:
        rng = np.random.default_rng(n + 100 * aligned)
        esz = 2
        for max_count in (9, 3000, 40_000 if n <= 8 else 6_000):
            sc, sd, rc, rd, in_sz, out_sz = a2a_case(rng, n, esz, max_count, aligned)
            ins = [rand_bytes(rng, in_sz * esz) for _ in range(n)]
            want = [np.full(out_sz * esz, FILL, dtype=np.uint8) for _ in range(n)]
            assert oracle.all_to_all_v(ins, want, sc, sd, rc, rd, int(DT.BFP16)) == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(out_sz * esz, fill=FILL) for _ in range(n)]
            w.all_to_all_v(sends, sc, sd, recvs, rc, rd, DT.BFP16)
            for r in range(n):
                assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), (n, aligned, max_count, r)
    finally:
        w.close()


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("n", [4, 7, 17, 64])
def test_all_gather_v_ragged_segments_many_destinations(monkeypatch, n, form):
    """AllGatherV over destination counts from 4 to 64: segments that end inside a tile, odd element
    displacements, differently aligned buffers (the two-kernel form then falls back to one kernel), empty
    segments."""
    w = world_with_form(monkeypatch, n, form)
    try:
        rng = np.random.default_rng(5000 + 10 * n)
        esz = 2
        for trial in range(3):
            counts = rng.integers(0, 9_000 if n <= 17 else 1_500, n).astype(np.uint64)
            counts[rng.integers(0, n)] = 0
            if trial == 2:
                counts = (counts // 8) * 8                      # everything 16-byte aligned
            displs = np.zeros(n, dtype=np.uint64)
            off = 0
            for j in rng.permutation(n):
                displs[j] = off
                off += int(counts[j]) + (0 if trial == 2 else int(rng.integers(0, 3)))
            total = off + 5
            ins = [rand_bytes(rng, max(int(c), 1) * esz) for c in counts]
            want = [np.full(total * esz, FILL, dtype=np.uint8) for _ in range(n)]
            assert oracle.all_gather_v(ins, want, counts, displs, int(DT.FP16)) == 0
            sends = [to_dev(x, pad_front=0 if trial == 2 else int(rng.integers(0, 8)) * 2) for x in ins]
            recvs = [dev_zeros(total * esz, pad_front=0 if trial != 1 else 2 * (r % 5), fill=FILL) for r in range(n)]
            w.all_gather_v(sends, recvs, counts, displs, DT.FP16)
            for r in range(n):
                assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), (n, trial, r)
    finally:
        w.close()


@pytest.mark.parametrize("n", [5, 9])
def test_broadcast_and_all_gather_of_half_a_gigabyte(n):
    """Large one-to-many copies, checked by equality with the source on the device (512 MiB broadcast to n - 1
    ranks, AllGather of n x 80 MiB): one kernel for five ranks, gather + fan-out over several 256 MiB windows for
    nine."""
    import torch
    nbytes = 512 << 20
    w = World(n)
    try:
        g = torch.Generator(device="cuda")
        g.manual_seed(77)
        bufs = [torch.randint(0, 256, (nbytes,), generator=g, device="cuda", dtype=torch.uint8) for _ in range(n)]
        want = bufs[3].clone()
        w.broadcast(bufs, nbytes, DT.UINT8, 3)
        for r in range(n):
            assert torch.equal(bufs[r], want), r
        del bufs, want
        per = 80 << 20
        sends = [torch.randint(0, 256, (per,), generator=g, device="cuda", dtype=torch.uint8) for _ in range(n)]
        recvs = [torch.zeros(n * per, device="cuda", dtype=torch.uint8) for _ in range(n)]
        w.all_gather(sends, recvs, per, DT.UINT8)
        whole = torch.cat(sends)
        for r in range(n):
            assert torch.equal(recvs[r], whole), r
    finally:
        w.close()


def test_all_to_all_v_moe_shape_zipf_small():
    """The MoE-dispatch shape of the headline AlltoAllV configuration at 1/64 of its token count:
    64 ranks, hidden 7168 bf16, per-destination token counts multinomial over Zipf(1.1) weights."""
    n, hidden, tokens = 64, 7168, 256
    w = World(n)
    try:
        rng = np.random.default_rng(0xC0FFEE + 4000)
        wts = 1.0 / np.arange(1, n + 1) ** 1.1
        wts /= wts.sum()
        tok = np.stack([rng.multinomial(tokens, wts) for _ in range(n)]).astype(np.uint64)
        sc = tok * hidden
        rc = sc.T.copy()
        sd = np.cumsum(sc, axis=1) - sc
        rd = np.cumsum(rc, axis=1) - rc
        ins = [rng.integers(0, 65536, tokens * hidden, dtype=np.uint16) for _ in range(n)]
        outs = [np.zeros(int(rc[i].sum()), dtype=np.uint16) for i in range(n)]
        assert oracle.all_to_all_v(ins, outs, sc, sd, rc, rd, int(DT.BFP16)) == 0
        sends = [to_dev(x) for x in ins]
        recvs = [dev_zeros(max(o.nbytes, 2)) for o in outs]
        w.all_to_all_v(sends, sc, sd, recvs, rc, rd, DT.BFP16)
        for i in range(n):
            assert np.array_equal(to_host(recvs[i], np.uint16)[:outs[i].size], outs[i]), i
    finally:
        w.close()


def test_rendezvous_mismatch_and_launch_time_checks():
    w = World(2)
    try:
        a = [to_dev(np.arange(16, dtype=np.float32)) for _ in range(2)]
        b = [dev_zeros(64) for _ in range(2)]
        hccl_amd.group_start()
        hccl_amd.all_reduce(w.comms[0], a[0], b[0], 16, DT.FP32, OP.SUM, w.stream)
        with pytest.raises(hccl_amd.HcclError) as e:
            hccl_amd.all_reduce(w.comms[1], a[1], b[1], 8, DT.FP32, OP.SUM, w.stream)   # different count
        assert e.value.code == 1
        with pytest.raises(hccl_amd.HcclError) as e:
            hccl_amd.group_end()                      # reports the verdict for the call that was queued
        assert e.value.code == 1
        # recvCounts of rank 0 disagree with sendCounts of rank 1
        sc = np.array([[1, 2], [3, 4]], dtype=np.uint64)
        rc = np.array([[1, 5], [2, 4]], dtype=np.uint64)
        z = np.zeros((2, 2), dtype=np.uint64)
        hccl_amd.group_start()
        hccl_amd.all_to_all_v(w.comms[0], a[0], sc[0], z[0], DT.FP32, b[0], rc[0], z[0], DT.FP32, w.stream)
        with pytest.raises(hccl_amd.HcclError) as e:
            hccl_amd.all_to_all_v(w.comms[1], a[1], sc[1], z[1], DT.FP32, b[1], rc[1], z[1], DT.FP32, w.stream)
        assert e.value.code == 1
        with pytest.raises(hccl_amd.HcclError) as e:
            hccl_amd.group_end()
        assert e.value.code == 1
        # the world is still usable afterwards
        with hccl_amd.group():
            for r in range(2):
                hccl_amd.all_reduce(w.comms[r], a[r], b[r], 16, DT.FP32, OP.SUM, w.stream)
        w.sync()
        assert np.array_equal(to_host(b[1], np.float32), 2 * np.arange(16, dtype=np.float32))
    finally:
        w.close()


def test_one_host_thread_per_rank_with_own_streams():
    """The calling pattern of the reference's examples: a thread per rank, each with its own stream,
    calls block until every rank has arrived (examples/02_collectives/01_allreduce/main.cc:76-85)."""
    import torch
    n, count = 4, 300_000
    info = hccl_amd.get_root_info()
    rng = np.random.default_rng(9)
    ins = [rng.standard_normal(count).astype(np.float32) for _ in range(n)]
    want = ins[0].copy()
    for r in range(1, n):
        want = ins[r] + want
    results, errors = [None] * n, []

    def rank_main(r):
        try:
            comm = hccl_amd.comm_init_root_info(n, info, r)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                send = to_dev(ins[r])
                recv = dev_zeros(4 * count)
            stream.synchronize()
            for _ in range(3):
                hccl_amd.all_reduce(comm, send, recv, count, DT.FP32, OP.SUM, stream)
            stream.synchronize()
            results[r] = to_host(recv, np.float32)
            hccl_amd.comm_destroy(comm)
        except Exception as exc:   # surfaced below
            errors.append((r, exc))

    threads = [threading.Thread(target=rank_main, args=(r,)) for r in range(n)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not errors, errors
    for r in range(n):
        assert np.array_equal(results[r].view(np.uint32), want.view(np.uint32)), r


@pytest.mark.parametrize("form", FORMS)
def test_all_gather_and_broadcast_into_differently_aligned_buffers(monkeypatch, form):
    """Every rank's buffers sit at their own offset from a 16-byte boundary: the stores to all but the first
    destination are unaligned 128-bit stores."""
    import hccl_amd
    n, count = 6, 33_333
    w = world_with_form(monkeypatch, n, form)
    try:
        rng = np.random.default_rng(404)
        ins = [rand_bytes(rng, count * 2) for _ in range(n)]
        want = [np.zeros(n * count * 2, dtype=np.uint8) for _ in range(n)]
        assert oracle.all_gather(ins, want, count, int(DT.FP16)) == 0
        sends = [to_dev(x, (2 * r) % 16) for r, x in enumerate(ins)]
        recvs = [dev_zeros(n * count * 2, (6 * r + 2) % 16) for r in range(n)]
        w.all_gather(sends, recvs, count, DT.FP16)
        for r in range(n):
            assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), r
        counts = np.array([100, 0, 7_777, 1, 40_001, 16], dtype=np.uint64)
        displs = np.array([3, 0, 200, 150, 9_000, 120], dtype=np.uint64)
        total = 50_000
        vins = [rand_bytes(rng, max(int(c), 1)) for c in counts]
        vwant = [np.full(total, FILL, dtype=np.uint8) for _ in range(n)]
        assert oracle.all_gather_v([x[:int(c)] for x, c in zip(vins, counts)], vwant, counts, displs, int(DT.UINT8)) == 0
        sends = [to_dev(x, (3 * r) % 16) for r, x in enumerate(vins)]
        recvs = [dev_zeros(total, (5 * r + 1) % 16, fill=FILL) for r in range(n)]
        w.all_gather_v(sends, recvs, counts, displs, DT.UINT8)
        for r in range(n):
            assert np.array_equal(to_host(recvs[r], np.uint8), vwant[r]), r
        bufs = [to_dev(rand_bytes(rng, 70_001), (7 * r) % 16) for r in range(n)]
        src = to_host(bufs[4], np.uint8)
        w.broadcast(bufs, 70_001, DT.UINT8, 4)
        for r in range(n):
            assert np.array_equal(to_host(bufs[r], np.uint8), src), r
    finally:
        w.close()


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("n,count", [(4, 10_001), (8, 65_536)])
def test_all_gather_with_the_send_buffer_inside_the_receive_buffer(monkeypatch, n, count, form):
    """Every rank sends the slice of its own recvBuf where its contribution belongs (the entry point puts no
    restriction on overlapping buffers, reference all_gather.cc:118-149): the own slot is copied onto itself."""
    import torch
    w = world_with_form(monkeypatch, n, form)
    try:
        rng = np.random.default_rng(n + count)
        parts = [rng.standard_normal(count).astype(np.float32) for _ in range(n)]
        recvs = [torch.zeros(n * count, dtype=torch.float32, device="cuda") for _ in range(n)]
        for r in range(n):
            recvs[r][r * count:(r + 1) * count] = torch.from_numpy(parts[r]).cuda()
        sends = [recvs[r][r * count:(r + 1) * count] for r in range(n)]
        w.all_gather(sends, recvs, count, DT.FP32)
        want = np.concatenate(parts)
        for r in range(n):
            assert np.array_equal(recvs[r].cpu().numpy().view(np.uint32), want.view(np.uint32)), r
    finally:
        w.close()


@pytest.mark.parametrize("n", [3, 8, 20])
def test_one_to_many_copies_as_gather_and_fan_out(monkeypatch, n):
    """The two-kernel form with buffers that share an offset of 4 bytes from a 16-byte boundary (the fan-out
    moves the bytes in front of and behind its aligned body one by one): AllGather over many windows, Broadcast
    from every kind of root, AllGatherV with adjacent and separate destination ranges."""
    w = world_with_form(monkeypatch, n, "two_kernels")
    try:
        rng = np.random.default_rng(900 + n)
        count = 3_001
        ins = [rand_bytes(rng, count * 4) for _ in range(n)]
        want = [np.zeros(n * count * 4, dtype=np.uint8) for _ in range(n)]
        assert oracle.all_gather(ins, want, count, int(DT.FP32)) == 0
        sends = [to_dev(x, 4) for x in ins]
        recvs = [dev_zeros(n * count * 4, 4) for _ in range(n)]
        w.all_gather(sends, recvs, count, DT.FP32)
        for r in range(n):
            assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), ("all_gather", r)
        for root, nbytes in ((0, 70_001), (n - 1, 5), (n // 2, 4_096), (1, 12_288)):
            bufs = [to_dev(rand_bytes(rng, nbytes), 4) for _ in range(n)]
            src = to_host(bufs[root], np.uint8)
            w.broadcast(bufs, nbytes, DT.UINT8, root)
            for r in range(n):
                assert np.array_equal(to_host(bufs[r], np.uint8), src), ("broadcast", root, nbytes, r)
        counts = rng.integers(1, 3_000, n).astype(np.uint64)
        displs = np.zeros(n, dtype=np.uint64)
        off = 0
        for j in range(n):                       # adjacent ranges, a gap after every third
            displs[j] = off
            off += int(counts[j]) + (7 if j % 3 == 2 else 0)
        total = off + 9
        vins = [rand_bytes(rng, int(c) * 2) for c in counts]
        vwant = [np.full(total * 2, FILL, dtype=np.uint8) for _ in range(n)]
        assert oracle.all_gather_v(vins, vwant, counts, displs, int(DT.BFP16)) == 0
        sends = [to_dev(x, 2 * (r % 3)) for r, x in enumerate(vins)]
        recvs = [dev_zeros(total * 2, 4, fill=FILL) for _ in range(n)]
        w.all_gather_v(sends, recvs, counts, displs, DT.BFP16)
        for r in range(n):
            assert np.array_equal(to_host(recvs[r], np.uint8), vwant[r]), ("all_gather_v", r)
    finally:
        w.close()


@pytest.mark.parametrize("n", [2, 8, 12])
def test_gather_step_as_the_copy_launched_from_its_arguments(monkeypatch, n):
    """One destination and up to eight equally long segments on 16-byte boundaries whose places in the destination
    start on 128-byte lines go through the copy kernel that finds everything in its arguments: the gather step of a
    two-kernel AllGather (128-byte multiples per rank; more than eight ranks and other lengths keep the general
    kernel) and the root's copy of a two-kernel Broadcast, lengths from one vector to many tiles and a tile and a
    half."""
    w = world_with_form(monkeypatch, n, "two_kernels")
    try:
        rng = np.random.default_rng(1300 + n)
        cases = [(nbytes, 0) for nbytes in (128, 16, 1_024, 1_536, 4_096 + 128, 65_536 + 16, 1_000_000 - 1_000_000 % 128)]
        # destinations on a 16-byte boundary that is no 128-byte line: everything aligned, yet the general kernel's
        cases += [(nbytes, 48) for nbytes in (16, 128, 4_096 + 128)]
        for nbytes, pad in cases:
            ins = [rand_bytes(rng, nbytes) for _ in range(n)]
            want = [np.zeros(n * nbytes, dtype=np.uint8) for _ in range(n)]
            assert oracle.all_gather(ins, want, nbytes, int(DT.UINT8)) == 0
            sends = [to_dev(x, 0) for x in ins]
            recvs = [dev_zeros(n * nbytes, pad) for _ in range(n)]
            w.all_gather(sends, recvs, nbytes, DT.UINT8)
            for r in range(n):
                assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), ("all_gather", nbytes, pad, r)
            bufs = [to_dev(rand_bytes(rng, nbytes), pad) for _ in range(n)]
            root = int(rng.integers(0, n))
            src = to_host(bufs[root], np.uint8)
            w.broadcast(bufs, nbytes, DT.UINT8, root)
            for r in range(n):
                assert np.array_equal(to_host(bufs[r], np.uint8), src), ("broadcast", root, nbytes, r)
    finally:
        w.close()
