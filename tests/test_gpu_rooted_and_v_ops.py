"""GPU parity of the entry points that marshal onto the hot path's kernels -- AlltoAll, AlltoAllVC,
ReduceScatterV, Reduce, Broadcast, Scatter -- against the CPU oracle, through the C ABI.  Same bar as
the other parity tests: bit-exact, except that arithmetic NaNs only have to be NaN on both sides."""
import threading

import numpy as np
import pytest

import hccl_amd
import oracle
from hccl_amd import HcclDataType as DT, HcclReduceOp as OP

from gpu_util import World, dev_zeros, require_library_on_gpu, to_dev, to_host
from test_gpu_parity import NP, check, gen

pytestmark = pytest.mark.gpu
SUM, PROD, MAX, MIN = range(4)
RSV_TYPES = [DT.INT8, DT.INT16, DT.INT32, DT.INT64, DT.FP16, DT.BFP16, DT.FP32]


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


@pytest.fixture(scope="module")
def worlds():
    made = {}

    def get(n):
        if n not in made:
            made[n] = World(n)
        return made[n]
    yield get
    for w in made.values():
        w.close()


# ---- AlltoAll / AlltoAllVC ---------------------------------------------------------------------------
@pytest.mark.parametrize("n,count,dtype", [(2, 1, DT.INT8), (3, 1000, DT.FP16), (8, 4099, DT.INT64),
                                           (16, 257, DT.UINT8), (8, 1 << 16, DT.BFP16)])
def test_all_to_all(worlds, n, count, dtype):
    w = worlds(n)
    rng = np.random.default_rng(n * 7 + count)
    esz = oracle.lib().orc_dtype_size(int(dtype))
    ins = [rng.integers(0, 256, n * count * esz, dtype=np.uint8) for _ in range(n)]
    want = [np.zeros(n * count * esz, dtype=np.uint8) for _ in range(n)]
    assert oracle.all_to_all(ins, want, count, int(dtype)) == 0
    sends = [to_dev(x) for x in ins]
    recvs = [dev_zeros(x.nbytes) for x in ins]
    w.all_to_all(sends, recvs, count, dtype)
    for r in range(n):
        assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), r


def vc_case(w, matrix, dtype, seed, pad=0):
    n = w.n
    m = np.asarray(matrix, dtype=np.uint64).reshape(n, n)
    rng = np.random.default_rng(seed)
    esz = oracle.lib().orc_dtype_size(int(dtype))
    ins = [rng.integers(0, 256, max(int(m[j].sum()), 1) * esz, dtype=np.uint8) for j in range(n)]
    want = [np.full(max(int(m[:, i].sum()), 1) * esz, 0xAB, dtype=np.uint8) for i in range(n)]
    assert oracle.all_to_all_vc(ins, want, m, int(dtype)) == 0
    sends = [to_dev(x, pad) for x in ins]
    recvs = [dev_zeros(x.nbytes, pad) for x in want]
    w.all_to_all_vc(sends, recvs, m, dtype)
    for r in range(n):
        assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), r


def test_all_to_all_vc_reference_matrices(worlds):
    vc_case(worlds(2), [10, 11, 1, 2222], DT.UINT32, 1)                 # alltoallvc_testcase.cc:184
    vc_case(worlds(6), [1] * 36, DT.INT8, 2)                             # :215
    vc_case(worlds(6), [0] * 36, DT.FP32, 3)                             # all-zero matrix: nothing moves


@pytest.mark.parametrize("n,dtype,pad", [(3, DT.FP16, 0), (8, DT.INT8, 3), (16, DT.FP32, 4), (64, DT.BFP16, 2)])
def test_all_to_all_vc_random_matrix_with_silent_ranks(worlds, n, dtype, pad):
    rng = np.random.default_rng(n)
    m = rng.integers(0, 3000, (n, n)).astype(np.uint64)
    m[rng.random((n, n)) < 0.2] = 0
    m[rng.integers(0, n), :] = 0
    m[:, rng.integers(0, n)] = 0
    vc_case(worlds(n), m, dtype, n + 100, pad)


# ---- ReduceScatterV ------------------------------------------------------------------------------------
def rsv_layout(rng, n, lo, hi, layout, esz):
    counts = rng.integers(lo, hi, n).astype(np.uint64)
    counts[rng.integers(0, n)] = 0
    displs = np.zeros(n, dtype=np.uint64)
    off = 0
    order = range(n) if layout == "prefix" else rng.permutation(n)
    for k in order:
        if layout == "gaps":
            off += int(rng.integers(0, 5))
        elif layout == "aligned":
            off = -(-off * esz // 16) * 16 // esz      # every slice starts on a 16-byte boundary
        displs[k] = off
        off += int(counts[k])
    return counts, displs, off + 5


def run_rsv(w, dtype, op, lo, hi, layout, seed, pad=0, algo="mesh"):
    n = w.n
    rng = np.random.default_rng(seed)
    esz = np.dtype(NP[dtype]).itemsize
    counts, displs, total = rsv_layout(rng, n, lo, hi, layout, esz)
    ins = [gen(dtype, op, rng, total) for _ in range(n)]
    want = [np.zeros(max(int(c), 1), dtype=NP[dtype]) for c in counts]
    assert oracle.reduce_scatter_v(ins, want, counts, displs, int(dtype), op, acc=oracle.ACC_FP32, algo=algo) == 0
    sends = [to_dev(x, pad) for x in ins]
    recvs = [dev_zeros(x.nbytes, pad) for x in want]
    w.reduce_scatter_v(sends, recvs, counts, displs, dtype, op, algo)
    for r in range(n):
        c = int(counts[r])
        got = to_host(recvs[r], NP[dtype])
        check(dtype, op, got[:c], want[r][:c], "reduce_scatter_v %s %s n=%d %s rank=%d" % (dtype.name, OP(op).name, n,
                                                                                         layout, r))
        if c == 0:
            assert np.all(got.view(np.uint8) == 0xAB)       # a rank that receives nothing is left alone


@pytest.mark.parametrize("dtype", RSV_TYPES)
@pytest.mark.parametrize("layout", ["prefix", "gaps", "aligned"])
def test_reduce_scatter_v_sum(worlds, dtype, layout):
    run_rsv(worlds(8), dtype, SUM, 1, 5000, layout, 17 + int(dtype))


@pytest.mark.parametrize("op", [PROD, MAX, MIN])
@pytest.mark.parametrize("dtype", [DT.INT32, DT.FP16, DT.FP32, DT.BFP16])
def test_reduce_scatter_v_other_ops(worlds, dtype, op):
    if op == PROD and dtype == DT.BFP16:
        pytest.skip("the reference rejects bf16 PROD")
    run_rsv(worlds(5), dtype, op, 1, 3000, "gaps", 31 + int(dtype) + op)


def test_reduce_scatter_v_large_uneven_slices(worlds):
    run_rsv(worlds(6), DT.BFP16, SUM, 1 << 18, 1 << 21, "aligned", 5)
    run_rsv(worlds(6), DT.FP32, SUM, 1 << 16, 1 << 19, "prefix", 6, pad=4)


@pytest.mark.parametrize("n", [2, 3, 8, 16])
def test_reduce_scatter_v_mesh_chunk_order(worlds, n):
    """Slices long enough for 4 KiB-aligned segments, slices dealt element-wise, and slices shorter than n - 1."""
    w = worlds(n)
    run_rsv(w, DT.FP32, SUM, 1, 40_000, "gaps", 900 + n, algo="mesh_chunk")
    run_rsv(w, DT.FP32, SUM, 1, 12, "prefix", 910 + n, algo="mesh_chunk")
    run_rsv(w, DT.BFP16, SUM, 1 << 14, 1 << 17, "aligned", 920 + n, algo="mesh_chunk")
    run_rsv(w, DT.FP32, MAX, 1, 9_000, "gaps", 930 + n, pad=4, algo="mesh_chunk")
    run_rsv(w, DT.FP32, SUM, 1, 5_000, "gaps", 940 + n)          # back to the plain mesh order


def test_reduce_scatter_v_mesh_chunk_refuses_more_than_the_staging_buffer_holds(worlds):
    w = worlds(3)
    hccl_amd.set_ccl_buffer_size(w.comms[0], 4096)
    try:
        run_rsv(w, DT.FP32, SUM, 900, 1024, "prefix", 950, algo="mesh_chunk")       # at most 4096 bytes per slice
        with pytest.raises(hccl_amd.HcclError) as e:
            run_rsv(w, DT.FP32, SUM, 1025, 1100, "prefix", 951, algo="mesh_chunk")
        assert e.value.code == 5
    finally:
        hccl_amd.set_ccl_buffer_size(w.comms[0], 0)
        w.set_algo(hccl_amd.OpKind.REDUCE_SCATTER, "mesh")


def test_reduce_scatter_v_counts_that_differ_between_ranks_are_rejected(worlds):
    w = worlds(3)
    bufs = [dev_zeros(64) for _ in range(6)]
    w.inputs_ready()
    codes = []
    hccl_amd.group_start()
    for r in range(3):
        counts = [4, 4, 4] if r != 2 else [4, 4, 5]
        try:
            codes.append(hccl_amd.reduce_scatter_v(w.comms[r], bufs[r], counts, [0, 4, 8], bufs[3 + r], counts[r],
                                                   DT.FP32, OP.SUM, w.stream))
        except hccl_amd.HcclError as e:
            codes.append(e.code)
    with pytest.raises(hccl_amd.HcclError) as ended:
        hccl_amd.group_end()
    assert ended.value.code == 1                            # the group's end reports it for the queued calls
    assert codes[-1] == 1                                   # HCCL_E_PARA, reported by the call that completes the set


# ---- Reduce ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n,root", [(2, 0), (5, 3), (8, 7), (16, 9)])
def test_reduce_two_shot_order(worlds, n, root):
    w = worlds(n)
    try:
        for dtype, op, count, ccl in ((DT.FP32, SUM, 100_003, 0), (DT.FP32, SUM, 5, 0), (DT.BFP16, SUM, 65_536, 0),
                                      (DT.FP16, MAX, 33_333, 0), (DT.FP64, SUM, 10_001, 0), (DT.INT32, PROD, 999, 0),
                                      (DT.FP32, SUM, 200_001, 1 << 18)):
            rng = np.random.default_rng(n * 37 + root + count)
            ins = [gen(dtype, op, rng, count) for _ in range(n)]
            want = [np.zeros(count, dtype=NP[dtype]) for _ in range(n)]
            hccl_amd.set_ccl_buffer_size(w.comms[0], ccl)
            per_loop = oracle.sole_max_count_per_loop(ccl, n, np.dtype(NP[dtype]).itemsize) if ccl else 0
            assert oracle.reduce(ins, want, count, int(dtype), op, root, acc=oracle.ACC_FP32, algo="mesh_two_shot",
                                 max_count_per_loop=per_loop) == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(x.nbytes) for x in ins]
            w.reduce(sends, recvs, count, dtype, op, root, "mesh_two_shot")
            check(dtype, op, to_host(recvs[root], NP[dtype]), want[root], "reduce two-shot %s n=%d" % (dtype.name, n))
            for r in range(n):
                if r != root:
                    assert np.all(to_host(recvs[r], np.uint8) == 0xAB)
    finally:
        hccl_amd.set_ccl_buffer_size(w.comms[0], 0)
        w.set_algo(hccl_amd.OpKind.REDUCE, "mesh")



@pytest.mark.parametrize("n,root", [(2, 1), (5, 3), (8, 0), (16, 9)])
@pytest.mark.parametrize("dtype,op", [(DT.FP32, SUM), (DT.BFP16, SUM), (DT.INT32, PROD), (DT.FP16, MAX),
                                      (DT.INT64, MIN), (DT.FP64, SUM)])
def test_reduce(worlds, n, root, dtype, op):
    w = worlds(n)
    rng = np.random.default_rng(n * 31 + root + int(dtype))
    count = 10_007
    ins = [gen(dtype, op, rng, count) for _ in range(n)]
    want = [np.zeros(count, dtype=NP[dtype]) for _ in range(n)]
    assert oracle.reduce(ins, want, count, int(dtype), op, root, acc=oracle.ACC_FP32) == 0
    sends = [to_dev(x) for x in ins]
    recvs = [dev_zeros(x.nbytes) for x in ins]
    w.reduce(sends, recvs, count, dtype, op, root)
    check(dtype, op, to_host(recvs[root], NP[dtype]), want[root], "reduce n=%d root=%d" % (n, root))
    for r in range(n):
        if r != root:
            assert np.all(to_host(recvs[r], np.uint8) == 0xAB), r   # only the root's recvBuf is written


# ---- Broadcast / Scatter -------------------------------------------------------------------------------
@pytest.mark.parametrize("n,root,count,dtype,pad", [(2, 0, 1, DT.INT8, 0), (3, 2, 1001, DT.FP16, 2),
                                                    (8, 5, 1 << 20, DT.FP32, 0), (16, 15, 77_777, DT.UINT8, 5),
                                                    (64, 31, 4096, DT.INT64, 0)])
def test_broadcast(worlds, n, root, count, dtype, pad):
    w = worlds(n)
    rng = np.random.default_rng(n + root)
    esz = oracle.lib().orc_dtype_size(int(dtype))
    host = [rng.integers(0, 256, count * esz, dtype=np.uint8) for _ in range(n)]
    bufs = [to_dev(x, pad) for x in host]
    w.broadcast(bufs, count, dtype, root)
    for r in range(n):
        assert np.array_equal(to_host(bufs[r], np.uint8), host[root]), r


@pytest.mark.parametrize("n,root,count,dtype,pad", [(2, 1, 1, DT.INT8, 0), (4, 0, 999, DT.FP16, 2),
                                                    (8, 7, 1 << 18, DT.FP32, 0), (64, 40, 1025, DT.UINT8, 1)])
def test_scatter(worlds, n, root, count, dtype, pad):
    w = worlds(n)
    rng = np.random.default_rng(n * 3 + root)
    esz = oracle.lib().orc_dtype_size(int(dtype))
    ins = [rng.integers(0, 256, n * count * esz, dtype=np.uint8) for _ in range(n)]
    want = [np.zeros(count * esz, dtype=np.uint8) for _ in range(n)]
    assert oracle.scatter(ins, want, count, int(dtype), root) == 0
    # only the root needs a send buffer
    sends = [to_dev(ins[r], pad) if r == root else None for r in range(n)]
    recvs = [dev_zeros(count * esz, pad) for _ in range(n)]
    w.scatter(sends, recvs, count, dtype, root)
    for r in range(n):
        assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), r


# ---- one host thread per rank, no group ----------------------------------------------------------------
def test_rooted_ops_with_one_blocking_thread_per_rank():
    import torch
    n, count, root = 4, 5000, 2
    w = World(n)
    try:
        rng = np.random.default_rng(9)
        ins = [rng.standard_normal(count).astype(np.float32) for _ in range(n)]
        want = [np.zeros(count, dtype=np.float32) for _ in range(n)]
        assert oracle.reduce(ins, want, count, int(DT.FP32), SUM, root) == 0
        sends = [to_dev(x) for x in ins]
        recvs = [dev_zeros(x.nbytes) for x in ins]
        streams = [torch.cuda.Stream() for _ in range(n)]
        torch.cuda.synchronize()
        errors = []

        def rank_main(r):
            try:
                hccl_amd.reduce(w.comms[r], sends[r], recvs[r], count, DT.FP32, OP.SUM, root, streams[r])
                hccl_amd.broadcast(w.comms[r], recvs[r], count, DT.FP32, root, streams[r])
                streams[r].synchronize()
            except Exception as e:   # noqa: BLE001 - reported below
                errors.append((r, e))

        threads = [threading.Thread(target=rank_main, args=(r,)) for r in range(n)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(120)
        assert not errors, errors
        for r in range(n):      # reduce to the root, then broadcast from it == all-reduce in rank order
            assert np.array_equal(to_host(recvs[r], np.float32).view(np.uint32), want[root].view(np.uint32)), r
    finally:
        w.close()
