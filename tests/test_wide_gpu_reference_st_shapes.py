"""GPU parity on the shapes of the reference's own system tests for the V operators, Broadcast and Scatter.

tests/golden/reference_st_shapes.json holds, as data, every case of test/st/algorithm/testcase/alltoallv_testcase.cc,
alltoallvc_testcase.cc, all_gather_v_testcase.cc, reduce_scatter_v_testcase*.cc, broadcast_testcase.cc and
scatter_testcase.cc whose numbers are written out: rank count, data type(s), the send-count matrix, the counts /
displacements or count and root, and for the cases that only assert a return code, that code.  The
reference runs them in a simulated world and verifies the task graph; here the same shapes go through the C ABI on
real buffers and are compared with the oracle, byte for byte.  Counts in the millions and beyond (the catalogue goes
up to 10 Gi elements) are folded down to a few thousand elements, keeping zero at zero, small counts as they are,
and the order and the holes of the displacements; the full sizes are the bench's business.
"""
import json
import os

import numpy as np
import pytest

import hccl_amd
import oracle
from hccl_amd import HcclDataType as DT, HcclReduceOp as OP

from gpu_util import World, dev_zeros, rand_bytes, require_library_on_gpu, to_dev, to_host
from test_gpu_parity import NP, check, gen

pytestmark = pytest.mark.gpu
FILL = 0xAB
CASES = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_st_shapes.json")))


def of_kind(kind):
    return [pytest.param(c, id=c["name"]) for c in CASES if c["kind"] == kind]


def fold(count):
    """Counts up to 6000 elements stay; larger ones become 3000 .. 5998, different for different counts."""
    return count if count <= 6000 else 3000 + count % 2999


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


def test_the_catalogue_is_whole():
    kinds = {}
    for c in CASES:
        kinds[c["kind"]] = kinds.get(c["kind"], 0) + 1
    assert kinds == {"all_to_all_v": 36, "all_to_all_vc": 36, "all_gather_v": 13, "reduce_scatter_v": 22,
                     "broadcast": 34, "scatter": 24}


def matrix_of(case):
    n = case["ranks"]
    return np.array([fold(v) for v in case["matrix"]], dtype=np.uint64).reshape(n, n)


@pytest.mark.parametrize("case", of_kind("all_to_all_v"))
def test_all_to_all_v_cases(worlds, case):
    """The reference derives each rank's arguments from the matrix: row = send counts, column = receive counts,
    both packed (alltoallv_testcase.cc GenAllToAllVParams)."""
    n = case["ranks"]
    w = worlds(n)
    m = matrix_of(case)
    sc = [m[r] for r in range(n)]
    rc = [m[:, r] for r in range(n)]
    sd = [np.concatenate(([0], np.cumsum(x)[:-1])).astype(np.uint64) for x in sc]
    rd = [np.concatenate(([0], np.cumsum(x)[:-1])).astype(np.uint64) for x in rc]
    for tname in case["types"]:
        dtype = DT[tname]
        esz = oracle.lib().orc_dtype_size(int(dtype))
        rng = np.random.default_rng(len(case["name"]) + int(dtype))
        ins = [rand_bytes(rng, max(int(sc[r].sum()), 1) * esz) for r in range(n)]
        want = [np.full(max(int(rc[r].sum()), 1) * esz, FILL, dtype=np.uint8) for r in range(n)]
        assert oracle.all_to_all_v(ins, want, sc, sd, rc, rd, int(dtype)) == 0
        sends = [to_dev(x) for x in ins]
        recvs = [dev_zeros(x.nbytes, fill=FILL) for x in want]
        w.all_to_all_v(sends, sc, sd, recvs, rc, rd, dtype)
        for r in range(n):
            assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), (case["source"], tname, r)


@pytest.mark.parametrize("case", of_kind("all_to_all_vc"))
def test_all_to_all_vc_cases(worlds, case):
    n = case["ranks"]
    w = worlds(n)
    m = matrix_of(case)
    for tname in case["types"]:
        dtype = DT[tname]
        esz = oracle.lib().orc_dtype_size(int(dtype))
        rng = np.random.default_rng(7 * len(case["name"]) + int(dtype))
        ins = [rand_bytes(rng, max(int(m[r].sum()), 1) * esz) for r in range(n)]
        want = [np.full(max(int(m[:, r].sum()), 1) * esz, FILL, dtype=np.uint8) for r in range(n)]
        assert oracle.all_to_all_vc(ins, want, m, int(dtype)) == 0
        sends = [to_dev(x) for x in ins]
        recvs = [dev_zeros(x.nbytes, fill=FILL) for x in want]
        w.all_to_all_vc(sends, recvs, m, dtype)
        for r in range(n):
            assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), (case["source"], tname, r)


def folded_layout(case):
    """Counts folded; displacements rebuilt in the original order with the original holes (capped at 64 elements)
    and, where the original intervals overlap, the original overlap."""
    counts = [fold(c) for c in case["counts"]]
    order = sorted(range(len(counts)), key=lambda i: (case["displs"][i], i))
    displs = [0] * len(counts)
    end_old, end_new = 0, 0
    for i in order:
        gap = case["displs"][i] - end_old                    # negative where intervals overlap
        displs[i] = max(end_new + min(gap, 64), 0)
        end_old = max(end_old, case["displs"][i] + case["counts"][i])
        end_new = max(end_new, displs[i] + counts[i])
    return np.array(counts, dtype=np.uint64), np.array(displs, dtype=np.uint64), end_new


def test_folding_keeps_small_layouts_as_they_are():
    for c in CASES:
        if "counts" in c and max(c["counts"]) <= 6000 and min(c["displs"]) == 0:
            counts, displs, _ = folded_layout(c)
            assert list(counts) == c["counts"] and list(displs) == c["displs"], c["name"]


@pytest.mark.parametrize("case", of_kind("all_gather_v"))
def test_all_gather_v_cases(worlds, case):
    n = case["ranks"]
    w = worlds(n)
    counts, displs, total = folded_layout(case)
    dtype = DT[case["types"][0]]
    esz = oracle.lib().orc_dtype_size(int(dtype))
    rng = np.random.default_rng(len(case["name"]))
    ins = [rand_bytes(rng, max(int(c), 1) * esz) for c in counts]
    sends = [to_dev(x) for x in ins]
    recvs = [dev_zeros(max(total, 1) * esz, fill=FILL) for _ in range(n)]
    if case.get("expect", "SUCCESS") != "SUCCESS":
        # all_gather_v_testcase.cc:259-289: overlapping receive intervals and in-place calls are HCCL_E_PARA
        assert case["expect"] == "E_PARA"
        w.inputs_ready()
        hccl_amd.group_start()
        codes = []
        for r in range(n):
            try:
                hccl_amd.all_gather_v(w.comms[r], sends[r], int(counts[r]), sends[r] if case["in_place"] else recvs[r],
                                      counts, displs, dtype, w.stream)
                codes.append(0)
            except hccl_amd.HcclError as e:
                codes.append(e.code)
        hccl_amd.group_end()                     # every call was refused at its entry: nothing is left in the group
        assert codes == [1] * n, (case["source"], codes)
        w.sync()
        for r in range(n):
            assert np.all(to_host(recvs[r], np.uint8) == FILL)      # a refused call writes nothing
        return
    want = [np.full(max(total, 1) * esz, FILL, dtype=np.uint8) for _ in range(n)]
    assert oracle.all_gather_v(ins, want, counts, displs, int(dtype)) == 0
    w.all_gather_v(sends, recvs, counts, displs, dtype)
    for r in range(n):
        assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), (case["source"], r)


@pytest.mark.parametrize("case", of_kind("reduce_scatter_v"))
def test_reduce_scatter_v_cases(worlds, case):
    """Sum where the case names no operation (reduce_scatter_v_testcase.cc:61), else the one it names.  Send
    displacements may overlap: reduce_scatter_v_testcase_a3.cc:140 hands three ranks the same slice; ranks may
    receive nothing (:285); counts may differ by a factor of 4096 (:293)."""
    n = case["ranks"]
    w = worlds(n)
    counts, displs, total = folded_layout(case)
    dtype = DT[case["types"][0]]
    op = int(OP[case.get("ops", ["SUM"])[0]])
    rng = np.random.default_rng(len(case["name"]) + 1)
    ins = [gen(dtype, op, rng, max(total, 1)) for _ in range(n)]
    want = [np.zeros(max(int(c), 1), dtype=NP[dtype]) for c in counts]
    assert oracle.reduce_scatter_v(ins, want, counts, displs, int(dtype), op, acc=oracle.ACC_FP32) == 0
    sends = [to_dev(x) for x in ins]
    recvs = [dev_zeros(x.nbytes) for x in want]
    w.reduce_scatter_v(sends, recvs, counts, displs, dtype, op)
    for r in range(n):
        c = int(counts[r])
        got = to_host(recvs[r], NP[dtype])
        check(dtype, op, got[:c], want[r][:c], "%s rank %d" % (case["source"], r))
        if c == 0:
            assert np.all(got.view(np.uint8) == FILL)           # a rank that receives nothing is left alone


@pytest.mark.parametrize("case", of_kind("broadcast"))
def test_broadcast_cases(worlds, case):
    """Up to 64 ranks, roots in every position of the reference's multi-level topologies (here one flat world)."""
    n, root, count = case["ranks"], case["root"], fold(case["count"])
    w = worlds(n)
    dtype = DT[case["types"][0]]
    esz = oracle.lib().orc_dtype_size(int(dtype))
    rng = np.random.default_rng(len(case["name"]) + root)
    host = [rand_bytes(rng, count * esz) for _ in range(n)]
    want = [x.copy() for x in host]
    assert oracle.broadcast(want, count, int(dtype), root) == 0
    bufs = [to_dev(x) for x in host]
    w.broadcast(bufs, count, dtype, root)
    for r in range(n):
        assert np.array_equal(to_host(bufs[r], np.uint8), want[r]), (case["source"], r)
        assert np.array_equal(want[r], host[root])


@pytest.mark.parametrize("case", of_kind("scatter"))
def test_scatter_cases(worlds, case):
    n, root, count = case["ranks"], case["root"], fold(case["count"])
    w = worlds(n)
    dtype = DT[case["types"][0]]
    esz = oracle.lib().orc_dtype_size(int(dtype))
    rng = np.random.default_rng(len(case["name"]) + 3 * root)
    ins = [rand_bytes(rng, n * count * esz) for _ in range(n)]
    want = [np.zeros(count * esz, dtype=np.uint8) for _ in range(n)]
    assert oracle.scatter(ins, want, count, int(dtype), root) == 0
    sends = [to_dev(ins[r]) if r == root else None for r in range(n)]      # only the root has a send buffer
    recvs = [dev_zeros(count * esz) for _ in range(n)]
    w.scatter(sends, recvs, count, dtype, root)
    for r in range(n):
        assert np.array_equal(to_host(recvs[r], np.uint8), want[r]), (case["source"], r)
