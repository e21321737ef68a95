"""Replays the shapes of the reference's own system tests for AllReduce, ReduceScatter, Reduce, AllGather and AlltoAll
(test/st/algorithm/testcase/all_reduce_testcase.cc, all_reduce_multilevel_testcase.cc, all_reduce_parallel_testcase.cc,
reduce_scatter_testcase.cc, reduce_scatter_aicpu_testcase*.cc, reduce_scatter_3level_testcase.cc,
reduce_scatter_meshchunk_concur_testcase.cc, reduce_testcase.cc, reduce_aicpu_testcase.cc, reduce_3level_testcase.cc,
reduce_sequence_testcase.cc, all_gather_aicpu_testcase.cc, all_gather_3level_testcase.cc, alltoall_testcase.cc;
transcribed as data into tests/golden/reference_st_reduce_shapes.json by
tests/golden/make_reference_st_reduce_shapes.py) through the C ABI against the oracle: the servers of the case's
topology become the level-0 groups of a loopback world and its pods the level-1 groups, the HCCL_ALGO string the case
sets is in the environment when the world is created, and the expected bits come from the oracle in the order that
string selects here (the two- and three-level orders where it names a sequence executor this library builds, the
one-level order otherwise).  The reference checks
these cases on a simulated task graph, not with values.  Counts above 6000 elements (the catalogue goes to 400 Mi) are
scaled down to about 3000; what they leave over after division by the rank count is kept, zero stays zero."""
import json
import os

import numpy as np
import pytest

import hccl_amd
import oracle
from hccl_amd import Algo, HcclDataType as DT, OpKind

from gpu_util import World, dev_zeros, rand_bytes, require_library_on_gpu, to_dev, to_host
from test_gpu_parity import NP, check, gen, order_of

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = json.load(open(os.path.join(HERE, "golden", "reference_st_reduce_shapes.json")))
TYPES = {"INT8": DT.INT8, "INT16": DT.INT16, "INT32": DT.INT32, "INT64": DT.INT64, "UINT64": DT.UINT64, "FP16": DT.FP16,
         "BFP16": DT.BFP16, "FP32": DT.FP32, "FP64": DT.FP64}
OPS = {"SUM": 0, "PROD": 1, "MAX": 2, "MIN": 3}
KINDS = {"all_reduce": OpKind.ALL_REDUCE, "reduce_scatter": OpKind.REDUCE_SCATTER, "reduce": OpKind.REDUCE}
COPIES = ("all_gather", "all_to_all")
SIZES = {"INT8": 1, "UINT8": 1, "INT16": 2, "UINT16": 2, "FP16": 2, "BFP16": 2, "INT32": 4, "UINT32": 4, "FP32": 4,
         "INT64": 8, "UINT64": 8, "FP64": 8, "HIF8": 1, "FP8E4M3": 1, "FP8E5M2": 1, "FP8E8M0": 1}
FILL = 0xAB
NAMES = {Algo.MESH: "mesh", Algo.RING: "ring", Algo.RHD: "rhd", Algo.NHR: "nhr", Algo.MESH_CHUNK: "mesh_chunk",
         Algo.ORDER_PRESERVED: "order_preserved", Algo.MESH_TWO_SHOT: "mesh_two_shot", Algo.AIV_MESH: "aiv_mesh",
         Algo.MESH_SYMMETRIC: "mesh_symmetric", Algo.MESH_CONCUR: "mesh_concur"}


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


def scaled(count, n):
    if count <= 6000:
        return count
    base = 3000 - 3000 % n
    return base + n * ((count // n) % 7) + count % n


def copy_shape(case, n):
    dtype, esz = DT[case["type"]], SIZES[case["type"]]
    count = scaled(case["count"], n)
    rng = np.random.default_rng(len(case["name"]) * 17 + count)
    w = World(n)
    try:
        if case["kind"] == "all_gather":
            ins = [rand_bytes(rng, max(count, 1) * esz) for _ in range(n)]
            want = [np.full(n * count * esz, FILL, dtype=np.uint8) for _ in range(n)]
            assert oracle.all_gather(ins, want, count, int(dtype)) == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(max(x.nbytes, 1), fill=FILL) for x in want]
            w.all_gather(sends, recvs, count, dtype)
        else:
            ins = [rand_bytes(rng, max(n * count, 1) * esz) for _ in range(n)]
            want = [np.full(n * count * esz, FILL, dtype=np.uint8) for _ in range(n)]
            assert oracle.all_to_all(ins, want, count, int(dtype)) == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(max(x.nbytes, 1), fill=FILL) for x in want]
            w.inputs_ready()
            with hccl_amd.group():
                for r in range(n):
                    hccl_amd.all_to_all(w.comms[r], sends[r], count, dtype, recvs[r], count, dtype, w.stream)
            w.sync()
        for r in range(n):
            assert np.array_equal(to_host(recvs[r], np.uint8)[:want[r].nbytes], want[r]), (case["name"], case["source"], r)
    finally:
        w.close()


def test_the_catalogue_is_what_the_generator_wrote():
    assert len(CASES) == 241
    assert {c["kind"] for c in CASES} == set(KINDS) | set(COPIES)
    assert all(c["type"] in (SIZES if c["kind"] in COPIES else TYPES) and c["op"] in OPS and sum(c["servers"]) <= 64
               for c in CASES)
    assert scaled(262148, 12) % 12 == 8 and scaled(5, 3) == 5 and scaled(0, 4) == 0 and scaled(419430400, 8) % 8 == 0


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_reference_system_test_shape(case):
    servers = case["servers"]
    n = sum(servers)
    if case["kind"] in COPIES:
        return copy_shape(case, n)
    kind, dtype, op = case["kind"], TYPES[case["type"]], OPS[case["op"]]
    level0 = servers[0] if len(servers) > 1 and len(set(servers)) == 1 and servers[0] > 1 else 1
    pods = case["pods"]
    level1 = pods[0] if level0 > 1 and len(pods) > 1 and len(set(pods)) == 1 else 0
    count = scaled(case["count"], n)
    env = {"HCCL_AMD_LEVEL0_RANKS": str(level0), "HCCL_AMD_LEVEL1_GROUPS": str(level1)}
    if case["hccl_algo"]:
        env["HCCL_ALGO"] = case["hccl_algo"]
    saved = {k: os.environ.get(k) for k in ("HCCL_ALGO", "HCCL_AMD_LEVEL0_RANKS", "HCCL_AMD_LEVEL1_GROUPS")}
    os.environ.pop("HCCL_ALGO", None)
    os.environ.update(env)
    try:
        w = World(n)
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    try:
        algo = NAMES[hccl_amd.get_algo(w.comms[0], KINDS[kind])]
        _, _, sequence = hccl_amd.select_from_hccl_algo(case["hccl_algo"] or "", KINDS[kind])
        host_only = op == OPS["PROD"] or dtype in (DT.INT64, DT.UINT64, DT.FP64)
        rng = np.random.default_rng(len(case["name"]) * 131 + count)
        what = "%s %s" % (case["name"], case["source"])
        # over levels: RHD / NHR unless a single-level executor was named, and the host-reduce fold where a sequence
        # executor with it was named (the order is then MESH for every type)
        two_level = level0 > 1 and ((sequence or not case["hccl_algo"]) and algo in ("rhd", "nhr") or
                                    (sequence and algo == "mesh"))
        host_only = host_only or (two_level and algo == "mesh")
        if kind == "reduce":
            root = case["root"]
            ins = [gen(dtype, op, rng, count) for _ in range(n)]
            want = [np.zeros(count, dtype=NP[dtype]) for _ in range(n)]
            if two_level:
                assert oracle.reduce_levels(ins, want, count, int(dtype), op, root, level0,
                                            n // level0 if host_only or not level1 else level1,
                                            "mesh" if host_only else algo) == 0
            else:   # one level: NHR, or the rank order (which the host-reduced types and a lone RHD fall back to)
                order = algo if algo in ("mesh", "ring", "mesh_two_shot") or (algo == "nhr" and not host_only) else "mesh"
                assert oracle.reduce(ins, want, count, int(dtype), op, root, algo=order) == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(max(x.nbytes, 1)) for x in ins]
            w.inputs_ready()
            with hccl_amd.group():
                for r in range(n):
                    hccl_amd.reduce(w.comms[r], sends[r], recvs[r], count, dtype, op, root, w.stream)
            w.sync()
            if count:
                check(dtype, op, to_host(recvs[root], NP[dtype])[:count], want[root], what)
            return
        between = "mesh" if host_only else algo
        if kind == "all_reduce":
            ins = [gen(dtype, op, rng, count) for _ in range(n)]
            want = [np.zeros(count, dtype=NP[dtype]) for _ in range(n)]
            if two_level and level1 and not host_only:
                assert oracle.all_reduce_three_level(ins, want, count, int(dtype), op, level0, level1, algo) == 0
            elif two_level:
                assert oracle.all_reduce_two_level(ins, want, count, int(dtype), op, level0, between) == 0
            else:
                assert oracle.all_reduce(ins, want, count, int(dtype), op, algo=order_of(algo, dtype, op, False)) == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(max(x.nbytes, 1)) for x in ins]
            w.inputs_ready()
            with hccl_amd.group():
                for r in range(n):
                    hccl_amd.all_reduce(w.comms[r], sends[r], recvs[r], count, dtype, op, w.stream)
        else:
            ins = [gen(dtype, op, rng, n * count) for _ in range(n)]
            want = [np.zeros(count, dtype=NP[dtype]) for _ in range(n)]
            if two_level and level1 and not host_only:
                assert oracle.reduce_scatter_three_level(ins, want, count, int(dtype), op, level0, level1, algo) == 0
            elif two_level:
                assert oracle.reduce_scatter_two_level(ins, want, count, int(dtype), op, level0, between) == 0
            else:
                assert oracle.reduce_scatter(ins, want, count, int(dtype), op, algo=order_of(algo, dtype, op, True)) == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(max(x.nbytes, 1)) for x in want]
            w.inputs_ready()
            with hccl_amd.group():
                for r in range(n):
                    hccl_amd.reduce_scatter(w.comms[r], sends[r], recvs[r], count, dtype, op, w.stream)
        w.sync()
        for r in range(n):
            if count:
                check(dtype, op, to_host(recvs[r], NP[dtype])[:count], want[r], "%s rank %d" % (what, r))
    finally:
        w.close()
