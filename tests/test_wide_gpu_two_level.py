"""GPU parity of the two-level AllReduce and ReduceScatter (level-0 groups of consecutive ranks, the configured
template between the groups; reference ins_v2_all_reduce_sequence_executor_aicpu.cc:592-852,
ins_v2_reduce_scatter_sequence_executor_aicpu.cc:298-500) against the CPU oracle, through the C ABI:
bit-exact for fp32 / integers / MAX, fp16 and bf16 SUM against the oracle's fp32-accumulate mode.  Also the reading
of HCCL_ALGO at world creation."""
import os

import numpy as np
import pytest

import hccl_amd
import oracle
from hccl_amd import Algo, HcclDataType as DT, OpKind

from gpu_util import World, dev_zeros, require_library_on_gpu, to_dev, to_host
from test_gpu_parity import MAX, MIN, NP, PROD, SUM, check, gen

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


def level1_of(algo, dtype, op):
    """PROD and the 64-bit types run on the host in the reference: between the groups they take its host-reduce
    template, which folds the own share first."""
    host_only = op == PROD or dtype in (DT.INT64, DT.UINT64, DT.FP64)
    return "mesh" if host_only else algo


def run(world, l0, algo, dtype, op, count, seed, pad=0, max_count_per_loop=0):
    n = world.n
    rng = np.random.default_rng(seed)
    ins = [gen(dtype, op, rng, count) for _ in range(n)]
    want = [np.zeros(count, dtype=NP[dtype]) for _ in range(n)]
    assert oracle.all_reduce_two_level(ins, want, count, int(dtype), op, l0, level1_of(algo, dtype, op),
                                       acc=oracle.ACC_FP32, max_count_per_loop=max_count_per_loop) == 0
    sends = [to_dev(x, (pad * (r + 1)) % 16 if pad else 0) for r, x in enumerate(ins)]
    recvs = [dev_zeros(x.nbytes, pad) for x in ins]
    world.all_reduce(sends, recvs, count, dtype, op, algo)
    for r in range(n):
        check(dtype, op, to_host(recvs[r], NP[dtype]), want[r],
              "two-level all_reduce %s %s %dx%d count=%d algo=%s rank=%d" % (dtype.name, op, l0, n // l0, count, algo, r))


@pytest.mark.parametrize("l0,l1", [(2, 3), (2, 4), (4, 2), (3, 2), (2, 6), (8, 8), (4, 4)])
def test_two_level_all_reduce_matches_the_oracle(l0, l1):
    n = l0 * l1
    w = World(n)
    try:
        hccl_amd.set_level0_rank_size(w.comms[0], l0)
        assert hccl_amd.get_level0_rank_size(w.comms[n - 1]) == l0
        seed = 100 * l0 + l1
        for algo in ("rhd", "nhr"):
            for count in (1, n - 1, n * 16, n * 16 + 3, 4093, 65543):
                run(w, l0, algo, DT.FP32, SUM, count, seed + count)
            run(w, l0, algo, DT.FP32, MAX, 3 * n + 1, seed + 1)
            run(w, l0, algo, DT.FP16, SUM, 2 * 4093, seed + 2, pad=2)
            run(w, l0, algo, DT.BFP16, SUM, 5000, seed + 3)
            run(w, l0, algo, DT.INT8, MIN, 70001, seed + 4, pad=1)
            run(w, l0, algo, DT.INT32, PROD, 4093, seed + 5)        # host-reduce fold between the groups
            run(w, l0, algo, DT.FP64, SUM, 1000 + n, seed + 6)
        # the other orders do not look at the groups
        rng = np.random.default_rng(seed)
        ins = [gen(DT.FP32, SUM, rng, 1234) for _ in range(n)]
        want = [np.zeros(1234, dtype=np.float32) for _ in range(n)]
        assert oracle.all_reduce(ins, want, 1234, int(DT.FP32), SUM, algo="mesh") == 0
        recvs = [dev_zeros(x.nbytes) for x in ins]
        w.all_reduce([to_dev(x) for x in ins], recvs, 1234, DT.FP32, SUM, "mesh")
        check(DT.FP32, SUM, to_host(recvs[0], np.float32), want[0], "mesh with groups")
    finally:
        w.close()


def run_rs(world, l0, algo, dtype, op, c, seed, pad=0):
    n = world.n
    rng = np.random.default_rng(seed)
    ins = [gen(dtype, op, rng, n * c) for _ in range(n)]
    want = [np.zeros(c, dtype=NP[dtype]) for _ in range(n)]
    assert oracle.reduce_scatter_two_level(ins, want, c, int(dtype), op, l0, level1_of(algo, dtype, op),
                                           acc=oracle.ACC_FP32) == 0
    sends = [to_dev(x, (pad * (r + 1)) % 16 if pad else 0) for r, x in enumerate(ins)]
    recvs = [dev_zeros(x.nbytes, pad) for x in want]
    world.reduce_scatter(sends, recvs, c, dtype, op, algo)
    for r in range(n):
        check(dtype, op, to_host(recvs[r], NP[dtype]), want[r],
              "two-level reduce_scatter %s %s %dx%d count=%d algo=%s rank=%d" % (dtype.name, op, l0, n // l0, c, algo, r))


@pytest.mark.parametrize("l0,l1", [(2, 3), (2, 4), (4, 2), (3, 2), (2, 6), (8, 8), (4, 4)])
def test_two_level_reduce_scatter_matches_the_oracle(l0, l1):
    """The reference's two-level ReduceScatter (ins_v2_reduce_scatter_sequence_executor_aicpu.cc:298-500): mesh inside
    the groups, RHD / NHR / the host-reduce fold between them; loops cover the same range of every slice and do not
    show, so a bounded staging buffer changes nothing."""
    n = l0 * l1
    w = World(n)
    try:
        hccl_amd.set_level0_rank_size(w.comms[0], l0)
        seed = 300 * l0 + l1
        for algo in ("rhd", "nhr"):
            for c in (1, 7, 256, 4093, 20011):
                run_rs(w, l0, algo, DT.FP32, SUM, c, seed + c)
            run_rs(w, l0, algo, DT.FP32, MAX, 3 * n + 1, seed + 1)
            run_rs(w, l0, algo, DT.FP16, SUM, 4093, seed + 2, pad=2)
            run_rs(w, l0, algo, DT.BFP16, SUM, 5000, seed + 3)
            run_rs(w, l0, algo, DT.INT8, MIN, 7001, seed + 4, pad=1)
            run_rs(w, l0, algo, DT.INT32, PROD, 1021, seed + 5)        # host-reduce fold between the groups
            run_rs(w, l0, algo, DT.FP64, SUM, 100 + n, seed + 6)
        w.set_ccl_buffer_size(64 * 1024)
        run_rs(w, l0, "rhd", DT.FP32, SUM, 30011, seed + 7)
        w.set_ccl_buffer_size(0)
        # the other orders do not look at the groups
        rng = np.random.default_rng(seed)
        ins = [gen(DT.FP32, SUM, rng, n * 321) for _ in range(n)]
        want = [np.zeros(321, dtype=np.float32) for _ in range(n)]
        assert oracle.reduce_scatter(ins, want, 321, int(DT.FP32), SUM, algo="mesh") == 0
        recvs = [dev_zeros(x.nbytes) for x in want]
        w.reduce_scatter([to_dev(x) for x in ins], recvs, 321, DT.FP32, SUM, "mesh")
        check(DT.FP32, SUM, to_host(recvs[n - 1], np.float32), want[n - 1], "mesh with groups")
    finally:
        w.set_ccl_buffer_size(0)
        w.close()


def test_two_level_as_fold_and_fan_out_and_in_loops():
    """The two-kernel form (forced, with small pieces) and the reference's staging-buffer loops give the same bits."""
    forced = {"HCCL_AMD_ALLREDUCE_TWO_KERNELS": "1", "HCCL_AMD_ALLREDUCE_PIECE_BYTES": "8192"}
    saved = {k: os.environ.get(k) for k in forced}
    os.environ.update(forced)
    try:
        w = World(6)
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    try:
        hccl_amd.set_level0_rank_size(w.comms[0], 2)
        for algo in ("rhd", "nhr"):
            run(w, 2, algo, DT.FP32, SUM, 6 * 4000 + 5, 41)
            run(w, 2, algo, DT.FP16, SUM, 6 * 4000, 42)
        # loops: half of the buffer receives, floored to 128 bytes and to a multiple of 6 elements
        ccl = 64 * 1024
        w.set_ccl_buffer_size(ccl)
        per_loop_nhr = ccl // 2 // 128 * 128 // 4 // 6 * 6
        run(w, 2, "nhr", DT.FP32, SUM, 3 * per_loop_nhr + 77, 43, max_count_per_loop=per_loop_nhr)
        count = 3 * per_loop_nhr + 77
        rc, per_loop_rhd = oracle.rhd_max_count_per_loop(ccl, count, 6, 4)
        assert rc == 0
        run(w, 2, "rhd", DT.FP32, SUM, count, 44, max_count_per_loop=per_loop_rhd)
    finally:
        w.set_ccl_buffer_size(0)
        w.close()


def test_hccl_algo_is_read_when_a_world_is_created():
    saved = {k: os.environ.get(k) for k in ("HCCL_ALGO", "HCCL_AMD_LEVEL0_RANKS")}
    try:
        os.environ["HCCL_ALGO"] = "allreduce:sequence{level0=mesh_concur,level1=rhd};reducescatter:nhr"
        os.environ["HCCL_AMD_LEVEL0_RANKS"] = "2"
        w = World(6)
        try:
            assert hccl_amd.get_algo(w.comms[0], OpKind.ALL_REDUCE) == Algo.RHD
            assert hccl_amd.get_algo(w.comms[0], OpKind.REDUCE_SCATTER) == Algo.NHR
            assert hccl_amd.get_level0_rank_size(w.comms[0]) == 2
            n, count = 6, 6 * 100 + 4
            rng = np.random.default_rng(5)
            ins = [gen(DT.FP32, SUM, rng, count) for _ in range(n)]
            want = [np.zeros(count, dtype=np.float32) for _ in range(n)]
            assert oracle.all_reduce_two_level(ins, want, count, int(DT.FP32), SUM, 2, "rhd") == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(x.nbytes) for x in ins]
            w.inputs_ready()
            with hccl_amd.group():
                for r in range(n):
                    hccl_amd.all_reduce(w.comms[r], sends[r], recvs[r], count, DT.FP32, SUM, w.stream)
            w.sync()
            for r in range(n):
                check(DT.FP32, SUM, to_host(recvs[r], np.float32), want[r], "HCCL_ALGO sequence rank %d" % r)
        finally:
            w.close()
        # a single-level executor keeps the world flat even with groups; a rejected string changes nothing
        os.environ["HCCL_ALGO"] = "allreduce:sole{nhr}"
        w = World(6)
        try:
            count = 6 * 50 + 1
            rng = np.random.default_rng(6)
            ins = [gen(DT.FP32, SUM, rng, count) for _ in range(6)]
            want = [np.zeros(count, dtype=np.float32) for _ in range(6)]
            assert oracle.all_reduce(ins, want, count, int(DT.FP32), SUM, algo="nhr") == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(x.nbytes) for x in ins]
            w.inputs_ready()
            with hccl_amd.group():
                for r in range(6):
                    hccl_amd.all_reduce(w.comms[r], sends[r], recvs[r], count, DT.FP32, SUM, w.stream)
            w.sync()
            check(DT.FP32, SUM, to_host(recvs[2], np.float32), want[2], "HCCL_ALGO sole{nhr} with groups")
        finally:
            w.close()
        # ReduceScatter: the strings of the reference's own system tests (reduce_scatter_aicpu_testcase*.cc)
        os.environ["HCCL_ALGO"] = "reducescatter:sequence{level0=meshconcur,level1=rhd}"
        w = World(6)
        try:
            assert hccl_amd.get_algo(w.comms[0], OpKind.REDUCE_SCATTER) == Algo.RHD
            n, c = 6, 1003
            rng = np.random.default_rng(8)
            ins = [gen(DT.FP32, SUM, rng, n * c) for _ in range(n)]
            want = [np.zeros(c, dtype=np.float32) for _ in range(n)]
            assert oracle.reduce_scatter_two_level(ins, want, c, int(DT.FP32), SUM, 2, "rhd") == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(x.nbytes) for x in want]
            w.inputs_ready()
            with hccl_amd.group():
                for r in range(n):
                    hccl_amd.reduce_scatter(w.comms[r], sends[r], recvs[r], c, DT.FP32, SUM, w.stream)
            w.sync()
            for r in range(n):
                check(DT.FP32, SUM, to_host(recvs[r], np.float32), want[r], "HCCL_ALGO reducescatter sequence rank %d" % r)
        finally:
            w.close()
        os.environ["HCCL_ALGO"] = "reducescatter:sole{level0=hdaicpureduce}"
        w = World(6)
        try:
            assert hccl_amd.get_algo(w.comms[0], OpKind.REDUCE_SCATTER) == Algo.RHD
            n, c = 6, 501
            rng = np.random.default_rng(9)
            ins = [gen(DT.FP32, SUM, rng, n * c) for _ in range(n)]
            want = [np.zeros(c, dtype=np.float32) for _ in range(n)]
            assert oracle.reduce_scatter(ins, want, c, int(DT.FP32), SUM, algo="rhd") == 0
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(x.nbytes) for x in want]
            w.inputs_ready()
            with hccl_amd.group():
                for r in range(n):
                    hccl_amd.reduce_scatter(w.comms[r], sends[r], recvs[r], c, DT.FP32, SUM, w.stream)
            w.sync()
            check(DT.FP32, SUM, to_host(recvs[4], np.float32), want[4], "HCCL_ALGO reducescatter sole{hd} with groups")
        finally:
            w.close()
        os.environ["HCCL_ALGO"] = "allreduce:sole{no_such_template}"
        w = World(4)
        try:
            assert hccl_amd.get_algo(w.comms[0], OpKind.ALL_REDUCE) == Algo.MESH
        finally:
            w.close()
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
