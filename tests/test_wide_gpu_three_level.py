"""GPU parity of the three-level AllReduce and ReduceScatter (level-0 groups inside level-1 groups; reference
ins_v2_all_reduce_sequence_executor_aicpu_3level.cc, ins_v2_reduce_scatter_sequence_executor_3level.cc) and of the
step-driven Reduce orders (NHR in one level, reduce_nhr.cc; RHD / NHR / the host-reduce fold in two and three levels,
reduce_sequence_executor_aicpu_3level.cc) against the CPU oracle, through the C ABI: bit-exact for fp32 / integers /
MAX, fp16 and bf16 SUM against the oracle's fp32-accumulate mode."""
import os

import numpy as np
import pytest

import hccl_amd
import oracle
from hccl_amd import Algo, HcclDataType as DT, OpKind

from gpu_util import World, dev_zeros, require_library_on_gpu, to_dev, to_host
from test_gpu_parity import MAX, MIN, NP, PROD, SUM, check, gen

pytestmark = pytest.mark.gpu

SHAPES = [(2, 2, 2), (2, 3, 2), (3, 2, 2), (2, 2, 3), (2, 1, 3), (4, 4, 4), (2, 4, 8), (4, 2, 3)]


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


def host_only(dtype, op):
    return op == PROD or dtype in (DT.INT64, DT.UINT64, DT.FP64)


def levels_world(l0, l1, l2):
    w = World(l0 * l1 * l2)
    hccl_amd.set_level0_rank_size(w.comms[0], l0)
    hccl_amd.set_level1_group_size(w.comms[0], l1)
    assert hccl_amd.get_level1_group_size(w.comms[-1]) == l1
    return w


def run_ar(w, l0, l1, algo, dtype, op, count, seed, pad=0, ccl=0):
    n = w.n
    rng = np.random.default_rng(seed)
    ins = [gen(dtype, op, rng, count) for _ in range(n)]
    want = [np.zeros(count, dtype=NP[dtype]) for _ in range(n)]
    if host_only(dtype, op):   # the host-reduce executor: two levels, every level-0 group a peer
        per_loop = ccl // 2 // 128 * 128 // ins[0].itemsize // n * n if ccl else 0
        assert oracle.all_reduce_two_level(ins, want, count, int(dtype), op, l0, "mesh", max_count_per_loop=per_loop) == 0
    else:
        assert oracle.all_reduce_three_level(ins, want, count, int(dtype), op, l0, l1, algo, ccl_bytes=ccl) == 0
    sends = [to_dev(x, (pad * (r + 1)) % 16 if pad else 0) for r, x in enumerate(ins)]
    recvs = [dev_zeros(x.nbytes, pad) for x in ins]
    w.all_reduce(sends, recvs, count, dtype, op, algo)
    for r in range(n):
        check(dtype, op, to_host(recvs[r], NP[dtype]), want[r],
              "three-level all_reduce %s %s %dx%dx%d count=%d algo=%s rank=%d" % (dtype.name, op, l0, l1, n // l0 // l1,
                                                                                  count, algo, r))


def run_rs(w, l0, l1, algo, dtype, op, c, seed, pad=0):
    n = w.n
    rng = np.random.default_rng(seed)
    ins = [gen(dtype, op, rng, n * c) for _ in range(n)]
    want = [np.zeros(c, dtype=NP[dtype]) for _ in range(n)]
    if host_only(dtype, op):
        assert oracle.reduce_scatter_two_level(ins, want, c, int(dtype), op, l0, "mesh") == 0
    else:
        assert oracle.reduce_scatter_three_level(ins, want, c, int(dtype), op, l0, l1, algo) == 0
    sends = [to_dev(x, (pad * (r + 1)) % 16 if pad else 0) for r, x in enumerate(ins)]
    recvs = [dev_zeros(x.nbytes, pad) for x in want]
    w.reduce_scatter(sends, recvs, c, dtype, op, algo)
    for r in range(n):
        check(dtype, op, to_host(recvs[r], NP[dtype]), want[r],
              "three-level reduce_scatter %s %s %dx%dx%d count=%d algo=%s rank=%d" % (dtype.name, op, l0, l1,
                                                                                      n // l0 // l1, c, algo, r))


def run_reduce(w, l0, l1, algo, dtype, op, count, root, seed, ccl=0, pad=0):
    """l0 of 1: one level."""
    n = w.n
    rng = np.random.default_rng(seed)
    ins = [gen(dtype, op, rng, count) for _ in range(n)]
    want = [np.zeros(count, dtype=NP[dtype]) for _ in range(n)]
    if l0 == 1:
        order = "mesh" if host_only(dtype, op) or algo == "rhd" else algo
        per_loop = ccl // 128 * 128 // ins[0].itemsize if ccl and order == "nhr" else 0
        assert oracle.reduce(ins, want, count, int(dtype), op, root, algo=order, max_count_per_loop=per_loop) == 0
    elif host_only(dtype, op):
        assert oracle.reduce_levels(ins, want, count, int(dtype), op, root, l0, n // l0, "mesh", ccl_bytes=ccl) == 0
    else:
        assert oracle.reduce_levels(ins, want, count, int(dtype), op, root, l0, l1, algo, ccl_bytes=ccl) == 0
    sends = [to_dev(x, (pad * (r + 1)) % 16 if pad else 0) for r, x in enumerate(ins)]
    recvs = [dev_zeros(x.nbytes, pad) for x in ins]
    w.reduce(sends, recvs, count, dtype, op, root, algo)
    check(dtype, op, to_host(recvs[root], NP[dtype]), want[root],
          "reduce %s %s levels %d/%d of %d count=%d algo=%s root=%d" % (dtype.name, op, l0, l1, n, count, algo, root))
    other = (root + 1) % n
    if other != root:   # only the root's buffer is written
        assert np.all(to_host(recvs[other], np.uint8) == 0xAB), (algo, other)


@pytest.mark.parametrize("l0,l1,l2", SHAPES)
def test_three_level_all_reduce_matches_the_oracle(l0, l1, l2):
    n = l0 * l1 * l2
    w = levels_world(l0, l1, l2)
    try:
        seed = 1000 * l0 + 100 * l1 + l2
        for algo in ("rhd", "nhr"):
            for count in (1, n - 1, n * 16, n * 16 + 3, 4093, 65543):
                run_ar(w, l0, l1, algo, DT.FP32, SUM, count, seed + count)
            run_ar(w, l0, l1, algo, DT.FP32, MAX, 3 * n + 1, seed + 1)
            run_ar(w, l0, l1, algo, DT.FP16, SUM, 2 * 4093, seed + 2, pad=2)
            run_ar(w, l0, l1, algo, DT.BFP16, SUM, 5000, seed + 3)
            run_ar(w, l0, l1, algo, DT.INT8, MIN, 70001, seed + 4, pad=1)
            run_ar(w, l0, l1, algo, DT.INT32, PROD, 4093, seed + 5)     # host-reduce fold, two levels
            run_ar(w, l0, l1, algo, DT.FP64, SUM, 1000 + n, seed + 6)
        # a staging buffer of 64 KiB: loops of the executor, each cut afresh
        w.set_ccl_buffer_size(64 * 1024)
        for algo in ("rhd", "nhr"):
            run_ar(w, l0, l1, algo, DT.FP32, SUM, 40003, seed + 7, ccl=64 * 1024)
            run_ar(w, l0, l1, algo, DT.INT32, PROD, 30011, seed + 8, ccl=64 * 1024)
    finally:
        w.set_ccl_buffer_size(0)
        w.close()


@pytest.mark.parametrize("l0,l1,l2", SHAPES)
def test_three_level_reduce_scatter_matches_the_oracle(l0, l1, l2):
    n = l0 * l1 * l2
    w = levels_world(l0, l1, l2)
    try:
        seed = 3000 * l0 + 100 * l1 + l2
        for algo in ("rhd", "nhr"):
            for c in (1, 7, 256, 4093):
                run_rs(w, l0, l1, algo, DT.FP32, SUM, c, seed + c)
            run_rs(w, l0, l1, algo, DT.FP32, MAX, 3 * n + 1, seed + 1)
            run_rs(w, l0, l1, algo, DT.FP16, SUM, 2047, seed + 2, pad=2)
            run_rs(w, l0, l1, algo, DT.BFP16, SUM, 1000, seed + 3)
            run_rs(w, l0, l1, algo, DT.INT8, MIN, 3001, seed + 4, pad=1)
            run_rs(w, l0, l1, algo, DT.INT32, PROD, 521, seed + 5)
            run_rs(w, l0, l1, algo, DT.FP64, SUM, 100 + n, seed + 6)
    finally:
        w.close()


@pytest.mark.parametrize("l0,l1,l2", [(1, 1, 2), (1, 1, 3), (1, 1, 6), (1, 1, 8), (1, 1, 13),
                                       (2, 3, 1), (3, 2, 1), (4, 4, 1), (2, 8, 1)] + SHAPES)
def test_reduce_in_the_step_driven_orders_matches_the_oracle(l0, l1, l2):
    """One level: NHR on slices of ceil(count / n) elements (RHD has no single-level Reduce in the reference and
    falls back to the rank order).  Two and three levels: the sequence executor with RHD, NHR or, for the types the
    reference reduces on the host, its host-reduce fold; chunks of floor(count / d) elements at every level."""
    n = l0 * l1 * l2
    w = World(n)
    try:
        if l0 > 1:
            hccl_amd.set_level0_rank_size(w.comms[0], l0)
            hccl_amd.set_level1_group_size(w.comms[0], l1 if l2 > 1 else 0)
        seed = 5000 * l0 + 100 * l1 + l2
        for algo in ("nhr", "rhd"):
            for k, count in enumerate((1, n - 1, n * 16, n * 16 + 3, 4093, 65543)):
                run_reduce(w, l0, l1, algo, DT.FP32, SUM, count, (k * 5 + 1) % n, seed + count)
            run_reduce(w, l0, l1, algo, DT.FP32, MIN, 3 * n + 1, n - 1, seed + 1)
            run_reduce(w, l0, l1, algo, DT.FP16, SUM, 2 * 4093, 0, seed + 2, pad=2)
            run_reduce(w, l0, l1, algo, DT.BFP16, SUM, 5000, n // 2, seed + 3)
            run_reduce(w, l0, l1, algo, DT.INT8, MAX, 70001, 1 % n, seed + 4, pad=1)
            run_reduce(w, l0, l1, algo, DT.INT32, PROD, 4093, n - 1, seed + 5)
            run_reduce(w, l0, l1, algo, DT.INT64, SUM, 1000 + n, 0, seed + 6)
        w.set_ccl_buffer_size(96 * 1024)
        for algo in ("nhr", "rhd"):
            run_reduce(w, l0, l1, algo, DT.FP32, SUM, 70001, n - 1, seed + 7, ccl=96 * 1024)
    finally:
        w.set_ccl_buffer_size(0)
        w.close()


def world_under(env, n):
    saved = {k: os.environ.get(k) for k in env}
    os.environ.update(env)
    try:
        return World(n)
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


def test_levels_and_orders_from_the_environment():
    """HCCL_AMD_LEVEL0_RANKS / HCCL_AMD_LEVEL1_GROUPS describe the topology, the reference's HCCL_ALGO names the
    executor: sequence{mesh_concur, nhr, nhr} and its relatives select the order that then runs over the levels the
    world has."""
    env = {"HCCL_AMD_LEVEL0_RANKS": "2", "HCCL_AMD_LEVEL1_GROUPS": "3",
           "HCCL_ALGO": "allreduce:sequence{level0=mesh_concur,level1=nhr,level2=nhr};"
                        "reducescatter:sequence{mesh_concur,rhd,rhd};reduce:sequence{level0=meshconcur,level1=rhd,level2=rhd}"}
    w = world_under(env, 12)
    try:
        assert hccl_amd.get_level0_rank_size(w.comms[0]) == 2 and hccl_amd.get_level1_group_size(w.comms[0]) == 3
        assert hccl_amd.get_algo(w.comms[0], OpKind.ALL_REDUCE) == Algo.NHR
        assert hccl_amd.get_algo(w.comms[0], OpKind.REDUCE_SCATTER) == Algo.RHD
        assert hccl_amd.get_algo(w.comms[0], OpKind.REDUCE) == Algo.RHD
        n, count = 12, 5003
        rng = np.random.default_rng(5)
        ins = [gen(DT.FP32, SUM, rng, count) for _ in range(n)]
        want = [np.zeros(count, np.float32) for _ in range(n)]
        assert oracle.all_reduce_three_level(ins, want, count, int(DT.FP32), SUM, 2, 3, "nhr") == 0
        recvs = [dev_zeros(x.nbytes) for x in ins]
        sends = [to_dev(x) for x in ins]
        w.inputs_ready()
        with hccl_amd.group():
            for r in range(n):
                hccl_amd.all_reduce(w.comms[r], sends[r], recvs[r], count, DT.FP32, SUM, w.stream)
        w.sync()
        check(DT.FP32, SUM, to_host(recvs[7], np.float32), want[7], "HCCL_ALGO three-level all_reduce")
        want = [np.zeros(count, np.float32) for _ in range(n)]
        assert oracle.reduce_levels(ins, want, count, int(DT.FP32), SUM, 5, 2, 3, "rhd") == 0
        recvs = [dev_zeros(x.nbytes) for x in ins]
        with hccl_amd.group():
            for r in range(n):
                hccl_amd.reduce(w.comms[r], sends[r], recvs[r], count, DT.FP32, SUM, 5, w.stream)
        w.sync()
        check(DT.FP32, SUM, to_host(recvs[5], np.float32), want[5], "HCCL_ALGO three-level reduce")
        c = 401
        ins = [gen(DT.FP32, SUM, rng, n * c) for _ in range(n)]
        want = [np.zeros(c, np.float32) for _ in range(n)]
        assert oracle.reduce_scatter_three_level(ins, want, c, int(DT.FP32), SUM, 2, 3, "rhd") == 0
        recvs = [dev_zeros(x.nbytes) for x in want]
        sends = [to_dev(x) for x in ins]
        w.inputs_ready()
        with hccl_amd.group():
            for r in range(n):
                hccl_amd.reduce_scatter(w.comms[r], sends[r], recvs[r], c, DT.FP32, SUM, w.stream)
        w.sync()
        for r in (0, 6, 11):
            check(DT.FP32, SUM, to_host(recvs[r], np.float32), want[r], "HCCL_ALGO three-level reduce_scatter %d" % r)
    finally:
        w.close()
    # a single-level executor asked for by name keeps one level whatever the topology
    w = world_under({"HCCL_AMD_LEVEL0_RANKS": "2", "HCCL_AMD_LEVEL1_GROUPS": "3", "HCCL_ALGO": "reduce:sole{nhr}"}, 12)
    try:
        n, count = 12, 1001
        rng = np.random.default_rng(6)
        ins = [gen(DT.FP32, SUM, rng, count) for _ in range(n)]
        want = [np.zeros(count, np.float32) for _ in range(n)]
        assert oracle.reduce(ins, want, count, int(DT.FP32), SUM, 3, algo="nhr") == 0
        recvs = [dev_zeros(x.nbytes) for x in ins]
        sends = [to_dev(x) for x in ins]
        w.inputs_ready()
        with hccl_amd.group():
            for r in range(n):
                hccl_amd.reduce(w.comms[r], sends[r], recvs[r], count, DT.FP32, SUM, 3, w.stream)
        w.sync()
        check(DT.FP32, SUM, to_host(recvs[3], np.float32), want[3], "reduce:sole{nhr} in a world with levels")
    finally:
        w.close()


# Another number here draws other cases (used for longer runs by hand, mostly on the CPU emulation).
SWEEP_SEED = int(os.environ.get("HCCL_AMD_TEST_SWEEP_SEED", "91000"))
TYPES = [DT.INT8, DT.INT16, DT.INT32, DT.INT64, DT.UINT64, DT.FP16, DT.BFP16, DT.FP32, DT.FP64]
LEVELS = [(2, 2, 2), (2, 2, 3), (3, 2, 2), (2, 3, 2), (2, 1, 4), (3, 3, 2), (2, 5, 2), (4, 2, 2), (2, 2, 5), (5, 2, 3),
          (2, 4, 4), (6, 2, 2)]


def pick_count(rng, n):
    kind = rng.integers(0, 4)
    if kind == 0:
        return int(rng.integers(1, 3 * n))                       # around one element per unit
    if kind == 1:
        return int(rng.integers(70, 5_000))
    if kind == 2:
        return int(rng.choice([4096, 8192, 65536]) + rng.integers(-3, 4))
    return n * int(rng.integers(1, 2_000))                       # everything divides


@pytest.mark.parametrize("l0,l1,l2", LEVELS)
def test_random_cases_over_levels(l0, l1, l2):
    """Seeded random sweep over (operator, type, operation, template, count, root, buffer alignment, staging-buffer
    size) in worlds of three levels."""
    n = l0 * l1 * l2
    rng = np.random.default_rng(SWEEP_SEED + 100 * l0 + 10 * l1 + l2)
    w = levels_world(l0, l1, l2)
    try:
        for case in range(24):
            dtype = TYPES[rng.integers(0, len(TYPES))]
            op = int(rng.integers(0, 4))
            if op == PROD and dtype in (DT.INT16, DT.BFP16):
                op = SUM
            algo = ("rhd", "nhr")[rng.integers(0, 2)]
            count = pick_count(rng, n)
            esz = np.dtype(NP[dtype]).itemsize
            pad = int(rng.integers(0, 16 // esz)) if rng.random() < 0.5 else 0
            which = rng.integers(0, 3)
            ccl = 0
            if which != 1 and rng.random() < 0.4:
                ccl = int(rng.choice([24_000, 1 << 16, 200_000]))
                host = host_only(dtype, op)
                if which == 0:      # AllReduce
                    fits = (ccl // 2 // 128 * 128 // esz // n * n > 0 if host
                            else oracle.sequence_max_count_per_loop(ccl, count, l0, n, esz, 128, algo == "rhd") is not None)
                else:               # Reduce
                    fits = oracle.sequence_max_count_per_loop(ccl, count, l0, n, esz, 4096, False) is not None
                if not fits:
                    ccl = 0
            w.set_ccl_buffer_size(ccl)
            seed = SWEEP_SEED + case * 139 + n
            if which == 0:
                run_ar(w, l0, l1, algo, dtype, op, count, seed, pad=pad, ccl=ccl)
            elif which == 1:
                run_rs(w, l0, l1, algo, dtype, op, max(1, count // n), seed, pad=pad)
            else:
                run_reduce(w, l0, l1, algo, dtype, op, count, int(rng.integers(0, n)), seed, ccl=ccl, pad=pad)
    finally:
        w.set_ccl_buffer_size(0)
        w.close()
