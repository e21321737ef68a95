"""CPU-only checks of the shipped library's host logic: it loads, exports what include/hccl.h
declares, rejects bad arguments with the reference's return codes before touching a GPU, and its
fold programs (the reduction plans the kernels execute) reproduce the oracle's results when
evaluated with numpy."""
import ctypes
import os
import re

import numpy as np
import pytest

import hccl_amd
from hccl_amd import Algo, HcclDataType as DT, HcclReduceOp as OP, OpKind

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32, U64 = 4, 6
SUM, PROD, MAX, MIN = range(4)


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "hccl.h")).read()
    names = set(re.findall(r"\b(Hccl[A-Za-z0-9]+)\s*\(", header))
    assert {"HcclAllReduce", "HcclReduceScatter", "HcclAllGather", "HcclAllGatherV", "HcclAlltoAllV", "HcclAlltoAll",
            "HcclAlltoAllVC", "HcclReduceScatterV", "HcclReduce", "HcclBroadcast", "HcclScatter"} <= names
    L = ctypes.CDLL(hccl_amd.LIB_PATH)
    for n in sorted(names):
        assert hasattr(L, n), n


# ---- fold programs ----------------------------------------------------------------------------------
def f32_fold(src, dst, op):
    with np.errstate(all="ignore"):
        if op == SUM:
            return src + dst
        if op == MAX:
            return np.where(src < dst, dst, src)
        return np.where(dst < src, dst, src)


def run_program(prog, leaf, op):
    """Evaluates a fold program; returns the value of the outermost level."""
    pos = 0

    def level():
        nonlocal pos
        acc = None
        while True:
            tok = prog[pos]
            pos += 1
            if tok in (0x81, 0xFF):
                return acc
            if tok == 0x80:
                sub = level()
                acc = sub if acc is None else f32_fold(sub, acc, op)
            else:
                n = tok & 0x3F if tok >= 0xC0 else 1
                ranks = prog[pos:pos + n] if tok >= 0xC0 else [tok]
                pos += n if tok >= 0xC0 else 0
                for r in ranks:
                    v = leaf(r)
                    acc = v if acc is None else f32_fold(v, acc, op)

    out = level()
    assert pos == len(prog) and prog[-1] == 0xFF
    return out


def program_ranks(prog):
    ranks, i = [], 0
    while i < len(prog):
        t = prog[i]
        i += 1
        if t >= 0xC0 and t != 0xFF:
            ranks += list(prog[i:i + (t & 0x3F)])
            i += t & 0x3F
        elif t < 0x40:
            ranks.append(t)
    return ranks


def wide(rng, n, count):
    return [(rng.standard_normal(count) * 10.0 ** rng.integers(-6, 6, count)).astype(np.float32) for _ in range(n)]


def tricky(rng, n, count):
    pool = np.array([0, 0x80000000, 0x7FC00001, 0x7FC00002, 0xFFC00003, 0x3F800000, 0xBF800000], dtype=np.uint32)
    return [pool[rng.integers(0, pool.size, count)].view(np.float32).copy() for _ in range(n)]


def same(a, b):
    nan = np.isnan(a) & np.isnan(b)
    return np.array_equal(a.view(np.uint32)[~nan], b.view(np.uint32)[~nan]) and np.array_equal(np.isnan(a), np.isnan(b))


RANKS = [1, 2, 3, 5, 6, 7, 8, 12, 16, 33, 64]
ALGO_NAME = {Algo.MESH_CHUNK: "mesh_chunk", Algo.MESH: "mesh", Algo.RING: "ring", Algo.RHD: "rhd", Algo.NHR: "nhr",
             Algo.ORDER_PRESERVED: "order_preserved", Algo.AIV_MESH: "aiv_mesh",
             Algo.MESH_SYMMETRIC: "mesh_symmetric"}


@pytest.mark.parametrize("n", RANKS)
def test_every_program_uses_every_rank_once(n):
    for kind in (OpKind.ALL_REDUCE, OpKind.REDUCE_SCATTER, OpKind.REDUCE):
        for algo in Algo:
            if kind == OpKind.ALL_REDUCE and algo == Algo.AIV_MESH:
                continue
            if kind != OpKind.ALL_REDUCE and algo == Algo.MESH_CONCUR:
                continue
            if (kind == OpKind.REDUCE) != (algo == Algo.MESH_TWO_SHOT) and not (
                    kind == OpKind.REDUCE and algo in (Algo.MESH, Algo.RING, Algo.NHR)):
                continue
            for prog in hccl_amd.fold_programs(kind, algo, n):
                assert sorted(program_ranks(prog)) == list(range(n)), (kind, algo, n)
                assert len(prog) <= 320


@pytest.mark.parametrize("n", RANKS)
@pytest.mark.parametrize("algo", [Algo.MESH, Algo.RING, Algo.RHD, Algo.NHR, Algo.ORDER_PRESERVED, Algo.AIV_MESH,
                                  Algo.MESH_SYMMETRIC, Algo.MESH_CHUNK])
def test_reduce_scatter_programs_match_oracle(orc, n, algo):
    progs = hccl_amd.fold_programs(OpKind.REDUCE_SCATTER, algo, n)
    c = 2 * n + 5
    for op, gen in ((SUM, wide), (MAX, tricky), (MIN, tricky)):
        rng = np.random.default_rng(1000 * n + 10 * int(algo) + op)
        ins = gen(rng, n, n * c)
        outs = [np.zeros(c, dtype=np.float32) for _ in range(n)]
        assert orc.reduce_scatter(ins, outs, c, F32, op, algo=ALGO_NAME[algo]) == 0
        for k in range(n):
            if algo == Algo.MESH_CHUNK and n > 1:
                got = np.zeros(c, dtype=np.float32)
                lo = 0
                for i, ln in enumerate(orc.mesh_chunk_segments(c, n, 4, True)):
                    if ln:
                        got[lo:lo + ln] = run_program(progs[k * (n - 1) + i],
                                                      lambda r: ins[r][k * c + lo:k * c + lo + ln], op)
                    lo += ln
            elif algo == Algo.AIV_MESH:
                per = c // n
                got = np.zeros(c, dtype=np.float32)
                for ch in range(n):
                    lo, hi = ch * per, (c if ch == n - 1 else (ch + 1) * per)
                    if hi > lo:
                        got[lo:hi] = run_program(progs[ch], lambda r: ins[r][k * c + lo:k * c + hi], op)
            else:
                prog = progs[k] if len(progs) > 1 else progs[0]
                got = run_program(prog, lambda r: ins[r][k * c:(k + 1) * c], op)
            assert same(got, outs[k]), (n, algo, op, k)


@pytest.mark.parametrize("n", RANKS)
@pytest.mark.parametrize("algo", [Algo.MESH, Algo.RING, Algo.RHD, Algo.NHR, Algo.ORDER_PRESERVED, Algo.MESH_SYMMETRIC,
                                  Algo.MESH_CHUNK])
def test_all_reduce_programs_match_oracle(orc, n, algo):
    progs = hccl_amd.fold_programs(OpKind.ALL_REDUCE, algo, n)
    count = 5 * n + 3
    for op, gen in ((SUM, wide), (MAX, tricky)):
        rng = np.random.default_rng(2000 * n + 10 * int(algo) + op)
        ins = gen(rng, n, count)
        outs = [np.zeros(count, dtype=np.float32) for _ in range(n)]
        assert orc.all_reduce(ins, outs, count, F32, op, algo=ALGO_NAME[algo]) == 0
        got = np.zeros(count, dtype=np.float32)
        if len(progs) == 1:
            got[:] = run_program(progs[0], lambda r: ins[r], op)
        elif algo == Algo.RHD:
            unit = count // n
            for i in range(n):
                lo, hi = i * unit, (i + 1) * unit
                if hi > lo:
                    got[lo:hi] = run_program(progs[i], lambda r: ins[r][lo:hi], op)
            for e in range(unit * n, count):
                got[e:e + 1] = run_program(progs[e - unit * n], lambda r: ins[r][e:e + 1], op)
        elif algo == Algo.MESH_CHUNK:
            sl = -(-count // n)
            for k in range(n):
                lo = min(count, k * sl)
                for i, ln in enumerate(orc.mesh_chunk_segments(max(0, min(sl, count - k * sl)), n, 4, False)):
                    if ln:
                        got[lo:lo + ln] = run_program(progs[k * (n - 1) + i], lambda r: ins[r][lo:lo + ln], op)
                    lo += ln
        elif algo == Algo.NHR:       # floor slices, the last one takes the rest
            sl = count // n
            for i in range(n):
                lo, hi = i * sl, (count if i == n - 1 else (i + 1) * sl)
                if hi > lo:
                    got[lo:hi] = run_program(progs[i], lambda r: ins[r][lo:hi], op)
        else:                        # ceil slices, the last ones may be short or empty
            sl = -(-count // n)
            for i in range(n):
                lo, hi = min(count, i * sl), min(count, (i + 1) * sl)
                if hi > lo:
                    got[lo:hi] = run_program(progs[i], lambda r: ins[r][lo:hi], op)
        assert same(got, outs[0]), (n, algo, op)


def test_known_programs():
    # rank order, one run of 8
    assert hccl_amd.fold_programs(OpKind.ALL_REDUCE, Algo.MESH, 8) == [bytes([0xC8, 0, 1, 2, 3, 4, 5, 6, 7, 0xFF])]
    # own slice first
    assert hccl_amd.fold_programs(OpKind.REDUCE_SCATTER, Algo.MESH, 4)[2] == bytes([0xC4, 2, 0, 1, 3, 0xFF])
    # mesh chunk, 4 ranks, slice 1: segments fold 1,2,3,0 / 1,3,0,2 / 1,0,2,3
    mc = hccl_amd.fold_programs(OpKind.REDUCE_SCATTER, Algo.MESH_CHUNK, 4)
    assert len(mc) == 12
    assert mc[3:6] == [bytes([0xC4, 1, 2, 3, 0, 0xFF]), bytes([0xC4, 1, 3, 0, 2, 0xFF]), bytes([0xC4, 1, 0, 2, 3, 0xFF])]
    assert hccl_amd.fold_programs(OpKind.ALL_REDUCE, Algo.MESH_CHUNK, 4) == mc
    # p = 6: ((x0+x2)+x4) + ((x1+x3)+x5) for the share of rank 0
    p6 = hccl_amd.fold_programs(OpKind.ALL_REDUCE, Algo.RHD, 6)
    assert p6[0] == bytes([0xC3, 0, 2, 4, 0x80, 0xC3, 1, 3, 5, 0x81, 0xFF])


# ---- argument validation (returns before any GPU work) ------------------------------------------------
@pytest.fixture(scope="module")
def world():
    comms = hccl_amd.comm_init_all(4)
    yield comms
    for c in comms:
        hccl_amd.comm_destroy(c)


def code_of(fn, *a, **k):
    try:
        return fn(*a, **k)
    except hccl_amd.HcclError as e:
        return e.code


def test_lifecycle_queries(world):
    assert [hccl_amd.get_rank_id(c) for c in world] == [0, 1, 2, 3]
    names = {hccl_amd.get_comm_name(c) for c in world}
    assert len(names) == 1 and 0 < len(names.pop()) < 128          # one name per world
    other = hccl_amd.comm_init_all(2)
    assert hccl_amd.get_comm_name(other[0]) == hccl_amd.get_comm_name(other[1]) != hccl_amd.get_comm_name(world[0])
    for c in other:
        hccl_amd.comm_destroy(c)
    assert code_of(hccl_amd.get_comm_name, other[0]) == 1          # a destroyed handle
    assert hccl_amd.get_rank_size(world[2]) == 4
    assert code_of(hccl_amd.comm_init_all, 0) == 1
    assert code_of(hccl_amd.comm_init_all, 65) == 1
    assert code_of(hccl_amd.comm_init_all, 2, [0, 1]) == 5
    info = hccl_amd.get_root_info()
    a = hccl_amd.comm_init_root_info(2, info, 0)
    assert code_of(hccl_amd.comm_init_root_info, 2, info, 0) == 1      # rank joined twice
    assert code_of(hccl_amd.comm_init_root_info, 3, info, 1) == 1      # size mismatch
    b = hccl_amd.comm_init_root_info(2, info, 1)
    assert hccl_amd.get_rank_id(b) == 1 and hccl_amd.get_rank_size(a) == 2
    hccl_amd.comm_destroy(a)
    hccl_amd.comm_destroy(b)
    assert code_of(hccl_amd.get_rank_id, a) == 1                       # destroyed handle


def test_algo_knob(world):
    assert hccl_amd.get_algo(world[0], OpKind.ALL_REDUCE) == Algo.MESH
    hccl_amd.set_algo(world[1], OpKind.ALL_REDUCE, Algo.RHD)
    assert hccl_amd.get_algo(world[3], OpKind.ALL_REDUCE) == Algo.RHD   # per world, not per rank
    assert code_of(hccl_amd.set_algo, world[0], OpKind.ALL_REDUCE, Algo.AIV_MESH) == 5
    hccl_amd.set_algo(world[0], OpKind.ALL_REDUCE, Algo.MESH)
    # Reduce knows its one-shot and two-shot orders, NHR, and RHD for worlds with levels; the two-shot order exists
    # for Reduce only
    assert hccl_amd.get_algo(world[0], OpKind.REDUCE) == Algo.MESH
    for algo in (Algo.MESH_TWO_SHOT, Algo.NHR, Algo.RHD):
        hccl_amd.set_algo(world[0], OpKind.REDUCE, algo)
        assert hccl_amd.get_algo(world[2], OpKind.REDUCE) == algo
    hccl_amd.set_algo(world[0], OpKind.REDUCE, Algo.MESH)
    for kind, algo in ((OpKind.REDUCE, Algo.ORDER_PRESERVED), (OpKind.REDUCE, Algo.MESH_CHUNK),
                       (OpKind.ALL_REDUCE, Algo.MESH_TWO_SHOT), (OpKind.REDUCE_SCATTER, Algo.MESH_TWO_SHOT)):
        assert code_of(hccl_amd.set_algo, world[0], kind, algo) == 5


@pytest.mark.parametrize("n", [1, 2, 5, 8, 33])
def test_reduce_programs_match_oracle(orc, n):
    count = 4 * n + 3
    rng = np.random.default_rng(3000 + n)
    ins = wide(rng, n, count)
    one = hccl_amd.fold_programs(OpKind.REDUCE, Algo.MESH, n)
    two = hccl_amd.fold_programs(OpKind.REDUCE, Algo.MESH_TWO_SHOT, n)
    assert len(one) == 1 and len(two) == n
    outs = [np.zeros(count, dtype=np.float32) for _ in range(n)]
    assert orc.reduce(ins, outs, count, F32, SUM, n - 1) == 0
    assert same(run_program(one[0], lambda r: ins[r], SUM), outs[n - 1])
    assert orc.reduce(ins, outs, count, F32, SUM, 0, algo="mesh_two_shot") == 0
    got = np.zeros(count, dtype=np.float32)
    lo = 0
    for k in range(n):
        ln = count // n + (1 if k < count % n else 0)
        got[lo:lo + ln] = run_program(two[k], lambda r: ins[r][lo:lo + ln], SUM)
        lo += ln
    assert same(got, outs[0])


def test_all_reduce_argument_checks(world):
    c, s, buf = world[0], 0x1000, 0x2000
    assert hccl_amd.all_reduce(c, None, None, 0, DT.FP32, OP.SUM, None) == 0        # count 0 wins over everything
    assert code_of(hccl_amd.all_reduce, c, buf, buf, 8, DT.FP32, OP.SUM, None) == 2   # null stream
    assert code_of(hccl_amd.all_reduce, None, buf, buf, 8, DT.FP32, OP.SUM, s) == 2   # null comm
    assert code_of(hccl_amd.all_reduce, c, None, buf, 8, DT.FP32, OP.SUM, s) == 2
    assert code_of(hccl_amd.all_reduce, c, buf, None, 8, DT.FP32, OP.SUM, s) == 2
    assert code_of(hccl_amd.all_reduce, c, buf, buf, 0x800000000, DT.FP32, OP.SUM, s) == 1
    for bad in (DT.UINT8, DT.UINT16, DT.UINT32, DT.INT128, DT.HIF8, DT.FP8E4M3, DT.FP8E5M2, DT.FP8E8M0, 13, 99):
        assert code_of(hccl_amd.all_reduce, c, buf, buf, 8, bad, OP.SUM, s) == 5
    for bad in (DT.INT16, DT.BFP16):
        assert code_of(hccl_amd.all_reduce, c, buf, buf, 8, bad, OP.PROD, s) == 5
    assert code_of(hccl_amd.all_reduce, c, buf, buf, 8, DT.FP32, 7, s) == 1


def test_other_entry_argument_checks(world):
    c, s, a, b = world[1], 0x1000, 0x2000, 0x3000
    assert hccl_amd.reduce_scatter(c, None, None, 0, DT.FP16, OP.SUM, None) == 0
    assert code_of(hccl_amd.reduce_scatter, c, a, b, 4, DT.FP16, OP.SUM, None) == 2
    assert code_of(hccl_amd.reduce_scatter, c, a, b, 4, DT.UINT8, OP.SUM, s) == 5
    assert hccl_amd.all_gather(c, None, None, 0, DT.UINT8, None) == 0
    assert code_of(hccl_amd.all_gather, c, a, None, 4, DT.UINT8, s) == 2
    assert code_of(hccl_amd.all_gather, c, a, b, 4, DT.INT128, s) == 5
    # AllGatherV
    z, cnt, dsp = [0, 0, 0, 0], [4, 4, 4, 4], [0, 4, 8, 12]
    assert hccl_amd.all_gather_v(c, None, 0, None, z, dsp, DT.FP16, s) == 0          # all-zero counts: no-op
    assert code_of(hccl_amd.all_gather_v, c, a, 4, a, cnt, dsp, DT.FP16, s) == 1     # in place rejected
    assert code_of(hccl_amd.all_gather_v, c, None, 4, b, cnt, dsp, DT.FP16, s) == 2
    assert code_of(hccl_amd.all_gather_v, c, a, 4, None, cnt, dsp, DT.FP16, s) == 2
    assert code_of(hccl_amd.all_gather_v, c, a, 4, b, cnt, [0, 2, 8, 12], DT.FP16, s) == 1   # overlap
    assert code_of(hccl_amd.all_gather_v, c, a, 4, b, cnt, [0, 4, 8, 2 ** 64 - 2], DT.FP16, s) == 1  # overflow
    assert code_of(hccl_amd.all_gather_v, c, a, 4, b, cnt, dsp, DT.FP16, None) == 2
    # AlltoAllV
    assert code_of(hccl_amd.all_to_all_v, c, a, cnt, dsp, DT.FP16, a, cnt, dsp, DT.FP16, s) == 1   # in place
    assert code_of(hccl_amd.all_to_all_v, c, None, cnt, dsp, DT.FP16, b, cnt, dsp, DT.FP16, s) == 2
    assert code_of(hccl_amd.all_to_all_v, c, a, cnt, dsp, DT.FP16, None, cnt, dsp, DT.FP16, s) == 2
    assert code_of(hccl_amd.all_to_all_v, c, a, cnt, dsp, DT.FP16, b, cnt, dsp, DT.INT128, s) == 5
    assert code_of(hccl_amd.all_to_all_v, c, a, [2 ** 40, 0, 0, 0], dsp, DT.FP16, b, cnt, dsp, DT.FP16, s) == 1


def test_rooted_and_v_entry_argument_checks(world):
    c, s, a, b = world[1], 0x1000, 0x2000, 0x3000
    cnt, dsp, z = [4, 4, 4, 4], [0, 4, 8, 12], [0, 0, 0, 0]
    # AlltoAll (reference all_to_all_v.cc:39-41, 475-515)
    assert hccl_amd.all_to_all(c, None, 0, DT.FP16, None, 0, DT.FP16, None) == 0          # both counts 0 wins
    assert code_of(hccl_amd.all_to_all, None, a, 4, DT.FP16, b, 4, DT.FP16, s) == 2
    assert code_of(hccl_amd.all_to_all, c, None, 4, DT.FP16, b, 4, DT.FP16, s) == 2
    assert code_of(hccl_amd.all_to_all, c, a, 4, DT.FP16, None, 4, DT.FP16, s) == 2
    assert code_of(hccl_amd.all_to_all, c, a, 4, DT.FP16, b, 5, DT.FP16, s) == 1          # counts differ
    assert code_of(hccl_amd.all_to_all, c, a, 4, DT.FP16, b, 4, DT.FP32, s) == 1          # types differ
    assert code_of(hccl_amd.all_to_all, c, a, 4, DT.FP16, b, 4, DT.FP16, None) == 2
    assert code_of(hccl_amd.all_to_all, c, a, 4, DT.FP16, a, 4, DT.FP16, s) == 1          # in place
    assert code_of(hccl_amd.all_to_all, c, a, 4, 99, b, 4, 99, s) == 1                    # unknown type: E_PARA here
    assert code_of(hccl_amd.all_to_all, c, a, 2 ** 40, DT.FP16, b, 2 ** 40, DT.FP16, s) == 1
    assert code_of(hccl_amd.all_to_all, c, a, 4, DT.INT128, b, 4, DT.INT128, s) == 5
    # AlltoAllVC (:153-209, 555-598)
    m = [1] * 16
    assert code_of(hccl_amd.all_to_all_vc, None, a, m, DT.FP16, b, DT.FP16, s) == 2
    assert code_of(hccl_amd.all_to_all_vc, c, a, m, DT.FP16, b, DT.FP16, None) == 2
    assert code_of(hccl_amd.all_to_all_vc, c, a, m, DT.FP16, a, DT.FP16, s) == 1          # in place
    assert code_of(hccl_amd.all_to_all_vc, c, a, [2 ** 40] + [1] * 15, DT.FP16, b, DT.FP16, s) == 1
    assert code_of(hccl_amd.all_to_all_vc, c, None, m, DT.FP16, b, DT.FP16, s) == 2       # row 1 is not all zero
    assert code_of(hccl_amd.all_to_all_vc, c, a, m, DT.FP16, None, DT.FP16, s) == 2
    assert code_of(hccl_amd.all_to_all_vc, c, a, m, DT.FP16, b, DT.INT128, s) == 5
    # ReduceScatterV (reduce_scatter_v.cc:48-79, 180-247)
    assert code_of(hccl_amd.reduce_scatter_v, c, a, cnt, dsp, b, 4, DT.FP16, OP.SUM, None) == 2
    assert code_of(hccl_amd.reduce_scatter_v, None, a, cnt, dsp, b, 4, DT.FP16, OP.SUM, s) == 2
    assert code_of(hccl_amd.reduce_scatter_v, c, a, cnt, dsp, None, 4, DT.FP16, OP.SUM, s) == 2
    assert hccl_amd.reduce_scatter_v(c, None, z, dsp, None, 0, DT.FP16, OP.SUM, s) == 0   # all-zero counts: no-op
    assert code_of(hccl_amd.reduce_scatter_v, c, None, cnt, dsp, b, 4, DT.FP16, OP.SUM, s) == 2
    assert code_of(hccl_amd.reduce_scatter_v, c, a, cnt, dsp, b, 2 ** 40, DT.FP16, OP.SUM, s) == 1
    for bad in (DT.UINT64, DT.FP64, DT.UINT8, DT.INT128, DT.HIF8):
        assert code_of(hccl_amd.reduce_scatter_v, c, a, cnt, dsp, b, 4, bad, OP.SUM, s) == 5
    assert code_of(hccl_amd.reduce_scatter_v, c, a, cnt, dsp, b, 4, DT.BFP16, OP.PROD, s) == 5
    # Reduce (reduce.cc:39, 106-153)
    assert hccl_amd.reduce(c, None, None, 0, DT.FP32, OP.SUM, 9, None) == 0
    assert code_of(hccl_amd.reduce, None, a, b, 4, DT.FP32, OP.SUM, 0, s) == 2
    assert code_of(hccl_amd.reduce, c, None, b, 4, DT.FP32, OP.SUM, 0, s) == 2
    assert code_of(hccl_amd.reduce, c, a, None, 4, DT.FP32, OP.SUM, 0, s) == 2
    assert code_of(hccl_amd.reduce, c, a, b, 4, DT.FP32, OP.SUM, 0, None) == 2
    assert code_of(hccl_amd.reduce, c, a, b, 2 ** 40, DT.FP32, OP.SUM, 0, s) == 1
    assert code_of(hccl_amd.reduce, c, a, b, 4, DT.UINT32, OP.SUM, 0, s) == 5
    assert code_of(hccl_amd.reduce, c, a, b, 4, DT.INT16, OP.PROD, 0, s) == 5
    assert code_of(hccl_amd.reduce, c, a, b, 4, DT.FP32, OP.SUM, 4, s) == 1               # root outside the world
    # Broadcast (broadcast.cc:38, 99-142)
    assert hccl_amd.broadcast(c, None, 0, DT.FP32, 9, None) == 0
    assert code_of(hccl_amd.broadcast, None, a, 4, DT.FP32, 0, s) == 2
    assert code_of(hccl_amd.broadcast, c, None, 4, DT.FP32, 0, s) == 2
    assert code_of(hccl_amd.broadcast, c, a, 4, DT.FP32, 0, None) == 2
    assert code_of(hccl_amd.broadcast, c, a, 4, DT.FP32, 4, s) == 1
    assert code_of(hccl_amd.broadcast, c, a, 2 ** 40, DT.FP32, 0, s) == 1
    assert code_of(hccl_amd.broadcast, c, a, 4, DT.INT128, 0, s) == 5
    # Scatter (scatter.cc:59-73)
    assert hccl_amd.scatter(c, None, None, 0, DT.FP32, 9, None) == 0
    assert code_of(hccl_amd.scatter, None, a, b, 4, DT.FP32, 0, s) == 2
    assert code_of(hccl_amd.scatter, c, a, None, 4, DT.FP32, 0, s) == 2
    assert code_of(hccl_amd.scatter, c, None, b, 4, DT.FP32, 1, s) == 2                   # this rank is the root
    assert code_of(hccl_amd.scatter, c, a, b, 4, DT.FP32, 4, s) == 1
    assert code_of(hccl_amd.scatter, c, a, b, 2 ** 40, DT.FP32, 0, s) == 1
    assert code_of(hccl_amd.scatter, c, a, b, 4, DT.INT128, 0, s) == 5
    assert code_of(hccl_amd.scatter, c, a, b, 4, DT.FP32, 0, None) == 2


def test_barrier_argument_checks(world):
    assert code_of(hccl_amd.barrier, world[0], None) == 2
    assert code_of(hccl_amd.barrier, None, 0x1000) == 2


def test_point_to_point_argument_checks(world):
    c, s, a = world[0], 0x1000, 0x2000
    # reference send.cc:33-38, 136-163 / recv.cc likewise: nothing to move is a success before any other check
    assert code_of(hccl_amd.send, c, None, 0, DT.FP32, 1, None) == 0
    assert code_of(hccl_amd.recv, c, None, 0, DT.FP32, 1, None) == 0
    assert code_of(hccl_amd.send, c, a, 4, DT.FP32, 1, None) == 2
    assert code_of(hccl_amd.send, None, a, 4, DT.FP32, 1, s) == 2
    assert code_of(hccl_amd.send, c, None, 4, DT.FP32, 1, s) == 2
    assert code_of(hccl_amd.recv, c, None, 4, DT.FP32, 1, s) == 2
    assert code_of(hccl_amd.send, c, a, 0x800000000, DT.FP32, 1, s) == 1
    assert code_of(hccl_amd.send, c, a, 4, DT.INT128, 1, s) == 5
    assert code_of(hccl_amd.send, c, a, 4, DT.FP32, 0, s) == 5              # to itself
    assert code_of(hccl_amd.recv, c, a, 4, DT.FP32, 0, s) == 5
    assert code_of(hccl_amd.send, c, a, 4, DT.FP32, 4, s) == 1              # no such rank
    assert code_of(hccl_amd.recv, c, a, 4, DT.FP32, 99, s) == 1
    # batch_send_recv.cc:34-60 and ins_v2_batch_send_recv_executor.cc:143-200
    item = hccl_amd.make_send_recv_item
    T = hccl_amd.HcclSendRecvType
    assert code_of(hccl_amd.batch_send_recv, c, [], None) == 0
    assert code_of(hccl_amd.batch_send_recv, c, [item(T.SEND, a, 4, DT.FP32, 1)], None) == 2
    assert code_of(hccl_amd.batch_send_recv, None, [item(T.SEND, a, 4, DT.FP32, 1)], s) == 2
    assert code_of(hccl_amd.batch_send_recv, c, [item(T.SEND, a, 0x800000000, DT.FP32, 1)], s) == 1
    assert code_of(hccl_amd.batch_send_recv, c, [item(T.SEND, a, 4, DT.INT128, 1)], s) == 5
    assert code_of(hccl_amd.batch_send_recv, c, [item(T.SEND, a, 4, DT.FP32, 4)], s) == 1
    assert code_of(hccl_amd.batch_send_recv, c, [item(T.SEND, None, 4, DT.FP32, 1)], s) == 2
    assert code_of(hccl_amd.batch_send_recv, c, [item(2, a, 4, DT.FP32, 1)], s) == 1
    assert code_of(hccl_amd.batch_send_recv, c, [item(T.SEND, a, 4, DT.FP32, 0)], s) == 1    # own rank, no receive
    assert code_of(hccl_amd.batch_send_recv, c, [item(T.SEND, None, 0, DT.FP32, 1)], s) == 0  # nothing to move
    with pytest.raises(TypeError):
        hccl_amd.batch_send_recv(c, [object()], s)


def test_a_send_whose_peer_never_receives_times_out(monkeypatch):
    monkeypatch.setenv("HCCL_EXEC_TIMEOUT", "1")
    comms = hccl_amd.comm_init_all(2)
    try:
        assert code_of(hccl_amd.send, comms[0], 0x2000, 8, DT.FP32, 1, 0x1000) == 9
        # the late receive finds the verdict: nothing is copied
        assert code_of(hccl_amd.recv, comms[1], 0x3000, 8, DT.FP32, 0, 0x1000) == 9
    finally:
        for c in comms:
            hccl_amd.comm_destroy(c)


def test_unparsable_hccl_deterministic_fails_every_collective(monkeypatch):
    # reference alg_env_config.cc:1113-1125: anything but true / false / strict is HCCL_E_PARA at the entry point
    monkeypatch.setenv("HCCL_DETERMINISTIC", "maybe")
    comms = hccl_amd.comm_init_all(2)
    try:
        assert code_of(hccl_amd.all_reduce, comms[0], 0x2000, 0x3000, 8, DT.FP32, OP.SUM, 0x1000) == 1
        assert code_of(hccl_amd.all_gather, comms[1], 0x2000, 0x3000, 8, DT.FP32, 0x1000) == 1
    finally:
        for c in comms:
            hccl_amd.comm_destroy(c)


def test_staging_buffer_size_knob_and_environment(monkeypatch):
    monkeypatch.delenv("HCCL_BUFFSIZE", raising=False)
    comms = hccl_amd.comm_init_all(2)
    try:
        assert hccl_amd.get_ccl_buffer_size(comms[0]) == 0                 # unset: one loop
        hccl_amd.set_ccl_buffer_size(comms[1], 65536)
        assert hccl_amd.get_ccl_buffer_size(comms[0]) == 65536             # a property of the world
    finally:
        for c in comms:
            hccl_amd.comm_destroy(c)
    # the reference's own known answers (test/ut/op_graph_utils/hccl_op_utils_test.cc:287-296)
    for env, want in (("100", 99 << 20), ("2048", 2047 << 20)):
        monkeypatch.setenv("HCCL_BUFFSIZE", env)
        comms = hccl_amd.comm_init_all(2)
        try:
            assert hccl_amd.get_ccl_buffer_size(comms[0]) == want
        finally:
            for c in comms:
                hccl_amd.comm_destroy(c)
    for env in ("abc", "-5", "0", "1", "12x", "4294967296"):              # :299-307
        monkeypatch.setenv("HCCL_BUFFSIZE", env)
        comms = hccl_amd.comm_init_all(2)
        try:
            assert code_of(hccl_amd.all_reduce, comms[0], 0x2000, 0x3000, 8, DT.FP32, OP.SUM, 0x1000) == 1, env
        finally:
            for c in comms:
                hccl_amd.comm_destroy(c)


def test_a_rank_whose_peers_never_call_times_out(monkeypatch):
    import time
    monkeypatch.setenv("HCCL_EXEC_TIMEOUT", "1")
    comms = hccl_amd.comm_init_all(2)
    try:
        t0 = time.perf_counter()
        assert code_of(hccl_amd.all_reduce, comms[0], 0x2000, 0x3000, 8, DT.FP32, OP.SUM, 0x1000) == 9   # HCCL_E_TIMEOUT
        assert 0.9 < time.perf_counter() - t0 < 5.0
        # the late peer completes the set: the collective is not launched, both sides learn about the time-out
        assert code_of(hccl_amd.all_reduce, comms[1], 0x2000, 0x3000, 8, DT.FP32, OP.SUM, 0x1000) == 9
    finally:
        for c in comms:
            hccl_amd.comm_destroy(c)


def test_calls_that_disagree_are_rejected_without_a_launch():
    comms = hccl_amd.comm_init_all(3)
    try:
        cases = [
            lambda r: hccl_amd.all_reduce(comms[r], 0x2000, 0x3000, 8 if r < 2 else 9, DT.FP32, OP.SUM, 0x1000),
            lambda r: hccl_amd.all_reduce(comms[r], 0x2000, 0x3000, 8, DT.FP32 if r < 2 else DT.FP16, OP.SUM, 0x1000),
            lambda r: hccl_amd.all_reduce(comms[r], 0x2000, 0x3000, 8, DT.FP32, OP.SUM if r < 2 else OP.MAX, 0x1000),
            lambda r: hccl_amd.reduce(comms[r], 0x2000, 0x3000, 8, DT.FP32, OP.SUM, 0 if r < 2 else 1, 0x1000),
            lambda r: (hccl_amd.all_reduce if r < 2 else hccl_amd.reduce_scatter)(comms[r], 0x2000, 0x3000, 8, DT.FP32,
                                                                                 OP.SUM, 0x1000),
        ]
        for case in cases:
            hccl_amd.group_start()
            codes = [code_of(case, r) for r in range(3)]
            assert codes == [0, 0, 1], codes          # the call that completes the set reports HCCL_E_PARA
            assert code_of(hccl_amd.group_end) == 1   # and the group's end reports it for the queued calls
    finally:
        for c in comms:
            hccl_amd.comm_destroy(c)


def test_group_end_without_start():
    assert code_of(hccl_amd.group_end) == 1


# ---- lifetime of handles, groups over several threads, rejected calls --------------------------------------------
FAKE_STREAM = 0x1000


def test_calls_on_a_destroyed_communicator_are_rejected():
    """A handle that was destroyed (its world possibly freed) is refused, not dereferenced."""
    comms = hccl_amd.comm_init_all(2)
    for c in comms:
        hccl_amd.comm_destroy(c)
    for c in comms:
        assert code_of(hccl_amd.comm_destroy, c) == 1                      # double destroy
        assert code_of(hccl_amd.get_rank_size, c) == 1
        assert code_of(hccl_amd.get_rank_id, c) == 1
        assert code_of(hccl_amd.all_reduce, c, 0x2000, 0x3000, 8, DT.FP32, OP.SUM, FAKE_STREAM) == 1
        assert code_of(hccl_amd.reduce_scatter, c, 0x2000, 0x3000, 8, DT.FP32, OP.SUM, FAKE_STREAM) == 1
        assert code_of(hccl_amd.all_gather, c, 0x2000, 0x3000, 8, DT.FP32, FAKE_STREAM) == 1
        assert code_of(hccl_amd.all_to_all_v, c, 0x2000, [1, 1], [0, 1], DT.FP32, 0x3000, [1, 1], [0, 1], DT.FP32,
                       FAKE_STREAM) == 1
        assert code_of(hccl_amd.barrier, c, FAKE_STREAM) == 1
        assert code_of(hccl_amd.send, c, 0x2000, 8, DT.FP32, 1, FAKE_STREAM) == 1
        assert code_of(hccl_amd.set_algo, c, OpKind.ALL_REDUCE, Algo.MESH) == 1
    assert code_of(hccl_amd.get_rank_size, ctypes.c_void_p(0x1234560)) == 1    # never issued


def test_a_live_rank_learns_that_a_peer_left():
    """Rank 0 waits in a collective; rank 1 destroys its communicator instead of joining: rank 0 wakes at once
    with an error, and nothing else runs in that world."""
    import threading
    import time
    comms = hccl_amd.comm_init_all(2)
    got = {}

    def waiter():
        t0 = time.perf_counter()
        got["code"] = code_of(hccl_amd.barrier, comms[0], FAKE_STREAM)
        got["seconds"] = time.perf_counter() - t0

    th = threading.Thread(target=waiter, daemon=True)
    th.start()
    time.sleep(0.3)
    assert th.is_alive()                                         # parked, waiting for rank 1
    hccl_amd.comm_destroy(comms[1])
    th.join(10)
    assert not th.is_alive()
    assert got["code"] == 7 and got["seconds"] < 5               # HCCL_E_UNAVAIL, long before the time-out
    assert code_of(hccl_amd.barrier, comms[0], FAKE_STREAM) == 7
    hccl_amd.comm_destroy(comms[0])
    assert code_of(hccl_amd.barrier, comms[0], FAKE_STREAM) == 1


def test_point_to_point_calls_after_a_peer_left_return_at_once():
    """A send, a receive or a batch towards a rank that has destroyed its communicator can never be completed: the
    call returns HCCL_E_UNAVAIL instead of waiting for the execution time-out."""
    import time
    comms = hccl_amd.comm_init_all(3)
    hccl_amd.comm_destroy(comms[2])
    t0 = time.perf_counter()
    assert code_of(hccl_amd.send, comms[0], 0x2000, 8, DT.FP32, 1, FAKE_STREAM) == 7
    assert code_of(hccl_amd.recv, comms[1], 0x2000, 8, DT.FP32, 0, FAKE_STREAM) == 7
    items = [hccl_amd.make_send_recv_item(hccl_amd.HcclSendRecvType.SEND, 0x2000, 8, DT.FP32, 1),
             hccl_amd.make_send_recv_item(hccl_amd.HcclSendRecvType.RECV, 0x3000, 8, DT.FP32, 2)]
    assert code_of(hccl_amd.batch_send_recv, comms[0], items, FAKE_STREAM) == 7
    assert time.perf_counter() - t0 < 5
    for c in comms[:2]:
        hccl_amd.comm_destroy(c)


def test_two_threads_each_grouping_half_of_the_ranks():
    """Every HcclGroupEnd returns only when the calls its thread queued are complete, whichever thread completed
    the set (a barrier over one stream launches nothing, so this runs without a GPU)."""
    import threading
    comms = hccl_amd.comm_init_all(4)
    codes = [None, None]
    try:
        def half(k):
            try:
                for _ in range(50):
                    with hccl_amd.group():
                        for r in (2 * k, 2 * k + 1):
                            hccl_amd.barrier(comms[r], FAKE_STREAM)
                codes[k] = 0
            except hccl_amd.HcclError as e:
                codes[k] = e.code

        ths = [threading.Thread(target=half, args=(k,), daemon=True) for k in range(2)]
        for th in ths:
            th.start()
        for th in ths:
            th.join(30)
            assert not th.is_alive()
        assert codes == [0, 0]
    finally:
        for c in comms:
            hccl_amd.comm_destroy(c)


def test_a_group_that_is_never_completed_ends_with_a_time_out(monkeypatch):
    import time
    monkeypatch.setenv("HCCL_EXEC_TIMEOUT", "1")
    comms = hccl_amd.comm_init_all(3)
    monkeypatch.delenv("HCCL_EXEC_TIMEOUT")
    try:
        hccl_amd.group_start()
        assert code_of(hccl_amd.barrier, comms[0], FAKE_STREAM) == 0      # queued
        assert code_of(hccl_amd.barrier, comms[1], FAKE_STREAM) == 0      # queued; rank 2 never calls
        t0 = time.perf_counter()
        assert code_of(hccl_amd.group_end) == 9                           # HCCL_E_TIMEOUT
        assert 0.9 < time.perf_counter() - t0 < 8.0
        # the late rank completes the set and finds the verdict
        assert code_of(hccl_amd.barrier, comms[2], FAKE_STREAM) == 9
        # nested groups: only the outermost end waits and reports
        hccl_amd.group_start()
        hccl_amd.group_start()
        for r in range(3):
            assert code_of(hccl_amd.barrier, comms[r], FAKE_STREAM) == 0
        assert code_of(hccl_amd.group_end) == 0
        assert code_of(hccl_amd.group_end) == 0
    finally:
        for c in comms:
            hccl_amd.comm_destroy(c)


def test_a_rejected_call_keeps_its_place_in_the_sequence():
    """Rank 1's AllReduce fails its argument checks: rank 0, already waiting in that collective, wakes with the
    same code instead of waiting for the time-out, and the next collective pairs up as usual."""
    import threading
    import time
    comms = hccl_amd.comm_init_all(2)
    got = {}
    try:
        def waiter():
            t0 = time.perf_counter()
            got["code"] = code_of(hccl_amd.all_reduce, comms[0], 0x2000, 0x3000, 8, DT.FP32, OP.SUM, FAKE_STREAM)
            got["seconds"] = time.perf_counter() - t0

        th = threading.Thread(target=waiter, daemon=True)
        th.start()
        time.sleep(0.3)
        assert code_of(hccl_amd.all_reduce, comms[1], None, 0x3000, 8, DT.FP32, OP.SUM, FAKE_STREAM) == 2   # HCCL_E_PTR
        th.join(10)
        assert not th.is_alive() and got["code"] == 2 and got["seconds"] < 5
        # the other way round: the rejected call comes first, the valid one finds the verdict
        assert code_of(hccl_amd.all_reduce, comms[0], 0x2000, 0x3000, 8, DT.UINT8, OP.SUM, FAKE_STREAM) == 5   # NOT_SUPPORT
        assert code_of(hccl_amd.all_reduce, comms[1], 0x2000, 0x3000, 8, DT.FP32, OP.SUM, FAKE_STREAM) == 5
        with hccl_amd.group():                                   # the numbering is intact
            for c in comms:
                hccl_amd.barrier(c, FAKE_STREAM)
    finally:
        for c in comms:
            hccl_amd.comm_destroy(c)


def test_stuck_counters_are_unavailable_unless_enabled(monkeypatch):
    monkeypatch.delenv("HCCL_AMD_STUCK_COUNTERS", raising=False)
    comms = hccl_amd.comm_init_all(2)
    try:
        assert code_of(hccl_amd.get_stuck_counters, comms[0]) == 7          # HCCL_E_UNAVAIL
    finally:
        for c in comms:
            hccl_amd.comm_destroy(c)
    assert code_of(hccl_amd.get_stuck_counters, comms[0]) == 1              # stale handle
