"""CPU tier: the two-level AllReduce and ReduceScatter orders (level-0 groups, reference
ins_v2_all_reduce_sequence_executor_aicpu.cc:592-852, ins_v2_reduce_scatter_sequence_executor_aicpu.cc:298-500) and the reading of the reference's HCCL_ALGO setting.

The oracle's two-level function is pinned by what does not depend on it: with one rank per group it must be the
(already pinned) one-level RHD / NHR oracle, with one group the own-first mesh order, integer sums must equal plain
modular sums, and on small worlds it must equal expression trees written out by hand from the reference's step
rules.  The library's fold programs are then evaluated with numpy against it.  The parser is checked against the
cases of the reference's own unit test (test/ut/common/alg_parse/alg_parse_test.cc), transcribed as data."""
import numpy as np
import pytest

import hccl_amd
from hccl_amd import Algo, OpKind

from test_host_plan import f32_fold, program_ranks, run_program, same, tricky, wide

F32, I32, F16 = 4, 2, 3
SUM, PROD, MAX, MIN = range(4)
L1 = {"rhd": Algo.RHD, "nhr": Algo.NHR, "mesh": Algo.MESH}
SHAPES = [(2, 3), (2, 4), (4, 2), (3, 2), (2, 6), (3, 5), (8, 8), (2, 2), (5, 3)]


# ---- the oracle against what is known without it ----------------------------------------------------
@pytest.mark.parametrize("p", [2, 3, 5, 6, 7, 8, 12])
def test_one_rank_per_group_is_the_one_level_order(orc, p):
    rng = np.random.default_rng(31 * p)
    for count in (p * 7, p * 7 + 3, 1, p - 1 if p > 1 else 1):
        for op, gen in ((SUM, wide), (MAX, tricky)):
            ins = gen(rng, p, count)
            for algo in ("rhd", "nhr"):
                want = [np.zeros(count, np.float32) for _ in range(p)]
                got = [np.zeros(count, np.float32) for _ in range(p)]
                assert orc.all_reduce(ins, want, count, F32, op, algo=algo) == 0
                assert orc.all_reduce_two_level(ins, got, count, F32, op, 1, algo) == 0
                for r in range(p):
                    assert same(got[r], want[r]), (p, count, op, algo, r)


@pytest.mark.parametrize("n", [2, 3, 4, 8])
def test_one_group_is_the_own_first_mesh_order(orc, n):
    """All ranks in one group: chunk i is folded by member i, its own input first, the others ascending; with a count
    that is a multiple of n that is the symmetric two-shot order, slice by slice."""
    rng = np.random.default_rng(17 * n)
    count = n * 9
    for op, gen in ((SUM, wide), (MIN, tricky)):
        ins = gen(rng, n, count)
        want = [np.zeros(count, np.float32) for _ in range(n)]
        assert orc.all_reduce(ins, want, count, F32, op, algo="mesh_symmetric") == 0
        for level1 in ("nhr", "mesh", "rhd"):
            got = [np.zeros(count, np.float32) for _ in range(n)]
            assert orc.all_reduce_two_level(ins, got, count, F32, op, n, level1) == 0
            for r in range(n):
                assert same(got[r], want[r]), (n, op, level1, r)


@pytest.mark.parametrize("l0,l1", SHAPES)
def test_every_rank_counts_exactly_once(orc, l0, l1):
    """int32 SUM of distinct powers of two per rank (n <= 30) or plain modular sums: order does not matter, every
    contribution must be there once, whatever the count leaves over."""
    n = l0 * l1
    rng = np.random.default_rng(5 * n + l0)
    for count in (n * 4, n * 4 + 1, n * 4 + n - 1, 3, 1):
        ins = [rng.integers(-2 ** 31, 2 ** 31, count, dtype=np.int64).astype(np.int32) for _ in range(n)]
        want = np.zeros(count, dtype=np.int64)
        for x in ins:
            want += x
        want = want.astype(np.int32)   # wraps
        for level1 in ("rhd", "nhr", "mesh"):
            got = [np.zeros(count, np.int32) for _ in range(n)]
            assert orc.all_reduce_two_level(ins, got, count, I32, SUM, l0, level1) == 0
            for r in range(n):
                assert np.array_equal(got[r], want), (l0, l1, count, level1, r)


def box(ins, l0, b, i, lo, hi, op):
    """What group b folds for chunk member i over elements [lo, hi): own input first, the others ascending."""
    acc = ins[b * l0 + i][lo:hi]
    for t in range(l0):
        if t != i:
            acc = f32_fold(ins[b * l0 + t][lo:hi], acc, op)
    return acc


def test_two_groups_of_three_and_three_groups_of_two_by_hand(orc):
    """Written out from the reference's step rules.
    RHD over 3 groups (template_utils.cc:117-208): r = 1, pair (0, 1), group 0 represents; PRE: group 1 is folded into
    group 0 on every unit; MAIN, one step: virtual rank 0 (group 0) keeps units 0 and 1 and receives group 2's, virtual
    rank 1 (group 2) keeps unit 2 and receives the pair's.  So units 0, 1 = B2 (+) (B1 (+) B0) with the pair as
    accumulator, unit 2 = (B1 (+) B0) (+) B2 with group 2 as accumulator.
    NHR over 2 groups (reduce_scatter_nhr.cc:458-506): one step, unit j stays at group j, the other group's share
    comes in: unit 0 = B1 (+) B0, unit 1 = B0 (+) B1 (accumulator written last)."""
    rng = np.random.default_rng(99)
    for op, gen in ((SUM, wide), (MAX, tricky), (MIN, tricky)):
        # 3 groups of 2 ranks, RHD between them; 36 elements: chunks of 18, units of 6
        l0, l1, count = 2, 3, 36
        ins = gen(rng, 6, count)
        got = [np.zeros(count, np.float32) for _ in range(6)]
        assert orc.all_reduce_two_level(ins, got, count, F32, op, l0, "rhd") == 0
        want = np.zeros(count, np.float32)
        for i in range(l0):
            for j in range(l1):
                lo = i * 18 + j * 6
                b = [box(ins, l0, g, i, lo, lo + 6, op) for g in range(l1)]
                pair = f32_fold(b[1], b[0], op)
                want[lo:lo + 6] = f32_fold(b[2], pair, op) if j < 2 else f32_fold(pair, b[2], op)
        for r in range(6):
            assert same(got[r], want), ("rhd", op, r)
        # 2 groups of 3 ranks, NHR between them; 31 elements: chunks 10, 10, 11; units 5 + 5 and 5 + 6
        l0, l1, count = 3, 2, 31
        ins = gen(rng, 6, count)
        got = [np.zeros(count, np.float32) for _ in range(6)]
        assert orc.all_reduce_two_level(ins, got, count, F32, op, l0, "nhr") == 0
        want = np.zeros(count, np.float32)
        for i, (lo, ln) in enumerate(((0, 10), (10, 10), (20, 11))):
            for j, (ulo, uhi) in enumerate(((lo, lo + 5), (lo + 5, lo + ln))):
                b = [box(ins, l0, g, i, ulo, uhi, op) for g in range(l1)]
                want[ulo:uhi] = f32_fold(b[1 - j], b[j], op)
        for r in range(6):
            assert same(got[r], want), ("nhr", op, r)
        # the host-reduce fold between 3 groups of 2: unit j starts from group j, the others ascending
        l0, l1, count = 2, 3, 13
        ins = gen(rng, 6, count)
        got = [np.zeros(count, np.float32) for _ in range(6)]
        assert orc.all_reduce_two_level(ins, got, count, F32, op, l0, "mesh") == 0
        want = np.zeros(count, np.float32)
        for i, (lo, ln) in enumerate(((0, 6), (6, 7))):
            unit = ln // 3
            for j in range(3):
                ulo, uhi = lo + j * unit, (lo + ln if j == 2 else lo + (j + 1) * unit)
                acc = box(ins, l0, j, i, ulo, uhi, op)
                for g in range(3):
                    if g != j:
                        acc = f32_fold(box(ins, l0, g, i, ulo, uhi, op), acc, op)
                want[ulo:uhi] = acc
        for r in range(6):
            assert same(got[r], want), ("mesh", op, r)


def test_loops_cut_the_count_like_the_executor(orc):
    """A bounded staging buffer: loops of maxCountPerLoop floored to a multiple of n, each sliced afresh; equal to
    running the collective loop by loop."""
    rng = np.random.default_rng(7)
    l0, l1 = 2, 3
    n, count, per_loop = 6, 100, 40          # 36 + 36 + 28
    ins = wide(rng, n, count)
    for level1 in ("rhd", "nhr"):
        got = [np.zeros(count, np.float32) for _ in range(n)]
        assert orc.all_reduce_two_level(ins, got, count, F32, SUM, l0, level1, max_count_per_loop=per_loop) == 0
        want = np.zeros(count, np.float32)
        pieces = ((0, 36), (36, 72), (72, 100)) if level1 == "nhr" else ((0, 36), (36, 72), (72, 96), (96, 100))
        for lo, hi in pieces:
            part = [x[lo:hi].copy() for x in ins]
            out = [np.zeros(hi - lo, np.float32) for _ in range(n)]
            assert orc.all_reduce_two_level(part, out, hi - lo, F32, SUM, l0, level1) == 0
            want[lo:hi] = out[0]
        assert same(got[3], want), level1


# ---- the library's programs against the oracle ---------------------------------------------------------
@pytest.mark.parametrize("l0,l1", SHAPES)
@pytest.mark.parametrize("level1", ["rhd", "nhr", "mesh"])
def test_two_level_programs_match_oracle(orc, l0, l1, level1):
    n = l0 * l1
    progs = hccl_amd.fold_programs(OpKind.ALL_REDUCE, L1[level1], n, level0=l0)
    assert len(progs) == n
    for prog in progs:
        assert sorted(program_ranks(prog)) == list(range(n)) and len(prog) <= 320
    for count in (n * 3, n * 3 + 5, 2):
        for op, gen in ((SUM, wide), (MAX, tricky)):
            rng = np.random.default_rng(1000 * n + 10 * l0 + op)
            ins = gen(rng, n, count)
            outs = [np.zeros(count, np.float32) for _ in range(n)]
            assert orc.all_reduce_two_level(ins, outs, count, F32, op, l0, level1) == 0
            got = np.zeros(count, np.float32)
            if level1 == "rhd":
                unit = count // n
                for u in range(n):
                    lo, hi = u * unit, (u + 1) * unit
                    if hi > lo:
                        got[lo:hi] = run_program(progs[u], lambda r: ins[r][lo:hi], op)
                for e in range(unit * n, count):
                    got[e:e + 1] = run_program(progs[e - unit * n], lambda r: ins[r][e:e + 1], op)
            else:
                chunk = count // l0
                for i in range(l0):
                    clo = i * chunk
                    chi = count if i == l0 - 1 else clo + chunk
                    unit = (chi - clo) // l1
                    for j in range(l1):
                        lo, hi = clo + j * unit, (chi if j == l1 - 1 else clo + (j + 1) * unit)
                        if hi > lo:
                            got[lo:hi] = run_program(progs[i * l1 + j], lambda r: ins[r][lo:hi], op)
            assert same(got, outs[0]), (l0, l1, level1, count, op)


def test_groups_must_divide_the_world():
    with pytest.raises(hccl_amd.HcclError) as e:
        hccl_amd.fold_programs(OpKind.ALL_REDUCE, Algo.RHD, 6, level0=4)
    assert e.value.code == 1
    # Reduce over groups runs the AllReduce's steps and hands the root the result
    assert hccl_amd.fold_programs(OpKind.REDUCE, Algo.MESH, 6, level0=2) == hccl_amd.fold_programs(
        OpKind.ALL_REDUCE, Algo.MESH, 6, level0=2)
    with pytest.raises(hccl_amd.HcclError) as e:
        hccl_amd.fold_programs(OpKind.REDUCE_SCATTER, Algo.ORDER_PRESERVED, 6, level0=2)
    assert e.value.code == 5
    # one rank per group, or all ranks in one: the one-level programs
    assert hccl_amd.fold_programs(OpKind.ALL_REDUCE, Algo.RHD, 6, level0=1) == hccl_amd.fold_programs(
        OpKind.ALL_REDUCE, Algo.RHD, 6)
    assert hccl_amd.fold_programs(OpKind.ALL_REDUCE, Algo.NHR, 6, level0=6) == hccl_amd.fold_programs(
        OpKind.ALL_REDUCE, Algo.NHR, 6)


# ---- two-level ReduceScatter (reference ins_v2_reduce_scatter_sequence_executor_aicpu.cc:298-500) ---------------
@pytest.mark.parametrize("p", [2, 3, 5, 6, 7, 8, 12])
def test_reduce_scatter_with_one_rank_per_group_is_the_one_level_order(orc, p):
    rng = np.random.default_rng(41 * p)
    for c in (7, 1):
        for op, gen in ((SUM, wide), (MAX, tricky)):
            ins = gen(rng, p, p * c)
            for algo in ("rhd", "nhr"):
                want = [np.zeros(c, np.float32) for _ in range(p)]
                got = [np.zeros(c, np.float32) for _ in range(p)]
                assert orc.reduce_scatter(ins, want, c, F32, op, algo=algo) == 0
                assert orc.reduce_scatter_two_level(ins, got, c, F32, op, 1, algo) == 0
                for r in range(p):
                    assert same(got[r], want[r]), (p, c, op, algo, r)


@pytest.mark.parametrize("n", [2, 3, 4, 8])
def test_reduce_scatter_with_one_group_is_the_own_first_mesh_order(orc, n):
    rng = np.random.default_rng(19 * n)
    c = 9
    for op, gen in ((SUM, wide), (MIN, tricky)):
        ins = gen(rng, n, n * c)
        want = [np.zeros(c, np.float32) for _ in range(n)]
        assert orc.reduce_scatter(ins, want, c, F32, op, algo="mesh") == 0
        for level1 in ("nhr", "mesh", "rhd"):
            got = [np.zeros(c, np.float32) for _ in range(n)]
            assert orc.reduce_scatter_two_level(ins, got, c, F32, op, n, level1) == 0
            for r in range(n):
                assert same(got[r], want[r]), (n, op, level1, r)


@pytest.mark.parametrize("l0,l1", SHAPES)
def test_reduce_scatter_counts_every_rank_exactly_once(orc, l0, l1):
    n = l0 * l1
    rng = np.random.default_rng(7 * n + l0)
    for c in (5, 1):
        ins = [rng.integers(-2 ** 31, 2 ** 31, n * c, dtype=np.int64).astype(np.int32) for _ in range(n)]
        want = np.zeros(n * c, dtype=np.int64)
        for x in ins:
            want += x
        want = want.astype(np.int32)   # wraps
        for level1 in ("rhd", "nhr", "mesh"):
            got = [np.zeros(c, np.int32) for _ in range(n)]
            assert orc.reduce_scatter_two_level(ins, got, c, I32, SUM, l0, level1) == 0
            for r in range(n):
                assert np.array_equal(got[r], want[r * c:(r + 1) * c]), (l0, l1, c, level1, r)


def test_two_level_reduce_scatter_by_hand(orc):
    """The trees of test_two_groups_of_three_and_three_groups_of_two_by_hand, slice by slice: rank j * l0 + i receives
    slice j * l0 + i, folded inside every group with member i's input first and between the groups by the level-1
    template's tree for unit j."""
    rng = np.random.default_rng(98)
    c = 6
    for op, gen in ((SUM, wide), (MAX, tricky), (MIN, tricky)):
        l0, l1 = 2, 3
        ins = gen(rng, 6, 6 * c)
        got = [np.zeros(c, np.float32) for _ in range(6)]
        assert orc.reduce_scatter_two_level(ins, got, c, F32, op, l0, "rhd") == 0
        for r in range(6):
            j, i = divmod(r, l0)
            b = [box(ins, l0, g, i, r * c, (r + 1) * c, op) for g in range(l1)]
            pair = f32_fold(b[1], b[0], op)
            want = f32_fold(b[2], pair, op) if j < 2 else f32_fold(pair, b[2], op)
            assert same(got[r], want), ("rhd", op, r)
        l0, l1 = 3, 2
        got = [np.zeros(c, np.float32) for _ in range(6)]
        assert orc.reduce_scatter_two_level(ins, got, c, F32, op, l0, "nhr") == 0
        for r in range(6):
            j, i = divmod(r, l0)
            b = [box(ins, l0, g, i, r * c, (r + 1) * c, op) for g in range(l1)]
            assert same(got[r], f32_fold(b[1 - j], b[j], op)), ("nhr", op, r)
        l0, l1 = 2, 3
        got = [np.zeros(c, np.float32) for _ in range(6)]
        assert orc.reduce_scatter_two_level(ins, got, c, F32, op, l0, "mesh") == 0
        for r in range(6):
            j, i = divmod(r, l0)
            acc = box(ins, l0, j, i, r * c, (r + 1) * c, op)
            for g in range(3):
                if g != j:
                    acc = f32_fold(box(ins, l0, g, i, r * c, (r + 1) * c, op), acc, op)
            assert same(got[r], acc), ("mesh", op, r)


@pytest.mark.parametrize("l0,l1", SHAPES)
@pytest.mark.parametrize("level1", ["rhd", "nhr", "mesh"])
def test_two_level_reduce_scatter_programs_match_oracle(orc, l0, l1, level1):
    n = l0 * l1
    progs = hccl_amd.fold_programs(OpKind.REDUCE_SCATTER, L1[level1], n, level0=l0)
    assert len(progs) == n
    all_reduce = hccl_amd.fold_programs(OpKind.ALL_REDUCE, L1[level1], n, level0=l0)
    for r, prog in enumerate(progs):
        assert sorted(program_ranks(prog)) == list(range(n)) and len(prog) <= 320
        assert prog == all_reduce[(r % l0) * l1 + r // l0]      # sub-slice r / l0 of chunk r % l0 of the AllReduce
    for c in (3, 1):
        for op, gen in ((SUM, wide), (MAX, tricky)):
            rng = np.random.default_rng(2000 * n + 10 * l0 + op)
            ins = gen(rng, n, n * c)
            outs = [np.zeros(c, np.float32) for _ in range(n)]
            assert orc.reduce_scatter_two_level(ins, outs, c, F32, op, l0, level1) == 0
            for r in range(n):
                got = run_program(progs[r], lambda k: ins[k][r * c:(r + 1) * c], op)
                assert same(got, outs[r]), (l0, l1, level1, c, op, r)


# ---- HCCL_ALGO ---------------------------------------------------------------------------------------
# (config, normal form) from test/ut/common/alg_parse/alg_parse_test.cc:29-213, 266-330
ACCEPTED = [
    ("allreduce:sequence{mesh2die,nhrmultilink};sole{nhr};allgather:sequence{mesh,nhr,nhr};concur{mesh,nhrmultilink}; "
     "not(meshoneshot)",
     "allreduce:sequence{mesh2die,nhrmultilink};sole{nhr};allgather:sequence{mesh,nhr,nhr};concur{mesh,nhrmultilink};"
     "not(sole{meshoneshot})"),
    ("not(parallel{mesh,nhr});allgather:sequence{mesh,nhr};allreduce:not(sequence{mesh_multi_link,nhr})",
     "not(parallel{mesh,nhr});allgather:sequence{mesh,nhr};allreduce:not(sequence{meshmultilink,nhr})"),
    ("allgather:not(sequence{level0=mesh2die,level1=nhrmultilink}); concur{not(mesh),meshchunktwoshot};mesh_chunk",
     "allgather:not(sequence{mesh2die,nhrmultilink});concur{not(mesh),meshchunktwoshot};sole{meshchunk}"),
    ("mesh_concur;sequence{meshtwoshot,not(nhrmultilink)};allgather:sequence{mesh,nhr}",
     "sole{meshconcur};sequence{meshtwoshot,not(nhrmultilink)};allgather:sequence{mesh,nhr}"),
    ("mesh2die; sequence{meshchunk  ,not( nhrmultilink)};allgather:sequence{mesh, nhr}",
     "sole{mesh2die};sequence{meshchunk,not(nhrmultilink)};allgather:sequence{mesh,nhr}"),
    ("alltoall:sole{mesh}", "alltoall:sole{mesh}"),
    ("reducescatter:sequence{level0=meshchunkconcur,level1=nhr}", "reducescatter:sequence{meshchunkconcur,nhr}"),
    ("", ""),
    ("nhrmultilink;meshoneshot;mesh2die", "sole{nhrmultilink};sole{meshoneshot};sole{mesh2die}"),
    ("allreduce:sequence{mesh2die,not(nhrmultilink),not(meshchunktwoshot)}",
     "allreduce:sequence{mesh2die,not(nhrmultilink),not(meshchunktwoshot)}"),
    ("reducescatter:sole{level0=hdaicpureduce}", "reducescatter:sole{hdaicpureduce}"),
    ("reducescatter:parallel{level0=mesh,level1=hd}", "reducescatter:parallel{mesh,hd}"),
    ("hd;reducescatter:not(parallel{level0=mesh,level1=hd});sole{level0=not(hdaicpureduce)}",
     "sole{hd};reducescatter:not(parallel{mesh,hd});sole{not(hdaicpureduce)}"),
    # explicit levels out of order land in level order (alg_parse.cc:156-190)
    ("allreduce:sequence{level1=rhd,level0=mesh_concur}", "allreduce:sequence{meshconcur,rhd}"),
]
REJECTED = [
    "invalid_op:sole{meshchunk}",
    "not(parallel{mesh2die,nhrmultilink};allgather:sequence{mesh,nhr}",
    "allgather:not(sequence{level0=mesh2die,level1=nhrmultilink}); concur{not(mesh2die),nhr;meshchunk}",
    "allreduce:sole{invalid_algo}",
    "allreduce:invalid_exec{meshchunktwoshot}",
    "alltoall:sole{meshwrite}",
    "allreduce:sole{nhr",
    "allreduce:sole{nhr}}",
    "level0:NA;level1:H-D_R",      # the older syntax of the other device generation is not this parser's
]


@pytest.mark.parametrize("config,normal", ACCEPTED)
def test_hccl_algo_strings_the_reference_accepts(config, normal):
    text, _, _ = hccl_amd.select_from_hccl_algo(config, OpKind.ALL_REDUCE)
    assert text == normal


@pytest.mark.parametrize("config", REJECTED)
def test_hccl_algo_strings_the_reference_rejects(config):
    with pytest.raises(hccl_amd.HcclError) as e:
        hccl_amd.select_from_hccl_algo(config, OpKind.ALL_REDUCE)
    assert e.value.code == 1


def st_strings():
    import json
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_st_hccl_algo_strings.json")
    return [e["config"] for e in json.load(open(path))]


@pytest.mark.parametrize("config", st_strings())
def test_every_hccl_algo_string_of_the_reference_system_tests_parses(config):
    """The configurations the reference's own system tests run with (test/st/algorithm/testcase/*.cc, collected as
    data by tests/golden/make_reference_st_hccl_algo_strings.py) are valid for its parser; they are for this one, and
    their normal form names the same operator, executor and templates."""
    text, _, _ = hccl_amd.select_from_hccl_algo(config, OpKind.ALL_REDUCE)
    strip = lambda t: t.replace("level0=", "").replace("level1=", "").replace("level2=", "").replace("_", "")
    assert text == strip(config)


def test_what_the_system_tests_two_level_strings_select():
    sel = hccl_amd.select_from_hccl_algo
    AR, RS, RD = OpKind.ALL_REDUCE, OpKind.REDUCE_SCATTER, OpKind.REDUCE
    # all_reduce_testcase.cc:317-345, all_reduce_dpu_testcase.cc: level-0 mesh inside a server, RHD / NHR between them
    assert sel("allreduce:sequence{level0=meshconcur,level1=rhd}", AR)[1:] == (Algo.RHD, True)
    assert sel("allreduce:sequence{mesh,nhr}", AR)[1:] == (Algo.NHR, True)
    # mixed templates above level 0, pipelines and parallel executors are orders this library does not build:
    # nothing is selected
    assert sel("allreduce:sequence{meshconcur,nhr,mesh}", AR)[1] is None
    assert sel("allreduce:pipeline{mesh,nhr,nhr}", AR)[1] is None
    assert sel("reducescatter:parallel{level0=mesh,level1=hd}", RS)[1] is None
    assert sel("reduce:parallel{nhr,nhr}", RD)[1] is None
    # one level
    assert sel("reducescatter:sole{level0=hdaicpureduce}", RS)[1] == Algo.RHD
    assert sel("reduce:sole{meshtwoshot}", RD)[1] == Algo.MESH_TWO_SHOT
    assert sel("reduce:sole{mesh}", RD)[1] == Algo.MESH
    assert sel("reducescatter:sole{level0=not(nhr)}", RS)[1] is None


def test_what_hccl_algo_selects():
    sel = hccl_amd.select_from_hccl_algo
    AR, RS, RD = OpKind.ALL_REDUCE, OpKind.REDUCE_SCATTER, OpKind.REDUCE
    assert sel("allreduce:sequence{level0=mesh_concur,level1=rhd}", AR)[1:] == (Algo.RHD, True)
    assert sel("allreduce:sequence{mesh_concur,nhr}", AR)[1:] == (Algo.NHR, True)
    assert sel("allreduce:sequence{mesh,nhr_aicpu_reduce}", AR)[1:] == (Algo.MESH, True)
    assert sel("allreduce:sequence{mesh_concur,rhd}", RS)[1] is None          # names another operator
    assert sel("allreduce:sole{mesh_one_shot}", AR)[1:] == (Algo.MESH, False)
    assert sel("allreduce:mesh_two_shot", AR)[1:] == (Algo.MESH, False)
    assert sel("allreduce:sole{mesh_chunk_two_shot}", AR)[1] == Algo.MESH_CHUNK
    assert sel("allreduce:nhr_aicpu_reduce", AR)[1] == Algo.RING
    assert sel("reducescatter:nhr_aicpu_reduce", RS)[1] == Algo.MESH
    assert sel("reducescatter:sole{hd_aicpu_reduce}", RS)[1] == Algo.RHD
    assert sel("reducescatterv:sole{mesh_chunk}", RS)[1] == Algo.MESH_CHUNK
    assert sel("reduce:mesh_two_shot", RD)[1] == Algo.MESH_TWO_SHOT
    assert sel("reduce:sole{nhr}", RD)[1:] == (Algo.NHR, False)                # reduce_nhr.cc
    assert sel("strictordered{mesh}", AR)[1] == Algo.ORDER_PRESERVED
    assert sel("strictordered{mesh}", RD)[1] is None
    # a clause without an operator applies to all of them; later clauses are read first
    assert sel("nhr", AR)[1] == Algo.NHR and sel("nhr", RS)[1] == Algo.NHR and sel("nhr", RD)[1] == Algo.NHR
    assert sel("mesh_chunk", AR)[1] == Algo.MESH_CHUNK and sel("mesh_chunk", RD)[1] is None
    assert sel("allreduce:sole{nhr};sole{mesh}", AR)[1] == Algo.MESH
    assert sel("sole{mesh};allreduce:sole{nhr}", AR)[1] == Algo.NHR
    assert sel("sole{mesh};allreduce:sole{nhr}", RS)[1] == Algo.MESH
    # negations exclude in the reference and select nothing here; copies have no order
    assert sel("allreduce:not(sole{nhr})", AR)[1] is None
    assert sel("allreduce:sole{not(nhr)}", AR)[1] is None
    assert sel("allgather:sole{mesh};alltoall:pairwise", AR)[1] is None
    assert sel("allreduce:sequence{mesh,nhr,nhr}", AR)[1:] == (Algo.NHR, True)  # the same template at both upper levels
    # ReduceScatter in two levels: the same executor family (ins_v2_reduce_scatter_sequence_executor_aicpu.cc:567-640)
    assert sel("reducescatter:sequence{level0=meshconcur,level1=rhd}", RS)[1:] == (Algo.RHD, True)
    assert sel("reducescatter:sequence{mesh_concur,nhr}", RS)[1:] == (Algo.NHR, True)
    assert sel("reducescatter:sequence{mesh,nhr_aicpu_reduce}", RS)[1:] == (Algo.MESH, True)
    assert sel("reducescatter:sequence{level0=meshchunkconcur,level1=nhr}", RS)[1] is None   # mesh chunk inside the groups
    assert sel("reducescatter:sequence{mesh,mesh}", RS)[1] is None
    assert sel("allreduce:parallel{mesh,nhr}", AR)[1] is None                  # another executor, another order
    assert sel("allreduce:pipeline{mesh,nhr}", AR)[1] is None
