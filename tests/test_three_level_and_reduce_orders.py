"""CPU tier: the three-level AllReduce / ReduceScatter orders (reference
ins_v2_all_reduce_sequence_executor_aicpu_3level.cc, ins_v2_reduce_scatter_sequence_executor_3level.cc) and the
step-driven Reduce orders (reduce_nhr.cc; reduce_sequence_executor_aicpu_3level.cc over two and three levels).

The oracle's functions are pinned by what does not depend on them: a world whose level-1 groups hold every box, or
one box each, must give the (already pinned) two-level oracle's bits; integer sums must equal plain modular sums;
small worlds must equal expression trees written out by hand from the reference's step rules; the Reduce of the
sequence executors must equal the AllReduce's value unit by unit, and where its chunks are cut unevenly the value
of the same unit of an evenly cut run; NHR Reduce must equal the pinned NHR ReduceScatter slice by slice.  The loop
rule is checked on numbers worked out by hand.  The library's fold programs are then evaluated with numpy against
the oracle, and the reading of HCCL_ALGO for three templates and for Reduce is checked."""
import numpy as np
import pytest

import hccl_amd
from hccl_amd import Algo, OpKind

from test_host_plan import f32_fold, program_ranks, run_program, same, tricky, wide

F32, I32 = 4, 2
SUM, PROD, MAX, MIN = range(4)
ALGO = {"rhd": Algo.RHD, "nhr": Algo.NHR, "mesh": Algo.MESH}
SHAPES = [(2, 2, 2), (2, 3, 2), (3, 2, 2), (2, 2, 3), (2, 4, 2), (4, 2, 2), (2, 2, 4), (2, 3, 3), (3, 5, 2), (4, 4, 4)]


def cuts(lo, ln, dims):
    """(index tuple, lo, hi) of every unit when [lo, lo + ln) is cut level by level into floor(ln / d) elements with
    the rest in the last."""
    if not dims:
        yield (), lo, lo + ln
        return
    d = dims[0]
    c = ln // d
    for i in range(d):
        cur = c if i < d - 1 else ln - c * (d - 1)
        for idx, a, b in cuts(lo + i * c, cur, dims[1:]):
            yield (i,) + idx, a, b


# ---- the oracle against what is known without it ------------------------------------------------------------------
@pytest.mark.parametrize("l0,boxes", [(2, 3), (2, 4), (3, 2), (4, 2), (2, 6), (3, 5)])
def test_one_pod_or_one_box_per_pod_is_the_two_level_order(orc, l0, boxes):
    """Level-1 groups that hold every box leave nothing between the pods; level-1 groups of one box leave nothing
    inside them, and the pods are what the boxes were."""
    n = l0 * boxes
    rng = np.random.default_rng(11 * n + l0)
    for count in (n * 5, n * 5 + 3, n - 1, 1):
        for op, gen in ((SUM, wide), (MAX, tricky)):
            ins = gen(rng, n, count)
            for algo in ("rhd", "nhr"):
                want = [np.zeros(count, np.float32) for _ in range(n)]
                assert orc.all_reduce_two_level(ins, want, count, F32, op, l0, algo) == 0
                for l1 in (boxes, 1):
                    got = [np.zeros(count, np.float32) for _ in range(n)]
                    assert orc.all_reduce_three_level(ins, got, count, F32, op, l0, l1, algo) == 0
                    for r in range(n):
                        assert same(got[r], want[r]), (l0, boxes, l1, count, op, algo, r)
        c = count
        ins = wide(rng, n, n * c)
        for algo in ("rhd", "nhr"):
            want = [np.zeros(c, np.float32) for _ in range(n)]
            assert orc.reduce_scatter_two_level(ins, want, c, F32, SUM, l0, algo) == 0
            for l1 in (boxes, 1):
                got = [np.zeros(c, np.float32) for _ in range(n)]
                assert orc.reduce_scatter_three_level(ins, got, c, F32, SUM, l0, l1, algo) == 0
                for r in range(n):
                    assert same(got[r], want[r]), ("rs", l0, boxes, l1, c, algo, r)


@pytest.mark.parametrize("l0,l1,l2", SHAPES)
def test_every_rank_counts_exactly_once(orc, l0, l1, l2):
    n = l0 * l1 * l2
    rng = np.random.default_rng(7 * n + l1)
    for count in (n * 3, n * 3 + 1, n * 3 + n - 1, 3, 1):
        ins = [rng.integers(-2 ** 31, 2 ** 31, count, dtype=np.int64).astype(np.int32) for _ in range(n)]
        want = np.zeros(count, dtype=np.int64)
        for x in ins:
            want += x
        want = want.astype(np.int32)
        for algo in ("rhd", "nhr"):
            got = [np.zeros(count, np.int32) for _ in range(n)]
            assert orc.all_reduce_three_level(ins, got, count, I32, SUM, l0, l1, algo) == 0
            for r in range(n):
                assert np.array_equal(got[r], want), (l0, l1, l2, count, algo, r)
            got = [np.zeros(count, np.int32) for _ in range(n)]
            assert orc.reduce_levels(ins, got, count, I32, SUM, n - 1, l0, l1, algo) == 0
            assert np.array_equal(got[n - 1], want) and not got[0].any(), (l0, l1, l2, count, algo)
            got = [np.zeros(count, np.int32) for _ in range(n)]
            assert orc.reduce(ins, got, count, I32, SUM, 1 % n, algo="nhr") == 0
            assert np.array_equal(got[1 % n], want)
    c = 5
    ins = [rng.integers(-2 ** 31, 2 ** 31, n * c, dtype=np.int64).astype(np.int32) for _ in range(n)]
    total = np.zeros(n * c, dtype=np.int64)
    for x in ins:
        total += x
    total = total.astype(np.int32)
    for algo in ("rhd", "nhr"):
        got = [np.zeros(c, np.int32) for _ in range(n)]
        assert orc.reduce_scatter_three_level(ins, got, c, I32, SUM, l0, l1, algo) == 0
        for r in range(n):
            assert np.array_equal(got[r], total[r * c:(r + 1) * c]), (l0, l1, l2, algo, r)


def box(ins, l0, first, i, lo, hi, op):
    """What the box whose first rank is `first` folds for member i over [lo, hi): own input first, the others ascending."""
    acc = ins[first + i][lo:hi]
    for t in range(l0):
        if t != i:
            acc = f32_fold(ins[first + t][lo:hi], acc, op)
    return acc


def test_two_by_two_by_two_and_two_by_two_by_three_by_hand(orc):
    """NHR between two participants (reduce_scatter_nhr.cc:458-506): one step, unit u stays with participant u and the
    other one's share comes in, value = other (+) own.  Eight ranks as 2 x 2 x 2, 24 elements: chunks of 12,
    sub-slices of 6, parts of 3.  Part k of sub-slice j of chunk i: the pods hold V_g = box(g, 1 - j) (+) box(g, j),
    the result is V_(1-k) (+) V_k.
    RHD between three pods (template_utils.cc:117-208): r = 1, pods 0 and 1 pair, pod 0 represents; PRE folds pod 1
    into pod 0 on every unit; one MAIN step: units 0 and 1 = V_2 (+) (V_1 (+) V_0), unit 2 = (V_1 (+) V_0) (+) V_2.
    Twelve ranks as 2 x 2 x 3 under RHD: inside a pod RHD between two boxes is one step between powers of two: unit u
    stays with box u, value = box(1 - u) (+) box(u)."""
    rng = np.random.default_rng(2024)
    for op, gen in ((SUM, wide), (MAX, tricky), (MIN, tricky)):
        l0, l1, l2, count = 2, 2, 2, 24
        ins = gen(rng, 8, count)
        got = [np.zeros(count, np.float32) for _ in range(8)]
        assert orc.all_reduce_three_level(ins, got, count, F32, op, l0, l1, "nhr") == 0
        want = np.zeros(count, np.float32)
        for (i, j, k), lo, hi in cuts(0, count, [l0, l1, l2]):
            v = [f32_fold(box(ins, l0, (g * l1 + 1 - j) * l0, i, lo, hi, op), box(ins, l0, (g * l1 + j) * l0, i, lo, hi, op), op)
                 for g in range(l2)]
            want[lo:hi] = f32_fold(v[1 - k], v[k], op)
        for r in range(8):
            assert same(got[r], want), ("nhr", op, r)
        # uneven: 29 elements: chunks 14 + 15, sub-slices 7 + 7 and 7 + 8, parts 3 + 4 and, of the 8, 4 + 4
        count = 29
        ins = gen(rng, 8, count)
        got = [np.zeros(count, np.float32) for _ in range(8)]
        assert orc.all_reduce_three_level(ins, got, count, F32, op, l0, l1, "nhr") == 0
        bounds = [0, 3, 7, 10, 14, 17, 21, 25, 29]
        want = np.zeros(count, np.float32)
        for u in range(8):
            i, j, k = u >> 2, (u >> 1) & 1, u & 1
            lo, hi = bounds[u], bounds[u + 1]
            v = [f32_fold(box(ins, l0, (g * l1 + 1 - j) * l0, i, lo, hi, op), box(ins, l0, (g * l1 + j) * l0, i, lo, hi, op), op)
                 for g in range(l2)]
            want[lo:hi] = f32_fold(v[1 - k], v[k], op)
        assert same(got[5], want), ("nhr uneven", op)
        # 2 x 2 x 3 under RHD, 36 elements: chunks of 18, sub-slices of 9, parts of 3
        l0, l1, l2, count = 2, 2, 3, 36
        ins = gen(rng, 12, count)
        got = [np.zeros(count, np.float32) for _ in range(12)]
        assert orc.all_reduce_three_level(ins, got, count, F32, op, l0, l1, "rhd") == 0
        want = np.zeros(count, np.float32)
        for (i, j, k), lo, hi in cuts(0, count, [l0, l1, l2]):
            v = [f32_fold(box(ins, l0, (g * l1 + 1 - j) * l0, i, lo, hi, op), box(ins, l0, (g * l1 + j) * l0, i, lo, hi, op), op)
                 for g in range(l2)]
            pair = f32_fold(v[1], v[0], op)
            want[lo:hi] = f32_fold(v[2], pair, op) if k < 2 else f32_fold(pair, v[2], op)
        for r in range(12):
            assert same(got[r], want), ("rhd", op, r)
        # the same trees for ReduceScatter: rank (g * l1 + b) * l0 + i ends with part g of sub-slice b of chunk i
        c = 5
        ins = gen(rng, 12, 12 * c)
        got = [np.zeros(c, np.float32) for _ in range(12)]
        assert orc.reduce_scatter_three_level(ins, got, c, F32, op, l0, l1, "rhd") == 0
        for r in range(12):
            i, b, g = r % l0, r // l0 % l1, r // (l0 * l1)
            lo, hi = r * c, (r + 1) * c
            v = [f32_fold(box(ins, l0, (q * l1 + 1 - b) * l0, i, lo, hi, op), box(ins, l0, (q * l1 + b) * l0, i, lo, hi, op), op)
                 for q in range(l2)]
            pair = f32_fold(v[1], v[0], op)
            want = f32_fold(v[2], pair, op) if g < 2 else f32_fold(pair, v[2], op)
            assert same(got[r], want), ("rs rhd", op, r)


@pytest.mark.parametrize("l0,l1,l2", SHAPES + [(2, 3, 1), (3, 2, 1), (4, 4, 1)])
def test_reduce_over_levels_is_the_all_reduce_value_unit_by_unit(orc, l0, l1, l2):
    """The sequence executor of Reduce runs the AllReduce's steps and hands the root the result.  NHR cuts the same
    way in both.  RHD cuts unevenly in Reduce (floor, rest in the last) and evenly in AllReduce: the value of a unit
    is that of the same unit of an even run over the same elements, which a count of n times the unit's length with
    the unit's elements in that unit's place supplies."""
    n = l0 * l1 * l2
    rng = np.random.default_rng(13 * n + l2)
    for count in (n * 4, n * 4 + 3, n + 1, 2):
        for op, gen in ((SUM, wide), (MIN, tricky)):
            ins = gen(rng, n, count)
            root = (count + op) % n
            got = [np.zeros(count, np.float32) for _ in range(n)]
            assert orc.reduce_levels(ins, got, count, F32, op, root, l0, l1, "nhr") == 0
            want = [np.zeros(count, np.float32) for _ in range(n)]
            if l2 > 1:
                assert orc.all_reduce_three_level(ins, want, count, F32, op, l0, l1, "nhr") == 0
            else:
                assert orc.all_reduce_two_level(ins, want, count, F32, op, l0, "nhr") == 0
            assert same(got[root], want[root]), ("nhr", l0, l1, l2, count, op)
            assert not got[(root + 1) % n].view(np.uint32).any()
            got = [np.zeros(count, np.float32) for _ in range(n)]
            assert orc.reduce_levels(ins, got, count, F32, op, root, l0, l1, "rhd") == 0
            for u, (idx, lo, hi) in enumerate(cuts(0, count, [l0, l1, l2])):
                ln = hi - lo
                if ln == 0:
                    continue
                even = [np.zeros(n * ln, np.float32) for _ in range(n)]
                for r in range(n):
                    even[r][u * ln:(u + 1) * ln] = ins[r][lo:hi]
                out = [np.zeros(n * ln, np.float32) for _ in range(n)]
                if l2 > 1:
                    assert orc.all_reduce_three_level(even, out, n * ln, F32, op, l0, l1, "rhd") == 0
                else:
                    assert orc.all_reduce_two_level(even, out, n * ln, F32, op, l0, "rhd") == 0
                assert same(got[root][lo:hi], out[0][u * ln:(u + 1) * ln]), ("rhd", l0, l1, l2, count, op, idx)
    if l2 == 1:
        # the host-reduce fold between the boxes, as the two-level AllReduce has it
        count = n * 3 + 2
        ins = wide(rng, n, count)
        got = [np.zeros(count, np.float32) for _ in range(n)]
        want = [np.zeros(count, np.float32) for _ in range(n)]
        assert orc.reduce_levels(ins, got, count, F32, SUM, 0, l0, l1, "mesh") == 0
        assert orc.all_reduce_two_level(ins, want, count, F32, SUM, l0, "mesh") == 0
        assert same(got[0], want[0])
    else:
        assert orc.reduce_levels(ins, got, count, F32, SUM, 0, l0, l1, "mesh") == 1   # two levels only


@pytest.mark.parametrize("n", [2, 3, 5, 6, 7, 8, 12, 16])
def test_nhr_reduce_is_the_nhr_reduce_scatter_slice_by_slice(orc, n):
    """reduce_nhr.cc: slices of ceil(count / n) elements, short or empty towards the end, each folded along the step
    tree of the NHR ReduceScatter: slice k of Reduce is output k of a ReduceScatter over the slices padded to one
    length."""
    rng = np.random.default_rng(17 * n)
    for count in (n * 4, n * 4 + 1, n * 4 + n - 1, n + 1, n - 1, 1):
        for op, gen in ((SUM, wide), (MAX, tricky)):
            ins = gen(rng, n, count)
            root = count % n
            got = [np.zeros(count, np.float32) for _ in range(n)]
            assert orc.reduce(ins, got, count, F32, op, root, algo="nhr") == 0
            slice_len = -(-count // n)
            padded = [np.zeros(n * slice_len, np.float32) for _ in range(n)]
            for r in range(n):
                padded[r][:count] = ins[r]
            outs = [np.zeros(slice_len, np.float32) for _ in range(n)]
            assert orc.reduce_scatter(padded, outs, slice_len, F32, op, algo="nhr") == 0
            want = np.concatenate(outs)[:count]
            assert same(got[root], want), (n, count, op)
    # loops of the executor: each sliced afresh
    count, per_loop = 10 * n + 3, 4 * n + 1
    ins = wide(rng, n, count)
    got = [np.zeros(count, np.float32) for _ in range(n)]
    assert orc.reduce(ins, got, count, F32, SUM, 0, algo="nhr", max_count_per_loop=per_loop) == 0
    want = np.zeros(count, np.float32)
    for lo in range(0, count, per_loop):
        hi = min(count, lo + per_loop)
        part = [x[lo:hi].copy() for x in ins]
        out = [np.zeros(hi - lo, np.float32) for _ in range(n)]
        assert orc.reduce(part, out, hi - lo, F32, SUM, 0, algo="nhr") == 0
        want[lo:hi] = out[0]
    assert same(got[0], want)


def test_loop_rule_of_the_three_level_executors_on_worked_numbers(orc):
    """A buffer of 5 KiB, boxes of four, sixteen ranks, fp32: five slices of 1024 bytes = 256 elements; four of them
    receive: 4096 bytes, already a multiple of 128 -> 1024 elements, a multiple of 16.  With 4096-byte alignment
    (Reduce) the same.  A last loop of 1023 elements would give the last member 255 + 3 = 258 > 256 elements:
    it is shortened to 254 * 4 + min(3, 256 - 254) = 1018 and 5 remain.  1021 -> 255 + 1 = 256 fits.
    RHD with a count that 16 does not divide: two tiles of 16 * 4 = 64 -> 128 bytes leave the buffer first:
    (5120 - 256) / 5 = 972 (a multiple of 4) -> 243 elements; 3888 bytes -> 3840 -> 960 elements."""
    assert orc.sequence_max_count_per_loop(5 * 1024, 100000, 4, 16, 4, 128, False) == (1024, 256)
    assert orc.sequence_max_count_per_loop(5 * 1024, 100000, 4, 16, 4, 4096, False) == (1024, 256)
    assert orc.sequence_max_count_per_loop(5 * 1024 + 4000, 100000, 4, 16, 4, 4096, False) == (1024, 456)
    assert orc.sequence_max_count_per_loop(5 * 1024, 100001, 4, 16, 4, 128, True) == (960, 243)
    assert orc.sequence_max_count_per_loop(5 * 1024, 100000 // 16 * 16, 4, 16, 4, 128, True) == (1024, 256)
    assert orc.sequence_max_count_per_loop(100, 1000, 4, 16, 4, 128, False) is None
    assert orc.sequence_select_loop_count(5000, 1024, 4, 256) == 1024
    assert orc.sequence_select_loop_count(1023, 1024, 4, 256) == 1018
    assert orc.sequence_select_loop_count(5, 1024, 4, 256) == 5
    assert orc.sequence_select_loop_count(1021, 1024, 4, 256) == 1021
    assert orc.sequence_select_loop_count(3, 1024, 4, 256) == 3        # fewer elements than members: nothing to give up
    # and in the collective: 2 x 2 x 2, a buffer of 3 KiB: slices of 1024 bytes, 512 elements a loop
    n, count = 8, 1300
    rng = np.random.default_rng(4)
    ins = wide(rng, n, count)
    for algo, pieces in (("nhr", ((0, 512), (512, 1024), (1024, 1300))),
                         ("rhd", ((0, 448), (448, 896), (896, 1296), (1296, 1300)))):
        got = [np.zeros(count, np.float32) for _ in range(n)]
        assert orc.all_reduce_three_level(ins, got, count, F32, SUM, 2, 2, algo, ccl_bytes=3 * 1024) == 0
        want = np.zeros(count, np.float32)
        for lo, hi in pieces:
            part = [x[lo:hi].copy() for x in ins]
            out = [np.zeros(hi - lo, np.float32) for _ in range(n)]
            assert orc.all_reduce_three_level(part, out, hi - lo, F32, SUM, 2, 2, algo) == 0
            want[lo:hi] = out[0]
        assert same(got[6], want), algo


# ---- the library's programs against the oracle -----------------------------------------------------------------------
@pytest.mark.parametrize("l0,l1,l2", SHAPES + [(2, 1, 3), (2, 2, 16), (2, 16, 2), (8, 4, 2)])
@pytest.mark.parametrize("algo", ["rhd", "nhr"])
def test_three_level_programs_match_oracle(orc, l0, l1, l2, algo):
    n = l0 * l1 * l2
    progs = hccl_amd.fold_programs(OpKind.ALL_REDUCE, ALGO[algo], n, level0=l0, level1=l1)
    assert len(progs) == n
    assert progs == hccl_amd.fold_programs(OpKind.REDUCE, ALGO[algo], n, level0=l0, level1=l1)
    for prog in progs:
        assert sorted(program_ranks(prog)) == list(range(n)) and len(prog) <= 320
    for count in (n * 3, n * 3 + 5, 2):
        for op, gen in ((SUM, wide), (MAX, tricky)):
            rng = np.random.default_rng(1000 * n + 10 * l1 + op)
            ins = gen(rng, n, count)
            outs = [np.zeros(count, np.float32) for _ in range(n)]
            assert orc.all_reduce_three_level(ins, outs, count, F32, op, l0, l1, algo) == 0
            got = np.zeros(count, np.float32)
            if algo == "rhd":
                unit = count // n
                for u in range(n):
                    lo, hi = u * unit, (u + 1) * unit
                    if hi > lo:
                        got[lo:hi] = run_program(progs[u], lambda r: ins[r][lo:hi], op)
                for e in range(unit * n, count):
                    got[e:e + 1] = run_program(progs[e - unit * n], lambda r: ins[r][e:e + 1], op)
            else:
                for (i, j, k), lo, hi in cuts(0, count, [l0, l1, l2]):
                    if hi > lo:
                        got[lo:hi] = run_program(progs[(i * l1 + j) * l2 + k], lambda r: ins[r][lo:hi], op)
            assert same(got, outs[0]), (l0, l1, l2, algo, count, op)
            root = n // 2
            outs = [np.zeros(count, np.float32) for _ in range(n)]
            assert orc.reduce_levels(ins, outs, count, F32, op, root, l0, l1, algo) == 0
            got = np.zeros(count, np.float32)
            for (i, j, k), lo, hi in cuts(0, count, [l0, l1, l2]):
                if hi > lo:
                    got[lo:hi] = run_program(progs[(i * l1 + j) * l2 + k], lambda r: ins[r][lo:hi], op)
            assert same(got, outs[root]), ("reduce", l0, l1, l2, algo, count, op)
    rs = hccl_amd.fold_programs(OpKind.REDUCE_SCATTER, ALGO[algo], n, level0=l0, level1=l1)
    assert [rs[(k * l1 + j) * l0 + i] for i in range(l0) for j in range(l1) for k in range(l2)] == progs
    c = 7
    rng = np.random.default_rng(31 * n)
    ins = wide(rng, n, n * c)
    outs = [np.zeros(c, np.float32) for _ in range(n)]
    assert orc.reduce_scatter_three_level(ins, outs, c, F32, SUM, l0, l1, algo) == 0
    for r in range(n):
        assert same(run_program(rs[r], lambda q: ins[q][r * c:(r + 1) * c], SUM), outs[r]), (l0, l1, l2, algo, r)


@pytest.mark.parametrize("n", [2, 3, 5, 6, 8, 12, 33, 64])
def test_nhr_reduce_programs_match_oracle(orc, n):
    progs = hccl_amd.fold_programs(OpKind.REDUCE, Algo.NHR, n)
    assert progs == hccl_amd.fold_programs(OpKind.REDUCE_SCATTER, Algo.NHR, n)
    rng = np.random.default_rng(41 * n)
    for count in (4 * n + 3, n - 1, 2 * n):
        ins = wide(rng, n, count)
        outs = [np.zeros(count, np.float32) for _ in range(n)]
        assert orc.reduce(ins, outs, count, F32, SUM, n - 1, algo="nhr") == 0
        slice_len = -(-count // n)
        got = np.zeros(count, np.float32)
        for k in range(n):
            lo, hi = min(count, k * slice_len), min(count, (k + 1) * slice_len)
            if hi > lo:
                got[lo:hi] = run_program(progs[k], lambda r: ins[r][lo:hi], SUM)
        assert same(got, outs[n - 1]), (n, count)


def test_levels_must_divide_and_the_host_reduce_fold_keeps_two():
    with pytest.raises(hccl_amd.HcclError) as e:
        hccl_amd.fold_programs(OpKind.ALL_REDUCE, Algo.NHR, 12, level0=2, level1=4)
    assert e.value.code == 1
    assert (hccl_amd.fold_programs(OpKind.ALL_REDUCE, Algo.MESH, 12, level0=2, level1=3)
            == hccl_amd.fold_programs(OpKind.ALL_REDUCE, Algo.MESH, 12, level0=2))
    assert (hccl_amd.fold_programs(OpKind.ALL_REDUCE, Algo.NHR, 12, level0=2, level1=6)
            == hccl_amd.fold_programs(OpKind.ALL_REDUCE, Algo.NHR, 12, level0=2))
    with pytest.raises(hccl_amd.HcclError) as e:
        hccl_amd.fold_programs(OpKind.REDUCE, Algo.RHD, 6)          # no single-level RHD Reduce
    assert e.value.code == 5
    comms = hccl_amd.comm_init_all(12)
    try:
        hccl_amd.set_level0_rank_size(comms[0], 2)
        hccl_amd.set_level1_group_size(comms[3], 3)
        assert hccl_amd.get_level1_group_size(comms[11]) == 3
        with pytest.raises(hccl_amd.HcclError) as e:
            hccl_amd.set_level1_group_size(comms[0], 4)
        assert e.value.code == 1
        hccl_amd.set_level0_rank_size(comms[0], 3)       # four groups: three of them no longer form level-1 groups
        assert hccl_amd.get_level1_group_size(comms[0]) == 0
        hccl_amd.set_algo(comms[0], OpKind.REDUCE, Algo.NHR)
        hccl_amd.set_algo(comms[0], OpKind.REDUCE, Algo.RHD)
        assert hccl_amd.get_algo(comms[5], OpKind.REDUCE) == Algo.RHD
    finally:
        for c in comms:
            hccl_amd.comm_destroy(c)


def test_what_hccl_algo_selects_for_three_levels_and_for_reduce():
    sel = hccl_amd.select_from_hccl_algo
    for op in (OpKind.ALL_REDUCE, OpKind.REDUCE_SCATTER, OpKind.REDUCE):
        assert sel("sequence{level0=mesh_concur,level1=nhr,level2=nhr}", op)[1:] == (Algo.NHR, True)
        assert sel("sequence{meshconcur,rhd,rhd}", op)[1:] == (Algo.RHD, True)
        assert sel("sequence{meshconcur,rhd}", op)[1:] == (Algo.RHD, True)
        assert sel("sequence{meshconcur,nhr,rhd}", op)[1] is None                 # no mixed executor is registered
        assert sel("sequence{mesh,nhr_aicpu_reduce,nhr_aicpu_reduce}", op)[1] is None
        assert sel("sequence{mesh,nhr_aicpu_reduce}", op)[1:] == (Algo.MESH, True)
        assert sel("sequence{mesh_chunk,nhr,nhr}", op)[1] is None
    # the string of the reference's own Reduce system test (test/st/algorithm/testcase/reduce_sequence_testcase.cc:57)
    assert sel("sequence{meshconcur,nhr,nhr}", OpKind.REDUCE)[1:] == (Algo.NHR, True)
    assert sel("reduce:sole{nhr}", OpKind.REDUCE)[1:] == (Algo.NHR, False)
    assert sel("reduce:sole{nhr_aicpu_reduce}", OpKind.REDUCE)[1:] == (Algo.MESH, False)
    assert sel("reduce:sole{mesh_two_shot}", OpKind.REDUCE)[1:] == (Algo.MESH_TWO_SHOT, False)
    assert sel("reduce:sole{mesh_chunk}", OpKind.REDUCE)[1] is None
    # Aicpu Reduce Sequence NHRAicpuReduce NHR: mesh inside the groups, the host-reduce fold between them
    assert sel("reduce:sequence{nhr_aicpu_reduce,nhr}", OpKind.REDUCE)[1:] == (Algo.MESH, True)
    assert sel("sequence{nhr_aicpu_reduce,nhr}", OpKind.ALL_REDUCE)[1] is None


def test_every_division_of_up_to_64_ranks_into_levels_has_programs_the_kernel_can_run():
    """Nesting depth and program length stay within what the kernel's interpreter takes (8 levels, 320 bytes) for every
    way of cutting 2 .. 64 ranks into boxes and pods, under both templates."""
    longest = 0
    for n in range(2, 65):
        for l0 in range(2, n):
            if n % l0:
                continue
            boxes = n // l0
            for l1 in range(1, boxes + 1):
                if boxes % l1:
                    continue
                for algo in (Algo.NHR, Algo.RHD):
                    progs = hccl_amd.fold_programs(OpKind.ALL_REDUCE, algo, n, level0=l0, level1=l1)
                    assert len(progs) == n
                    longest = max(longest, max(len(p) for p in progs))
    assert longest <= 320


@pytest.mark.parametrize("n", [2, 3, 5, 6, 8, 12, 33])
def test_all_reduce_of_the_two_shot_executor_over_one_mesh(orc, n):
    """Aicpu AllReduce Sole MeshConcur (ins_v2_all_reduce_two_shot_sole_executor.cc): a mesh ReduceScatter on slices
    of floor(len / n) elements with the rest in the last, slice k folded own input first, then the AllGather.  Where
    n divides the count the slices are those of the symmetric two-shot order (pinned elsewhere); all ranks in one
    level-0 group is the same executor seen from the two-level one; uneven counts by hand."""
    rng = np.random.default_rng(23 * n)
    for count in (n * 6, n * 6 + 1, n * 6 + n - 1, n - 1, 1):
        for op, gen in ((SUM, wide), (MIN, tricky)):
            ins = gen(rng, n, count)
            got = [np.zeros(count, np.float32) for _ in range(n)]
            assert orc.all_reduce(ins, got, count, F32, op, algo="mesh_concur") == 0
            if count % n == 0:
                want = [np.zeros(count, np.float32) for _ in range(n)]
                assert orc.all_reduce(ins, want, count, F32, op, algo="mesh_symmetric") == 0
                assert same(got[0], want[0]), (n, count, op)
            want = [np.zeros(count, np.float32) for _ in range(n)]
            assert orc.all_reduce_two_level(ins, want, count, F32, op, n, "nhr") == 0
            assert same(got[n - 1], want[n - 1]), (n, count, op)
            by_hand = np.zeros(count, np.float32)
            slice_len = count // n
            for k in range(n):
                lo = k * slice_len
                hi = count if k == n - 1 else lo + slice_len
                by_hand[lo:hi] = box(ins, n, 0, k, lo, hi, op)
            for r in range(n):
                assert same(got[r], by_hand), (n, count, op, r)
    # loops: floored to a multiple of n, each cut afresh
    count, per_loop = 11 * n + 3, 4 * n + n - 1
    ins = wide(rng, n, count)
    got = [np.zeros(count, np.float32) for _ in range(n)]
    assert orc.all_reduce(ins, got, count, F32, SUM, algo="mesh_concur", max_count_per_loop=per_loop) == 0
    want = np.zeros(count, np.float32)
    for lo in range(0, count, 4 * n):
        hi = min(count, lo + 4 * n)
        part = [x[lo:hi].copy() for x in ins]
        out = [np.zeros(hi - lo, np.float32) for _ in range(n)]
        assert orc.all_reduce(part, out, hi - lo, F32, SUM, algo="mesh_concur") == 0
        want[lo:hi] = out[0]
    assert same(got[0], want)
    # the library's programs: those of the mesh ReduceScatter, one per slice
    progs = hccl_amd.fold_programs(OpKind.ALL_REDUCE, Algo.MESH_CONCUR, n)
    assert progs == hccl_amd.fold_programs(OpKind.REDUCE_SCATTER, Algo.MESH, n)
    with pytest.raises(hccl_amd.HcclError) as e:
        hccl_amd.fold_programs(OpKind.REDUCE_SCATTER, Algo.MESH_CONCUR, n)
    assert e.value.code == 5
    sel = hccl_amd.select_from_hccl_algo
    assert sel("allreduce:sole{mesh_concur}", OpKind.ALL_REDUCE)[1:] == (Algo.MESH_CONCUR, False)
    assert sel("mesh_concur", OpKind.REDUCE_SCATTER)[1:] == (Algo.MESH, False)
    assert sel("allreduce:sequence{mesh,mesh_concur}", OpKind.ALL_REDUCE)[1] is None
