"""Pins the oracle's restatement of the ops built on the same kernels as the hot path: AlltoAll,
AlltoAllVC (matrix -> counts / displacements conversion), ReduceScatterV, Reduce, Broadcast, Scatter.

Nothing here retypes the oracle's loops: data movement is checked against numpy slicing / reshapes,
the conversion against values worked out by hand for the count matrices the reference's own system
tests use (test/st/algorithm/testcase/alltoallvc_testcase.cc:184, 215), reductions against exact
integer arithmetic, the written association order in fp32, and the ops they must degenerate to.
"""
import numpy as np
import pytest

I8, I16, I32, F16, F32, I64, U64, F64, BF16 = 0, 1, 2, 3, 4, 5, 6, 10, 11
SUM, PROD, MAX, MIN = range(4)


def wide_f32(rng, n, count):
    return [(rng.standard_normal(count) * 10.0 ** rng.integers(-6, 6, count)).astype(np.float32) for _ in range(n)]


# ---- AlltoAll ----------------------------------------------------------------------------------
@pytest.mark.parametrize("n,count", [(1, 5), (2, 1), (3, 7), (8, 33), (16, 4)])
def test_all_to_all_is_a_block_transpose(orc, n, count):
    rng = np.random.default_rng(n * 100 + count)
    ins = [rng.integers(-2 ** 31, 2 ** 31 - 1, n * count).astype(np.int32) for _ in range(n)]
    outs = [np.zeros(n * count, dtype=np.int32) for _ in range(n)]
    assert orc.all_to_all(ins, outs, count, I32) == 0
    want = np.stack([x.reshape(n, count) for x in ins]).transpose(1, 0, 2)   # [dst][src][elem]
    for i in range(n):
        assert np.array_equal(outs[i].reshape(n, count), want[i])


# ---- AlltoAllVC --------------------------------------------------------------------------------
def test_all_to_all_vc_params_reference_2x2_matrix(orc):
    # matrix {10, 11, 1, 2222}: row = sender, column = receiver
    m = np.array([10, 11, 1, 2222], dtype=np.uint64)
    sc, rc, sd, rd = orc.all_to_all_vc_params(2, 0, m)
    assert (list(sc), list(rc), list(sd), list(rd)) == ([10, 11], [10, 1], [0, 10], [0, 10])
    sc, rc, sd, rd = orc.all_to_all_vc_params(2, 1, m)
    assert (list(sc), list(rc), list(sd), list(rd)) == ([1, 2222], [11, 2222], [0, 1], [0, 11])


def test_all_to_all_vc_params_all_ones_6x6(orc):
    m = np.ones(36, dtype=np.uint64)
    for r in range(6):
        sc, rc, sd, rd = orc.all_to_all_vc_params(6, r, m)
        assert list(sc) == [1] * 6 and list(rc) == [1] * 6
        assert list(sd) == list(range(6)) and list(rd) == list(range(6))


@pytest.mark.parametrize("n,seed", [(2, 0), (3, 1), (6, 2), (8, 3)])
def test_all_to_all_vc_moves_what_numpy_slicing_moves(orc, n, seed):
    rng = np.random.default_rng(seed)
    m = rng.integers(0, 40, (n, n)).astype(np.uint64)
    m[rng.integers(0, n), :] = 0                      # one silent sender
    m[:, rng.integers(0, n)] = 0                      # one rank that receives nothing
    ins = [rng.integers(0, 65535, max(int(m[j].sum()), 1)).astype(np.uint16) for j in range(n)]
    outs = [np.full(max(int(m[:, i].sum()), 1), 0xAAAA, dtype=np.uint16) for i in range(n)]
    assert orc.all_to_all_vc(ins, outs, m, 8) == 0    # uint16
    for i in range(n):
        parts = []
        for j in range(n):
            lo = int(m[j, :i].sum())
            parts.append(ins[j][lo:lo + int(m[j, i])])
        want = np.concatenate(parts) if int(m[:, i].sum()) else np.zeros(0, dtype=np.uint16)
        assert np.array_equal(outs[i][:want.size], want)
        assert np.all(outs[i][want.size:] == 0xAAAA)


def test_all_to_all_vc_equals_all_to_all_for_a_constant_matrix(orc):
    n, count = 5, 9
    rng = np.random.default_rng(7)
    ins = [rng.integers(0, 255, n * count).astype(np.uint8) for _ in range(n)]
    a = [np.zeros(n * count, dtype=np.uint8) for _ in range(n)]
    b = [np.zeros(n * count, dtype=np.uint8) for _ in range(n)]
    assert orc.all_to_all(ins, a, count, 7) == 0
    assert orc.all_to_all_vc(ins, b, np.full(n * n, count, dtype=np.uint64), 7) == 0
    for x, y in zip(a, b):
        assert np.array_equal(x, y)


# ---- ReduceScatterV ------------------------------------------------------------------------------
def rsv_layout(rng, n, lo, hi, gaps):
    counts = rng.integers(lo, hi, n).astype(np.uint64)
    counts[rng.integers(0, n)] = 0
    displs = np.zeros(n, dtype=np.uint64)
    off = 0
    for k in rng.permutation(n) if gaps else range(n):
        off += int(rng.integers(0, 5)) if gaps else 0
        displs[k] = off
        off += int(counts[k])
    return counts, displs, off + 3


@pytest.mark.parametrize("n", [2, 3, 6, 8])
@pytest.mark.parametrize("gaps", [False, True])
def test_reduce_scatter_v_int32_sum_and_max_match_exact_arithmetic(orc, n, gaps):
    rng = np.random.default_rng(n + 10 * gaps)
    counts, displs, total = rsv_layout(rng, n, 1, 50, gaps)
    ins = [rng.integers(-2 ** 31, 2 ** 31 - 1, total).astype(np.int32) for _ in range(n)]
    for op in (SUM, MAX, MIN, PROD):
        outs = [np.full(max(int(c), 1), 77, dtype=np.int32) for c in counts]
        assert orc.reduce_scatter_v(ins, outs, counts, displs, I32, op) == 0
        for k in range(n):
            sl = np.stack([x[int(displs[k]):int(displs[k]) + int(counts[k])] for x in ins])
            if op == SUM:
                want = sl.astype(np.int64).sum(axis=0).astype(np.int32)          # wraps mod 2^32
            elif op == PROD:
                want = np.ones(sl.shape[1], dtype=np.uint32)
                for row in sl:
                    want = want * row.view(np.uint32)
                want = want.view(np.int32)
            else:
                want = sl.max(axis=0) if op == MAX else sl.min(axis=0)
            assert np.array_equal(outs[k][:int(counts[k])], want), (op, k)
            if counts[k] == 0:
                assert outs[k][0] == 77


def test_reduce_scatter_v_fp32_starts_with_the_own_slice_then_ranks_ascending(orc):
    n = 5
    rng = np.random.default_rng(3)
    counts, displs, total = rsv_layout(rng, n, 40, 90, True)
    ins = wide_f32(rng, n, total)
    outs = [np.zeros(max(int(c), 1), dtype=np.float32) for c in counts]
    assert orc.reduce_scatter_v(ins, outs, counts, displs, F32, SUM) == 0
    differs_from_rank_order = False
    for k in range(n):
        lo, c = int(displs[k]), int(counts[k])
        acc = ins[k][lo:lo + c].copy()
        for t in range(n):
            if t != k:
                acc = ins[t][lo:lo + c] + acc
        assert np.array_equal(outs[k][:c].view(np.uint32), acc.view(np.uint32)), k
        plain = ins[0][lo:lo + c].copy()
        for t in range(1, n):
            plain = ins[t][lo:lo + c] + plain
        differs_from_rank_order |= not np.array_equal(plain.view(np.uint32), acc.view(np.uint32))
    assert differs_from_rank_order        # the inputs do tell the two orders apart


@pytest.mark.parametrize("dtype,np_dt", [(BF16, np.uint16), (F16, np.uint16), (I8, np.int8), (I64, np.int64)])
def test_reduce_scatter_v_with_uniform_counts_is_reduce_scatter(orc, dtype, np_dt):
    n, c = 6, 37
    rng = np.random.default_rng(11)
    if dtype == BF16:
        ins = [orc.np_fp32_to_bf16_bits(rng.standard_normal(n * c).astype(np.float32)) for _ in range(n)]
    elif dtype == F16:
        ins = [rng.standard_normal(n * c).astype(np.float16).view(np.uint16) for _ in range(n)]
    else:
        ins = [rng.integers(-100, 100, n * c).astype(np_dt) for _ in range(n)]
    a = [np.zeros(c, dtype=np_dt) for _ in range(n)]
    b = [np.zeros(c, dtype=np_dt) for _ in range(n)]
    counts = np.full(n, c, dtype=np.uint64)
    displs = (np.arange(n) * c).astype(np.uint64)
    assert orc.reduce_scatter_v(ins, a, counts, displs, dtype, SUM) == 0
    assert orc.reduce_scatter(ins, b, c, dtype, SUM, algo="mesh") == 0
    for x, y in zip(a, b):
        assert np.array_equal(x, y)


@pytest.mark.parametrize("dtype", [U64, F64])
def test_reduce_scatter_v_rejects_the_types_its_entry_point_rejects(orc, dtype):
    ins = [np.zeros(4, dtype=np.uint64) for _ in range(2)]
    outs = [np.zeros(2, dtype=np.uint64) for _ in range(2)]
    rc = orc.reduce_scatter_v(ins, outs, np.array([2, 2], dtype=np.uint64), np.array([0, 2], dtype=np.uint64),
                              dtype, SUM)
    assert rc == 5   # HCCL_E_NOT_SUPPORT


# ---- Reduce ----------------------------------------------------------------------------------------
@pytest.mark.parametrize("n,root", [(1, 0), (2, 1), (5, 3), (8, 0), (8, 7)])
def test_reduce_writes_the_rank_order_fold_to_the_root_only(orc, n, root):
    rng = np.random.default_rng(n * 8 + root)
    count = 257
    ins = wide_f32(rng, n, count)
    outs = [np.full(count, 123.0, dtype=np.float32) for _ in range(n)]
    assert orc.reduce(ins, outs, count, F32, SUM, root) == 0
    acc = ins[0].copy()
    for r in range(1, n):
        acc = ins[r] + acc
    assert np.array_equal(outs[root].view(np.uint32), acc.view(np.uint32))
    for r in range(n):
        if r != root:
            assert np.all(outs[r] == 123.0)


def test_reduce_equals_all_reduce_mesh_at_the_root_for_bf16_and_int_prod(orc):
    n, count, root = 6, 129, 4
    rng = np.random.default_rng(5)
    for dtype, make in ((BF16, lambda: orc.np_fp32_to_bf16_bits(rng.standard_normal(count).astype(np.float32))),
                        (I32, lambda: rng.integers(-3, 4, count).astype(np.int32))):
        ins = [make() for _ in range(n)]
        for op in ((SUM, MAX, MIN) if dtype == BF16 else (SUM, PROD, MAX, MIN)):   # no bf16 PROD in the reference
            a = [np.zeros(count, dtype=ins[0].dtype) for _ in range(n)]
            b = [np.zeros(count, dtype=ins[0].dtype) for _ in range(n)]
            assert orc.reduce(ins, a, count, dtype, op, root) == 0
            assert orc.all_reduce(ins, b, count, dtype, op, algo="mesh") == 0
            assert np.array_equal(a[root], b[root])


@pytest.mark.parametrize("n,root,count", [(2, 1, 257), (5, 3, 1003), (8, 0, 8 * 100), (8, 7, 5), (3, 2, 2)])
def test_reduce_two_shot_deals_slices_and_folds_the_own_slice_first(orc, n, root, count):
    """Slices: count // n elements, the first count % n one longer; slice k = x_k, then the others ascending."""
    rng = np.random.default_rng(n * 80 + root + count)
    ins = wide_f32(rng, n, count)
    outs = [np.full(count, 123.0, dtype=np.float32) for _ in range(n)]
    assert orc.reduce(ins, outs, count, F32, SUM, root, algo="mesh_two_shot") == 0
    want = np.zeros(count, dtype=np.float32)
    lo = 0
    for k in range(n):
        ln = count // n + (1 if k < count % n else 0)
        acc = ins[k][lo:lo + ln].copy()
        for t in range(n):
            if t != k:
                acc = ins[t][lo:lo + ln] + acc
        want[lo:lo + ln] = acc
        lo += ln
    assert lo == count
    assert np.array_equal(outs[root].view(np.uint32), want.view(np.uint32))
    for r in range(n):
        if r != root:
            assert np.all(outs[r] == 123.0)


def test_reduce_two_shot_loops_deal_afresh_and_integers_do_not_care(orc):
    rng = np.random.default_rng(81)
    n, count, per_loop = 4, 1000, 300
    ins = wide_f32(rng, n, count)
    outs = [np.zeros(count, dtype=np.float32) for _ in range(n)]
    assert orc.reduce(ins, outs, count, F32, SUM, 2, algo="mesh_two_shot", max_count_per_loop=per_loop) == 0
    want = np.zeros(count, dtype=np.float32)
    for done in range(0, count, per_loop):
        cur = min(per_loop, count - done)
        lo = done
        for k in range(n):
            ln = cur // n + (1 if k < cur % n else 0)
            acc = ins[k][lo:lo + ln].copy()
            for t in range(n):
                if t != k:
                    acc = ins[t][lo:lo + ln] + acc
            want[lo:lo + ln] = acc
            lo += ln
    assert np.array_equal(outs[2].view(np.uint32), want.view(np.uint32))
    ints = [rng.integers(-2 ** 31, 2 ** 31 - 1, count, dtype=np.int32) for _ in range(n)]
    a = [np.zeros(count, dtype=np.int32) for _ in range(n)]
    b = [np.zeros(count, dtype=np.int32) for _ in range(n)]
    assert orc.reduce(ints, a, count, I32, SUM, 1) == 0
    assert orc.reduce(ints, b, count, I32, SUM, 1, algo="mesh_two_shot", max_count_per_loop=77) == 0
    assert np.array_equal(a[1], b[1])


def test_reduce_rejects_a_root_outside_the_world(orc):
    ins = [np.zeros(4, dtype=np.float32) for _ in range(2)]
    assert orc.reduce(ins, [x.copy() for x in ins], 4, F32, SUM, 2) == 1   # HCCL_E_PARA


# ---- Broadcast / Scatter -------------------------------------------------------------------------
@pytest.mark.parametrize("n,root", [(1, 0), (3, 2), (8, 5)])
def test_broadcast_copies_the_root_buffer_to_every_rank(orc, n, root):
    rng = np.random.default_rng(n + root)
    count = 77
    bufs = [rng.integers(0, 2 ** 16, count).astype(np.uint16) for _ in range(n)]
    src = bufs[root].copy()
    assert orc.broadcast(bufs, count, F16, root) == 0
    for b in bufs:
        assert np.array_equal(b, src)


@pytest.mark.parametrize("n,root", [(1, 0), (4, 1), (8, 7)])
def test_scatter_hands_slice_r_of_the_root_to_rank_r(orc, n, root):
    rng = np.random.default_rng(n * 3 + root)
    c = 19
    ins = [rng.integers(-2 ** 63, 2 ** 63 - 1, n * c).astype(np.int64) for _ in range(n)]
    outs = [np.zeros(c, dtype=np.int64) for _ in range(n)]
    assert orc.scatter(ins, outs, c, I64, root) == 0
    for r in range(n):
        assert np.array_equal(outs[r], ins[root].reshape(n, c)[r])
