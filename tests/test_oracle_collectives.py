"""Pins the association order and data movement of every executor the oracle restates
(rows a5-a15), by brute force on small inputs against the order written in the reference's
templates, its worked examples, and independent closed forms.

fp32 inputs span ~12 decades so that a different association order changes low bits in most
elements; MAX / MIN inputs are drawn from {+0, -0, NaNs with distinct payloads, 1} so that a swapped
src / dst role changes the result.
"""
import json
import os

import numpy as np
import pytest

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "rhd_nhr_tables.json")))
I8, I16, I32, F16, F32, I64, U64, F64, BF16 = 0, 1, 2, 3, 4, 5, 6, 10, 11
SUM, PROD, MAX, MIN = range(4)


def wide_f32(rng, n, count):
    return [(rng.standard_normal(count) * 10.0 ** rng.integers(-6, 6, count)).astype(np.float32) for _ in range(n)]


def tricky_f32(rng, n, count):
    pool = np.array([0x00000000, 0x80000000, 0x7FC00001, 0x7FC00002, 0xFFC00003, 0x3F800000, 0xBF800000],
                    dtype=np.uint32)
    return [pool[rng.integers(0, pool.size, count)].view(np.float32).copy() for _ in range(n)]


def f32_op(src, dst, op):
    """dst <- src (+) dst with the reference's operand roles."""
    with np.errstate(all="ignore"):
        if op == SUM:
            return src + dst
        if op == PROD:
            return src * dst
        if op == MAX:
            return np.where(src < dst, dst, src)
        return np.where(dst < src, dst, src)


def bits_equal_nan_class(a, b):
    """Bit-exact except that arithmetic NaNs only need to be NaN on both sides."""
    a32, b32 = a.view(np.uint32), b.view(np.uint32)
    both_nan = np.isnan(a) & np.isnan(b)
    return np.array_equal(a32[~both_nan], b32[~both_nan]) and np.array_equal(np.isnan(a), np.isnan(b))


def outs_like(ins, count=None):
    return [np.zeros(ins[0].size if count is None else count, dtype=ins[0].dtype) for _ in ins]


# ---------------------------------------------------------------------------------------------
# AllReduce in rank order (a6, a7, a8)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 2, 3, 8, 16])
@pytest.mark.parametrize("algo", ["mesh", "two_shot"])
def test_all_reduce_rank_order_fp32(orc, n, algo):
    rng = np.random.default_rng(n)
    count = 1031
    ins = wide_f32(rng, n, count)
    outs = outs_like(ins)
    assert orc.all_reduce(ins, outs, count, F32, SUM, algo=algo) == 0
    acc = ins[0].copy()
    for r in range(1, n):
        acc = ins[r] + acc
    for o in outs:
        assert np.array_equal(o.view(np.uint32), acc.view(np.uint32))
    if n >= 8:   # the check discriminates: pairwise-tree order gives different bits
        tree = [x.copy() for x in ins]
        while len(tree) > 1:
            tree = [tree[i] + tree[i + 1] for i in range(0, len(tree), 2)]
        assert np.count_nonzero(tree[0] != acc) > count // 10


@pytest.mark.parametrize("op", [MAX, MIN])
def test_all_reduce_rank_order_roles(orc, op):
    rng = np.random.default_rng(3)
    n, count = 5, 4096
    ins = tricky_f32(rng, n, count)
    outs = outs_like(ins)
    assert orc.all_reduce(ins, outs, count, F32, op) == 0
    acc = ins[0].copy()
    for r in range(1, n):
        acc = f32_op(ins[r], acc, op)
    assert np.array_equal(outs[0].view(np.uint32), acc.view(np.uint32))
    # swapping the roles is observable on this input
    swapped = ins[0].copy()
    for r in range(1, n):
        swapped = f32_op(swapped, ins[r], op)
    assert np.count_nonzero(swapped.view(np.uint32) != acc.view(np.uint32)) > 100


def test_all_reduce_in_place(orc):
    rng = np.random.default_rng(4)
    ins = [rng.integers(-100, 100, 257, dtype=np.int32) for _ in range(4)]
    want = sum(x.astype(np.int64) for x in ins).astype(np.int32)
    assert orc.all_reduce(ins, ins, 257, I32, SUM) == 0
    for x in ins:
        assert np.array_equal(x, want)


# ---------------------------------------------------------------------------------------------
# ReduceScatter orders (a9, a10, a12, vector-core mesh)
# ---------------------------------------------------------------------------------------------
def rs_expected(ins, n, c, k, leaf_order):
    """Left fold over leaf_order of rank t's slice k."""
    acc = ins[leaf_order[0]][k * c:(k + 1) * c].copy()
    for t in leaf_order[1:]:
        acc = ins[t][k * c:(k + 1) * c] + acc
    return acc


@pytest.mark.parametrize("n", [1, 2, 5, 8])
def test_reduce_scatter_mesh_own_rank_first(orc, n):
    rng = np.random.default_rng(10 + n)
    c = 333
    ins = wide_f32(rng, n, n * c)
    outs = outs_like(ins, c)
    assert orc.reduce_scatter(ins, outs, c, F32, SUM, algo="mesh") == 0
    for k in range(n):
        order = [k] + [t for t in range(n) if t != k]
        assert np.array_equal(outs[k].view(np.uint32), rs_expected(ins, n, c, k, order).view(np.uint32))
    if n == 8:
        plain = rs_expected(ins, n, c, 5, list(range(n)))
        assert np.count_nonzero(plain != outs[5]) > c // 10


def test_reduce_scatter_nhr_tree_n8(orc):
    """Slice k ends as ((x_k+x_k+1)+(x_k+2+x_k+3)) + ((x_k+4+x_k+5)+(x_k+6+x_k+7)), indices mod 8,
    the receiver's partial being dst at every step."""
    rng = np.random.default_rng(21)
    n, c = 8, 257
    ins = wide_f32(rng, n, n * c)
    outs = outs_like(ins, c)
    assert orc.reduce_scatter(ins, outs, c, F32, SUM, algo="nhr") == 0
    for k in range(n):
        x = [ins[(k + i) % n][k * c:(k + 1) * c] for i in range(n)]
        a = (x[1] + x[0])
        b = (x[3] + x[2])
        cc = (x[5] + x[4])
        d = (x[7] + x[6])
        want = (((d + cc)) + (b + a))
        assert np.array_equal(outs[k].view(np.uint32), want.view(np.uint32)), k


def test_reduce_scatter_nhr_roles_n4(orc):
    """N=4 from the reference's hand table: step 0 rank m receives slices {m, m-2} from m+1; step 1 slice m
    from m+2.  Slice k at rank k: step0 acc = x_{k+1} (+) x_k ; rank k+2 holds x_{k+3} (+) x_{k+2};
    step1 acc = (x_{k+3} (+) x_{k+2}) (+) acc."""
    rng = np.random.default_rng(22)
    n, c = 4, 512
    ins = tricky_f32(rng, n, n * c)
    for op in (MAX, MIN):
        outs = outs_like(ins, c)
        assert orc.reduce_scatter(ins, outs, c, F32, op, algo="nhr") == 0
        for k in range(n):
            x = [ins[(k + i) % n][k * c:(k + 1) * c] for i in range(n)]
            own = f32_op(x[1], x[0], op)
            far = f32_op(x[3], x[2], op)
            want = f32_op(far, own, op)
            assert np.array_equal(outs[k].view(np.uint32), want.view(np.uint32))


def nhr_tree_n8(x):
    """The N=8 tree of one slice, x[i] = rank (k + i) mod 8's values of slice k."""
    return ((x[7] + x[6]) + (x[5] + x[4])) + ((x[3] + x[2]) + (x[1] + x[0]))


def nhr_all_reduce_expected_n8(ins, lo, hi):
    """Elements [lo, hi) handled by one run of the one-level NHR AllReduce template: seven slices of
    floor((hi - lo) / 8) elements and the last slice with the rest."""
    want = np.zeros(hi - lo, dtype=np.float32)
    cnt = hi - lo
    sl = cnt // 8
    for k in range(8):
        a, b = k * sl, (cnt if k == 7 else (k + 1) * sl)
        want[a:b] = nhr_tree_n8([ins[(k + i) % 8][lo + a:lo + b] for i in range(8)])
    return want


@pytest.mark.parametrize("count", [8 * 300, 8 * 300 + 5, 5, 8, 15])
def test_all_reduce_nhr_floor_slices_last_takes_rest(orc, count):
    rng = np.random.default_rng(23 + count)
    ins = wide_f32(rng, 8, count)
    outs = outs_like(ins)
    assert orc.all_reduce(ins, outs, count, F32, SUM, algo="nhr") == 0
    want = nhr_all_reduce_expected_n8(ins, 0, count)
    for o in outs:
        assert np.array_equal(o.view(np.uint32), want.view(np.uint32))


def test_all_reduce_nhr_loop_re_cuts_slices(orc):
    """Each loop over the staging buffer slices its own share afresh."""
    rng = np.random.default_rng(24)
    count, per_loop = 2000, 640
    ins = wide_f32(rng, 8, count)
    outs = outs_like(ins)
    assert orc.all_reduce(ins, outs, count, F32, SUM, algo="nhr", max_count_per_loop=per_loop) == 0
    want = np.concatenate([nhr_all_reduce_expected_n8(ins, lo, min(count, lo + per_loop))
                           for lo in range(0, count, per_loop)])
    for o in outs:
        assert np.array_equal(o.view(np.uint32), want.view(np.uint32))
    one_loop = outs_like(ins)
    assert orc.all_reduce(ins, one_loop, count, F32, SUM, algo="nhr") == 0
    assert np.count_nonzero(one_loop[0] != outs[0]) > 0           # wide-range inputs: the order shows


# ---- mesh chunk ----------------------------------------------------------------------------------
def test_mesh_chunk_segment_sizes(orc):
    """ReduceScatter(V): floor(bytes / (n-1)) down to 4 KiB, the last takes the rest; too small: element-wise,
    the first len mod (n-1) one longer.  AllReduce: always element-wise."""
    # 8 ranks, fp32: 100000 el = 400000 B / 7 = 57142 -> 53248 B = 13312 el; last = 100000 - 6 * 13312
    assert orc.mesh_chunk_segments(100000, 8, 4, True) == [13312] * 6 + [100000 - 6 * 13312]
    # below 4 KiB per segment: 7000 B / 7 = 1000 B -> element-wise: 1750 el = 7 * 250
    assert orc.mesh_chunk_segments(1750, 8, 4, True) == [250] * 7
    assert orc.mesh_chunk_segments(1753, 8, 4, True) == [251] * 3 + [250] * 4
    assert orc.mesh_chunk_segments(3, 8, 4, True) == [1, 1, 1, 0, 0, 0, 0]
    # two ranks: a single segment, never the aligned rule
    assert orc.mesh_chunk_segments(1 << 20, 2, 4, True) == [1 << 20]
    # exactly 4 KiB per segment
    assert orc.mesh_chunk_segments(7 * 1024, 8, 4, True) == [1024] * 7
    assert orc.mesh_chunk_segments(7 * 1024 - 1, 8, 4, True) == [1024] * 6 + [1023]     # 28668 B / 7 = 4095 -> 0 -> element-wise
    assert orc.mesh_chunk_segments(100000, 8, 4, False) == [14286] * 5 + [14285] * 2
    # bf16: 3 ranks, 10000 el = 20000 B / 2 = 10000 -> 8192 B = 4096 el
    assert orc.mesh_chunk_segments(10000, 3, 2, True) == [4096, 5904]
    for n in (2, 3, 5, 8, 64):
        for ln in (0, 1, n - 2, n - 1, 4097, 1 << 16):
            for align in (True, False):
                assert sum(orc.mesh_chunk_segments(ln, n, 2, align)) == ln


def mesh_chunk_order(n, k, i):
    """Ranks folded into segment i of slice k, worked out by hand from the step loop: step s delivers the
    segment from the rank s + i + 1 places above k, places n .. n+i-1 standing for 1 .. i after the sender
    skips itself: k, k+i+1, ..., k+n-1, k+1, ..., k+i."""
    return [k] + [(k + d) % n for d in list(range(i + 1, n)) + list(range(1, i + 1))]


def test_mesh_chunk_order_n4_by_hand():
    # n = 4, slice 1: segment 0 <- 2, 3, 0 ; segment 1 <- 3, 0, 2 ; segment 2 <- 0, 2, 3
    assert [mesh_chunk_order(4, 1, i) for i in range(3)] == [[1, 2, 3, 0], [1, 3, 0, 2], [1, 0, 2, 3]]


@pytest.mark.parametrize("n,c", [(4, 3 * 5000), (8, 100000), (8, 1753), (3, 10000), (2, 777), (5, 3)])
def test_reduce_scatter_mesh_chunk_rotation(orc, n, c):
    rng = np.random.default_rng(300 + n + c)
    ins = wide_f32(rng, n, n * c)
    outs = outs_like(ins, c)
    assert orc.reduce_scatter(ins, outs, c, F32, SUM, algo="mesh_chunk") == 0
    segs = orc.mesh_chunk_segments(c, n, 4, True)
    for k in range(n):
        lo = 0
        for i, ln in enumerate(segs):
            order = mesh_chunk_order(n, k, i)
            acc = ins[order[0]][k * c + lo:k * c + lo + ln].copy()
            for t in order[1:]:
                acc = ins[t][k * c + lo:k * c + lo + ln] + acc
            assert np.array_equal(outs[k][lo:lo + ln].view(np.uint32), acc.view(np.uint32)), (k, i)
            lo += ln
    if n == 8 and c == 100000:
        plain = rs_expected(ins, n, c, 3, [3] + [t for t in range(n) if t != 3])
        assert np.count_nonzero(plain != outs[3]) > c // 10       # not the plain mesh order


def test_reduce_scatter_mesh_chunk_loops_re_cut_segments(orc):
    rng = np.random.default_rng(310)
    n, c, per_loop = 4, 40000, 16384
    ins = wide_f32(rng, n, n * c)
    outs = outs_like(ins, c)
    assert orc.reduce_scatter(ins, outs, c, F32, SUM, algo="mesh_chunk", max_count_per_loop=per_loop) == 0
    for k in range(n):
        for done in range(0, c, per_loop):
            cur = min(per_loop, c - done)
            lo = done
            for i, ln in enumerate(orc.mesh_chunk_segments(cur, n, 4, True)):
                order = mesh_chunk_order(n, k, i)
                acc = ins[order[0]][k * c + lo:k * c + lo + ln].copy()
                for t in order[1:]:
                    acc = ins[t][k * c + lo:k * c + lo + ln] + acc
                assert np.array_equal(outs[k][lo:lo + ln].view(np.uint32), acc.view(np.uint32)), (k, done, i)
                lo += ln


@pytest.mark.parametrize("n,count", [(4, 40003), (8, 100000), (8, 5), (3, 7), (2, 1001), (6, 6 * 7 * 100 + 11)])
def test_all_reduce_mesh_chunk_rotation(orc, n, count):
    rng = np.random.default_rng(320 + n + count)
    ins = wide_f32(rng, n, count)
    outs = outs_like(ins)
    assert orc.all_reduce(ins, outs, count, F32, SUM, algo="mesh_chunk") == 0
    chunk = -(-count // n)
    want = np.zeros(count, dtype=np.float32)
    for k in range(n):
        base, ln_k = min(count, k * chunk), max(0, min(chunk, count - k * chunk))
        lo = base
        for i, ln in enumerate(orc.mesh_chunk_segments(ln_k, n, 4, False)):
            order = mesh_chunk_order(n, k, i)
            acc = ins[order[0]][lo:lo + ln].copy()
            for t in order[1:]:
                acc = ins[t][lo:lo + ln] + acc
            want[lo:lo + ln] = acc
            lo += ln
    for o in outs:
        assert np.array_equal(o.view(np.uint32), want.view(np.uint32))


def test_reduce_scatter_v_mesh_chunk_rotation(orc):
    rng = np.random.default_rng(330)
    n = 5
    counts = [30000, 0, 7, 4100, 12345]
    displs = [100, 40000, 31000, 50000, 60000]
    total = 80000
    ins = wide_f32(rng, n, total)
    outs = [np.zeros(max(c, 1), dtype=np.float32) for c in counts]
    assert orc.reduce_scatter_v(ins, outs, counts, displs, F32, SUM, algo="mesh_chunk") == 0
    for k in range(n):
        lo = 0
        for i, ln in enumerate(orc.mesh_chunk_segments(counts[k], n, 4, True)):
            order = mesh_chunk_order(n, k, i)
            a, b = displs[k] + lo, displs[k] + lo + ln
            acc = ins[order[0]][a:b].copy()
            for t in order[1:]:
                acc = ins[t][a:b] + acc
            assert np.array_equal(outs[k][lo:lo + ln].view(np.uint32), acc.view(np.uint32)), (k, i)
            lo += ln


def test_order_preserved_six_block_example(orc):
    """The worked example in the reference's own comment: E->A, F->B, C->(AE), D->(BF), (BFD)->(AEC)."""
    rng = np.random.default_rng(30)
    n, c = 6, 300
    ins = wide_f32(rng, n, n * c)
    outs = outs_like(ins, c)
    assert orc.reduce_scatter(ins, outs, c, F32, SUM, algo="order_preserved") == 0
    for k in range(n):
        slot = [ins[t][k * c:(k + 1) * c].copy() for t in range(n)]
        for src, dst in GOLD["order_preserved_six_blocks"]["steps"]:
            slot[dst] = slot[src] + slot[dst]
        assert np.array_equal(outs[k].view(np.uint32), slot[0].view(np.uint32))


def test_order_preserved_n8_tree(orc):
    rng = np.random.default_rng(31)
    n, count = 8, 999
    x = wide_f32(rng, n, count)
    outs = outs_like(x)
    assert orc.all_reduce(x, outs, count, F32, SUM, algo="order_preserved") == 0
    want = ((x[4] + x[0]) + (x[6] + x[2])) + ((x[5] + x[1]) + (x[7] + x[3]))
    # association: ((x0+x4)+(x2+x6)) + ((x1+x5)+(x3+x7)); fp add is commutative bit for bit
    assert np.array_equal(outs[3].view(np.uint32), want.view(np.uint32))


def test_aiv_mesh_chunk_rotation(orc):
    rng = np.random.default_rng(40)
    n, c = 4, 103     # 103 = 4*25 + 3: the last chunk takes the remainder
    ins = wide_f32(rng, n, n * c)
    outs = outs_like(ins, c)
    assert orc.reduce_scatter(ins, outs, c, F32, SUM, algo="aiv_mesh") == 0
    per = c // n
    for k in range(n):
        for ch in range(n):
            lo = ch * per
            hi = c if ch == n - 1 else lo + per
            acc = ins[ch][k * c + lo:k * c + hi].copy()
            for i in range(1, n):
                acc = ins[(ch + i) % n][k * c + lo:k * c + hi] + acc
            assert np.array_equal(outs[k][lo:hi].view(np.uint32), acc.view(np.uint32))


# ---------------------------------------------------------------------------------------------
# RHD (a11): message-passing simulation vs an independent recursive closed form
# ---------------------------------------------------------------------------------------------
def rhd_tree(x, p, i, op):
    """Value of data unit i after RHD: holder f folds, at halving step k, the partial of f ^ (P >> (k+1))
    (incoming = src) into its own (dst); virtual rank v < r starts from x[v+r] (+) x[v]."""
    hp = 1
    while hp <= p // 2:
        hp *= 2
    r, P = p - hp, hp
    K = P.bit_length() - 1
    f = i if i < r else i - r

    def leaf(v):
        return f32_op(x[v + r], x[v], op) if v < r else x[v + r]

    def held(k, v):
        if k < 0:
            return leaf(v)
        dist = P >> (k + 1)
        return f32_op(held(k - 1, v ^ dist), held(k - 1, v), op)

    return held(K - 1, f)


def test_rhd_p6_worked_example(orc):
    rng = np.random.default_rng(50)
    p, c = 6, 200
    ins = wide_f32(rng, p, p * c)
    outs = outs_like(ins, c)
    assert orc.reduce_scatter(ins, outs, c, F32, SUM, algo="rhd") == 0
    for k in range(p):
        x = [ins[t][k * c:(k + 1) * c] for t in range(p)]
        want = ((x[0] + x[2]) + x[4]) + ((x[1] + x[3]) + x[5])
        assert np.array_equal(outs[k].view(np.uint32), want.view(np.uint32)), k


@pytest.mark.parametrize("p", [2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 17])
@pytest.mark.parametrize("op", [SUM, MAX, MIN])
def test_rhd_reduce_scatter_matches_closed_form(orc, p, op):
    rng = np.random.default_rng(100 * p + op)
    c = 64
    ins = wide_f32(rng, p, p * c) if op == SUM else tricky_f32(rng, p, p * c)
    outs = outs_like(ins, c)
    assert orc.reduce_scatter(ins, outs, c, F32, op, algo="rhd") == 0
    for k in range(p):
        x = [ins[t][k * c:(k + 1) * c] for t in range(p)]
        assert bits_equal_nan_class(outs[k], rhd_tree(x, p, k, op)), (p, k)


@pytest.mark.parametrize("p,count", [(6, 6 * 40), (6, 6 * 40 + 5), (5, 3), (3, 100), (12, 1000), (7, 7), (8, 64)])
@pytest.mark.parametrize("op", [SUM, MAX])
def test_rhd_all_reduce_units_and_tail(orc, p, count, op):
    rng = np.random.default_rng(p * 7 + count)
    ins = wide_f32(rng, p, count) if op == SUM else tricky_f32(rng, p, count)
    outs = outs_like(ins)
    assert orc.all_reduce(ins, outs, count, F32, op, algo="rhd") == 0
    unit = count // p
    want = np.zeros(count, dtype=np.float32)
    for i in range(p):
        lo, hi = i * unit, (i + 1) * unit
        want[lo:hi] = rhd_tree([x[lo:hi] for x in ins], p, i, op)
    for e in range(unit * p, count):       # padded tail: element e sits alone in unit e - unit*p
        want[e:e + 1] = rhd_tree([x[e:e + 1] for x in ins], p, e - unit * p, op)
    for o in outs:
        assert bits_equal_nan_class(o, want)


def test_rhd_all_reduce_loop_bound_changes_only_roles(orc):
    """A bounded staging buffer re-cuts the units per loop; integer results cannot depend on it."""
    rng = np.random.default_rng(60)
    p, count = 6, 1000
    ins = [rng.integers(-2 ** 31, 2 ** 31 - 1, count, dtype=np.int32) for _ in range(p)]
    a, b = outs_like(ins), outs_like(ins)
    assert orc.all_reduce(ins, a, count, I32, SUM, algo="rhd") == 0
    assert orc.all_reduce(ins, b, count, I32, SUM, algo="rhd", max_count_per_loop=120) == 0
    want = np.sum(np.stack(ins).astype(np.int64), axis=0).astype(np.int32)
    assert np.array_equal(a[0], want) and np.array_equal(b[5], want)


# ---------------------------------------------------------------------------------------------
# Every algorithm uses every rank exactly once; integer results are order independent
# ---------------------------------------------------------------------------------------------
AR_ALGOS = ["mesh", "two_shot", "rhd", "nhr", "order_preserved", "mesh_chunk"]
RS_ALGOS = ["mesh", "nhr", "rhd", "order_preserved", "aiv_mesh", "mesh_chunk"]


@pytest.mark.parametrize("n", [1, 2, 3, 5, 6, 7, 8, 16, 33, 64])
def test_every_rank_contributes_once(orc, n):
    count = 2 * n + 3
    ins = [np.full(count, np.uint64(1) << np.uint64(r), dtype=np.uint64) for r in range(n)]
    full = np.uint64((1 << n) - 1)
    for algo in AR_ALGOS:
        outs = outs_like(ins)
        assert orc.all_reduce(ins, outs, count, U64, SUM, algo=algo) == 0, algo
        for o in outs:
            assert np.all(o == full), (algo, n)
    c = 7
    ins = [np.full(n * c, np.uint64(1) << np.uint64(r), dtype=np.uint64) for r in range(n)]
    for algo in RS_ALGOS:
        outs = outs_like(ins, c)
        assert orc.reduce_scatter(ins, outs, c, U64, SUM, algo=algo) == 0, algo
        for o in outs:
            assert np.all(o == full), (algo, n)


@pytest.mark.parametrize("dtype,npdt", [(I8, np.int8), (I16, np.int16), (I32, np.int32), (I64, np.int64)])
def test_integer_results_match_modular_closed_form(orc, dtype, npdt):
    rng = np.random.default_rng(int(dtype) + 70)
    n, count = 6, 1234
    info = np.iinfo(npdt)
    ins = [rng.integers(info.min, info.max, count, dtype=npdt, endpoint=True) for _ in range(n)]
    stack = np.stack(ins).astype(object)
    bits = info.bits
    for op in (SUM, PROD, MAX, MIN):
        if op == PROD and dtype == I16:
            continue
        if op == SUM:
            want = [sum(int(v) for v in col) for col in stack.T]
        elif op == PROD:
            want = []
            for col in stack.T:
                acc = 1
                for v in col:
                    acc *= int(v)
                want.append(acc)
        elif op == MAX:
            want = [max(int(v) for v in col) for col in stack.T]
        else:
            want = [min(int(v) for v in col) for col in stack.T]
        want = np.array([w % (1 << bits) for w in want], dtype=object)
        for algo in AR_ALGOS:
            outs = outs_like(ins)
            assert orc.all_reduce(ins, outs, count, dtype, op, algo=algo) == 0
            got = np.array([int(v) % (1 << bits) for v in outs[n - 1]], dtype=object)
            assert np.array_equal(got, want), (algo, op)


def test_half_accumulation_modes(orc):
    """ACC_FP32: one rounding at the end; ACC_STEP: the host pattern rounds after every pair."""
    rng = np.random.default_rng(80)
    n, count = 8, 5000
    f = [rng.standard_normal(count).astype(np.float32) for _ in range(n)]
    for dtype, narrow, widen in ((F16, lambda a: a.astype(np.float16).view(np.uint16),
                                  lambda h: h.view(np.float16).astype(np.float32)),
                                 (BF16, orc.np_fp32_to_bf16_bits, orc.bf16_bits_to_fp32)):
        ins = [narrow(x) for x in f]
        w = [widen(h) for h in ins]
        outs = outs_like(ins)
        assert orc.all_reduce(ins, outs, count, dtype, SUM, acc=orc.ACC_FP32) == 0
        acc = w[0].copy()
        for r in range(1, n):
            acc = w[r] + acc
        assert np.array_equal(outs[0], narrow(acc))
        assert orc.all_reduce(ins, outs, count, dtype, SUM, acc=orc.ACC_STEP) == 0
        acc = w[0].copy()
        for r in range(1, n):
            acc = widen(narrow(w[r] + acc))
        assert np.array_equal(outs[0], narrow(acc))
        # fp32 accumulation is within 1 ulp of the exactly-rounded sum
        exact = narrow(np.sum(np.stack(w).astype(np.float64), axis=0).astype(np.float32))
        assert orc.all_reduce(ins, outs, count, dtype, SUM, acc=orc.ACC_FP32) == 0
        d = np.abs(outs[0].astype(np.int32) - exact.astype(np.int32))
        same_sign = (outs[0] >> 15) == (exact >> 15)
        assert np.all(d[same_sign] <= 1)


def test_admission(orc):
    a = [np.zeros(8, dtype=np.uint16) for _ in range(2)]
    o = outs_like(a)
    assert orc.all_reduce(a, o, 8, 7, SUM) == 5         # uint8 cannot be reduced
    assert orc.all_reduce(a, o, 8, I16, PROD) == 5      # PROD not defined for int16
    assert orc.all_reduce(a, o, 8, BF16, PROD) == 5
    assert orc.all_reduce(a, o, 8, BF16, MAX) == 0
    assert orc.all_reduce(a, o, 0, F16, SUM) == 0


# ---------------------------------------------------------------------------------------------
# Copies (a13, a14, a15): index maps on distinct byte patterns
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 2, 3, 8])
def test_all_gather_index_map(orc, n):
    c = 37
    ins = [(np.arange(c, dtype=np.uint16) + 1000 * r).astype(np.uint16) for r in range(n)]
    outs = [np.zeros(n * c, dtype=np.uint16) for _ in range(n)]
    assert orc.all_gather(ins, outs, c, F16) == 0
    for o in outs:
        for r in range(n):
            assert np.array_equal(o[r * c:(r + 1) * c], ins[r])


def test_all_gather_v_unordered_with_holes(orc):
    n = 4
    counts = [5, 0, 9, 3]
    displs = [20, 7, 0, 11]            # unordered, holes at [9,11) and [14,20)
    ins = [np.full(max(c, 1), 10 + r, dtype=np.int32) for r, c in enumerate(counts)]
    outs = [np.full(25, -1, dtype=np.int32) for _ in range(n)]
    assert orc.all_gather_v(ins, outs, counts, displs, I32) == 0
    want = np.full(25, -1, dtype=np.int32)
    want[20:25], want[0:9], want[11:14] = 10, 12, 13
    for o in outs:
        assert np.array_equal(o, want)
    assert orc.all_gather_v(ins, outs, [5, 5, 0, 0], [0, 4, 0, 0], I32) == 1   # overlap


@pytest.mark.parametrize("n", [2, 3, 8])
def test_all_to_all_v_index_map(orc, n):
    rng = np.random.default_rng(n)
    send_counts = rng.integers(0, 6, size=(n, n)).astype(np.uint64)
    recv_counts = send_counts.T.copy()
    # displacements with gaps, in shuffled block order
    sdispls = np.zeros((n, n), dtype=np.uint64)
    rdispls = np.zeros((n, n), dtype=np.uint64)
    for r in range(n):
        for tab, cnts in ((sdispls, send_counts), (rdispls, recv_counts)):
            off = 1
            for j in rng.permutation(n):
                tab[r, j] = off
                off += int(cnts[r, j]) + int(rng.integers(0, 3))
    in_sz = int((sdispls + send_counts).max()) + 2
    out_sz = int((rdispls + recv_counts).max()) + 2
    ins = [(np.arange(in_sz, dtype=np.int64) + 10_000 * r) for r in range(n)]
    outs = [np.full(out_sz, -7, dtype=np.int64) for _ in range(n)]
    assert orc.all_to_all_v(ins, outs, send_counts, sdispls, recv_counts, rdispls, I64) == 0
    for i in range(n):
        want = np.full(out_sz, -7, dtype=np.int64)
        for j in range(n):
            c = int(send_counts[j, i])
            want[int(rdispls[i, j]):int(rdispls[i, j]) + c] = ins[j][int(sdispls[j, i]):int(sdispls[j, i]) + c]
        assert np.array_equal(outs[i], want)
    bad = recv_counts.copy()
    bad[0, 1] += 1
    assert orc.all_to_all_v(ins, outs, send_counts, sdispls, bad, rdispls, I64) == 1


# ---------------------------------------------------------------------------------------------
# AllReduce two-shot over symmetric memory: slice k starts from rank k's input (two_shot.cc:341-357)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n,count", [(2, 7), (3, 100), (5, 3), (8, 1031), (16, 40)])
def test_all_reduce_symmetric_two_shot_slice_k_starts_from_rank_k(orc, n, count):
    rng = np.random.default_rng(n * 10 + count)
    ins = wide_f32(rng, n, count)
    outs = outs_like(ins)
    assert orc.all_reduce(ins, outs, count, F32, SUM, algo="mesh_symmetric") == 0
    sl = -(-count // n)                               # ceil(count / n), two_shot.cc:184
    want = np.zeros(count, dtype=np.float32)
    for k in range(n):
        lo, hi = min(count, k * sl), min(count, (k + 1) * sl)
        acc = ins[k][lo:hi].copy()
        for t in range(n):
            if t != k:
                acc = ins[t][lo:hi] + acc
        want[lo:hi] = acc
    for r in range(n):
        assert np.array_equal(outs[r].view(np.uint32), want.view(np.uint32)), r
    if n > 2 and count > n:                             # and it is a different order from the plain two-shot
        plain = outs_like(ins)
        assert orc.all_reduce(ins, plain, count, F32, SUM, algo="two_shot") == 0
        assert not np.array_equal(plain[0].view(np.uint32), want.view(np.uint32))
