"""GPU parity: the HIP data plane, called through the C ABI, against the CPU oracle on the same seeded
inputs.  Bar: bit-exact for integers, copies / packs, fp32 / fp64 and every MAX / MIN; fp16 / bf16 SUM
are compared bit-exactly with the oracle's fp32-accumulate mode and within 1 ulp of a float64
reference (the tolerance the task states for half precision).  A NaN produced by arithmetic only has
to be a NaN on both sides (payloads of arithmetic NaNs are machine specific)."""
import numpy as np
import pytest

import oracle
import hccl_amd
from hccl_amd import HcclDataType as DT, HcclReduceOp as OP, OpKind

from gpu_util import World, dev_zeros, require_library_on_gpu, same_bits_nan_class, to_dev, to_host

pytestmark = pytest.mark.gpu

SUM, PROD, MAX, MIN = range(4)
NP = {DT.INT8: np.int8, DT.INT16: np.int16, DT.INT32: np.int32, DT.INT64: np.int64, DT.UINT64: np.uint64,
      DT.FP16: np.uint16, DT.BFP16: np.uint16, DT.FP32: np.float32, DT.FP64: np.float64}
FLOAT_VIEW = {DT.FP16: lambda a: a.view(np.float16), DT.BFP16: oracle.bf16_bits_to_fp32,
              DT.FP32: lambda a: a, DT.FP64: lambda a: a}
REDUCE_TYPES = [DT.INT8, DT.INT16, DT.INT32, DT.INT64, DT.UINT64, DT.FP16, DT.BFP16, DT.FP32, DT.FP64]


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


def gen(dtype, op, rng, count):
    """Inputs that make a wrong order, a wrong operand role or a wrong rounding visible."""
    npdt = NP[dtype]
    if dtype in (DT.INT8, DT.INT16, DT.INT32, DT.INT64, DT.UINT64):
        info = np.iinfo(npdt)
        a = rng.integers(info.min, info.max, count, dtype=npdt, endpoint=True)
        if op == PROD:   # keep half of the lanes small so that products stay informative
            small = rng.choice(np.array([-2, -1, 1, 2, 3] if info.min < 0 else [1, 2, 3], dtype=npdt), count)
            a = np.where(rng.random(count) < 0.5, small, a)
        return a
    if op in (MAX, MIN):
        pools = {DT.FP32: np.array([0, 0x80000000, 0x7FC00001, 0x7FC00002, 0xFFC00003, 0x3F800000, 0xBF800000,
                                    0x7F800000, 0xFF800000, 0x00000001], dtype=np.uint32),
                 DT.FP64: np.array([0, 1 << 63, 0x7FF8000000000001, 0xFFF8000000000003, 0x3FF0000000000000,
                                    0xBFF0000000000000, 0x7FF0000000000000], dtype=np.uint64),
                 DT.FP16: np.array([0, 0x8000, 0x7E01, 0x7E02, 0xFE03, 0x3C00, 0xBC00, 0x7C00, 0xFC00, 0x0001, 0x7D01],
                                   dtype=np.uint16),
                 DT.BFP16: np.array([0, 0x8000, 0x7FC1, 0x7FC2, 0xFFC3, 0x3F80, 0xBF80, 0x7F80, 0xFF80, 0x0001, 0x7FA1],
                                    dtype=np.uint16)}
        pool = pools[dtype]
        a = pool[rng.integers(0, pool.size, count)]
        rnd = rng.standard_normal(count)
        mix = rng.random(count) < 0.5
        if dtype == DT.FP32:
            return np.where(mix, rnd.astype(np.float32).view(np.uint32), a).view(np.float32)
        if dtype == DT.FP64:
            return np.where(mix, rnd.view(np.uint64), a).view(np.float64)
        if dtype == DT.FP16:
            return np.where(mix, rnd.astype(np.float16).view(np.uint16), a)
        return np.where(mix, oracle.np_fp32_to_bf16_bits(rnd.astype(np.float32)), a)
    scale = 10.0 ** rng.integers(-3, 3, count) if op == SUM else 1.0 + 0.0 * rng.random(count)
    base = rng.standard_normal(count) * scale
    if op == PROD:
        base = 1.0 + 0.5 * rng.standard_normal(count)
    if dtype == DT.FP32:
        a = base.astype(np.float32)
        a[::97] = np.float32(1e-41)      # fp32 subnormals must survive
        a[5::101] = np.float32(np.inf)
        return a
    if dtype == DT.FP64:
        return base.astype(np.float64)
    if dtype == DT.FP16:
        h = base.astype(np.float16)
        h[::89] = np.float16(6e-8)       # fp16 subnormal
        h[7::103] = np.float16(60000.0)  # sums overflow to Inf
        return h.view(np.uint16)
    return oracle.np_fp32_to_bf16_bits(base.astype(np.float32))


def check(dtype, op, got, want, what):
    fv = FLOAT_VIEW.get(dtype)
    if fv is not None and op in (SUM, PROD):
        ok = same_bits_nan_class(got, want, fv)
    else:
        ok = np.array_equal(got.view(np.uint8), want.view(np.uint8))
    if not ok:
        diff = np.nonzero(got.view(np.uint8).reshape(got.size, -1) != want.view(np.uint8).reshape(want.size, -1))[0]
        diff = np.unique(diff)
        raise AssertionError("%s: %d of %d elements differ, first at %s (got %r want %r)" % (
            what, diff.size, got.size, diff[:4], got[diff[:4]], want[diff[:4]]))


def pad_of(pad, r, which):
    """pad may be a number (every buffer alike) or a function (rank, 'send' | 'recv') -> bytes."""
    return pad(r, which) if callable(pad) else pad


def order_of(algo, dtype, op, reduce_scatter):
    """PROD and the 64-bit types are not offered by the reference's write-reduce templates: mesh order."""
    host_only = op == PROD or dtype in (DT.INT64, DT.UINT64, DT.FP64)
    if host_only and (algo in ("nhr", "rhd", "mesh_chunk", "mesh_concur", "aiv_mesh") or (algo == "ring" and reduce_scatter)):
        return "mesh"
    return algo


def run_all_reduce(world, dtype, op, count, algo, seed, pad=0, in_place=False, max_count_per_loop=0):
    rng = np.random.default_rng(seed)
    n = world.n
    ins = [gen(dtype, op, rng, count) for _ in range(n)]
    want = [np.zeros(count, dtype=NP[dtype]) for _ in range(n)]
    assert oracle.all_reduce(ins, want, count, int(dtype), op, acc=oracle.ACC_FP32,
                             algo=order_of(algo, dtype, op, False), max_count_per_loop=max_count_per_loop) == 0
    sends = [to_dev(x, pad_of(pad, r, "send")) for r, x in enumerate(ins)]
    recvs = sends if in_place else [dev_zeros(x.nbytes, pad_of(pad, r, "recv")) for r, x in enumerate(ins)]
    world.all_reduce(sends, recvs, count, dtype, op, algo)
    for r in range(n):
        check(dtype, op, to_host(recvs[r], NP[dtype]), want[r],
              "all_reduce %s %s n=%d count=%d algo=%s rank=%d" % (dtype.name, OP(op).name, n, count, algo, r))


def run_reduce_scatter(world, dtype, op, c, algo, seed, pad=0, max_count_per_loop=0):
    rng = np.random.default_rng(seed)
    n = world.n
    ins = [gen(dtype, op, rng, n * c) for _ in range(n)]
    want = [np.zeros(c, dtype=NP[dtype]) for _ in range(n)]
    kw = {"max_count_per_loop": max_count_per_loop} if max_count_per_loop else {}
    assert oracle.reduce_scatter(ins, want, c, int(dtype), op, acc=oracle.ACC_FP32,
                                 algo=order_of(algo, dtype, op, True), **kw) == 0
    sends = [to_dev(x, pad_of(pad, r, "send")) for r, x in enumerate(ins)]
    recvs = [dev_zeros(c * ins[0].itemsize, pad_of(pad, r, "recv")) for r in range(n)]
    world.reduce_scatter(sends, recvs, c, dtype, op, algo)
    for r in range(n):
        check(dtype, op, to_host(recvs[r], NP[dtype]), want[r],
              "reduce_scatter %s %s n=%d c=%d algo=%s rank=%d" % (dtype.name, OP(op).name, n, c, algo, r))


# ---------------------------------------------------------------------------------------------
# Type / op matrix
# ---------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def world8():
    w = World(8)
    yield w
    w.close()


@pytest.mark.parametrize("dtype", REDUCE_TYPES)
@pytest.mark.parametrize("op", [SUM, PROD, MAX, MIN])
def test_all_reduce_type_op_matrix(world8, dtype, op):
    if op == PROD and dtype in (DT.INT16, DT.BFP16):
        pytest.skip("PROD is not defined for this type (reference op_common.cc:4392-4413)")
    run_all_reduce(world8, dtype, op, 40_007, "mesh", seed=int(dtype) * 10 + op)


@pytest.mark.parametrize("dtype", REDUCE_TYPES)
@pytest.mark.parametrize("op", [SUM, MAX])
def test_reduce_scatter_type_matrix(world8, dtype, op):
    run_reduce_scatter(world8, dtype, op, 8_192 + 16, "mesh", seed=500 + int(dtype) * 10 + op)


# ---------------------------------------------------------------------------------------------
# Algorithms x rank counts x ragged counts (the sweep of the reference's vector-core unit tests:
# ranks {1,2,3,4,8,16,32}, counts not divisible by the rank count and smaller than it)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 2, 3, 5, 6, 7, 8, 16, 33, 64])
def test_all_reduce_algorithms_and_ragged_counts(n):
    w = World(n)
    try:
        for algo in ("mesh", "ring", "rhd", "nhr", "order_preserved", "mesh_symmetric", "mesh_chunk", "mesh_concur"):
            for count in (1, 3, 17, 129, 1023, 4093, 65_543):
                run_all_reduce(w, DT.FP32, SUM, count, algo, seed=n * 1000 + count)
            run_all_reduce(w, DT.FP32, MAX, 2_051, algo, seed=n)
            run_all_reduce(w, DT.BFP16, SUM, 4_099, algo, seed=n + 1)
            run_all_reduce(w, DT.INT32, PROD, 1_025, algo, seed=n + 2)
    finally:
        w.close()


@pytest.mark.parametrize("n", [1, 2, 3, 5, 6, 8, 16, 64])
def test_reduce_scatter_algorithms_and_ragged_counts(n):
    w = World(n)
    try:
        for algo in ("mesh", "ring", "nhr", "rhd", "order_preserved", "aiv_mesh", "mesh_symmetric", "mesh_chunk"):
            for c in (1, 3, 17, 129, 1024, 4093):
                run_reduce_scatter(w, DT.FP32, SUM, c, algo, seed=n * 2000 + c)
            run_reduce_scatter(w, DT.FP32, MIN, 515, algo, seed=n + 3)
            run_reduce_scatter(w, DT.FP16, SUM, 2_048, algo, seed=n + 4)
    finally:
        w.close()


def test_unaligned_buffers_and_in_place(world8):
    for pad in (2, 4, 8):          # payload starts 2 / 4 / 8 bytes past a 16-byte boundary
        run_all_reduce(world8, DT.FP16, SUM, 5_001, "mesh", seed=pad, pad=pad)
        run_reduce_scatter(world8, DT.BFP16, SUM, 999, "mesh", seed=pad + 10, pad=pad)
    # every buffer at its own offset from a 16-byte boundary: sources are read unaligned; AllReduce into
    # differently aligned recvBufs is the one case left to the element path
    mixed = lambda r, which: (2 * r + (4 if which == "recv" else 0)) % 16
    run_all_reduce(world8, DT.FP16, SUM, 20_011, "mesh", seed=31, pad=mixed)
    run_all_reduce(world8, DT.BFP16, MAX, 4_097, "rhd", seed=32, pad=mixed)
    run_all_reduce(world8, DT.FP16, SUM, 20_011, "nhr", seed=33, pad=lambda r, which: 2 * r % 16 if which == "send" else 6)
    run_reduce_scatter(world8, DT.BFP16, SUM, 5_003, "ring", seed=34, pad=mixed)
    run_reduce_scatter(world8, DT.INT8, SUM, 5_003, "mesh", seed=35, pad=lambda r, which: (r * 5 + 1) % 16)
    run_reduce_scatter(world8, DT.INT32, MAX, 1_001, "rhd", seed=36, pad=lambda r, which: 4 * (r % 4))
    run_all_reduce(world8, DT.FP32, SUM, 70_001, "mesh", seed=77, in_place=True)
    run_all_reduce(world8, DT.INT64, MAX, 9_999, "rhd", seed=78, in_place=True)


# ---------------------------------------------------------------------------------------------
# The benchmark configurations (C1 at its real size; the others at sizes the oracle finishes in seconds;
# their full sizes are covered by tests/test_gpu_full_size.py through size-independent properties)
# ---------------------------------------------------------------------------------------------
def test_config1_all_reduce_fp32_n8_rank_order(world8):
    rng = np.random.default_rng(0xC0FFEE + 1000)
    count = 1_048_576
    ins = [rng.uniform(-1.0, 1.0, count).astype(np.float32) for _ in range(8)]
    want = ins[0].copy()
    for r in range(1, 8):
        want = ins[r] + want                      # (((x0+x1)+x2)...+x7)
    o = [np.zeros(count, dtype=np.float32) for _ in range(8)]
    assert oracle.all_reduce(ins, o, count, 4, SUM, algo="ring") == 0
    assert np.array_equal(o[0].view(np.uint32), want.view(np.uint32))
    sends = [to_dev(x) for x in ins]
    recvs = [dev_zeros(x.nbytes) for x in ins]
    world8.all_reduce(sends, recvs, count, DT.FP32, SUM, "ring")
    for r in range(8):
        assert np.array_equal(to_host(recvs[r], np.uint32), want.view(np.uint32))


def test_config2_reduce_scatter_bf16_n8(world8):
    rng = np.random.default_rng(0xC0FFEE + 2000)
    c = 1 << 20
    f = [rng.standard_normal(8 * c).astype(np.float32) for _ in range(8)]
    ins = [oracle.np_fp32_to_bf16_bits(x) for x in f]
    sends = [to_dev(x) for x in ins]
    for algo in ("ring", "mesh"):
        want = [np.zeros(c, dtype=np.uint16) for _ in range(8)]
        assert oracle.reduce_scatter(ins, want, c, 11, SUM, acc=oracle.ACC_FP32, algo=algo) == 0
        recvs = [dev_zeros(2 * c) for _ in range(8)]
        world8.reduce_scatter(sends, recvs, c, DT.BFP16, SUM, algo)
        w64 = np.stack([oracle.bf16_bits_to_fp32(x).astype(np.float64) for x in ins])
        for k in range(8):
            got = to_host(recvs[k], np.uint16)
            assert np.array_equal(got, want[k]), (algo, k)
            # within 1 ulp of the correctly rounded exact sum
            exact = oracle.np_fp32_to_bf16_bits(w64[:, k * c:(k + 1) * c].sum(axis=0).astype(np.float32))
            d = np.abs(got.astype(np.int32) - exact.astype(np.int32))
            assert d[(got >> 15) == (exact >> 15)].max() <= 1


def test_config3_all_reduce_int32_n16_max_and_prod():
    w = World(16)
    try:
        rng = np.random.default_rng(0xC0FFEE + 3000)
        count = 1 << 20
        mx = [rng.integers(-2 ** 31, 2 ** 31 - 1, count, dtype=np.int32, endpoint=True) for _ in range(16)]
        pr = [rng.choice(np.array([-2, -1, 1, 2], dtype=np.int32), count) for _ in range(16)]
        for ins, op in ((mx, MAX), (pr, PROD)):
            stack = np.stack(ins).astype(np.int64)
            if op == MAX:
                want = stack.max(axis=0).astype(np.int32)
            else:
                acc = np.ones(count, dtype=np.uint64)
                for x in ins:
                    acc = (acc * x.astype(np.int64).astype(np.uint64)) & np.uint64(0xFFFFFFFF)
                want = acc.astype(np.uint32).view(np.int32)
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(4 * count) for _ in ins]
            w.all_reduce(sends, recvs, count, DT.INT32, op, "mesh")
            for r in (0, 7, 15):
                assert np.array_equal(to_host(recvs[r], np.int32), want)
    finally:
        w.close()


def test_config5a_all_reduce_fp16_rhd_n6():
    w = World(6)
    try:
        rng = np.random.default_rng(0xC0FFEE + 5000)
        count = (1 << 20) + 5           # not a multiple of 6: exercises the padded remainder
        ins = [(rng.standard_normal(count) * 0.5).astype(np.float16).view(np.uint16) for _ in range(6)]
        x = [h.view(np.float16).astype(np.float32) for h in ins]
        tree = ((x[0] + x[2]) + x[4]) + ((x[1] + x[3]) + x[5])      # the p = 6 association, fp32 accumulate
        want = tree.astype(np.float16).view(np.uint16)
        o = [np.zeros(count, dtype=np.uint16) for _ in range(6)]
        assert oracle.all_reduce(ins, o, count, 3, SUM, acc=oracle.ACC_FP32, algo="rhd") == 0
        assert np.array_equal(o[3], want)
        sends = [to_dev(h) for h in ins]
        recvs = [dev_zeros(2 * count) for _ in ins]
        w.all_reduce(sends, recvs, count, DT.FP16, SUM, "rhd")
        for r in range(6):
            assert np.array_equal(to_host(recvs[r], np.uint16), want)
    finally:
        w.close()


def test_hccl_deterministic_strict_selects_the_order_preserved_fold(monkeypatch):
    """reference order_preserved_common.h:104-114: strict + float + SUM/PROD + more than two ranks."""
    import hccl_amd
    monkeypatch.setenv("HCCL_DETERMINISTIC", "Strict")
    n, count = 6, 4099
    w = World(n)                                     # the variable is read when the world is created
    monkeypatch.delenv("HCCL_DETERMINISTIC")
    try:
        rng = np.random.default_rng(77)
        ins = [gen(DT.FP32, SUM, rng, count) for _ in range(n)]
        strict = [np.zeros(count, dtype=np.float32) for _ in range(n)]
        plain = [np.zeros(count, dtype=np.float32) for _ in range(n)]
        assert oracle.all_reduce(ins, strict, count, int(DT.FP32), SUM, algo="order_preserved") == 0
        assert oracle.all_reduce(ins, plain, count, int(DT.FP32), SUM, algo="mesh") == 0
        assert not np.array_equal(strict[0].view(np.uint32), plain[0].view(np.uint32))   # the orders are told apart
        sends = [to_dev(x) for x in ins]
        recvs = [dev_zeros(x.nbytes) for x in ins]
        w.all_reduce(sends, recvs, count, DT.FP32, SUM, "mesh")                  # configured: mesh; strict wins
        check(DT.FP32, SUM, to_host(recvs[2], np.float32), strict[2], "strict all_reduce")
        # MAX is not covered by the rule: the configured order applies
        ins = [gen(DT.FP32, MAX, rng, count) for _ in range(n)]
        want = [np.zeros(count, dtype=np.float32) for _ in range(n)]
        assert oracle.all_reduce(ins, want, count, int(DT.FP32), MAX, algo="mesh") == 0
        sends = [to_dev(x) for x in ins]
        w.all_reduce(sends, recvs, count, DT.FP32, MAX, "mesh")
        check(DT.FP32, MAX, to_host(recvs[4], np.float32), want[4], "strict all_reduce MAX")
        # ReduceScatter follows the same rule
        c = 1031
        ins = [gen(DT.FP32, SUM, rng, n * c) for _ in range(n)]
        want = [np.zeros(c, dtype=np.float32) for _ in range(n)]
        assert oracle.reduce_scatter(ins, want, c, int(DT.FP32), SUM, algo="order_preserved") == 0
        sends = [to_dev(x) for x in ins]
        recvs = [dev_zeros(4 * c) for _ in range(n)]
        w.reduce_scatter(sends, recvs, c, DT.FP32, SUM, "mesh")
        for r in range(n):
            check(DT.FP32, SUM, to_host(recvs[r], np.float32), want[r], "strict reduce_scatter rank %d" % r)
    finally:
        w.close()


def test_element_by_element_path_for_every_type(monkeypatch):
    """The path heads, tails and single elements take, forced for whole buffers (HCCL_AMD_REDUCE_VECTOR=0)."""
    monkeypatch.setenv("HCCL_AMD_REDUCE_VECTOR", "0")
    w = World(5)                                     # the variable is read when the world is created
    monkeypatch.delenv("HCCL_AMD_REDUCE_VECTOR")
    try:
        for dtype in REDUCE_TYPES:
            for op in (SUM, PROD, MAX, MIN):
                if op == PROD and dtype in (DT.INT16, DT.BFP16):
                    continue
                run_all_reduce(w, dtype, op, 1_237, "mesh", seed=900 + int(dtype) * 4 + op)
            run_reduce_scatter(w, dtype, SUM, 333, "nhr", seed=950 + int(dtype))
            run_all_reduce(w, dtype, MAX, 515, "rhd", seed=960 + int(dtype))
    finally:
        w.close()


def test_workgroups_that_loop_over_several_positions(monkeypatch):
    """With the grid capped (HCCL_AMD_REDUCE_BLOCKS) every workgroup strides over many vector positions."""
    monkeypatch.setenv("HCCL_AMD_REDUCE_BLOCKS", "7")
    w = World(6)
    monkeypatch.delenv("HCCL_AMD_REDUCE_BLOCKS")
    try:
        run_all_reduce(w, DT.FP32, SUM, 70_001, "mesh", seed=1)
        run_all_reduce(w, DT.BFP16, SUM, 50_003, "rhd", seed=2)
        run_all_reduce(w, DT.FP16, MAX, 33_333, "nhr", seed=3, pad=2)
        run_reduce_scatter(w, DT.INT8, SUM, 20_011, "ring", seed=4)
        run_reduce_scatter(w, DT.INT32, PROD, 9_999, "aiv_mesh", seed=5)
    finally:
        w.close()


@pytest.mark.parametrize("n", [2, 5, 16, 33])
def test_all_reduce_as_fold_and_fan_out(monkeypatch, n):
    """The two-kernel form of AllReduce (fold into the first recvBuf, that range to the other recvBufs with a
    wavefront per destination), forced for small messages with pieces of 4 KiB: counts that span several pieces and
    end in a ragged one, orders with a fold program per sub-segment (pieces of whole sub-segments, and parts of a
    sub-segment that is longer than a piece), recvBufs that share their misalignment and recvBufs that do not."""
    monkeypatch.setenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS", "1")
    monkeypatch.setenv("HCCL_AMD_ALLREDUCE_PIECE_BYTES", "4096")
    w = World(n)
    monkeypatch.delenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS")
    monkeypatch.delenv("HCCL_AMD_ALLREDUCE_PIECE_BYTES")
    try:
        seed = 2000 + n
        for dtype in REDUCE_TYPES:
            for op in (SUM, MAX):
                run_all_reduce(w, dtype, op, 4_093, "mesh", seed=seed)
                seed += 1
        run_all_reduce(w, DT.INT32, PROD, 17, "mesh", seed=seed)            # less than one piece
        run_all_reduce(w, DT.FP32, SUM, 1_024, "ring", seed=seed + 1)       # exactly one piece
        run_all_reduce(w, DT.FP32, SUM, 65_543, "ring", seed=seed + 2, pad=4)   # every buffer 4 bytes off: shared misalignment
        run_all_reduce(w, DT.BFP16, SUM, 10_007, "mesh", seed=seed + 3, pad=lambda r, which: 2 * r + (6 if which == "recv" else 0))
        run_all_reduce(w, DT.FP16, MIN, 9_001, "mesh", seed=seed + 4, in_place=True)
        run_all_reduce(w, DT.FP32, SUM, 5_000, "rhd", seed=seed + 5)        # sub-segments shorter than a piece
        run_all_reduce(w, DT.FP16, SUM, 70_001, "rhd", seed=seed + 6)       # remainder frame after the whole frames
        run_all_reduce(w, DT.BFP16, SUM, 50_003, "nhr", seed=seed + 7, pad=2)
        run_all_reduce(w, DT.INT32, SUM, 200_003, "nhr", seed=seed + 8)     # sub-segments longer than a piece
        run_all_reduce(w, DT.FP32, SUM, 33_333, "order_preserved", seed=seed + 9)
        run_all_reduce(w, DT.FP32, MAX, 20_011, "mesh_symmetric", seed=seed + 11, in_place=True)
        run_all_reduce(w, DT.FP16, SUM, 40_009, "mesh_concur", seed=seed + 16, pad=2)   # uneven last slice
        run_all_reduce(w, DT.INT8, SUM, 30_011, "mesh_chunk", seed=seed + 12)   # pieces of whole slices
        run_all_reduce(w, DT.FP32, SUM, 257, "mesh_chunk", seed=seed + 14)      # slices shorter than a piece, short last slice
        run_all_reduce(w, DT.BFP16, SUM, 3 * n + 1, "mesh_chunk", seed=seed + 15, pad=2)
        run_all_reduce(w, DT.INT8, SUM, 3, "nhr", seed=seed + 13)           # fewer elements than ranks
    finally:
        w.close()


@pytest.mark.parametrize("n,waves", [(2, 2), (5, 2), (6, 3), (8, 4), (16, 4), (3, 4)])
def test_all_reduce_with_the_stores_of_a_tile_shared_by_wavefronts(monkeypatch, n, waves):
    """The many-destination form of the fused kernel (wavefront 0 folds a tile, `waves` wavefronts store it),
    forced for small messages and with the two-kernel form off; a small grid makes every workgroup loop over tiles."""
    monkeypatch.setenv("HCCL_AMD_REDUCE_STORE_WAVES", str(waves))
    monkeypatch.setenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS", "0")
    monkeypatch.setenv("HCCL_AMD_REDUCE_BLOCKS", "24")
    w = World(n)
    monkeypatch.delenv("HCCL_AMD_REDUCE_STORE_WAVES")
    monkeypatch.delenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS")
    monkeypatch.delenv("HCCL_AMD_REDUCE_BLOCKS")
    try:
        seed = 5200 + 10 * n + waves
        for dtype in REDUCE_TYPES:
            run_all_reduce(w, dtype, SUM, 20_011, "mesh", seed=seed)
            seed += 1
        run_all_reduce(w, DT.FP32, SUM, 70_001, "nhr", seed=seed)                # nested order, LDS stack in wavefront 0
        run_all_reduce(w, DT.BFP16, SUM, 50_003, "rhd", seed=seed + 1)
        run_all_reduce(w, DT.FP16, MAX, 33_333, "order_preserved", seed=seed + 2, pad=2)   # unaligned: head and tail elements
        run_all_reduce(w, DT.INT8, MIN, 9, "mesh", seed=seed + 3)                # less than one vector
        run_all_reduce(w, DT.INT32, PROD, 4_099, "mesh", seed=seed + 4, in_place=True)
        run_all_reduce(w, DT.FP64, SUM, 12_345, "mesh", seed=seed + 5, pad=lambda r, which: r + (3 if which == "recv" else 0))
        run_reduce_scatter(w, DT.FP32, SUM, 5_001, "mesh", seed=seed + 6)        # one result stream: form not taken
    finally:
        w.close()


@pytest.mark.parametrize("n,blocks", [(2, 0), (3, 24), (5, 0), (8, 0), (8, 7)])
def test_all_reduce_and_reduce_scatter_with_two_tiles_per_wavefront(monkeypatch, n, blocks):
    """The form for launches of about one generation of wavefronts (a wavefront takes two adjacent tiles and issues
    the loads of both before it folds either), forced for every size: even and odd numbers of tiles, less than one
    tile, heads and tails off the 16-byte grid, every element type; with a small grid every workgroup strides over
    pairs.  Orders whose programs nest keep the one-tile kernel."""
    monkeypatch.setenv("HCCL_AMD_REDUCE_PAIR", "1")
    monkeypatch.setenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS", "0")
    if blocks:
        monkeypatch.setenv("HCCL_AMD_REDUCE_BLOCKS", str(blocks))
    w = World(n)
    monkeypatch.delenv("HCCL_AMD_REDUCE_PAIR")
    monkeypatch.delenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS")
    if blocks:
        monkeypatch.delenv("HCCL_AMD_REDUCE_BLOCKS")
    try:
        seed = 6100 + 10 * n + blocks
        for dtype in REDUCE_TYPES:
            run_all_reduce(w, dtype, SUM, 20_011, "mesh", seed=seed)
            seed += 1
        for count in (1, 255, 256, 257, 511, 512, 513, 768, 4096 * 3, 4096 * 4 + 1, 100_003):
            run_all_reduce(w, DT.FP32, SUM, count, "ring", seed=seed)            # 256 fp32 = one tile
            seed += 1
        run_all_reduce(w, DT.FP16, MAX, 33_333, "mesh", seed=seed, pad=2)        # unaligned: head and tail elements
        run_all_reduce(w, DT.BFP16, SUM, 50_003, "mesh", seed=seed + 1, pad=lambda r, which: 2 * r + (6 if which == "recv" else 0))
        run_all_reduce(w, DT.INT8, MIN, 9, "mesh", seed=seed + 2)                # less than one vector
        run_all_reduce(w, DT.INT32, PROD, 4_099, "mesh", seed=seed + 3, in_place=True)
        run_all_reduce(w, DT.FP64, SUM, 12_345, "mesh", seed=seed + 4, pad=lambda r, which: r + (3 if which == "recv" else 0))
        run_all_reduce(w, DT.FP32, SUM, 70_001, "nhr", seed=seed + 5)            # nested program: form not taken
        run_all_reduce(w, DT.FP32, SUM, 70_001, "mesh_symmetric", seed=seed + 6)
        run_reduce_scatter(w, DT.FP32, SUM, 5_001, "mesh", seed=seed + 7)        # one result stream, own rank first
        run_reduce_scatter(w, DT.BFP16, SUM, 10_007, "mesh", seed=seed + 8)
        run_reduce_scatter(w, DT.INT16, MAX, 513, "aiv_mesh", seed=seed + 9)
    finally:
        w.close()


@pytest.mark.parametrize("n,waves,blocks", [(2, 2, 0), (3, 4, 24), (5, 3, 0), (8, 3, 0), (8, 4, 7), (16, 2, 0), (12, 3, 5)])
def test_all_reduce_with_wavefronts_that_exchange_their_tiles_and_store_their_own_destinations(monkeypatch, n, waves, blocks):
    """The form for many destinations and a few MiB per rank (every wavefront of a workgroup folds a tile, the results
    change hands through LDS, wavefront k stores all of them to destinations k, k + waves, ...), forced for every size:
    tile counts that the workgroup's wavefronts divide and do not, less than one tile, heads and tails off the 16-byte
    grid, every element type, more wavefronts than destinations and fewer; with a small grid every workgroup strides
    on.  Results cut into sub-segments with programs of their own take it too; orders whose programs nest and results
    with one destination keep the plain kernel."""
    monkeypatch.setenv("HCCL_AMD_REDUCE_ALL_FOLD", str(waves))
    monkeypatch.setenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS", "0")
    if blocks:
        monkeypatch.setenv("HCCL_AMD_REDUCE_BLOCKS", str(blocks))
    w = World(n)
    monkeypatch.delenv("HCCL_AMD_REDUCE_ALL_FOLD")
    monkeypatch.delenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS")
    if blocks:
        monkeypatch.delenv("HCCL_AMD_REDUCE_BLOCKS")
    try:
        seed = 6500 + 10 * n + waves
        for dtype in REDUCE_TYPES:
            run_all_reduce(w, dtype, SUM, 20_011, "mesh", seed=seed)
            seed += 1
        for count in (1, 255, 256, 257, 256 * waves - 1, 256 * waves, 256 * waves + 1, 256 * (2 * waves + 1), 4096 * 3,
                      4096 * 4 + 1, 100_003):
            run_all_reduce(w, DT.FP32, SUM, count, "ring", seed=seed)            # 256 fp32 = one tile
            seed += 1
        run_all_reduce(w, DT.FP16, MAX, 33_333, "mesh", seed=seed, pad=2)        # unaligned: head and tail elements
        run_all_reduce(w, DT.BFP16, SUM, 50_003, "mesh", seed=seed + 1, pad=lambda r, which: 2 * r + (6 if which == "recv" else 0))
        run_all_reduce(w, DT.INT8, MIN, 9, "mesh", seed=seed + 2)                # less than one vector
        run_all_reduce(w, DT.INT32, PROD, 4_099, "mesh", seed=seed + 3, in_place=True)
        run_all_reduce(w, DT.FP64, SUM, 12_345, "mesh", seed=seed + 4, pad=lambda r, which: r + (3 if which == "recv" else 0))
        run_all_reduce(w, DT.FP32, SUM, 70_001, "nhr", seed=seed + 5)            # nested program: form not taken
        run_all_reduce(w, DT.FP32, SUM, 70_001, "mesh_symmetric", seed=seed + 6)     # n sub-segments, flat programs
        run_all_reduce(w, DT.BFP16, SUM, 30_011, "mesh_concur", seed=seed + 7, pad=2)
        run_all_reduce(w, DT.FP32, MIN, 9_973, "mesh_chunk", seed=seed + 8)
        run_reduce_scatter(w, DT.FP32, SUM, 5_001, "mesh", seed=seed + 9)        # one result stream: form not taken
    finally:
        w.close()


@pytest.mark.parametrize("n,waves", [(2, 2), (3, 8), (5, 3), (6, 4), (8, 2), (8, 3), (8, 8)])
def test_all_reduce_launched_from_its_arguments_alone(monkeypatch, n, waves):
    """The kernel for a flat fold of up to eight ranks to up to eight destinations that finds everything in its
    arguments (no program image), forced for every size: tile counts that the workgroup's wavefronts divide and do
    not, less than one tile and less than one vector, elements behind the last whole vector, every element type and
    operator, in place, more wavefronts than destinations and fewer.  Operands off the 16-byte grid, nested programs,
    results cut into sub-segments and results with one destination keep the general kernel."""
    monkeypatch.setenv("HCCL_AMD_REDUCE_DIRECT", str(waves))
    monkeypatch.setenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS", "0")
    w = World(n)
    monkeypatch.delenv("HCCL_AMD_REDUCE_DIRECT")
    monkeypatch.delenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS")
    try:
        seed = 6900 + 10 * n + waves
        for dtype in REDUCE_TYPES:
            for op in (SUM, PROD, MAX, MIN):
                if op == PROD and dtype in (DT.INT16, DT.BFP16):
                    continue   # not defined for these types
                run_all_reduce(w, dtype, op, 20_011, "mesh", seed=seed)
                seed += 1
        for count in (1, 3, 4, 5, 255, 256, 257, 256 * waves - 1, 256 * waves, 256 * waves + 1, 256 * (2 * waves + 1),
                      4096 * 3, 4096 * 4 + 1, 100_003):
            run_all_reduce(w, DT.FP32, SUM, count, "ring", seed=seed)            # 256 fp32 = one tile
            seed += 1
        # whole workgroups of eight tiles only (eight ranks and eight wavefronts: the straight-line instantiation)
        for dtype in REDUCE_TYPES:
            esz = np.dtype(NP[dtype]).itemsize
            for op in (SUM, PROD, MAX, MIN):
                if op == PROD and dtype in (DT.INT16, DT.BFP16):
                    continue
                run_all_reduce(w, dtype, op, 3 * 8192 // esz, "mesh", seed=seed, in_place=(op == MAX))
                seed += 1
        run_all_reduce(w, DT.INT8, MIN, 9, "mesh", seed=seed)                    # less than one vector
        run_all_reduce(w, DT.INT8, SUM, 16 * 64 * 3 + 15, "mesh", seed=seed + 1)  # fifteen elements behind the vectors
        run_all_reduce(w, DT.INT32, PROD, 4_099, "mesh", seed=seed + 2, in_place=True)
        run_all_reduce(w, DT.BFP16, SUM, 30_011, "mesh", seed=seed + 3, in_place=True)
        run_all_reduce(w, DT.FP16, MAX, 33_333, "mesh", seed=seed + 4, pad=2)    # off the 16-byte grid: general kernel
        run_all_reduce(w, DT.FP64, SUM, 12_345, "mesh", seed=seed + 5, pad=lambda r, which: r + (3 if which == "recv" else 0))
        run_all_reduce(w, DT.FP32, SUM, 70_001, "nhr", seed=seed + 6)            # nested program: general kernel
        run_all_reduce(w, DT.FP32, SUM, 70_001, "mesh_symmetric", seed=seed + 7)   # n sub-segments: general kernel
        run_all_reduce(w, DT.FP32, MIN, 9_973, "mesh_chunk", seed=seed + 8)
        run_reduce_scatter(w, DT.FP32, SUM, 5_001, "mesh", seed=seed + 9)        # one result stream: general kernel
    finally:
        w.close()


@pytest.mark.parametrize("n,waves", [(8, 8), (8, 4), (2, 4), (3, 8), (4, 8), (5, 2), (6, 8), (7, 3)])
def test_all_reduce_launched_from_its_arguments_with_two_tiles_per_wavefront(monkeypatch, n, waves):
    """The instantiations that take two tiles per wavefront (whole workgroups of 2 * waves tiles only; straight-line
    code for eight ranks and eight wavefronts), asked for by name: every type and operator at sizes they take, and
    sizes that only the one-tile kernels take (half a workgroup more, elements behind the last vector)."""
    monkeypatch.setenv("HCCL_AMD_REDUCE_DIRECT", str(waves))
    monkeypatch.setenv("HCCL_AMD_REDUCE_DIRECT_TILES", "2")
    monkeypatch.setenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS", "0")
    w = World(n)
    for k in ("HCCL_AMD_REDUCE_DIRECT", "HCCL_AMD_REDUCE_DIRECT_TILES", "HCCL_AMD_ALLREDUCE_TWO_KERNELS"):
        monkeypatch.delenv(k)
    try:
        seed = 7300 + 100 * n + waves
        group = 2 * waves * 1024           # bytes of one workgroup
        for dtype in REDUCE_TYPES:
            esz = np.dtype(NP[dtype]).itemsize
            for op in (SUM, PROD, MAX, MIN):
                if op == PROD and dtype in (DT.INT16, DT.BFP16):
                    continue
                run_all_reduce(w, dtype, op, 3 * group // esz, "mesh", seed=seed, in_place=(op == MIN))
                seed += 1
        for groups2 in (2, 1, 3, 5, 8):    # halves of a workgroup
            run_all_reduce(w, DT.FP32, SUM, groups2 * group // 8, "mesh", seed=seed + groups2)
        run_all_reduce(w, DT.FP32, SUM, group // 4 + 4, "mesh", seed=seed + 11)
        run_all_reduce(w, DT.BFP16, SUM, 2 * group // 2 - 8, "mesh", seed=seed + 12)
        run_all_reduce(w, DT.INT8, MAX, group + 5, "mesh", seed=seed + 13)
    finally:
        w.close()


@pytest.mark.parametrize("n,waves", [(9, 2), (12, 8), (13, 4), (16, 8), (16, 2)])
def test_all_reduce_of_nine_to_sixteen_ranks_launched_from_its_arguments(monkeypatch, n, waves):
    """The instantiation for nine to sixteen leaves and destinations (whole workgroups of `waves` tiles only), asked
    for by name: every type and operator at sizes it takes, and sizes that fall to the general kernel (half a
    workgroup more, elements behind the last vector, operands off the 16-byte grid)."""
    monkeypatch.setenv("HCCL_AMD_REDUCE_DIRECT", str(waves))
    monkeypatch.setenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS", "0")
    w = World(n)
    for k in ("HCCL_AMD_REDUCE_DIRECT", "HCCL_AMD_ALLREDUCE_TWO_KERNELS"):
        monkeypatch.delenv(k)
    try:
        seed = 7700 + 100 * n + waves
        group = waves * 1024               # bytes of one workgroup
        for dtype in REDUCE_TYPES:
            esz = np.dtype(NP[dtype]).itemsize
            for op in (SUM, PROD, MAX, MIN):
                if op == PROD and dtype in (DT.INT16, DT.BFP16):
                    continue
                run_all_reduce(w, dtype, op, 5 * group // esz, "mesh", seed=seed, in_place=(op == MIN))
                seed += 1
        for halves in (2, 1, 3, 7, 16):
            run_all_reduce(w, DT.FP32, SUM, halves * group // 8, "mesh", seed=seed + halves)
        run_all_reduce(w, DT.FP32, SUM, group // 4 + 4, "mesh", seed=seed + 21)
        run_all_reduce(w, DT.BFP16, SUM, 3 * group // 2, "mesh", seed=seed + 22, pad=2)
        run_all_reduce(w, DT.FP32, SUM, 3 * group // 4, "nhr", seed=seed + 23)      # nested program: general kernel
    finally:
        w.close()


def test_prepared_group_issues_the_same_collective():
    """hccl_amd.prepared_group converts the arguments of a group's calls once; what it runs is the plain sequence
    HcclGroupStart, the entry points, HcclGroupEnd, and a bad argument still raises with the entry point's code."""
    n, count = 4, 10_007
    w = World(n)
    try:
        rng = np.random.default_rng(808)
        host = [rng.standard_normal(count).astype(np.float32) for _ in range(n)]
        want = [np.zeros(count, dtype=np.float32) for _ in range(n)]
        assert oracle.all_reduce(host, want, count, int(DT.FP32), SUM, algo="mesh") == 0
        ins = [to_dev(x) for x in host]
        w.set_algo(OpKind.ALL_REDUCE, "mesh")
        w.inputs_ready()
        for _ in range(3):
            outs = [dev_zeros(count * 4) for _ in range(n)]
            w.inputs_ready()
            run = hccl_amd.prepared_group([("HcclAllReduce", (ins[r], outs[r], count, DT.FP32, SUM, w.comms[r], w.stream))
                                           for r in range(n)])
            run()
            w.sync()
            for r in range(n):
                assert np.array_equal(to_host(outs[r], np.uint32), want[r].view(np.uint32)), r
        bad = hccl_amd.prepared_group([("HcclAllReduce", (ins[0], None, count, DT.FP32, SUM, w.comms[0], w.stream))])
        with pytest.raises(hccl_amd.HcclError):
            bad()
    finally:
        w.close()


def test_two_kernel_all_reduce_can_be_captured_into_a_graph(monkeypatch):
    """Once its fold program is on the device (one eager call of the same kind) the fold + fan-out AllReduce is
    kernel launches only."""
    import torch
    monkeypatch.setenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS", "1")
    monkeypatch.setenv("HCCL_AMD_ALLREDUCE_PIECE_BYTES", "65536")
    n, count = 8, 40_003
    w = World(n)
    monkeypatch.delenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS")
    monkeypatch.delenv("HCCL_AMD_ALLREDUCE_PIECE_BYTES")
    try:
        rng = np.random.default_rng(4343)
        host = [rng.standard_normal(count).astype(np.float32) for _ in range(n)]
        want = [np.zeros(count, dtype=np.float32) for _ in range(n)]
        assert oracle.all_reduce(host, want, count, int(DT.FP32), SUM, algo="mesh") == 0
        ins = [torch.from_numpy(x).cuda() for x in host]
        outs = [torch.zeros(count, device="cuda") for _ in range(n)]

        def step():
            with hccl_amd.group():
                for r in range(n):
                    hccl_amd.all_reduce(w.comms[r], ins[r], outs[r], count, DT.FP32, OP.SUM, w.stream)

        torch.cuda.synchronize()
        step()
        w.sync()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=w.stream):
            step()
        for replay in range(3):
            for t in outs:
                t.fill_(float(replay))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for r in range(n):
                assert np.array_equal(outs[r].cpu().numpy().view(np.uint32), want[r].view(np.uint32)), (replay, r)
    finally:
        w.close()


def test_head_and_tail_counters_follow_the_collectives(monkeypatch):
    """HCCL_AMD_STUCK_COUNTERS=1: the launch stream writes the number of every collective in front of and behind its
    kernels; after a synchronisation both words hold the number of the last collective, and results are unchanged."""
    monkeypatch.setenv("HCCL_AMD_STUCK_COUNTERS", "1")
    w = World(4)
    monkeypatch.delenv("HCCL_AMD_STUCK_COUNTERS")
    try:
        assert hccl_amd.get_stuck_counters(w.comms[0]) == (0, 0)
        run_all_reduce(w, DT.FP32, SUM, 10_007, "mesh", seed=31)
        assert hccl_amd.get_stuck_counters(w.comms[1]) == (1, 1)
        run_reduce_scatter(w, DT.BFP16, SUM, 4_099, "nhr", seed=32)
        run_all_reduce(w, DT.INT32, MAX, 77, "rhd", seed=33)
        assert hccl_amd.get_stuck_counters(w.comms[3]) == (3, 3)
    finally:
        w.close()


def test_all_reduce_larger_than_a_million_workgroups():
    """2 x 1 GiB of fp16 per rank: 2^26 vector positions, one per lane, 2^20 workgroups per destination."""
    import torch
    n, count = 2, 1 << 29
    w = World(n)
    try:
        g = torch.Generator(device="cuda")
        g.manual_seed(99)
        sends = [torch.randn(count, generator=g, device="cuda", dtype=torch.float16) for _ in range(n)]
        recvs = [torch.empty(count, dtype=torch.float16, device="cuda") for _ in range(n)]
        w.all_reduce(sends, recvs, count, DT.FP16, OP.SUM, "mesh")
        step = 1 << 27
        for lo in range(0, count, step):
            want = (sends[1][lo:lo + step].float() + sends[0][lo:lo + step].float()).half()
            for r in range(n):
                assert torch.equal(recvs[r][lo:lo + step].view(torch.int16), want.view(torch.int16)), (lo, r)
            del want
    finally:
        w.close()


# ---------------------------------------------------------------------------------------------
# Loops over a bounded staging buffer: every loop is sliced afresh (NHR, RHD)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [6, 8])
@pytest.mark.parametrize("algo", ["nhr", "rhd"])
def test_all_reduce_follows_staging_buffer_loops(n, algo):
    w = World(n)
    try:
        for dtype, count, ccl in ((DT.FP32, 100_003, 65536), (DT.FP32, 6 * 8 * 1000, 4096), (DT.FP16, 33_333, 8192),
                                  (DT.INT32, 5, 65536)):
            esz = np.dtype(NP[dtype]).itemsize
            if algo == "nhr":
                per_loop = oracle.sole_max_count_per_loop(ccl, 1, esz)
            else:
                rc, per_loop = oracle.rhd_max_count_per_loop(ccl, count, n, esz)
                assert rc == 0
            w.set_ccl_buffer_size(ccl)
            run_all_reduce(w, dtype, SUM, count, algo, seed=n * 100 + count % 97, max_count_per_loop=per_loop)
        # one loop again: differs from the looped result for wide-range fp32 inputs, equals the oracle's one loop
        w.set_ccl_buffer_size(0)
        run_all_reduce(w, DT.FP32, SUM, 100_003, algo, seed=77)
        # a buffer that holds no loop is refused like in the reference
        w.set_ccl_buffer_size(16 if algo == "rhd" else 2)
        x = [to_dev(np.ones(64, dtype=np.float32)) for _ in range(n)]
        y = [dev_zeros(256) for _ in range(n)]
        with pytest.raises(hccl_amd.HcclError) as e:
            w.all_reduce(x, y, 64, DT.FP32, SUM, algo)
        assert e.value.code == 4
        # orders that fold every position alike ignore the buffer
        w.set_ccl_buffer_size(4096)
        run_all_reduce(w, DT.FP32, SUM, 10_001, "mesh", seed=78)
        run_all_reduce(w, DT.FP32, SUM, 10_001, "mesh_symmetric", seed=79)
    finally:
        w.set_ccl_buffer_size(0)
        w.close()


@pytest.mark.parametrize("two_kernels", [False, True])
@pytest.mark.parametrize("n", [2, 3, 8, 16])
def test_mesh_chunk_order_with_aligned_segments_and_staging_loops(monkeypatch, n, two_kernels):
    """Slices long enough for the 4 KiB rule, odd sizes, several types; then the executor's loops, which cut
    every loop's share into segments of its own.  Also with the AllReduce forced into fold + fan-out over pieces of
    64 KiB (pieces of whole slices; slices longer than a piece keep the fused kernel)."""
    if two_kernels:
        monkeypatch.setenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS", "1")
        monkeypatch.setenv("HCCL_AMD_ALLREDUCE_PIECE_BYTES", "65536")
    w = World(n)
    monkeypatch.delenv("HCCL_AMD_ALLREDUCE_TWO_KERNELS", raising=False)
    monkeypatch.delenv("HCCL_AMD_ALLREDUCE_PIECE_BYTES", raising=False)
    try:
        for dtype, c in ((DT.FP32, 100_000), (DT.FP32, 7 * 1024 * (n - 1) - 1), (DT.BFP16, 300_001), (DT.INT8, 77_777),
                         (DT.FP16, 65_536)):
            run_reduce_scatter(w, dtype, SUM, c, "mesh_chunk", seed=n * 7 + c % 91)
            run_all_reduce(w, dtype, SUM, c + 13, "mesh_chunk", seed=n * 9 + c % 89)
        run_reduce_scatter(w, DT.FP32, MAX, 50_001, "mesh_chunk", seed=5, pad=lambda r, which: 4 * (r % 4))
        run_all_reduce(w, DT.FP32, MIN, 50_001, "mesh_chunk", seed=6, in_place=True)
        ccl = 1 << 20
        w.set_ccl_buffer_size(ccl)
        run_reduce_scatter(w, DT.FP32, SUM, 300_000, "mesh_chunk", seed=7,
                           max_count_per_loop=oracle.sole_max_count_per_loop(ccl, n - 1, 4))
        run_all_reduce(w, DT.FP32, SUM, 700_001, "mesh_chunk", seed=8,
                       max_count_per_loop=oracle.sole_max_count_per_loop(ccl, 2, 4))
    finally:
        w.set_ccl_buffer_size(0)
        w.close()


def test_prod_and_64_bit_types_fold_in_mesh_order_under_write_reduce_algorithms(world8):
    """The reference offers NHR / RHD / mesh chunk / vector-core mesh neither PROD nor 64-bit types and falls back
    to its host-reduce mesh templates: those calls must equal the oracle's MESH order bit for bit."""
    def all_reduce_as_mesh(dtype, op, count, algo, seed):
        rng = np.random.default_rng(seed)
        ins = [gen(dtype, op, rng, count) for _ in range(8)]
        want = [np.zeros(count, dtype=NP[dtype]) for _ in range(8)]
        assert oracle.all_reduce(ins, want, count, int(dtype), op, acc=oracle.ACC_FP32, algo="mesh") == 0
        sends = [to_dev(x) for x in ins]
        recvs = [dev_zeros(x.nbytes) for x in ins]
        world8.all_reduce(sends, recvs, count, dtype, op, algo)
        for r in range(8):
            check(dtype, op, to_host(recvs[r], NP[dtype]), want[r], "all_reduce %s as mesh, rank %d" % (algo, r))

    def reduce_scatter_as_mesh(dtype, op, c, algo, seed):
        rng = np.random.default_rng(seed)
        ins = [gen(dtype, op, rng, 8 * c) for _ in range(8)]
        want = [np.zeros(c, dtype=NP[dtype]) for _ in range(8)]
        assert oracle.reduce_scatter(ins, want, c, int(dtype), op, acc=oracle.ACC_FP32, algo="mesh") == 0
        sends = [to_dev(x) for x in ins]
        recvs = [dev_zeros(c * ins[0].itemsize) for _ in range(8)]
        world8.reduce_scatter(sends, recvs, c, dtype, op, algo)
        for r in range(8):
            check(dtype, op, to_host(recvs[r], NP[dtype]), want[r], "reduce_scatter %s as mesh, rank %d" % (algo, r))

    for algo in ("nhr", "rhd", "mesh_chunk"):
        all_reduce_as_mesh(DT.FP64, SUM, 30_001, algo, 1)
        all_reduce_as_mesh(DT.FP32, PROD, 30_001, algo, 2)
        all_reduce_as_mesh(DT.FP64, MAX, 5_001, algo, 3)
    for algo in ("nhr", "ring", "rhd", "mesh_chunk", "aiv_mesh"):
        reduce_scatter_as_mesh(DT.FP64, SUM, 9_001, algo, 4)
        reduce_scatter_as_mesh(DT.FP32, PROD, 9_001, algo, 5)
        reduce_scatter_as_mesh(DT.FP16, PROD, 9_001, algo, 6)


def test_fp16_prod_carries_the_payload_of_a_single_nan_operand_bit_for_bit():
    """fp16 PROD is the one half-precision reduction whose arithmetic the reference holds itself (AicpuReduceFp16,
    alg_data_trans_wrapper.cc:1237-1257): widen, multiply in fp32, narrow with Fp32ToFp16, whose NaN rule keeps
    the top ten mantissa bits (:1196-1207).  With exactly one NaN among the operands of an element the result is
    defined on every machine (the multiply returns that NaN, quieted), so it is compared bit for bit: every payload,
    both signs, quiet and signalling, the NaN at any rank, next to finite values, zeros, subnormals and infinities."""
    payloads = np.arange(1, 0x400, dtype=np.uint16)
    nans = np.concatenate([0x7C00 | payloads, 0xFC00 | payloads]).astype(np.uint16)     # 2046 patterns
    # Two pools, so that the other operands never make a NaN of their own (0 * Inf): one with infinities and nothing
    # that can underflow to zero, one with zeros and subnormals and nothing that can overflow.
    with_inf = np.array([0x3C00, 0xBC00, 0x7C00, 0xFC00, 0x3555, 0xC100, 0x4000], dtype=np.uint16)
    with_zero = np.array([0x3C00, 0xBC00, 0x0000, 0x8000, 0x0001, 0x0400, 0x3555, 0x3800], dtype=np.uint16)
    for n, algo in ((2, "mesh"), (3, "ring"), (8, "mesh"), (6, "rhd")):
        w = World(n)
        try:
            rng = np.random.default_rng(900 + n)
            count = 3 * nans.size + 5
            even = np.arange(count) % 2 == 0
            ins = [np.where(even, with_inf[rng.integers(0, with_inf.size, count)],
                            with_zero[rng.integers(0, with_zero.size, count)]) for _ in range(n)]
            holder = rng.integers(0, n, count)
            pattern = np.resize(nans, count)
            for r in range(n):
                ins[r] = np.where(holder == r, pattern, ins[r]).astype(np.uint16)
            want = [np.zeros(count, dtype=np.uint16) for _ in range(n)]
            assert oracle.all_reduce(ins, want, count, int(DT.FP16), PROD, acc=oracle.ACC_FP32,
                                     algo=order_of(algo, DT.FP16, PROD, False)) == 0
            # the closed form of the reference's rule: the operand's NaN with its quiet bit set
            assert np.array_equal(want[0], pattern | 0x0200)
            sends = [to_dev(x) for x in ins]
            recvs = [dev_zeros(2 * count) for _ in range(n)]
            w.all_reduce(sends, recvs, count, DT.FP16, PROD, algo)
            for r in range(n):
                got = to_host(recvs[r], np.uint16)
                bad = np.nonzero(got != want[r])[0]
                assert bad.size == 0, "n=%d rank %d: %d differ, first %s got %s want %s" % (
                    n, r, bad.size, bad[:4], [hex(x) for x in got[bad[:4]]], [hex(x) for x in want[r][bad[:4]]])
            # ReduceScatter takes the element path for its ragged tail as well
            c = count // n
            rs_want = [np.zeros(c, dtype=np.uint16) for _ in range(n)]
            rs_ins = [x[:n * c] for x in ins]
            assert oracle.reduce_scatter(rs_ins, rs_want, c, int(DT.FP16), PROD, acc=oracle.ACC_FP32, algo="mesh") == 0
            rs_recvs = [dev_zeros(2 * c) for _ in range(n)]
            w.reduce_scatter([to_dev(x) for x in rs_ins], rs_recvs, c, DT.FP16, PROD, "mesh")
            for r in range(n):
                assert np.array_equal(to_host(rs_recvs[r], np.uint16), rs_want[r]), "reduce_scatter n=%d rank %d" % (n, r)
        finally:
            w.close()


def test_warmed_up_collectives_can_be_captured_into_a_graph_and_replayed():
    """After one eager call (which uploads the fold programs) AllReduce, ReduceScatter and AllGather are plain kernel
    launches on the caller's stream: a captured graph of them must reproduce the eager results on every replay,
    with eager work and synchronisations between the replays."""
    import torch
    n, count = 8, 50_000
    w = World(n)
    try:
        rng = np.random.default_rng(4242)
        ins = [torch.from_numpy(rng.standard_normal(n * count).astype(np.float32)).cuda() for _ in range(n)]
        ar = [torch.zeros(n * count, device="cuda") for _ in range(n)]
        rs = [torch.zeros(count, device="cuda") for _ in range(n)]
        ag = [torch.zeros(n * count, device="cuda") for _ in range(n)]
        w.set_algo(OpKind.ALL_REDUCE, "rhd")
        w.set_algo(OpKind.REDUCE_SCATTER, "nhr")

        def step():
            with hccl_amd.group():
                for r in range(n):
                    hccl_amd.all_reduce(w.comms[r], ins[r], ar[r], n * count, DT.FP32, OP.SUM, w.stream)
            with hccl_amd.group():
                for r in range(n):
                    hccl_amd.reduce_scatter(w.comms[r], ins[r], rs[r], count, DT.FP32, OP.SUM, w.stream)
            with hccl_amd.group():
                for r in range(n):
                    hccl_amd.all_gather(w.comms[r], rs[r], ag[r], count, DT.FP32, w.stream)

        torch.cuda.synchronize()
        step()
        w.sync()
        eager = [[t.clone() for t in group] for group in (ar, rs, ag)]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=w.stream):
            step()
        for replay in range(4):
            for group in (ar, rs, ag):
                for t in group:
                    t.fill_(float(replay))                  # eager work between the replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for got, want in zip((ar, rs, ag), eager):
                for r in range(n):
                    assert torch.equal(got[r], want[r]), (replay, r)
        # new inputs through the same graph: the kernels read the buffers, not a snapshot
        for t in ins:
            t.mul_(-0.5)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        step()
        w.sync()
        for r in range(n):
            assert torch.equal(ar[r], ar[0]) and torch.equal(ag[r], ag[0])
        want = [np.zeros(count, dtype=np.float32) for _ in range(n)]
        host = [t.cpu().numpy() for t in ins]
        assert oracle.reduce_scatter(host, want, count, int(DT.FP32), SUM, acc=oracle.ACC_FP32, algo="nhr") == 0
        for r in range(n):
            assert np.array_equal(rs[r].cpu().numpy().view(np.uint32), want[r].view(np.uint32))
    finally:
        w.close()


@pytest.mark.parametrize("algo", ["mesh", "nhr", "rhd", "mesh_chunk"])
def test_reduce_scatter_into_the_own_slice_of_the_send_buffer(algo):
    """recvBuf = sendBuf + rank * recvCount: every position of a rank's own slice is read and then overwritten by
    the one lane that folds it, so the overlap is harmless."""
    import torch
    n, c = 8, 30_011
    w = World(n)
    try:
        rng = np.random.default_rng(7070)
        ins = [rng.standard_normal(n * c).astype(np.float32) for _ in range(n)]
        want = [np.zeros(c, dtype=np.float32) for _ in range(n)]
        assert oracle.reduce_scatter(ins, want, c, int(DT.FP32), SUM, acc=oracle.ACC_FP32, algo=algo) == 0
        sends = [torch.from_numpy(x).cuda() for x in ins]
        recvs = [sends[r][r * c:(r + 1) * c] for r in range(n)]
        w.reduce_scatter(sends, recvs, c, DT.FP32, OP.SUM, algo)
        for r in range(n):
            assert np.array_equal(recvs[r].cpu().numpy().view(np.uint32), want[r].view(np.uint32)), (algo, r)
            other = (r + 1) % n          # the slices a rank does not own are untouched
            assert np.array_equal(sends[r][other * c:(other + 1) * c].cpu().numpy(), ins[r][other * c:(other + 1) * c])
    finally:
        w.close()
