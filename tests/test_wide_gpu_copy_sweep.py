"""Seeded random sweep over the copy operators (AllGather(V), AlltoAll(V/VC), Broadcast, Scatter): rank count,
element size, counts with empty contributions, shuffled displacements with holes, and buffers that start anywhere
on an element boundary, so that sources and destinations meet at every combination of offsets from a 16-byte
boundary (the aligned, the congruent and the lane-shifting form of the copy kernels).  Every case is compared with
the oracle byte for byte, including the bytes a collective must leave alone."""
import os

import numpy as np
import pytest

import oracle
from hccl_amd import HcclDataType as DT

from gpu_util import World, a2a_case, dev_zeros, rand_bytes, require_library_on_gpu, to_dev, to_host

pytestmark = pytest.mark.gpu
FILL = 0xAB
# Another number here draws other cases (used for longer runs by hand, mostly on the CPU emulation).
SWEEP_SEED = int(os.environ.get("HCCL_AMD_TEST_SWEEP_SEED", "70000"))
TYPES = [(DT.UINT8, 1), (DT.FP16, 2), (DT.HIF8, 1), (DT.FP32, 4), (DT.INT64, 8), (DT.BFP16, 2), (DT.FP64, 8)]
OPS = ["all_gather", "all_gather_v", "all_to_all", "all_to_all_v", "all_to_all_vc", "broadcast", "scatter"]
FORMS = {"by_size": {}, "two_kernels": {"HCCL_AMD_COPY_TWO_KERNELS": "1", "HCCL_AMD_ALLREDUCE_PIECE_BYTES": "4096"}}


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


def pick_count(rng, n):
    kind = rng.integers(0, 4)
    if kind == 0:
        return int(rng.integers(1, 40))
    if kind == 1:
        return int(rng.integers(40, 3000))
    top = 60_000 if n <= 8 else 6_000
    return int(rng.integers(3000, top))


def check(recvs, want, what):
    for r, (got, exp) in enumerate(zip(recvs, want)):
        assert np.array_equal(to_host(got, np.uint8), exp), what + (r,)


@pytest.mark.parametrize("form", list(FORMS))
@pytest.mark.parametrize("n", [2, 3, 5, 8, 13, 16])
def test_random_copy_cases(monkeypatch, n, form):
    rng = np.random.default_rng(SWEEP_SEED + n)
    for k, v in FORMS[form].items():
        monkeypatch.setenv(k, v)
    w = World(n)
    for k in FORMS[form]:
        monkeypatch.delenv(k)
    try:
        for case in range(21):
            op = OPS[case % len(OPS)]
            dtype, esz = TYPES[rng.integers(0, len(TYPES))]
            count = pick_count(rng, n)
            skew = rng.random() < 0.6                       # buffers off the 16-byte grid, each by its own amount
            pad = lambda: int(rng.integers(0, 16 // esz)) * esz if skew else 0
            what = (op, n, form, case, dtype.name, count)
            if op == "all_gather":
                ins = [rand_bytes(rng, count * esz) for _ in range(n)]
                want = [np.full(n * count * esz, FILL, dtype=np.uint8) for _ in range(n)]
                assert oracle.all_gather(ins, want, count, int(dtype)) == 0
                sends = [to_dev(x, pad()) for x in ins]
                recvs = [dev_zeros(x.nbytes, pad(), fill=FILL) for x in want]
                w.all_gather(sends, recvs, count, dtype)
            elif op == "all_gather_v":
                counts = rng.integers(0, count + 1, n).astype(np.uint64)
                counts[rng.integers(0, n)] = 0
                displs = np.zeros(n, dtype=np.uint64)
                off = int(rng.integers(0, 4))
                for j in rng.permutation(n):
                    displs[j] = off
                    off += int(counts[j]) + int(rng.integers(0, 5))
                ins = [rand_bytes(rng, max(int(c), 1) * esz) for c in counts]
                want = [np.full((off + 3) * esz, FILL, dtype=np.uint8) for _ in range(n)]
                assert oracle.all_gather_v(ins, want, counts, displs, int(dtype)) == 0
                sends = [to_dev(x, pad()) for x in ins]
                recvs = [dev_zeros(x.nbytes, pad(), fill=FILL) for x in want]
                w.all_gather_v(sends, recvs, counts, displs, dtype)
            elif op == "all_to_all":
                count = max(1, count // n)
                ins = [rand_bytes(rng, n * count * esz) for _ in range(n)]
                want = [np.full(n * count * esz, FILL, dtype=np.uint8) for _ in range(n)]
                assert oracle.all_to_all(ins, want, count, int(dtype)) == 0
                sends = [to_dev(x, pad()) for x in ins]
                recvs = [dev_zeros(x.nbytes, pad(), fill=FILL) for x in want]
                w.all_to_all(sends, recvs, count, dtype)
            elif op == "all_to_all_v":
                sc, sd, rc, rd, in_sz, out_sz = a2a_case(rng, n, esz, max(2, count // n), aligned=bool(rng.random() < 0.3))
                ins = [rand_bytes(rng, in_sz * esz) for _ in range(n)]
                want = [np.full(out_sz * esz, FILL, dtype=np.uint8) for _ in range(n)]
                assert oracle.all_to_all_v(ins, want, sc, sd, rc, rd, int(dtype)) == 0
                sends = [to_dev(x, pad()) for x in ins]
                recvs = [dev_zeros(x.nbytes, pad(), fill=FILL) for x in want]
                w.all_to_all_v(sends, sc, sd, recvs, rc, rd, dtype)
            elif op == "all_to_all_vc":
                m = rng.integers(0, max(2, count // n), (n, n)).astype(np.uint64)
                m[rng.random((n, n)) < 0.2] = 0
                ins = [rand_bytes(rng, max(int(m[r].sum()), 1) * esz) for r in range(n)]
                want = [np.full(max(int(m[:, r].sum()), 1) * esz, FILL, dtype=np.uint8) for r in range(n)]
                assert oracle.all_to_all_vc(ins, want, m, int(dtype)) == 0
                sends = [to_dev(x, pad()) for x in ins]
                recvs = [dev_zeros(x.nbytes, pad(), fill=FILL) for x in want]
                w.all_to_all_vc(sends, recvs, m, dtype)
            elif op == "broadcast":
                root = int(rng.integers(0, n))
                host = [rand_bytes(rng, count * esz) for _ in range(n)]
                want = [x.copy() for x in host]
                assert oracle.broadcast(want, count, int(dtype), root) == 0
                recvs = [to_dev(x, pad()) for x in host]
                w.broadcast(recvs, count, dtype, root)
            else:
                root = int(rng.integers(0, n))
                count = max(1, count // n)
                ins = [rand_bytes(rng, n * count * esz) for _ in range(n)]
                want = [np.full(count * esz, FILL, dtype=np.uint8) for _ in range(n)]
                assert oracle.scatter(ins, want, count, int(dtype), root) == 0
                sends = [to_dev(ins[r], pad()) if r == root else None for r in range(n)]
                recvs = [dev_zeros(x.nbytes, pad(), fill=FILL) for x in want]
                w.scatter(sends, recvs, count, dtype, root)
            check(recvs, want, what)
    finally:
        w.close()
