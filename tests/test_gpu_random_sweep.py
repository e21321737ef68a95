"""Seeded random sweep over (collective, type, op, algorithm, rank count, element count, buffer alignment,
staging-buffer size): every case is compared with the oracle like the hand-picked cases of test_gpu_parity.py."""
import os

import numpy as np
import pytest

import oracle
from hccl_amd import HcclDataType as DT

from gpu_util import World, require_library_on_gpu
from test_gpu_parity import MAX, MIN, NP, PROD, SUM, run_all_reduce, run_reduce_scatter

pytestmark = pytest.mark.gpu
# Another number here draws other cases (used for longer runs by hand, mostly on the CPU emulation).
SWEEP_SEED = int(os.environ.get("HCCL_AMD_TEST_SWEEP_SEED", "90000"))

TYPES = [DT.INT8, DT.INT16, DT.INT32, DT.INT64, DT.UINT64, DT.FP16, DT.BFP16, DT.FP32, DT.FP64]
AR_ALGOS = ["mesh", "ring", "rhd", "nhr", "order_preserved", "mesh_symmetric", "mesh_chunk", "mesh_concur"]
RS_ALGOS = ["mesh", "ring", "nhr", "rhd", "order_preserved", "aiv_mesh", "mesh_symmetric", "mesh_chunk"]


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


def pick_count(rng):
    kind = rng.integers(0, 4)
    if kind == 0:
        return int(rng.integers(1, 70))                         # fewer elements than lanes, often than ranks
    if kind == 1:
        return int(rng.integers(70, 5_000))
    if kind == 2:
        return int(rng.choice([4096, 8192, 65536]) + rng.integers(-3, 4))     # around vector / tile boundaries
    return int(rng.integers(5_000, 120_000))


FORMS = {
    "by_size": {},
    # without the kernel that is launched from its arguments alone: the general kernel on the short messages too
    "general_kernel": {"HCCL_AMD_REDUCE_DIRECT": "0"},
    # AllReduce as fold + fan-out whatever the size, pieces of a few KiB
    "two_kernels": {"HCCL_AMD_ALLREDUCE_TWO_KERNELS": "1", "HCCL_AMD_ALLREDUCE_PIECE_BYTES": None},
    # the fused kernel with a tile's stores shared by wavefronts, on a grid so small that workgroups loop
    "shared_stores": {"HCCL_AMD_ALLREDUCE_TWO_KERNELS": "0", "HCCL_AMD_REDUCE_STORE_WAVES": None,
                      "HCCL_AMD_REDUCE_BLOCKS": "40"},
}


@pytest.mark.parametrize("form", list(FORMS))
@pytest.mark.parametrize("n", [2, 3, 4, 6, 7, 8, 12, 16])
def test_random_reduce_cases(monkeypatch, n, form):
    rng = np.random.default_rng(SWEEP_SEED + n)
    env = dict(FORMS[form])
    if "HCCL_AMD_ALLREDUCE_PIECE_BYTES" in env:
        env["HCCL_AMD_ALLREDUCE_PIECE_BYTES"] = str([4096, 20_480, 65_536][n % 3])
    if "HCCL_AMD_REDUCE_STORE_WAVES" in env:
        env["HCCL_AMD_REDUCE_STORE_WAVES"] = str(2 + n % 3)
    for k, v in env.items():
        monkeypatch.setenv(k, v)
    w = World(n)
    for k in env:
        monkeypatch.delenv(k)
    try:
        for case in range(28):
            dtype = TYPES[rng.integers(0, len(TYPES))]
            op = int(rng.integers(0, 4))
            if op == PROD and dtype in (DT.INT16, DT.BFP16):
                op = SUM
            count = pick_count(rng)
            esz = np.dtype(NP[dtype]).itemsize
            offs = [int(rng.integers(0, 16 // esz)) * esz if rng.random() < 0.5 else 0 for _ in range(2 * n)]
            pad = lambda r, which, offs=offs: offs[r if which == "send" else n + r]
            if rng.random() < 0.5:
                algo = AR_ALGOS[rng.integers(0, len(AR_ALGOS))]
                loop, ccl = 0, 0
                if algo in ("nhr", "rhd", "mesh_chunk", "mesh_concur") and rng.random() < 0.4 and op != PROD and esz < 8:
                    ccl = int(rng.choice([4096, 20_000, 1 << 16]))
                    if algo == "nhr":
                        loop = oracle.sole_max_count_per_loop(ccl, 1, esz)
                    elif algo == "mesh_chunk":
                        loop = oracle.sole_max_count_per_loop(ccl, 2, esz)
                    elif algo == "mesh_concur":
                        loop = ccl // 2 // 128 * 128 // esz // n * n
                        if loop == 0:
                            ccl = 0
                    else:
                        rc, loop = oracle.rhd_max_count_per_loop(ccl, count, n, esz)
                        if rc != 0:
                            ccl, loop = 0, 0
                w.set_ccl_buffer_size(ccl)
                run_all_reduce(w, dtype, op, count, algo, seed=case * 131 + n, pad=pad,
                               in_place=bool(rng.random() < 0.15), max_count_per_loop=loop)
            else:
                algo = RS_ALGOS[rng.integers(0, len(RS_ALGOS))]
                loop, ccl = 0, 0
                if algo == "mesh_chunk" and rng.random() < 0.4 and op != PROD and esz < 8:
                    ccl = int(rng.choice([4096 * n, 1 << 16]))
                    loop = oracle.sole_max_count_per_loop(ccl, n - 1, esz)
                w.set_ccl_buffer_size(ccl)
                run_reduce_scatter(w, dtype, op, max(1, count // n), algo, seed=case * 137 + n, pad=pad,
                                   max_count_per_loop=loop)
    finally:
        w.set_ccl_buffer_size(0)
        w.close()
