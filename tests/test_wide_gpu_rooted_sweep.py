"""Seeded random sweep over the two reduce operators tests/test_gpu_random_sweep.py leaves out: Reduce (rank order and
two-shot, any root, buffers off the 16-byte grid) and ReduceScatterV (mesh and mesh-chunk order; packed, holed and
16-byte-aligned layouts with an empty slice).  Every case is compared with the oracle."""
import numpy as np
import pytest

import hccl_amd
import oracle
from hccl_amd import HcclDataType as DT

from gpu_util import World, dev_zeros, require_library_on_gpu, to_dev, to_host
from test_gpu_parity import MAX, NP, PROD, SUM, check, gen
from test_gpu_random_sweep import SWEEP_SEED, TYPES, pick_count
from test_gpu_rooted_and_v_ops import RSV_TYPES, run_rsv

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


@pytest.mark.parametrize("n", [2, 3, 5, 8, 13, 16])
def test_random_reduce_and_reduce_scatter_v_cases(n):
    rng = np.random.default_rng(SWEEP_SEED + 500 + n)
    w = World(n)
    try:
        for case in range(20):
            op = int(rng.integers(0, 4))
            if case % 2 == 0:
                dtype = TYPES[rng.integers(0, len(TYPES))]
                if op == PROD and dtype in (DT.INT16, DT.BFP16):
                    op = SUM
                esz = np.dtype(NP[dtype]).itemsize
                count, root = pick_count(rng), int(rng.integers(0, n))
                algo = "mesh_two_shot" if rng.random() < 0.5 else "mesh"
                pads = [int(rng.integers(0, 16 // esz)) * esz if rng.random() < 0.5 else 0 for _ in range(2 * n)]
                ins = [gen(dtype, op, rng, count) for _ in range(n)]
                want = [np.zeros(count, dtype=NP[dtype]) for _ in range(n)]
                assert oracle.reduce(ins, want, count, int(dtype), op, root, acc=oracle.ACC_FP32, algo=algo) == 0
                sends = [to_dev(x, pads[r]) for r, x in enumerate(ins)]
                recvs = [dev_zeros(x.nbytes, pads[n + r]) for r, x in enumerate(ins)]
                w.reduce(sends, recvs, count, dtype, op, root, algo)
                check(dtype, op, to_host(recvs[root], NP[dtype]), want[root],
                      "reduce %s %s n=%d root=%d count=%d case=%d" % (algo, dtype.name, n, root, count, case))
                for r in range(n):
                    if r != root:
                        assert np.all(to_host(recvs[r], np.uint8) == 0xAB), (case, r)
            else:
                dtype = RSV_TYPES[rng.integers(0, len(RSV_TYPES))]
                if op == PROD and dtype in (DT.INT16, DT.BFP16):
                    op = SUM
                hi = int(rng.choice([12, 700, 9000, 40_000]))
                layout = ["prefix", "gaps", "aligned"][rng.integers(0, 3)]
                algo = "mesh_chunk" if rng.random() < 0.4 and op != PROD and dtype != DT.INT64 else "mesh"
                run_rsv(w, dtype, op, 1, hi, layout, SWEEP_SEED + 1000 * n + case, pad=int(rng.integers(0, 2)) * 8, algo=algo)
    finally:
        w.set_algo(hccl_amd.OpKind.REDUCE, "mesh")
        w.set_algo(hccl_amd.OpKind.REDUCE_SCATTER, "mesh")
        w.close()


@pytest.mark.parametrize("n", [2, 9, 16, 17, 33])
def test_reduce_scatter_v_rank_counts_either_side_of_the_sixteen_group_table(n):
    """Up to sixteen slices a workgroup finds its slice by counting the slices' ends, which it reads in one go;
    beyond that it searches.  Both with an empty slice among them."""
    w = World(n)
    try:
        run_rsv(w, DT.INT32, SUM, 1, 3000, "gaps", 70 + n)
        run_rsv(w, DT.FP16, MAX, 200, 2000, "prefix", 90 + n)
    finally:
        w.close()
