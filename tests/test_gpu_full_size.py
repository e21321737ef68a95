"""The five benchmark configurations at their full sizes.  The CPU oracle would take minutes there, so the
results are checked on the GPU through properties that do not depend on size: the reduction is recomputed
slice by slice with torch in the association order the algorithm fixes (fp32 accumulate, one rounding),
integer reductions against torch's exact integer ops, AlltoAllV by a round trip through its inverse plus
a conserved checksum, AllGatherV by comparing every landed block with its source."""
import numpy as np
import pytest

import hccl_amd
from hccl_amd import HcclDataType as DT, HcclReduceOp as OP, OpKind

from gpu_util import World, require_library_on_gpu

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


def gen(seed):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return g


def test_config2_reduce_scatter_bf16_full_size():
    import torch
    n, c = 8, 1 << 24
    w = World(n)
    try:
        sends = [torch.randn(n * c, generator=gen(0xC0FFEE + 2000 + r), device="cuda", dtype=torch.bfloat16)
                 for r in range(n)]
        recvs = [torch.empty(c, dtype=torch.bfloat16, device="cuda") for _ in range(n)]
        for algo in ("ring", "mesh"):
            w.reduce_scatter(sends, recvs, c, DT.BFP16, OP.SUM, algo)
            for k in range(n):
                x = [sends[(k + i) % n][k * c:(k + 1) * c].float() for i in range(n)]
                if algo == "ring":   # NHR tree of slice k, fp32
                    want = ((x[1] + x[0]) + (x[3] + x[2])) + ((x[5] + x[4]) + (x[7] + x[6]))
                else:                # own slice first, then ranks ascending
                    o = [sends[k][k * c:(k + 1) * c].float()] + [sends[t][k * c:(k + 1) * c].float()
                                                                 for t in range(n) if t != k]
                    want = o[0]
                    for v in o[1:]:
                        want = v + want
                assert torch.equal(recvs[k].view(torch.int16), want.bfloat16().view(torch.int16)), (algo, k)
                del x, want
    finally:
        w.close()


def test_config3_all_reduce_int32_full_size():
    import torch
    n, count = 16, 1 << 26
    w = World(n)
    try:
        lut = torch.tensor([-2, -1, 1, 2], dtype=torch.int32, device="cuda")
        for op in (OP.MAX, OP.PROD):
            if op == OP.MAX:
                sends = [torch.randint(-2 ** 31, 2 ** 31 - 1, (count,), generator=gen(3000 + r), device="cuda",
                                       dtype=torch.int32) for r in range(n)]
            else:
                sends = [lut[torch.randint(0, 4, (count,), generator=gen(3100 + r), device="cuda")] for r in range(n)]
            recvs = [torch.empty(count, dtype=torch.int32, device="cuda") for _ in range(n)]
            w.all_reduce(sends, recvs, count, DT.INT32, op, "mesh")
            want = sends[0].clone()
            for r in range(1, n):
                want = torch.maximum(want, sends[r]) if op == OP.MAX else want * sends[r]   # int32 mul wraps
            for r in (0, 5, 15):
                assert torch.equal(recvs[r], want), (op, r)
            del sends, recvs, want
            torch.cuda.empty_cache()
    finally:
        w.close()


def test_config5a_all_reduce_fp16_rhd_full_size():
    import torch
    n, count = 6, 1 << 28
    w = World(n)
    try:
        sends = [(torch.randn(count, generator=gen(5000 + r), device="cuda", dtype=torch.float32) * 0.5).half()
                 for r in range(n)]
        recvs = [torch.empty(count, dtype=torch.float16, device="cuda") for _ in range(n)]
        w.all_reduce(sends, recvs, count, DT.FP16, OP.SUM, "rhd")
        step = 1 << 26
        for lo in range(0, count, step):
            x = [s[lo:lo + step].float() for s in sends]
            want = (((x[0] + x[2]) + x[4]) + ((x[1] + x[3]) + x[5])).half()
            for r in (0, 3, 5):
                assert torch.equal(recvs[r][lo:lo + step].view(torch.int16), want.view(torch.int16)), (lo, r)
            del x, want
    finally:
        w.close()


def test_config5b_all_gather_v_full_size():
    import torch
    n = 6
    w = World(n)
    try:
        rng = np.random.default_rng(0xC0FFEE + 5001)
        counts = rng.integers(1 << 20, (32 << 20) + 1, n).astype(np.uint64)
        for layout in ("prefix", "shuffled_with_gaps"):
            if layout == "prefix":
                displs = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.uint64)
                total = int(counts.sum())
            else:
                displs = np.zeros(n, dtype=np.uint64)
                off = 3
                for j in rng.permutation(n):
                    displs[j] = off
                    off += int(counts[j]) + int(rng.integers(1, 9))
                total = off
            sends = [torch.randn(int(c), generator=gen(5100 + r), device="cuda", dtype=torch.float16)
                     for r, c in enumerate(counts)]
            recvs = [torch.full((total,), -7.0, dtype=torch.float16, device="cuda") for _ in range(n)]
            w.all_gather_v(sends, recvs, counts, displs, DT.FP16)
            covered = 0
            for d in range(n):
                for r in range(n):
                    lo = int(displs[r])
                    assert torch.equal(recvs[d][lo:lo + int(counts[r])].view(torch.int16), sends[r].view(torch.int16))
                covered = int((recvs[d] != -7.0).sum().item())
                assert covered <= int(counts.sum())          # nothing outside the blocks was written
            del sends, recvs
            torch.cuda.empty_cache()
    finally:
        w.close()


def test_config4_all_to_all_v_moe_full_size_round_trip():
    import torch
    n, hidden, tokens = 64, 7168, 16384
    w = World(n)
    try:
        rng = np.random.default_rng(0xC0FFEE + 4000)
        wts = 1.0 / np.arange(1, n + 1) ** 1.1
        wts /= wts.sum()
        tok = np.stack([rng.multinomial(tokens, wts) for _ in range(n)]).astype(np.uint64)
        sc = tok * hidden
        rc = sc.T.copy()
        sd = np.cumsum(sc, axis=1) - sc
        rd = np.cumsum(rc, axis=1) - rc
        sends = [torch.randint(-32768, 32767, (tokens * hidden,), generator=gen(4100 + r), device="cuda",
                               dtype=torch.int16) for r in range(n)]
        recvs = [torch.empty(max(int(rc[i].sum()), 8), dtype=torch.int16, device="cuda") for i in range(n)]
        w.all_to_all_v(sends, sc, sd, recvs, rc, rd, DT.BFP16)
        # conservation: nothing lost, nothing duplicated
        total_in = sum(int(s.sum(dtype=torch.int64).item()) for s in sends)
        total_out = sum(int(recvs[i][:int(rc[i].sum())].sum(dtype=torch.int64).item()) for i in range(n))
        assert total_in == total_out
        # a few segments checked directly: recv_i[rdispls_i[j] ...] == send_j[sdispls_j[i] ...]
        for i, j in ((0, 0), (0, 63), (63, 0), (17, 5), (5, 17), (31, 31)):
            cnt = int(sc[j, i])
            assert torch.equal(recvs[i][int(rd[i, j]):int(rd[i, j]) + cnt], sends[j][int(sd[j, i]):int(sd[j, i]) + cnt])
        # the inverse exchange brings every token home
        back = [torch.zeros(tokens * hidden, dtype=torch.int16, device="cuda") for _ in range(n)]
        w.all_to_all_v(recvs, rc, rd, back, sc, sd, DT.BFP16)
        for r in range(n):
            assert torch.equal(back[r], sends[r]), r
    finally:
        w.close()


def test_reduce_scatter_v_uneven_slices_full_size():
    import torch
    n = 8
    w = World(n)
    try:
        rng = np.random.default_rng(0xC0FFEE + 6000)
        counts = (rng.integers(1 << 20, 3 << 20, n) * 8).astype(np.uint64)
        counts[3] += 5                                     # one slice that ends off a 16-byte boundary
        displs = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.uint64)
        total = int(counts.sum())
        sends = [torch.randn(total, generator=gen(6100 + r), device="cuda", dtype=torch.bfloat16) for r in range(n)]
        recvs = [torch.empty(int(c), dtype=torch.bfloat16, device="cuda") for c in counts]
        w.reduce_scatter_v(sends, recvs, counts, displs, DT.BFP16, OP.SUM)
        for k in range(n):
            lo, c = int(displs[k]), int(counts[k])
            want = sends[k][lo:lo + c].float()               # own slice first, then ranks ascending, fp32
            for t in range(n):
                if t != k:
                    want = sends[t][lo:lo + c].float() + want
            assert torch.equal(recvs[k].view(torch.int16), want.bfloat16().view(torch.int16)), k
            del want
    finally:
        w.close()


def test_reduce_then_broadcast_equals_all_reduce_full_size():
    import torch
    n, count, root = 8, 1 << 26, 3
    w = World(n)
    try:
        sends = [torch.randn(count, generator=gen(6200 + r), device="cuda", dtype=torch.float32) for r in range(n)]
        recvs = [torch.full((count,), -1.0, dtype=torch.float32, device="cuda") for _ in range(n)]
        w.reduce(sends, recvs, count, DT.FP32, OP.SUM, root)
        want = sends[0].clone()
        for r in range(1, n):
            want = sends[r] + want                           # rank order, bit exact in fp32
        assert torch.equal(recvs[root].view(torch.int32), want.view(torch.int32))
        assert all(bool((recvs[r] == -1.0).all()) for r in range(n) if r != root)
        w.broadcast(recvs, count, DT.FP32, root)
        for r in range(n):
            assert torch.equal(recvs[r].view(torch.int32), want.view(torch.int32)), r
        allr = [torch.empty(count, dtype=torch.float32, device="cuda") for _ in range(n)]
        w.all_reduce(sends, allr, count, DT.FP32, OP.SUM, "mesh")
        assert torch.equal(allr[5].view(torch.int32), want.view(torch.int32))
    finally:
        w.close()


def test_scatter_and_all_to_all_full_size():
    import torch
    n = 16
    w = World(n)
    try:
        count = 1 << 22
        sends = [torch.randint(-32768, 32767, (n * count,), generator=gen(6500 + r), device="cuda", dtype=torch.int16)
                 for r in range(n)]
        recvs = [torch.empty(n * count, dtype=torch.int16, device="cuda") for _ in range(n)]
        w.all_to_all(sends, recvs, count, DT.BFP16)
        for i in (0, 7, 15):
            got = recvs[i].view(n, count)
            for j in range(n):
                assert torch.equal(got[j], sends[j].view(n, count)[i]), (i, j)
        # applying the exchange twice is the identity (a block transpose)
        back = [torch.empty(n * count, dtype=torch.int16, device="cuda") for _ in range(n)]
        w.all_to_all(recvs, back, count, DT.BFP16)
        for r in range(n):
            assert torch.equal(back[r], sends[r]), r
        root = 9
        outs = [torch.empty(count, dtype=torch.int16, device="cuda") for _ in range(n)]
        w.scatter([sends[r] if r == root else None for r in range(n)], outs, count, DT.INT16, root)
        for r in range(n):
            assert torch.equal(outs[r], sends[root].view(n, count)[r]), r
    finally:
        w.close()
