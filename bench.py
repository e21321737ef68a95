#!/usr/bin/env python3
"""Benchmark of the loopback data plane on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2] [--no-others] [--no-cpu]

A step is one collective over all N loopback ranks (N per-rank calls through the C ABI inside a
group, one fused kernel launch).  The headline workload is the configuration the metric is quoted
on: ReduceScatter SUM bf16, rankSize 8, 134,217,728 elements in / 16,777,216 out per rank, "ring"
algorithm.  Inputs are synthetic (seeded torch generators, seed = 0xC0FFEE + 1000 * config + rank) and
resident in HBM before timing starts.

Prints ONE JSON line: the headline workload with its roofline and CPU baseline, and under "others" the
remaining benchmark configurations (c1, c3max, c3prod, c4, c5a, c5b), each with its GPU timing, bandwidths,
fraction of the HBM roofline and its own CPU baseline (the reference's host reduce / copy pattern restated
in C, same operator, rank count, data type and fold order, on a bounded sample; one thread and all cores).
"""
import argparse
import json
import os
import re
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
SEED = 0xC0FFEE
CONFIGS = ("c1", "c2", "c3max", "c3prod", "c4", "c5a", "c5b")
EXTRA = ("rsv", "reduce", "bcast", "ag", "scatter", "a2a")


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2", choices=list(CONFIGS) + ["copycal"] + list(EXTRA))
    ap.add_argument("--algo", default=None, help="override the algorithm of the workload (mesh/ring/rhd/nhr/...)")
    ap.add_argument("--no-others", action="store_true", help="time the selected workload only")
    ap.add_argument("--extra", action="store_true", help="also time the entry points outside the benchmark configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU time of the headline's one-thread baseline")
    ap.add_argument("--cpu-seconds-others", type=float, default=2.5)
    return ap.parse_args()


def zipf_routing(np, n, tokens, seed):
    """Per-source token counts over n destinations, multinomial with Zipf(1.1) weights over the destination index."""
    rng = np.random.default_rng(seed)
    wts = 1.0 / np.arange(1, n + 1) ** 1.1
    wts /= wts.sum()
    return np.stack([rng.multinomial(tokens, wts) for _ in range(n)]).astype(np.uint64)


def gather_v_counts(np, n, lo, hi, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(lo, hi + 1, n).astype(np.uint64)


# ---------------------------------------------------------------------------------------------
# GPU workloads.  Each returns (step, algorithmic_bytes, bytes_for_algbw, busbw_factor, keepalive, description,
# dtype, n, algorithm)
# ---------------------------------------------------------------------------------------------
class Workloads:
    def __init__(self, torch, hccl):
        self.torch = torch
        self.h = hccl
        self.stream = torch.cuda.Stream()
        self.worlds = {}

    def world(self, n):
        if n not in self.worlds:
            self.worlds[n] = self.h.comm_init_all(n)
        return self.worlds[n]

    def gen(self, seed):
        g = self.torch.Generator(device="cuda")
        g.manual_seed(seed)
        return g

    def _reduce(self, kind, cfg, n, count, tdtype, hdtype, op, algo, make, sets=1):
        """`sets` buffer sets are used in turn, so that a small workload does not stay in the 256 MB last-level cache."""
        t, h = self.torch, self.h
        comms = self.world(n)
        per_rank_in = count * n if kind == "rs" else count
        sends = [[make(per_rank_in, SEED + 1000 * cfg + 100 * k + r) for r in range(n)] for k in range(sets)]
        recvs = [[t.empty(count, dtype=tdtype, device="cuda") for _ in range(n)] for _ in range(sets)]
        opk = h.OpKind.REDUCE_SCATTER if kind == "rs" else h.OpKind.ALL_REDUCE
        h.set_algo(comms[0], opk, h.Algo[algo.upper()])
        entry = "HcclReduceScatter" if kind == "rs" else "HcclAllReduce"
        stream = self.stream
        turn = [0]
        # one collective = the n per-rank calls of the C ABI inside a group; their arguments are converted to C types
        # once per buffer set (a collective of 15 us would otherwise wait for Python's conversions)
        groups = [h.prepared_group([(entry, (sends[k][r], recvs[k][r], count, hdtype, op, comms[r], stream))
                                    for r in range(n)]) for k in range(sets)]

        def step():
            k = turn[0]
            turn[0] = (k + 1) % sets
            groups[k]()

        esz = sends[0][0].element_size()
        if kind == "rs":
            hbm = n * n * count * esz + n * count * esz
            alg = n * count * esz
            bus = (n - 1) / n
        else:
            hbm = 2 * n * count * esz
            alg = count * esz
            bus = 2 * (n - 1) / n
        return step, hbm, alg, bus, (sends, recvs)

    def c1(self, algo):
        t, h = self.torch, self.h
        mk = lambda cnt, seed: t.rand(cnt, generator=self.gen(seed), device="cuda", dtype=t.float32) * 2 - 1
        algo = algo or "ring"
        # 6 buffer sets of 64 MiB: 384 MiB in rotation, more than the last-level cache holds
        return self._reduce("ar", 1, 8, 1 << 20, t.float32, h.HcclDataType.FP32, h.HcclReduceOp.SUM, algo, mk, sets=6) + (
            "AllReduce SUM fp32 rankSize=8 1Mi el/rank, 6 buffer sets in rotation", "f32", 8, algo)

    def c2(self, algo):
        t, h = self.torch, self.h
        mk = lambda cnt, seed: t.randn(cnt, generator=self.gen(seed), device="cuda", dtype=t.bfloat16)
        algo = algo or "ring"
        return self._reduce("rs", 2, 8, 1 << 24, t.bfloat16, h.HcclDataType.BFP16, h.HcclReduceOp.SUM, algo, mk) + (
            "ReduceScatter SUM bf16 rankSize=8 128Mi el in / 16Mi out per rank", "bf16", 8, algo)

    def c3max(self, algo):
        t, h = self.torch, self.h
        mk = lambda cnt, seed: t.randint(-2 ** 31, 2 ** 31 - 1, (cnt,), generator=self.gen(seed), device="cuda",
                                         dtype=t.int32)
        algo = algo or "mesh"
        return self._reduce("ar", 3, 16, 1 << 26, t.int32, h.HcclDataType.INT32, h.HcclReduceOp.MAX, algo, mk) + (
            "AllReduce MAX int32 rankSize=16 64Mi el/rank", "int32", 16, algo)

    def c3prod(self, algo):
        t, h = self.torch, self.h
        lut = t.tensor([-2, -1, 1, 2], dtype=t.int32, device="cuda")
        mk = lambda cnt, seed: lut[t.randint(0, 4, (cnt,), generator=self.gen(seed + 50), device="cuda")]
        algo = algo or "mesh"
        return self._reduce("ar", 3, 16, 1 << 26, t.int32, h.HcclDataType.INT32, h.HcclReduceOp.PROD, algo, mk) + (
            "AllReduce PROD int32 rankSize=16 64Mi el/rank", "int32", 16, algo)

    def c5a(self, algo):
        t, h = self.torch, self.h
        mk = lambda cnt, seed: (t.randn(cnt, generator=self.gen(seed), device="cuda", dtype=t.float32) * 0.5).half()
        algo = algo or "rhd"
        return self._reduce("ar", 5, 6, 1 << 28, t.float16, h.HcclDataType.FP16, h.HcclReduceOp.SUM, algo, mk) + (
            "AllReduce SUM fp16 rankSize=6 RHD 256Mi el/rank", "f16", 6, algo)

    def c5b(self, algo):
        import numpy as np
        t, h = self.torch, self.h
        n, sets = 6, 4   # 4 buffer sets of 0.9 GB in rotation: no step finds its source in the last-level cache
        comms = self.world(n)
        counts = gather_v_counts(np, n, 1 << 20, 32 << 20, SEED + 5000 + 500)
        displs = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.uint64)
        total = int(counts.sum())
        sends = [[t.randn(int(c), generator=self.gen(SEED + 5000 + 600 + 10 * k + r), device="cuda", dtype=t.float16)
                  for r, c in enumerate(counts)] for k in range(sets)]
        recvs = [[t.empty(total, dtype=t.float16, device="cuda") for _ in range(n)] for _ in range(sets)]
        stream = self.stream
        turn = [0]

        def step():
            k = turn[0]
            turn[0] = (k + 1) % sets
            with h.group():
                for r in range(n):
                    h.all_gather_v(comms[r], sends[k][r], int(counts[r]), recvs[k][r], counts, displs,
                                   h.HcclDataType.FP16, stream)

        hbm = (1 + n) * total * 2
        return step, hbm, total * 2, (n - 1) / n, (sends, recvs), \
            "AllGatherV fp16 rankSize=6 counts U[1Mi,32Mi], 4 buffer sets in rotation", "f16", n, "mesh"

    def copycal(self, algo):
        """Plain copy of known size (the rankSize == 1 shortcut): calibrates the HBM byte counters."""
        t, h = self.torch, self.h
        comms = self.world(1)
        nbytes = 1 << 30
        src = t.randint(0, 255, (nbytes,), generator=self.gen(1), device="cuda", dtype=t.uint8)
        dst = t.empty(nbytes, dtype=t.uint8, device="cuda")
        stream = self.stream

        def step():
            h.all_gather(comms[0], src, dst, nbytes, h.HcclDataType.UINT8, stream)

        return step, 2 * nbytes, nbytes, 1.0, (src, dst), "plain copy 1 GiB (rankSize=1 AllGather)", "u8", 1, "copy"

    # ---- the entry points that marshal onto the same kernels (not among the five benchmark configurations) ----------
    def rsv(self, algo):
        """ReduceScatterV bf16, 8 ranks, uneven slices between 8 Mi and 24 Mi elements (16-byte aligned starts)."""
        import numpy as np
        t, h = self.torch, self.h
        n = 8
        comms = self.world(n)
        rng = np.random.default_rng(SEED + 6000)
        counts = (rng.integers(1 << 20, 3 << 20, n) * 8).astype(np.uint64)
        displs = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.uint64)
        total = int(counts.sum())
        sends = [t.randn(total, generator=self.gen(SEED + 6100 + r), device="cuda", dtype=t.bfloat16)
                 for r in range(n)]
        recvs = [t.empty(int(c), dtype=t.bfloat16, device="cuda") for c in counts]
        stream = self.stream
        cu, du = h.u64_array(counts), h.u64_array(displs)
        algo = algo or "mesh"
        h.set_algo(comms[0], h.OpKind.REDUCE_SCATTER, h.Algo[algo.upper()])

        def step():
            with h.group():
                for r in range(n):
                    h.reduce_scatter_v(comms[r], sends[r], cu, du, recvs[r], int(counts[r]), h.HcclDataType.BFP16,
                                       h.HcclReduceOp.SUM, stream)

        return step, (n + 1) * total * 2, total * 2, (n - 1) / n, (sends, recvs), \
            "ReduceScatterV SUM bf16 rankSize=8 slices U[8Mi,24Mi]", "bf16", n, algo

    def reduce(self, algo):
        t, h = self.torch, self.h
        n, count, root = 8, 1 << 26, 3
        comms = self.world(n)
        sends = [t.randn(count, generator=self.gen(SEED + 6200 + r), device="cuda", dtype=t.float32)
                 for r in range(n)]
        recv = t.empty(count, dtype=t.float32, device="cuda")
        stream = self.stream

        def step():
            with h.group():
                for r in range(n):
                    h.reduce(comms[r], sends[r], recv, count, h.HcclDataType.FP32, h.HcclReduceOp.SUM, root, stream)

        return step, (n + 1) * count * 4, count * 4, 1.0, (sends, recv), \
            "Reduce SUM fp32 rankSize=8 64Mi el/rank", "f32", n, "mesh"

    def bcast(self, algo):
        t, h = self.torch, self.h
        n, count, root, sets = 8, 1 << 27, 5, 4   # 4 buffer sets of 1 GiB in rotation
        comms = self.world(n)
        bufs = [[t.randint(0, 255, (count,), generator=self.gen(SEED + 6300 + 10 * k + r), device="cuda", dtype=t.uint8)
                 for r in range(n)] for k in range(sets)]
        stream = self.stream
        turn = [0]

        def step():
            k = turn[0]
            turn[0] = (k + 1) % sets
            with h.group():
                for r in range(n):
                    h.broadcast(comms[r], bufs[k][r], count, h.HcclDataType.UINT8, root, stream)

        return step, n * count, count, 1.0, bufs, "Broadcast rankSize=8 128 MiB, 4 buffer sets in rotation", "u8", n, "mesh"

    def ag(self, algo):
        """AllGather bf16, 16 ranks, 32 Mi elements (64 MiB) from every rank: 1 GiB into every recvBuf."""
        t, h = self.torch, self.h
        n, count = 16, 1 << 25
        comms = self.world(n)
        sends = [t.randint(-32768, 32767, (count,), generator=self.gen(SEED + 6600 + r), device="cuda", dtype=t.int16)
                 for r in range(n)]
        recvs = [t.empty(n * count, dtype=t.int16, device="cuda") for _ in range(n)]
        stream = self.stream

        def step():
            with h.group():
                for r in range(n):
                    h.all_gather(comms[r], sends[r], recvs[r], count, h.HcclDataType.BFP16, stream)

        total = n * count * 2
        return step, (1 + n) * total, total, (n - 1) / n, (sends, recvs), \
            "AllGather bf16 rankSize=16 32Mi el/rank", "bf16", n, "mesh"

    def scatter(self, algo):
        t, h = self.torch, self.h
        n, count, root = 8, 1 << 27, 2
        comms = self.world(n)
        send = t.randint(0, 255, (n * count,), generator=self.gen(SEED + 6400), device="cuda", dtype=t.uint8)
        recvs = [t.empty(count, dtype=t.uint8, device="cuda") for _ in range(n)]
        stream = self.stream

        def step():
            with h.group():
                for r in range(n):
                    h.scatter(comms[r], send if r == root else None, recvs[r], count, h.HcclDataType.UINT8, root,
                              stream)

        return step, 2 * n * count, n * count, (n - 1) / n, (send, recvs), "Scatter rankSize=8 128 MiB per rank", \
            "u8", n, "mesh"

    def a2a(self, algo):
        t, h = self.torch, self.h
        n, count = 16, 1 << 22
        comms = self.world(n)
        sends = [t.randint(-32768, 32767, (n * count,), generator=self.gen(SEED + 6500 + r), device="cuda",
                           dtype=t.int16) for r in range(n)]
        recvs = [t.empty(n * count, dtype=t.int16, device="cuda") for _ in range(n)]
        stream = self.stream

        def step():
            with h.group():
                for r in range(n):
                    h.all_to_all(comms[r], sends[r], count, h.HcclDataType.BFP16, recvs[r], count,
                                 h.HcclDataType.BFP16, stream)

        total = n * n * count * 2
        return step, 2 * total, total // n, (n - 1) / n, (sends, recvs), \
            "AlltoAll bf16 rankSize=16 4Mi el per pair", "bf16", n, "mesh"

    def c4(self, algo):
        import numpy as np
        t, h = self.torch, self.h
        n, hidden, tokens = 64, 7168, 16384
        comms = self.world(n)
        sc = zipf_routing(np, n, tokens, SEED + 4000 + 500) * hidden
        rc = sc.T.copy()
        sd = np.cumsum(sc, axis=1) - sc
        rd = np.cumsum(rc, axis=1) - rc
        sends = [t.randint(-32768, 32767, (tokens * hidden,), generator=self.gen(SEED + 4000 + r), device="cuda",
                           dtype=t.int16) for r in range(n)]
        recvs = [t.empty(max(int(rc[i].sum()), 8), dtype=t.int16, device="cuda") for i in range(n)]
        stream = self.stream
        rows = [tuple(h.u64_array(x[r]) for x in (sc, sd, rc, rd)) for r in range(n)]

        def step():
            with h.group():
                for r in range(n):
                    a, b, c, d = rows[r]
                    h.all_to_all_v(comms[r], sends[r], a, b, h.HcclDataType.BFP16, recvs[r], c, d,
                                   h.HcclDataType.BFP16, stream)

        total = int(sc.sum()) * 2
        return step, 2 * total, total // n, (n - 1) / n, (sends, recvs), \
            "AlltoAllV bf16 rankSize=64 16384 tokens x 7168 per rank, Zipf(1.1) routing", "bf16", n, "mesh"


def time_steps(torch, stream, step, steps, warmup):
    """HIP events on the stream the kernels are launched on, around exactly `steps` steps."""
    torch.cuda.synchronize()   # inputs were generated on torch's default stream
    for _ in range(warmup):
        step()
    stream.synchronize()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record(stream)
    for _ in range(steps):
        step()
    stop.record(stream)
    stream.synchronize()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    dev_ms = start.elapsed_time(stop) / steps
    return dev_ms, wall_ms


def measure(torch, wl, name, algo, steps, warmup):
    step, hbm, alg, bus, keep, desc, dtype, n, algo_used = getattr(wl, name)(algo)
    dev_ms, wall_ms = time_steps(torch, wl.stream, step, steps, warmup)
    t = dev_ms * 1e-3
    out = {"workload": desc, "algorithm": algo_used, "n_ranks": n, "steps": steps, "ms_per_step": round(dev_ms, 5 if dev_ms < 0.1 else 4),
           "wall_ms_per_step": round(wall_ms, 5 if wall_ms < 0.1 else 4),
           "algbw_GBs": round(alg / t / 1e9, 2), "busbw_GBs": round(alg / t / 1e9 * bus, 2),
           "hbm_GBs": round(hbm / t / 1e9, 2), "hbm_frac": round(hbm / t / 1e9 / HBM_PEAK_GBS, 4),
           "algorithmic_bytes": hbm, "dtype": dtype}
    del keep, step
    torch.cuda.empty_cache()
    return out


# ---------------------------------------------------------------------------------------------
# CPU baselines: the oracle's restatement of the reference's host path (pairwise reduce passes in the
# template's order, rounding after every step for 16-bit floats; one memcpy per slice for the copies), timed
# on a bounded sample of the same workload.  A case is built at a fraction `frac` of the per-rank size; the
# same rank count, data type, operator and fold order as the GPU leg.
# ---------------------------------------------------------------------------------------------
class CpuCase:
    def __init__(self, run, alg_bytes, bus, what, frac):
        self.run, self.alg_bytes, self.bus, self.what, self.frac = run, alg_bytes, bus, what, frac


def cpu_case(name, frac, algo, salt=0):
    import numpy as np
    import oracle

    def reduce_case(kind, cfg, n, full, np_make, dtype, op, acc, order, esz, label):
        c = max(64, int(full * frac)) // 64 * 64
        per_in = c * n if kind == "rs" else c
        ins = [np_make(np.random.default_rng(SEED + 1000 * cfg + r + 7919 * salt), per_in) for r in range(n)]
        outs = [np.zeros(c, dtype=ins[0].dtype) for _ in range(n)]
        fn = oracle.reduce_scatter if kind == "rs" else oracle.all_reduce

        def run():
            assert fn(ins, outs, c, dtype, op, acc=acc, algo=order) == 0

        alg = (n * c if kind == "rs" else c) * esz
        bus = (n - 1) / n if kind == "rs" else 2 * (n - 1) / n
        return CpuCase(run, alg, bus, "%s, %d of %d elements per rank, order '%s'" % (label, c, full, order), c / full)

    if name == "c1":
        mk = lambda rng, cnt: rng.uniform(-1, 1, cnt).astype(np.float32)
        return reduce_case("ar", 1, 8, 1 << 20, mk, oracle.FP32, oracle.SUM, oracle.ACC_STEP, algo or "ring", 4,
                           "fp32 host loop in rank order")
    if name == "c2":
        def mk(rng, cnt):   # N(0,1) rounded to nearest even bf16 (no NaN or overflow can occur)
            u = rng.standard_normal(cnt, dtype=np.float32).view(np.uint32)
            u += 0x7FFF + ((u >> 16) & 1)
            return (u >> 16).astype(np.uint16)

        return reduce_case("rs", 2, 8, 1 << 24, mk, oracle.BF16, oracle.SUM, oracle.ACC_STEP, algo or "ring", 2,
                           "bf16 by analogy with the fp16 host pattern (widen, fp32 add, narrow after every pairwise step)")
    if name == "c3max":
        mk = lambda rng, cnt: rng.integers(-2 ** 31, 2 ** 31, cnt, dtype=np.int64).astype(np.int32)
        return reduce_case("ar", 3, 16, 1 << 26, mk, oracle.INT32, oracle.MAX, oracle.ACC_STEP, algo or "mesh", 4,
                           "int32 MAX host loop")
    if name == "c3prod":
        mk = lambda rng, cnt: np.array([-2, -1, 1, 2], dtype=np.int32)[rng.integers(0, 4, cnt)]
        return reduce_case("ar", 3, 16, 1 << 26, mk, oracle.INT32, oracle.PROD, oracle.ACC_STEP, algo or "mesh", 4,
                           "int32 PROD host loop (wraparound)")
    if name == "c5a":
        mk = lambda rng, cnt: (rng.standard_normal(cnt, dtype=np.float32) * 0.5).astype(np.float16).view(np.uint16)
        return reduce_case("ar", 5, 6, 1 << 28, mk, oracle.FP16, oracle.SUM, oracle.ACC_STEP, algo or "rhd", 2,
                           "fp16 host pattern (widen, fp32 add, narrow after every pairwise step)")
    if name == "c4":
        n, hidden = 64, 7168
        tokens = max(n, int(16384 * frac))
        sc = zipf_routing(np, n, tokens, SEED + 4000 + 500 + salt) * hidden
        rc = sc.T.copy()
        sd = np.cumsum(sc, axis=1) - sc
        rd = np.cumsum(rc, axis=1) - rc
        rng = np.random.default_rng(SEED + 4000 + salt)
        ins = [rng.integers(0, 65536, tokens * hidden, dtype=np.uint16) for _ in range(n)]
        outs = [np.zeros(max(int(rc[i].sum()), 1), dtype=np.uint16) for i in range(n)]

        def run():
            assert oracle.all_to_all_v(ins, outs, sc, sd, rc, rd, oracle.BF16) == 0

        return CpuCase(run, int(sc.sum()) * 2 // n, (n - 1) / n,
                       "memcpy per (source, destination) segment, %d of 16384 tokens per rank" % tokens, tokens / 16384)
    if name == "c5b":
        n = 6
        counts = gather_v_counts(np, n, 1 << 20, 32 << 20, SEED + 5000 + 500)
        counts = np.maximum(1, (counts * frac).astype(np.uint64))
        displs = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.uint64)
        total = int(counts.sum())
        rng = np.random.default_rng(SEED + 5000 + 600 + salt)
        ins = [rng.integers(0, 65536, int(c), dtype=np.uint16) for c in counts]
        outs = [np.zeros(total, dtype=np.uint16) for _ in range(n)]

        def run():
            assert oracle.all_gather_v(ins, outs, counts, displs, oracle.FP16) == 0

        return CpuCase(run, total * 2, (n - 1) / n,
                       "memcpy per slice, counts scaled to %.4g of U[1Mi,32Mi]" % frac, frac)
    return None


# Largest sample of each workload, as a fraction of its per-rank size: bounds host memory and set-up time.
CPU_MAX_FRAC = {"c1": 1.0, "c2": 1 / 8, "c3max": 1 / 16, "c3prod": 1 / 16, "c5a": 1 / 32, "c4": 1 / 32, "c5b": 1 / 8}


def timed(run, passes=1):
    t0 = time.perf_counter()
    for _ in range(passes):
        run()
    return (time.perf_counter() - t0) / passes


def cpu_baseline(name, algo, seconds):
    """One-thread figure (faithful: the reference's loop is single-threaded) and an all-cores figure (the sample
    cut into as many independent collectives as there are cores, one thread each)."""
    top = CPU_MAX_FRAC.get(name)
    if top is None:
        return None
    probe = cpu_case(name, top / 64, algo)
    probe.run()                                  # page in the outputs
    per_frac = timed(probe.run) / probe.frac     # seconds per unit fraction
    frac = min(top, max(probe.frac, seconds / per_frac))
    case = cpu_case(name, frac, algo) if frac > probe.frac else probe
    case.run()
    passes = max(1, int(round(seconds / (per_frac * case.frac))))
    dt = timed(case.run, passes)
    one = case.alg_bytes / dt / 1e9 * case.bus
    cores = min(16, os.cpu_count() or 1)
    parts = [cpu_case(name, frac / cores, algo, salt=1 + k) for k in range(cores)]
    for p in parts:
        p.run()
    threads = [threading.Thread(target=timed, args=(p.run, passes)) for p in parts]
    t0 = time.perf_counter()
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    dt_mt = time.perf_counter() - t0
    many = passes * sum(p.alg_bytes for p in parts) / dt_mt / 1e9 * parts[0].bus
    return {"value": round(one, 4), "unit": "GB/s busBW", "cores": 1, "kind": "port",
            "sample": "%d pass(es) over %s; %.1f s in all" % (passes, case.what, dt * passes),
            "all_cores": {"value": round(many, 4), "cores": cores, "seconds": round(dt_mt, 2),
                          "sample": "%d independent collectives of 1/%d of that sample, one thread each, %d pass(es)" % (cores, cores, passes)}}


TRAFFIC_FILE = os.path.join("profiles", "reduce_scatter_bf16_n8_pmc.txt")


def traffic_from_profiles():
    """HBM bytes per launch of the headline kernel as counted with rocprofv3 --pmc in an earlier run (the committed
    summary); this run does not measure it."""
    path = os.path.join(ROOT, TRAFFIC_FILE)
    if not os.path.exists(path):
        return None
    m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", open(path).read(), re.M)
    return float(m.group(1)) if m else None


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures the one-GPU loopback data plane; --gpus %d is not supported "
              "(every box has one GPU and nothing here uses a second)." % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    import hccl_amd
    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    torch.cuda.set_device(0)
    hccl_amd.lib()
    wl = Workloads(torch, hccl_amd)

    main_res = measure(torch, wl, args.workload, args.algo, args.steps, args.warmup)
    others = {}
    if not args.no_others:
        names = [n for n in CONFIGS if n != args.workload]
        if args.extra:
            names += [n for n in EXTRA if n != args.workload]
        for name in names:
            # the tiny configuration needs many steps for a stable figure, the large ones few
            steps = max(args.steps, 200) if name == "c1" else max(3, args.steps // 2)
            others[name] = measure(torch, wl, name, None, steps, 3)
    del wl
    torch.cuda.empty_cache()

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(args.workload, args.algo, args.cpu_seconds)
        for name, res in others.items():
            res["cpu_baseline"] = cpu_baseline(name, None, args.cpu_seconds_others)

    hbm = main_res["algorithmic_bytes"]
    t = main_res["ms_per_step"] * 1e-3
    traffic = traffic_from_profiles() if (args.workload == "c2" and args.algo in (None, "ring")) else None
    line = {
        "metric": "busBW GB/s + % of HBM peak, AllReduce/ReduceScatter 8-rank loopback, 1 MI355X",
        "value": main_res["busbw_GBs"], "unit": "GB/s busBW", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": main_res["dtype"], "data": "synthetic",
        "config": {"workload": main_res["workload"], "algorithm": main_res["algorithm"],
                   "rank_size": main_res["n_ranks"], "algbw_GBs": main_res["algbw_GBs"],
                   "hbm_percent_of_peak": round(100 * main_res["hbm_frac"], 2)},
        "roofline": {"bound": "hbm", "achieved": round(hbm / t / 1e9, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(hbm / t / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": traffic,
                     "traffic_source": (TRAFFIC_FILE + " (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE of this kernel in a "
                                        "profiling run of this command, calibrated against a plain copy; the "
                                        "counters cannot be read while timing)") if traffic else None,
                     "algorithmic_bytes_per_launch": hbm, "launch_ms": main_res["ms_per_step"],
                     "timing": "HIP events on the launch stream around the timed steps, one kernel launch per step "
                               "(the rocprofv3 kernel duration of the same command is in profiles/)"},
        "cpu_baseline": cpu,
    }
    if others:
        line["others"] = others
    print(json.dumps(line))


if __name__ == "__main__":
    main()
