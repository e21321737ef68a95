#!/usr/bin/env python3
"""Benchmark of the loopback data plane on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2] [--others]

A step is one collective over all N loopback ranks (N per-rank calls through the C ABI inside a
group, one fused kernel launch).  The headline workload is the configuration the metric is quoted
on: ReduceScatter SUM bf16, rankSize 8, 134,217,728 elements in / 16,777,216 out per rank, "ring"
algorithm.  Inputs are synthetic (seeded torch generators) and resident in HBM before timing starts.
Prints ONE JSON line.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
GIB = float(1 << 30)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3max", "c3prod", "c4", "c5a", "c5b", "copycal", "rsv", "reduce", "bcast", "scatter",
                             "a2a"])
    ap.add_argument("--algo", default=None, help="override the algorithm of the workload (mesh/ring/rhd/nhr/...)")
    ap.add_argument("--others", action="store_true", help="also time the other benchmark configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    return ap.parse_args()


# ---------------------------------------------------------------------------------------------
# Workloads.  Each returns (run_step, algorithmic_bytes, alg_bytes_for_algbw, n, description, dtype)
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

    def _reduce(self, kind, n, count, tdtype, hdtype, op, algo, make):
        t, h = self.torch, self.h
        comms = self.world(n)
        per_rank_in = count * n if kind == "rs" else count
        sends = [make(per_rank_in, 0xC0FFEE + r) for r in range(n)]
        recvs = [t.empty(count, dtype=tdtype, device="cuda") for _ in range(n)]
        opk = h.OpKind.REDUCE_SCATTER if kind == "rs" else h.OpKind.ALL_REDUCE
        h.set_algo(comms[0], opk, h.Algo[algo.upper()])
        fn = h.reduce_scatter if kind == "rs" else h.all_reduce
        stream = self.stream

        def step():
            with h.group():
                for r in range(n):
                    fn(comms[r], sends[r], recvs[r], count, hdtype, op, stream)

        esz = sends[0].element_size()
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
        return self._reduce("ar", 8, 1 << 20, t.float32, h.HcclDataType.FP32, h.HcclReduceOp.SUM, algo or "ring", mk) + (
            "AllReduce SUM fp32 rankSize=8 1Mi el/rank", "f32", 8)

    def c2(self, algo):
        t, h = self.torch, self.h
        mk = lambda cnt, seed: t.randn(cnt, generator=self.gen(seed), device="cuda", dtype=t.bfloat16)
        return self._reduce("rs", 8, 1 << 24, t.bfloat16, h.HcclDataType.BFP16, h.HcclReduceOp.SUM, algo or "ring", mk) + (
            "ReduceScatter SUM bf16 rankSize=8 128Mi el in / 16Mi out per rank", "bf16", 8)

    def c3max(self, algo):
        t, h = self.torch, self.h
        mk = lambda cnt, seed: t.randint(-2 ** 31, 2 ** 31 - 1, (cnt,), generator=self.gen(seed), device="cuda",
                                         dtype=t.int32)
        return self._reduce("ar", 16, 1 << 26, t.int32, h.HcclDataType.INT32, h.HcclReduceOp.MAX, algo or "mesh", mk) + (
            "AllReduce MAX int32 rankSize=16 64Mi el/rank", "int32", 16)

    def c3prod(self, algo):
        t, h = self.torch, self.h
        lut = t.tensor([-2, -1, 1, 2], dtype=t.int32, device="cuda")
        mk = lambda cnt, seed: lut[t.randint(0, 4, (cnt,), generator=self.gen(seed), device="cuda")]
        return self._reduce("ar", 16, 1 << 26, t.int32, h.HcclDataType.INT32, h.HcclReduceOp.PROD, algo or "mesh", mk) + (
            "AllReduce PROD int32 rankSize=16 64Mi el/rank", "int32", 16)

    def c5a(self, algo):
        t, h = self.torch, self.h
        mk = lambda cnt, seed: (t.randn(cnt, generator=self.gen(seed), device="cuda", dtype=t.float32) * 0.5).half()
        return self._reduce("ar", 6, 1 << 28, t.float16, h.HcclDataType.FP16, h.HcclReduceOp.SUM, algo or "rhd", mk) + (
            "AllReduce SUM fp16 rankSize=6 RHD 256Mi el/rank", "f16", 6)

    def c5b(self, algo):
        import numpy as np
        t, h = self.torch, self.h
        n = 6
        comms = self.world(n)
        rng = np.random.default_rng(0xC0FFEE + 5001)
        counts = rng.integers(1 << 20, (32 << 20) + 1, n).astype(np.uint64)
        displs = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.uint64)
        total = int(counts.sum())
        sends = [t.randn(int(c), generator=self.gen(0xC0FFEE + 5100 + r), device="cuda", dtype=t.float16)
                 for r, c in enumerate(counts)]
        recvs = [t.empty(total, dtype=t.float16, device="cuda") for _ in range(n)]
        stream = self.stream

        def step():
            with h.group():
                for r in range(n):
                    h.all_gather_v(comms[r], sends[r], int(counts[r]), recvs[r], counts, displs,
                                   h.HcclDataType.FP16, stream)

        hbm = (1 + n) * total * 2
        return step, hbm, total * 2, (n - 1) / n, (sends, recvs), \
            "AllGatherV fp16 rankSize=6 counts U[1Mi,32Mi]", "u8", n

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

        return step, 2 * nbytes, nbytes, 1.0, (src, dst), "plain copy 1 GiB (rankSize=1 AllGather)", "u8", 1

    # ---- the entry points that marshal onto the same kernels (not among the five benchmark configurations) ----------
    def rsv(self, algo):
        """ReduceScatterV bf16, 8 ranks, uneven slices between 8 Mi and 24 Mi elements (16-byte aligned starts)."""
        import numpy as np
        t, h = self.torch, self.h
        n = 8
        comms = self.world(n)
        rng = np.random.default_rng(0xC0FFEE + 6000)
        counts = (rng.integers(1 << 20, 3 << 20, n) * 8).astype(np.uint64)
        displs = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.uint64)
        total = int(counts.sum())
        sends = [t.randn(total, generator=self.gen(0xC0FFEE + 6100 + r), device="cuda", dtype=t.bfloat16)
                 for r in range(n)]
        recvs = [t.empty(int(c), dtype=t.bfloat16, device="cuda") for c in counts]
        stream = self.stream
        cu, du = h.u64_array(counts), h.u64_array(displs)

        def step():
            with h.group():
                for r in range(n):
                    h.reduce_scatter_v(comms[r], sends[r], cu, du, recvs[r], int(counts[r]), h.HcclDataType.BFP16,
                                       h.HcclReduceOp.SUM, stream)

        return step, (n + 1) * total * 2, total * 2, (n - 1) / n, (sends, recvs), \
            "ReduceScatterV SUM bf16 rankSize=8 slices U[8Mi,24Mi]", "bf16", n

    def reduce(self, algo):
        t, h = self.torch, self.h
        n, count, root = 8, 1 << 26, 3
        comms = self.world(n)
        sends = [t.randn(count, generator=self.gen(0xC0FFEE + 6200 + r), device="cuda", dtype=t.float32)
                 for r in range(n)]
        recv = t.empty(count, dtype=t.float32, device="cuda")
        stream = self.stream

        def step():
            with h.group():
                for r in range(n):
                    h.reduce(comms[r], sends[r], recv, count, h.HcclDataType.FP32, h.HcclReduceOp.SUM, root, stream)

        return step, (n + 1) * count * 4, count * 4, 1.0, (sends, recv), \
            "Reduce SUM fp32 rankSize=8 64Mi el/rank", "f32", n

    def bcast(self, algo):
        t, h = self.torch, self.h
        n, count, root = 8, 1 << 27, 5
        comms = self.world(n)
        bufs = [t.randint(0, 255, (count,), generator=self.gen(0xC0FFEE + 6300 + r), device="cuda", dtype=t.uint8)
                for r in range(n)]
        stream = self.stream

        def step():
            with h.group():
                for r in range(n):
                    h.broadcast(comms[r], bufs[r], count, h.HcclDataType.UINT8, root, stream)

        return step, n * count, count, 1.0, bufs, "Broadcast rankSize=8 128 MiB", "u8", n

    def scatter(self, algo):
        t, h = self.torch, self.h
        n, count, root = 8, 1 << 27, 2
        comms = self.world(n)
        send = t.randint(0, 255, (n * count,), generator=self.gen(0xC0FFEE + 6400), device="cuda", dtype=t.uint8)
        recvs = [t.empty(count, dtype=t.uint8, device="cuda") for _ in range(n)]
        stream = self.stream

        def step():
            with h.group():
                for r in range(n):
                    h.scatter(comms[r], send if r == root else None, recvs[r], count, h.HcclDataType.UINT8, root,
                              stream)

        return step, 2 * n * count, n * count, (n - 1) / n, (send, recvs), "Scatter rankSize=8 128 MiB per rank", "u8", n

    def a2a(self, algo):
        t, h = self.torch, self.h
        n, count = 16, 1 << 22
        comms = self.world(n)
        sends = [t.randint(-32768, 32767, (n * count,), generator=self.gen(0xC0FFEE + 6500 + r), device="cuda",
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
            "AlltoAll bf16 rankSize=16 4Mi el per pair", "u8", n

    def c4(self, algo):
        import numpy as np
        t, h = self.torch, self.h
        n, hidden, tokens = 64, 7168, 16384
        comms = self.world(n)
        rng = np.random.default_rng(0xC0FFEE + 4000)
        wts = 1.0 / np.arange(1, n + 1) ** 1.1
        wts /= wts.sum()
        tok = np.stack([rng.multinomial(tokens, wts) for _ in range(n)]).astype(np.uint64)
        sc = tok * hidden
        rc = sc.T.copy()
        sd = np.cumsum(sc, axis=1) - sc
        rd = np.cumsum(rc, axis=1) - rc
        sends = [t.randint(-32768, 32767, (tokens * hidden,), generator=self.gen(0xC0FFEE + 4100 + r), device="cuda",
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
            "AlltoAllV bf16 rankSize=64 16384 tokens x 7168 per rank, Zipf(1.1) routing", "u8", n


def time_steps(torch, stream, step, steps, warmup):
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
    step, hbm, alg, bus, keep, desc, dtype, n = getattr(wl, name)(algo)
    dev_ms, wall_ms = time_steps(torch, wl.stream, step, steps, warmup)
    t = dev_ms * 1e-3
    out = {"workload": desc, "n_ranks": n, "ms_per_step": round(dev_ms, 4), "wall_ms_per_step": round(wall_ms, 4),
           "algbw_GBs": round(alg / t / 1e9, 2), "busbw_GBs": round(alg / t / 1e9 * bus, 2),
           "hbm_GBs": round(hbm / t / 1e9, 2), "hbm_frac": round(hbm / t / 1e9 / HBM_PEAK_GBS, 4),
           "algorithmic_bytes": hbm, "dtype": dtype}
    del keep
    torch.cuda.empty_cache()
    return out


# ---------------------------------------------------------------------------------------------
# CPU baseline: the oracle's restatement of the reference's host reduce path (pairwise passes that
# round after every step), on a bounded sample of the same workload.
# ---------------------------------------------------------------------------------------------
def cpu_baseline_c2(seconds):
    import numpy as np
    import oracle
    n, sz = 8, 2
    rng = np.random.default_rng(0xC0FFEE + 2000)

    made = {}

    def run(c, threads, passes=1):
        if c not in made:
            made.clear()
            made[c] = [oracle.np_fp32_to_bf16_bits(rng.standard_normal(n * c, dtype=np.float32)) for _ in range(n)]
        ins = made[c]
        outs = [np.zeros(c, dtype=np.uint16) for _ in range(n)]
        t0 = time.perf_counter()
        for _ in range(passes):
            if threads == 1:
                rc = oracle.reduce_scatter(ins, outs, c, oracle.BF16, oracle.SUM, acc=oracle.ACC_STEP, algo="mesh")
            else:
                rc = oracle.reduce_scatter_mt(ins, outs, c, oracle.BF16, oracle.SUM, oracle.ACC_STEP, threads)
            assert rc == 0
        return (time.perf_counter() - t0) / passes

    probe_c = 1 << 15
    rate = probe_c / run(probe_c, 1)                       # output elements per rank per second
    c = int(min(1 << 24, max(1 << 15, rate * seconds)))
    c -= c % 8
    # the whole workload may take less than the time asked for: then time several passes over it
    passes = max(1, int(round(seconds / (c / rate))))
    dt = run(c, 1, passes)
    busbw = n * c * sz / dt / 1e9 * (n - 1) / n
    cores = min(16, os.cpu_count() or 1)
    dt_mt = run(c, cores)
    return {"value": round(busbw, 4), "unit": "GB/s busBW", "cores": 1, "kind": "port",
            "sample": "%d pass(es) over recvCount %d of 16777216 per rank (same 8-rank bf16 ReduceScatter, host "
                      "pattern: widen, fp32 add, narrow after every pairwise step), %.1f s in all" % (passes, c, dt * passes),
            "all_cores": {"value": round(n * c * sz / dt_mt / 1e9 * (n - 1) / n, 4), "cores": cores,
                          "seconds": round(dt_mt, 2)}}


def traffic_from_profiles():
    """HBM bytes per launch measured with rocprofv3 --pmc, if a summary has been committed."""
    path = os.path.join(ROOT, "profiles", "reduce_scatter_bf16_n8_pmc.txt")
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
    if args.others:
        for name in ("c1", "c2", "c3max", "c3prod", "c4", "c5a", "c5b"):
            if name != args.workload:
                others[name] = measure(torch, wl, name, None, max(3, args.steps // 2), 2)
        if args.workload == "c2":
            others["c2_mesh_order"] = measure(torch, wl, "c2", "mesh", args.steps, 2)
        for name in ("rsv", "reduce", "bcast", "scatter", "a2a"):
            if name != args.workload:
                others[name] = measure(torch, wl, name, None, max(3, args.steps // 2), 2)

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline_c2(args.cpu_seconds)

    hbm = main_res["algorithmic_bytes"]
    t = main_res["ms_per_step"] * 1e-3
    line = {
        "metric": "busBW GB/s + % of HBM peak, AllReduce/ReduceScatter 8-rank loopback, 1 MI355X",
        "value": main_res["busbw_GBs"], "unit": "GB/s busBW", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": main_res["dtype"], "data": "synthetic",
        "config": {"workload": main_res["workload"], "algorithm": args.algo or "default of the workload",
                   "rank_size": main_res["n_ranks"], "algbw_GBs": main_res["algbw_GBs"],
                   "hbm_percent_of_peak": round(100 * main_res["hbm_frac"], 2)},
        "roofline": {"bound": "hbm", "achieved": round(hbm / t / 1e9, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(hbm / t / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": traffic_from_profiles() if args.workload == "c2" else None,
                     "algorithmic_bytes_per_launch": hbm, "kernel_ms": main_res["ms_per_step"]},
        "cpu_baseline": cpu,
    }
    if others:
        line["others"] = others
    print(json.dumps(line))


if __name__ == "__main__":
    main()
