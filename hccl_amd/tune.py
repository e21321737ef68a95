"""Times both sides of the launch-form thresholds of hccl_amd/csrc/launch_policy.h on the GPU at hand.

    python -m hccl_amd.tune [--quick]
    python -m hccl_amd.tune --all-gather 16:1,2 8:2,4,6 --broadcast 9:16,24,32     (ranks:MiB per rank,... per table)
    python -m hccl_amd.tune --all-reduce-small 8:2048,4096                          (ranks:KiB per rank,...)

For every shape of a small grid the forms the policy chooses between are run on the same buffers, interleaved
(worlds created with the overriding environment variable set), and the table shows each form's fraction of the 8 TB/s
HBM peak, the form the library picks by itself and whether a forced form beats it by more than two per cent: a row
marked `<-- ` is a threshold to look at after a kernel change or on another part.  Buffer sets rotate where one
set would fit the last-level cache.  Needs the built library and a GPU; nothing here is used by the library itself.
"""
import argparse
import os
import statistics
import sys

HBM_PEAK = 8e12


def _time(torch, stream, step, steps):
    for _ in range(3):
        step()
    stream.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record(stream)
    for _ in range(steps):
        step()
    b.record(stream)
    stream.synchronize()
    return a.elapsed_time(b) / steps


def _forms(torch, h, make_step, forms, moved, rounds, steps):
    """forms: [(name, {env})]; make_step(comms) -> step().  Returns {name: fraction of peak} (median over rounds)."""
    times = {name: [] for name, _ in forms}
    stream = torch.cuda.Stream()
    for _ in range(rounds):
        for name, env in forms:
            saved = {k: os.environ.get(k) for k in env}
            os.environ.update(env)
            try:
                n, step = make_step(stream)
                times[name].append(_time(torch, stream, step, steps))
                for c in n:
                    h.comm_destroy(c)
            finally:
                for k, v in saved.items():
                    if v is None:
                        os.environ.pop(k, None)
                    else:
                        os.environ[k] = v
    return {name: moved / (statistics.median(t) * 1e-3) / HBM_PEAK for name, t in times.items()}


def _row(label, fracs, own="auto"):
    """Prints one row and returns (label, fracs)."""
    best = max((v, k) for k, v in fracs.items() if k != own)
    flag = "   <-- %s is %.1f %% ahead of the library's choice" % (best[1], 100 * (best[0] / fracs[own] - 1)) \
        if best[0] > 1.02 * fracs[own] else ""
    print("%-34s %s%s" % (label, "  ".join("%s %.3f" % (k, v) for k, v in fracs.items()), flag), flush=True)
    return label, fracs


def all_reduce_rows(torch, h, ranks, mibs, rounds):
    print("# AllReduce fp32 SUM in rank order: fused kernel with 1 / 2 / 3 wavefronts sharing a tile's stores, fold + "
          "fan-out, the library's own choice")
    rows = []
    for n in ranks:
        for mib in mibs:
            count = (mib << 20) // 4
            per_set = 2 * n * count * 4
            sets = max(1, min(8, -(-(600 << 20) // per_set)))
            sends = [[torch.randn(count, device="cuda") for _ in range(n)] for _ in range(sets)]
            recvs = [[torch.empty(count, device="cuda") for _ in range(n)] for _ in range(sets)]
            torch.cuda.synchronize()

            def make_step(stream):
                comms = h.comm_init_all(n)
                turn = [0]

                def step():
                    k = turn[0]
                    turn[0] = (k + 1) % sets
                    with h.group():
                        for r in range(n):
                            h.all_reduce(comms[r], sends[k][r], recvs[k][r], count, h.HcclDataType.FP32,
                                         h.HcclReduceOp.SUM, stream)
                return comms, step

            fused = {"HCCL_AMD_ALLREDUCE_TWO_KERNELS": "0"}
            forms = [("w1", dict(fused, HCCL_AMD_REDUCE_STORE_WAVES="1")),
                     ("w2", dict(fused, HCCL_AMD_REDUCE_STORE_WAVES="2")),
                     ("w3", dict(fused, HCCL_AMD_REDUCE_STORE_WAVES="3")),
                     ("two", {"HCCL_AMD_ALLREDUCE_TWO_KERNELS": "1"}), ("auto", {})]
            steps = 10 if per_set > (200 << 20) else 50
            rows.append(_row("%2d ranks x %4d MiB" % (n, mib), _forms(torch, h, make_step, forms, per_set, rounds, steps)))
            del sends, recvs
            torch.cuda.empty_cache()
    return rows


def all_reduce_small_rows(torch, h, ranks, kibs, rounds, only=None):
    print("# AllReduce fp32 SUM in rank order, a few MiB per rank: the general kernel with one tile per wavefront, two, "
          "workgroups of 2 / 3 / 4 wavefronts that exchange their tiles and store one or two streams each; up to eight "
          "ranks also the kernel launched from its arguments alone with 2 / 3 / 4 / 6 / 8 wavefronts; the library's own "
          "choice (collectives issued with their arguments converted once)")
    rows = []
    for n in ranks:
        for kib in kibs:
            count = (kib << 10) // 4
            per_set = 2 * n * count * 4
            sets = max(1, min(12, -(-(600 << 20) // per_set)))
            sends = [[torch.randn(count, device="cuda") for _ in range(n)] for _ in range(sets)]
            recvs = [[torch.empty(count, device="cuda") for _ in range(n)] for _ in range(sets)]
            torch.cuda.synchronize()

            def make_step(stream):
                comms = h.comm_init_all(n)
                groups = [h.prepared_group([("HcclAllReduce", (sends[k][r], recvs[k][r], count, h.HcclDataType.FP32,
                                                               h.HcclReduceOp.SUM, comms[r], stream))
                                            for r in range(n)]) for k in range(sets)]
                turn = [0]

                def step():
                    k = turn[0]
                    turn[0] = (k + 1) % sets
                    groups[k]()
                return comms, step

            off = {"HCCL_AMD_REDUCE_DIRECT": "0"}
            forms = [("one", dict(off, HCCL_AMD_REDUCE_PAIR="0", HCCL_AMD_REDUCE_ALL_FOLD="0")),
                     ("pair", dict(off, HCCL_AMD_REDUCE_PAIR="1", HCCL_AMD_REDUCE_ALL_FOLD="0")),
                     ("fold2", dict(off, HCCL_AMD_REDUCE_ALL_FOLD="2")), ("fold3", dict(off, HCCL_AMD_REDUCE_ALL_FOLD="3")),
                     ("fold4", dict(off, HCCL_AMD_REDUCE_ALL_FOLD="4"))]
            if n <= 8:
                forms += [("direct%d" % k, {"HCCL_AMD_REDUCE_DIRECT": str(k), "HCCL_AMD_REDUCE_DIRECT_TILES": "1"})
                          for k in (2, 3, 4, 6, 8)]
                forms += [("direct%dx2" % k, {"HCCL_AMD_REDUCE_DIRECT": str(k), "HCCL_AMD_REDUCE_DIRECT_TILES": "2"})
                          for k in (4, 8)]
            elif n <= 16:
                forms += [("direct%d" % k, {"HCCL_AMD_REDUCE_DIRECT": str(k)}) for k in (2, 4, 8)]
            if only is not None:
                forms = [f for f in forms if f[0] in only]
            forms.append(("auto", {}))
            fracs = _forms(torch, h, make_step, forms, per_set, rounds, 200)
            us = "/".join("%.1f" % (per_set / (v * HBM_PEAK) * 1e6) for v in fracs.values())
            rows.append(_row("%2d ranks x %5d KiB  %s us" % (n, kib, us), fracs))
            del sends, recvs
            torch.cuda.empty_cache()
    return rows


COPY_FORMS = [("one", {"HCCL_AMD_COPY_TWO_KERNELS": "0"}), ("two", {"HCCL_AMD_COPY_TWO_KERNELS": "1"}), ("auto", {})]


def all_gather_rows(torch, h, ranks, mibs, rounds):
    print("# AllGather: one kernel, gather + fan-out, the library's own choice")
    rows = []
    for n in ranks:
        for mib in mibs:
            nbytes = mib << 20
            per_set = (1 + n) * n * nbytes
            sets = max(1, min(6, -(-(600 << 20) // per_set)))
            sends = [[torch.randint(0, 255, (nbytes,), device="cuda", dtype=torch.uint8) for _ in range(n)]
                     for _ in range(sets)]
            recvs = [[torch.empty(n * nbytes, device="cuda", dtype=torch.uint8) for _ in range(n)] for _ in range(sets)]
            torch.cuda.synchronize()

            def make_step(stream):
                comms = h.comm_init_all(n)
                turn = [0]

                def step():
                    k = turn[0]
                    turn[0] = (k + 1) % sets
                    with h.group():
                        for r in range(n):
                            h.all_gather(comms[r], sends[k][r], recvs[k][r], nbytes, h.HcclDataType.UINT8, stream)
                return comms, step

            forms = COPY_FORMS
            steps = 10 if per_set > (200 << 20) else 50
            rows.append(_row("%2d ranks x %4d MiB" % (n, mib), _forms(torch, h, make_step, forms, per_set, rounds, steps)))
            del sends, recvs
            torch.cuda.empty_cache()
    return rows


def broadcast_rows(torch, h, ranks, mibs, rounds):
    print("# Broadcast from rank 0: one kernel, copy + fan-out, the library's own choice")
    rows = []
    for n in ranks:
        for mib in mibs:
            nbytes = mib << 20
            per_set = n * nbytes
            sets = max(1, min(8, -(-(600 << 20) // per_set)))
            bufs = [[torch.randint(0, 255, (nbytes,), device="cuda", dtype=torch.uint8) for _ in range(n)]
                    for _ in range(sets)]
            torch.cuda.synchronize()

            def make_step(stream):
                comms = h.comm_init_all(n)
                turn = [0]

                def step():
                    k = turn[0]
                    turn[0] = (k + 1) % sets
                    with h.group():
                        for r in range(n):
                            h.broadcast(comms[r], bufs[k][r], nbytes, h.HcclDataType.UINT8, 0, stream)
                return comms, step

            forms = COPY_FORMS
            steps = 10 if per_set > (200 << 20) else 50
            rows.append(_row("%2d ranks x %4d MiB" % (n, mib), _forms(torch, h, make_step, forms, per_set, rounds, steps)))
            del bufs
            torch.cuda.empty_cache()
    return rows


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--quick", action="store_true", help="a third of the grid, one round")
    ap.add_argument("--all-reduce", nargs="*", metavar="RANKS:MIB,..", help="AllReduce rows of these shapes only")
    ap.add_argument("--all-reduce-small", nargs="*", metavar="RANKS:KIB,..", help="small AllReduce rows of these shapes only")
    ap.add_argument("--all-gather", nargs="*", metavar="RANKS:MIB,..", help="AllGather rows of these shapes only")
    ap.add_argument("--broadcast", nargs="*", metavar="RANKS:MIB,..", help="Broadcast rows of these shapes only")
    args = ap.parse_args()
    import torch
    import hccl_amd as h
    if not torch.cuda.is_available():
        sys.exit("hccl_amd.tune needs the GPU")
    torch.cuda.set_device(0)
    h.lib()
    rounds = 1 if args.quick else 3
    chosen = [(args.all_reduce, all_reduce_rows), (args.all_reduce_small, all_reduce_small_rows),
              (args.all_gather, all_gather_rows), (args.broadcast, broadcast_rows)]
    if any(specs is not None for specs, _ in chosen):
        for specs, rows in chosen:
            for spec in specs or []:
                ranks, mibs = spec.split(":")
                rows(torch, h, [int(ranks)], [int(m) for m in mibs.split(",")], rounds)
        return
    all_reduce_rows(torch, h, [3, 4, 6, 8, 16] if not args.quick else [4, 8], [16, 64, 256] if not args.quick else [64],
                    rounds)
    all_reduce_small_rows(torch, h, [2, 8] if not args.quick else [8], [2048, 4096, 8192] if not args.quick else [4096], rounds)
    all_gather_rows(torch, h, [4, 6, 8, 16] if not args.quick else [8], [8, 64] if not args.quick else [64], rounds)
    broadcast_rows(torch, h, [6, 8, 16] if not args.quick else [8], [16, 64] if not args.quick else [64], rounds)


if __name__ == "__main__":
    main()
