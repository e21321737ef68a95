"""The reference's own Python suites (experimental/eco_system/python/tests/run_reduce_op_suite.py and
run_dtype_suite.py), replayed call for call through the mirror of hccl4py.ops: one host thread per rank, blocking
calls, the same tiny buffers and closed-form expectations (tests/golden/hccl4py_closed_form_suites.json)."""
import json
import os
import threading

import numpy as np
import pytest

import hccl_amd as h
import oracle
from hccl_amd import HcclDataType as DT, HcclReduceOp as OP

import gpu_util
from gpu_util import require_library_on_gpu

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "hccl4py_closed_form_suites.json")))
NP = {"INT8": np.int8, "INT16": np.int16, "INT32": np.int32, "INT64": np.int64, "UINT8": np.uint8,
      "UINT16": np.uint16, "UINT32": np.uint32, "UINT64": np.uint64, "FP16": np.float16, "FP32": np.float32,
      "FP64": np.float64, "BFP16": None}
# reduce ops do not admit these types (reference op_common.cc:4349-4413, reduce_scatter_v.cc:225-247)
NOT_REDUCIBLE = {"UINT8", "UINT16", "UINT32"}
NOT_REDUCIBLE_V = NOT_REDUCIBLE | {"UINT64", "FP64"}


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


def pack(name, values):
    if name == "BFP16":
        return oracle.np_fp32_to_bf16_bits(np.asarray(values, dtype=np.float32))
    return np.asarray(values).astype(NP[name])


def unpack(name, raw, n):
    if name == "BFP16":
        return oracle.bf16_bits_to_fp32(raw.view(np.uint16)[:n]).astype(np.float64)
    return raw.view(NP[name])[:n].astype(np.float64)


def run_ranks(nranks, body):
    """body(rank, comm, stream, to_dev, to_host) in one thread per rank; returns the per-rank results."""
    if not gpu_util.EMU:
        import torch
    info = h.get_root_info()
    out = [None] * nranks
    errors = []
    # A rank that is through may not destroy its communicator while a peer still has point-to-point calls to make:
    # destroying one rank ends the world for all of them.
    all_through = threading.Barrier(nranks)

    def main(rank):
        try:
            comm = h.comm_init_root_info(nranks, info, rank)
            if gpu_util.EMU:   # the CPU emulation run: host buffers, launches run to completion
                out[rank] = body(rank, comm, gpu_util._EmuStream(), gpu_util.to_dev, lambda t: t.read())
                all_through.wait(90)
                h.comm_destroy(comm)
                return
            stream = torch.cuda.Stream()

            def to_dev(arr):
                t = torch.from_numpy(np.ascontiguousarray(arr).view(np.uint8).reshape(-1).copy()).cuda()
                torch.cuda.current_stream().synchronize()
                return t

            def to_host(t):
                stream.synchronize()
                return t.cpu().numpy()
            out[rank] = body(rank, comm, stream, to_dev, to_host)
            stream.synchronize()
            all_through.wait(90)
            h.comm_destroy(comm)
        except Exception as e:   # noqa: BLE001 - reported below
            errors.append((rank, repr(e)))

    threads = [threading.Thread(target=main, args=(r,)) for r in range(nranks)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(100)
    assert not errors, errors
    return out


def zeros(nbytes):
    """A cleared device buffer; the fill (on torch's current stream) has finished when this returns, so that a
    collective on another stream, possibly a peer's, cannot be overtaken by it."""
    if gpu_util.EMU:
        return gpu_util.dev_zeros(max(nbytes, 1), fill=0)
    import torch
    t = torch.zeros(max(nbytes, 1), dtype=torch.uint8, device="cuda")
    torch.cuda.current_stream().synchronize()
    return t


@pytest.mark.parametrize("collective", GOLD["reduce_op_suite"]["collectives"])
@pytest.mark.parametrize("rop", ["SUM", "PROD", "MAX", "MIN"])
def test_reduce_op_suite(collective, rop):
    vals = GOLD["reduce_op_suite"]["rank_values"]
    expect = GOLD["reduce_op_suite"]["expect"][rop]
    nranks = len(vals)

    def body(rank, comm, stream, to_dev, to_host):
        op = getattr(OP, rop)
        if collective in ("all_reduce", "reduce"):
            count = 4
            sbuf, rbuf = to_dev(np.full(count, vals[rank], dtype=np.float32)), zeros(count * 4)
            if collective == "all_reduce":
                h.all_reduce(comm, sbuf, rbuf, count, data_type=DT.FP32, reduce_op=op, stream=stream)
            else:
                h.reduce(comm, sbuf, rbuf, count, data_type=DT.FP32, reduce_op=op, root=0, stream=stream)
            got = to_host(rbuf).view(np.float32)[:count]
            return True if (collective == "reduce" and rank != 0) else bool(np.all(np.abs(got - expect) < 1e-3))
        sbuf, rbuf = to_dev(np.full(nranks, vals[rank], dtype=np.float32)), zeros(4)
        if collective == "reduce_scatter":
            h.reduce_scatter(comm, sbuf, rbuf, 1, data_type=DT.FP32, reduce_op=op, stream=stream)
        else:
            h.reduce_scatter_v(comm, sbuf, [1] * nranks, list(range(nranks)), rbuf, 1, data_type=DT.FP32,
                               reduce_op=op, stream=stream)
        return bool(abs(float(to_host(rbuf).view(np.float32)[0]) - expect) < 1e-3)

    assert all(run_ranks(nranks, body))


@pytest.mark.parametrize("nranks", [2, 4])
@pytest.mark.parametrize("dtype_name", GOLD["dtype_suite"]["dtypes"])
def test_dtype_suite(dtype_name, nranks):
    dt = getattr(DT, dtype_name)
    esize = 2 if dtype_name == "BFP16" else np.dtype(NP[dtype_name]).itemsize
    tol = GOLD["dtype_suite"]["float_tolerance"] if dtype_name in ("FP16", "BFP16", "FP32", "FP64") else 0.5
    sum_expect = float(sum(range(1, nranks + 1)))
    gathered = [float(i + 1) for i in range(nranks)]

    def close(got, want):
        return bool(np.all(np.abs(np.asarray(got, dtype=np.float64) - np.asarray(want, dtype=np.float64)) < tol))

    def body(rank, comm, stream, to_dev, to_host):
        res = {}
        mine = float(rank + 1)
        ones = [1] * nranks
        ramp = list(range(nranks))
        for op in GOLD["dtype_suite"]["ops"]:
            reducing = op in ("all_reduce", "reduce", "reduce_scatter", "reduce_scatter_v")
            refused = dtype_name in (NOT_REDUCIBLE_V if op == "reduce_scatter_v" else NOT_REDUCIBLE)
            try:
                if op == "all_reduce":
                    s, r = to_dev(pack(dtype_name, [mine] * 4)), zeros(4 * esize)
                    h.all_reduce(comm, s, r, 4, data_type=dt, stream=stream)
                    ok = close(unpack(dtype_name, to_host(r), 4), sum_expect)
                elif op == "reduce":
                    s, r = to_dev(pack(dtype_name, [mine] * 4)), zeros(4 * esize)
                    h.reduce(comm, s, r, 4, data_type=dt, root=0, stream=stream)
                    ok = close(unpack(dtype_name, to_host(r), 4), sum_expect) if rank == 0 else True
                elif op == "broadcast":
                    b = to_dev(pack(dtype_name, [7.0 if rank == 0 else 0.0] * 4))
                    h.broadcast(comm, b, 4, data_type=dt, root=0, stream=stream)
                    ok = close(unpack(dtype_name, to_host(b), 4), 7.0)
                elif op == "all_gather":
                    s, r = to_dev(pack(dtype_name, [mine])), zeros(nranks * esize)
                    h.all_gather(comm, s, r, 1, data_type=dt, stream=stream)
                    ok = close(unpack(dtype_name, to_host(r), nranks), gathered)
                elif op == "all_gather_v":
                    s, r = to_dev(pack(dtype_name, [mine])), zeros(nranks * esize)
                    h.all_gather_v(comm, s, 1, r, ones, ramp, data_type=dt, stream=stream)
                    ok = close(unpack(dtype_name, to_host(r), nranks), gathered)
                elif op == "scatter":
                    root_vals = [float((i + 1) * 10) for i in range(nranks)]
                    s = to_dev(pack(dtype_name, root_vals if rank == 0 else [0.0] * nranks))
                    r = zeros(esize)
                    h.scatter(comm, s, r, 1, data_type=dt, root=0, stream=stream)
                    ok = close(unpack(dtype_name, to_host(r), 1), float((rank + 1) * 10))
                elif op == "reduce_scatter":
                    s, r = to_dev(pack(dtype_name, [mine] * nranks)), zeros(esize)
                    h.reduce_scatter(comm, s, r, 1, data_type=dt, stream=stream)
                    ok = close(unpack(dtype_name, to_host(r), 1), sum_expect)
                elif op == "reduce_scatter_v":
                    s, r = to_dev(pack(dtype_name, [mine] * nranks)), zeros(esize)
                    h.reduce_scatter_v(comm, s, ones, ramp, r, 1, data_type=dt, stream=stream)
                    ok = close(unpack(dtype_name, to_host(r), 1), sum_expect)
                elif op == "all_to_all":
                    s, r = to_dev(pack(dtype_name, [mine] * nranks)), zeros(nranks * esize)
                    h.all_to_all(comm, s, 1, dt, r, 1, dt, stream=stream)
                    ok = close(unpack(dtype_name, to_host(r), nranks), gathered)
                elif op == "all_to_all_v":
                    s, r = to_dev(pack(dtype_name, [mine] * nranks)), zeros(nranks * esize)
                    h.all_to_all_v(comm, s, ones, ramp, dt, r, ones, ramp, dt, stream=stream)
                    ok = close(unpack(dtype_name, to_host(r), nranks), gathered)
                elif op == "all_to_all_vc":
                    s, r = to_dev(pack(dtype_name, [mine] * nranks)), zeros(nranks * esize)
                    h.all_to_all_vc(comm, s, [1] * (nranks * nranks), dt, r, dt, stream=stream)
                    ok = close(unpack(dtype_name, to_host(r), nranks), gathered)
                elif op == "send_recv":
                    if nranks != 2:
                        res[op] = True           # the reference runs this case on two ranks only
                        continue
                    peer = 1 - rank
                    s, r = to_dev(pack(dtype_name, [mine] * 4)), zeros(4 * esize)
                    if rank == 0:
                        h.send(comm, s, 4, dt, dest_rank=peer, stream=stream)
                        h.recv(comm, r, 4, dt, src_rank=peer, stream=stream)
                    else:
                        h.recv(comm, r, 4, dt, src_rank=peer, stream=stream)
                        h.send(comm, s, 4, dt, dest_rank=peer, stream=stream)
                    ok = close(unpack(dtype_name, to_host(r), 4), float(peer + 1))
                else:
                    nxt, prv = (rank + 1) % nranks, (rank - 1 + nranks) % nranks
                    s, r = to_dev(pack(dtype_name, [mine] * 4)), zeros(4 * esize)
                    items = [h.make_send_recv_item(h.HcclSendRecvType.SEND, s, 4, dt, nxt),
                             h.make_send_recv_item(h.HcclSendRecvType.RECV, r, 4, dt, prv)]
                    h.batch_send_recv(comm, items, stream=stream)
                    ok = close(unpack(dtype_name, to_host(r), 4), float(prv + 1))
                res[op] = ok and not (reducing and refused)
            except h.HcclError as e:
                res[op] = reducing and refused and e.code == 5      # HCCL_E_NOT_SUPPORT, like the reference
        return res

    for rank, res in enumerate(run_ranks(nranks, body)):
        bad = [op for op, ok in res.items() if not ok]
        assert not bad, (dtype_name, nranks, rank, bad)
