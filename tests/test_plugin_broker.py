"""The algorithm-plugin function table (include/hccl_algo_plugin.h).  CPU part: what the reference's plugin
manager checks before it accepts a broker (reference src/algo_plugin/hccl_algo_plugin_mgr.cc:
LoadPluginTable, ValidatePluginTable) and the select / query contract; nothing here reaches a GPU.
GPU part: an operator executed through the table matches the oracle."""
import ctypes
import os

import numpy as np
import pytest

import hccl_amd
from hccl_amd import HcclDataType as DT, HcclReduceOp as OP, plugin

FIXED_COUNT_OPS = ["AllReduce", "ReduceScatter", "AllGather", "Reduce", "Broadcast", "Scatter", "AllToAll", "Send",
                   "Recv"]


def test_param_struct_has_the_reference_layout():
    # 3*u32 + int + char[32] + u64 + u32 + int + char[32] + 2*u32 + 3 pointers + 2 enums + 5*u32 + bool + 7*u32
    P = plugin.HcclAlgoPluginParam
    assert P.opName.offset == 16 and P.count.offset == 48 and P.root.offset == 56 and P.topoName.offset == 64
    assert P.rankNum.offset == 96 and P.sendBuf.offset == 104 and P.stream.offset == 120
    assert P.dataType.offset == 128 and P.isAsymmetricTopo.offset == 156 and P.reserved.offset == 160
    assert ctypes.sizeof(P) == 192


def test_table_passes_the_managers_validation():
    t = plugin.table()
    assert t.version == plugin.API_VERSION
    for fn in (t.IsReady, t.FetchContext, t.SelectAlg, t.ExecuteAlg, t.QueryAlgs):
        assert fn
    assert t.IsReady() is True
    assert t.FetchContext() is not None


@pytest.mark.parametrize("op", FIXED_COUNT_OPS)
def test_select_and_query_agree(op):
    t = plugin.table()
    ctx = t.FetchContext()
    name = ctypes.create_string_buffer(128)
    assert t.SelectAlg(ctx, ctypes.byref(plugin.make_param(op, 8)), name, 128) is True
    listed = ctypes.create_string_buffer(256)
    assert t.QueryAlgs(ctx, op.encode(), listed, 256) == 0
    assert listed.raw.split(b"\0")[0] == name.value and name.value.startswith(b"HcclAmdLoopback")


def test_operators_without_a_plugin_signature_are_not_taken():
    t = plugin.table()
    ctx = t.FetchContext()
    name = ctypes.create_string_buffer(128)
    for op in ("AllToAllV", "AllToAllVC", "AllGatherV", "ReduceScatterV", "BatchSendRecv", ""):
        assert t.SelectAlg(ctx, ctypes.byref(plugin.make_param(op, 8)), name, 128) is False
        listed = ctypes.create_string_buffer(16)
        assert t.QueryAlgs(ctx, op.encode(), listed, 16) == 0 and listed.raw[0:1] == b"\0"
        assert t.ExecuteAlg(ctx, b"x", op.encode(), ctypes.byref(plugin.make_param(op, 8)), None) == 5


def test_malformed_requests_are_rejected():
    t = plugin.table()
    ctx = t.FetchContext()
    name = ctypes.create_string_buffer(128)
    bad = plugin.make_param("AllReduce", 8)
    bad.magic = 0
    assert t.SelectAlg(ctx, ctypes.byref(bad), name, 128) is False
    assert t.ExecuteAlg(ctx, b"HcclAmdLoopbackAllReduce", b"AllReduce", ctypes.byref(bad), None) == 1
    short = plugin.make_param("AllReduce", 8)
    short.structSize = 100
    assert t.SelectAlg(ctx, ctypes.byref(short), name, 128) is False
    ok = plugin.make_param("AllReduce", 8)
    assert t.SelectAlg(None, ctypes.byref(ok), name, 128) is False                          # foreign context
    assert t.SelectAlg(ctx, ctypes.byref(ok), name, 4) is False                              # name does not fit
    assert t.ExecuteAlg(ctx, b"SomethingElse", b"AllReduce", ctypes.byref(ok), None) == 6    # HCCL_E_NOT_FOUND
    tiny = ctypes.create_string_buffer(8)
    assert t.QueryAlgs(ctx, b"AllReduce", tiny, 8) == 3                                      # HCCL_E_MEMORY
    # the entry point's own checks still apply: null stream -> HCCL_E_PTR
    assert t.ExecuteAlg(ctx, b"HcclAmdLoopbackAllReduce", b"AllReduce", ctypes.byref(ok), None) == 2


# ---- selector libraries for the reference's own broker --------------------------------------------------
ENTRY_POINT = {"AllReduce": "HcclAllReduce", "ReduceScatter": "HcclReduceScatter", "AllGather": "HcclAllGather",
               "Reduce": "HcclReduce", "Broadcast": "HcclBroadcast", "Scatter": "HcclScatter", "AllToAll": "HcclAlltoAll",
               "Send": "HcclSend", "Recv": "HcclRecv"}


def test_entry_struct_has_the_reference_layout():
    E = plugin.HcclAlgoPluginAlgEntry
    assert E.algName.offset == 12 and E.soPath.offset == 140 and E.fnSymbol.offset == 652
    assert ctypes.sizeof(E) == 780


@pytest.mark.parametrize("op", FIXED_COUNT_OPS)
def test_selector_library_registers_the_entry_point_of_the_data_plane(op):
    """What the reference's broker does with a selector library (plugin_broker.cc:140-207, 280-330): query the
    entries, check their magic, later dlopen soPath and dlsym fnSymbol."""
    sel = plugin.load_selector(op)
    n = ctypes.c_int(-1)
    entries = sel.HcclAlgoPluginQueryEntries(ctypes.byref(n))
    assert n.value == 1
    e = entries[0]
    assert (e.version, e.magic, e.structSize) == (1, plugin.ENTRY_MAGIC, 780)
    assert e.algName == b"HcclAmdLoopback" + op.encode()
    assert e.fnSymbol == ENTRY_POINT[op].encode()
    impl = e.soPath.decode()
    assert os.path.realpath(impl) == os.path.realpath(hccl_amd.LIB_PATH)
    assert getattr(ctypes.CDLL(impl), e.fnSymbol.decode())           # the symbol resolves in that library
    assert sel.HcclAlgoPluginQueryEntries(None)[0].algName == e.algName      # a null count is tolerated


@pytest.mark.parametrize("op", FIXED_COUNT_OPS)
def test_selector_takes_what_the_entry_point_admits_and_nothing_else(op, monkeypatch):
    sel = plugin.load_selector(op)
    name = ctypes.create_string_buffer(128)
    assert sel.Select(ctypes.byref(plugin.make_param(op, 8, DT.FP32, OP.SUM)), name, 128) is True
    assert name.value == b"HcclAmdLoopback" + op.encode()
    other = "Broadcast" if op != "Broadcast" else "AllReduce"
    assert sel.Select(ctypes.byref(plugin.make_param(other, 8)), name, 128) is False      # another operator
    bad = plugin.make_param(op, 8)
    bad.magic = 0
    assert sel.Select(ctypes.byref(bad), name, 128) is False
    assert sel.Select(ctypes.byref(plugin.make_param(op, 8)), name, 8) is False          # the name does not fit
    assert sel.Select(None, name, 128) is False
    assert sel.Select(ctypes.byref(plugin.make_param(op, 8, DT.INT128)), name, 128) is False
    reduces = op in ("AllReduce", "ReduceScatter", "Reduce")
    assert sel.Select(ctypes.byref(plugin.make_param(op, 8, DT.UINT8)), name, 128) is (not reduces)
    assert sel.Select(ctypes.byref(plugin.make_param(op, 8, DT.BFP16, OP.PROD)), name, 128) is (not reduces)
    monkeypatch.setenv("HCCL_AMD_PLUGIN_SELECT", "0")
    assert sel.Select(ctypes.byref(plugin.make_param(op, 8, DT.FP32, OP.SUM)), name, 128) is False


def test_selector_honours_an_explicit_library_path(monkeypatch, tmp_path):
    """HCCL_AMD_LIBRARY is read when the entries are first built, so a fresh copy of the library is loaded."""
    import shutil
    src = plugin.selector_path("AllGather")
    dst = tmp_path / "AllGather" / "libhccl_plugin_allgather_selector.so"
    dst.parent.mkdir()
    shutil.copy(src, dst)
    monkeypatch.setenv("HCCL_AMD_LIBRARY", "/opt/somewhere/libhccl_amd.so")
    lib = ctypes.CDLL(str(dst))
    lib.HcclAlgoPluginQueryEntries.restype = ctypes.POINTER(plugin.HcclAlgoPluginAlgEntry)
    n = ctypes.c_int(0)
    assert lib.HcclAlgoPluginQueryEntries(ctypes.byref(n))[0].soPath == b"/opt/somewhere/libhccl_amd.so"


@pytest.mark.gpu
def test_all_reduce_through_a_selector_library_like_the_reference_broker_would_run_it():
    """Select, then dlopen(soPath), dlsym(fnSymbol) and a call with the operator's hccl.h signature."""
    import oracle
    from gpu_util import World, dev_zeros, require_library_on_gpu, to_dev, to_host
    require_library_on_gpu()
    sel = plugin.load_selector("AllReduce")
    cnt = ctypes.c_int(0)
    entry = sel.HcclAlgoPluginQueryEntries(ctypes.byref(cnt))[0]
    impl = ctypes.CDLL(entry.soPath.decode())
    fn = getattr(impl, entry.fnSymbol.decode())
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                   ctypes.c_void_p]
    n, count = 4, 20_011
    w = World(n)
    try:
        rng = np.random.default_rng(13)
        ins = [rng.standard_normal(count).astype(np.float32) for _ in range(n)]
        want = [np.zeros(count, dtype=np.float32) for _ in range(n)]
        assert oracle.all_reduce(ins, want, count, int(DT.FP32), 0, algo="mesh") == 0
        sends = [to_dev(x) for x in ins]
        recvs = [dev_zeros(x.nbytes) for x in ins]
        name = ctypes.create_string_buffer(128)
        w.inputs_ready()
        hccl_amd.group_start()
        for r in range(n):
            p = plugin.make_param("AllReduce", count, DT.FP32, OP.SUM, 0, sends[r].data_ptr(), recvs[r].data_ptr(),
                                  w.stream.cuda_stream, n)
            assert sel.Select(ctypes.byref(p), name, 128) and name.value == entry.algName
            assert fn(p.sendBuf, p.recvBuf, p.count, p.dataType, p.reduceOp, w.comms[r], p.stream) == 0
        hccl_amd.group_end()
        w.sync()
        for r in range(n):
            assert np.array_equal(to_host(recvs[r], np.float32).view(np.uint32), want[r].view(np.uint32)), r
    finally:
        w.close()


@pytest.mark.gpu
def test_all_reduce_and_broadcast_through_the_table_match_the_oracle():
    import oracle
    from gpu_util import World, dev_zeros, require_library_on_gpu, to_dev, to_host
    require_library_on_gpu()
    t = plugin.table()
    ctx = t.FetchContext()
    n, count, root = 4, 10_007, 1
    w = World(n)
    try:
        rng = np.random.default_rng(12)
        ins = [rng.standard_normal(count).astype(np.float32) for _ in range(n)]
        want = [np.zeros(count, dtype=np.float32) for _ in range(n)]
        assert oracle.all_reduce(ins, want, count, int(DT.FP32), 0, algo="mesh") == 0
        sends = [to_dev(x) for x in ins]
        recvs = [dev_zeros(x.nbytes) for x in ins]
        name = ctypes.create_string_buffer(128)
        w.inputs_ready()
        hccl_amd.group_start()
        for r in range(n):
            p = plugin.make_param("AllReduce", count, DT.FP32, OP.SUM, 0, sends[r].data_ptr(), recvs[r].data_ptr(),
                                  w.stream.cuda_stream, n)
            assert t.SelectAlg(ctx, ctypes.byref(p), name, 128)
            assert t.ExecuteAlg(ctx, name.value, b"AllReduce", ctypes.byref(p), w.comms[r]) == 0
        hccl_amd.group_end()
        w.sync()
        for r in range(n):
            assert np.array_equal(to_host(recvs[r], np.float32).view(np.uint32), want[r].view(np.uint32)), r
        # Send / Recv: the peer travels as remoteRank
        outs = [dev_zeros(ins[0].nbytes) for _ in range(n)]
        w.inputs_ready()
        hccl_amd.group_start()
        for r in range(n):
            ps = plugin.make_param("Send", count, DT.FP32, 0, 0, sends[r].data_ptr(), None, w.stream.cuda_stream, n,
                                   remote_rank=(r + 1) % n)
            pr = plugin.make_param("Recv", count, DT.FP32, 0, 0, None, outs[r].data_ptr(), w.stream.cuda_stream, n,
                                   remote_rank=(r - 1) % n)
            assert t.ExecuteAlg(ctx, b"HcclAmdLoopbackSend", b"Send", ctypes.byref(ps), w.comms[r]) == 0
            assert t.ExecuteAlg(ctx, b"HcclAmdLoopbackRecv", b"Recv", ctypes.byref(pr), w.comms[r]) == 0
        hccl_amd.group_end()
        w.sync()
        for r in range(n):
            assert np.array_equal(to_host(outs[r], np.float32).view(np.uint32), ins[(r - 1) % n].view(np.uint32)), r
        # Broadcast: the one buffer travels as sendBuf
        bufs = [to_dev(x) for x in ins]
        w.inputs_ready()
        hccl_amd.group_start()
        for r in range(n):
            p = plugin.make_param("Broadcast", count, DT.FP32, 0, root, bufs[r].data_ptr(), None, w.stream.cuda_stream, n)
            assert t.ExecuteAlg(ctx, b"HcclAmdLoopbackBroadcast", b"Broadcast", ctypes.byref(p), w.comms[r]) == 0
        hccl_amd.group_end()
        w.sync()
        for r in range(n):
            assert np.array_equal(to_host(bufs[r], np.float32).view(np.uint32), ins[root].view(np.uint32)), r
    finally:
        w.close()
