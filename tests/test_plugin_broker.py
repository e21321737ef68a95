"""The algorithm-plugin function table (include/hccl_algo_plugin.h).  CPU part: what the reference's plugin
manager checks before it accepts a broker (reference src/algo_plugin/hccl_algo_plugin_mgr.cc:
LoadPluginTable, ValidatePluginTable) and the select / query contract; nothing here reaches a GPU.
GPU part: an operator executed through the table matches the oracle."""
import ctypes

import numpy as np
import pytest

import hccl_amd
from hccl_amd import HcclDataType as DT, HcclReduceOp as OP, plugin

FIXED_COUNT_OPS = ["AllReduce", "ReduceScatter", "AllGather", "Reduce", "Broadcast", "Scatter", "AllToAll"]


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
    for op in ("AllToAllV", "AllGatherV", "ReduceScatterV", "Send", "Recv", ""):
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
