"""ctypes bindings of libhccl_amd.so, shaped like the reference's hccl4py.ops
(reference experimental/eco_system/python/hccl4py/ops.py:48-80): every collective takes
``(hccl_comm, send_buf, recv_buf, count, data_type, reduce_op, stream)`` with element counts and
device pointers, returns the HcclResult code and raises :class:`HcclError` when it is not zero.

The library is loaded from ``hccl_amd/libhccl_amd.so`` (built by ``make -C hccl_amd/csrc``).  There
is no fallback: if the shared object is missing the import of any collective fails loudly.
"""
import ctypes
import enum
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhccl_amd.so")
MAX_RANKS = 64


class HcclDataType(enum.IntEnum):
    INT8 = 0
    INT16 = 1
    INT32 = 2
    FP16 = 3
    FP32 = 4
    INT64 = 5
    UINT64 = 6
    UINT8 = 7
    UINT16 = 8
    UINT32 = 9
    FP64 = 10
    BFP16 = 11
    INT128 = 12
    HIF8 = 14
    FP8E4M3 = 15
    FP8E5M2 = 16
    FP8E8M0 = 17
    RESERVED = 255


class HcclReduceOp(enum.IntEnum):
    SUM = 0
    PROD = 1
    MAX = 2
    MIN = 3
    RESERVED = 4


class HcclResult(enum.IntEnum):
    SUCCESS = 0
    E_PARA = 1
    E_PTR = 2
    E_MEMORY = 3
    E_INTERNAL = 4
    E_NOT_SUPPORT = 5
    E_TIMEOUT = 9
    E_RUNTIME = 15


class Algo(enum.IntEnum):
    MESH = 0
    RING = 1
    RHD = 2
    NHR = 3
    ORDER_PRESERVED = 4
    AIV_MESH = 5
    MESH_SYMMETRIC = 6
    MESH_CHUNK = 7
    MESH_TWO_SHOT = 8
    MESH_CONCUR = 9


class HcclSendRecvType(enum.IntEnum):
    SEND = 0
    RECV = 1


class HcclSendRecvItem(ctypes.Structure):
    """One transfer of batch_send_recv (include/hccl_types.h)."""
    _fields_ = [("sendRecvType", ctypes.c_int), ("buf", ctypes.c_void_p), ("count", ctypes.c_uint64),
                ("dataType", ctypes.c_int), ("remoteRank", ctypes.c_uint32)]


class OpKind(enum.IntEnum):
    ALL_REDUCE = 0
    REDUCE_SCATTER = 1
    REDUCE = 2


DTYPE_SIZE = {0: 1, 1: 2, 2: 4, 3: 2, 4: 4, 5: 8, 6: 8, 7: 1, 8: 2, 9: 4, 10: 8, 11: 2, 12: 16, 14: 1, 15: 1,
              16: 1, 17: 1}


class HcclError(RuntimeError):
    def __init__(self, code, where):
        self.code = int(code)
        super().__init__("%s failed with HcclResult %d (%s)" % (where, self.code, error_string(self.code)))


def build(jobs=8):
    """Compiles the gfx950 kernels and the host layer into libhccl_amd.so."""
    subprocess.check_call(["make", "-s", "-C", os.path.join(_HERE, "csrc"), "-j%d" % jobs])
    return LIB_PATH


_lib = None


def lib():
    """Loads libhccl_amd.so; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("%s is missing: run `make -C hccl_amd/csrc` (or hccl_amd.build()) first" % LIB_PATH)
    _lib = _bind(ctypes.CDLL(LIB_PATH))
    return _lib


def _bind(L):
    """Declares the argument and result types of the library's entry points on the loaded library L."""
    vp, u64, u32, i32 = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_int
    L.HcclAllReduce.argtypes = [vp, vp, u64, i32, i32, vp, vp]
    L.HcclReduceScatter.argtypes = [vp, vp, u64, i32, i32, vp, vp]
    L.HcclAllGather.argtypes = [vp, vp, u64, i32, vp, vp]
    L.HcclAllGatherV.argtypes = [vp, u64, vp, vp, vp, i32, vp, vp]
    L.HcclAlltoAllV.argtypes = [vp, vp, vp, i32, vp, vp, vp, i32, vp, vp]
    L.HcclAmdAlltoAllVNoAlloc.argtypes = [vp, vp, vp, i32, vp, vp, vp, i32, vp, vp]
    L.HcclAlltoAll.argtypes = [vp, u64, i32, vp, u64, i32, vp, vp]
    L.HcclAlltoAllVC.argtypes = [vp, vp, i32, vp, i32, vp, vp]
    L.HcclReduceScatterV.argtypes = [vp, vp, vp, vp, u64, i32, i32, vp, vp]
    L.HcclReduce.argtypes = [vp, vp, u64, i32, i32, u32, vp, vp]
    L.HcclBroadcast.argtypes = [vp, u64, i32, u32, vp, vp]
    L.HcclScatter.argtypes = [vp, vp, u64, i32, u32, vp, vp]
    L.HcclBarrier.argtypes = [vp, vp]
    L.HcclSend.argtypes = [vp, u64, i32, u32, vp, vp]
    L.HcclRecv.argtypes = [vp, u64, i32, u32, vp, vp]
    L.HcclBatchSendRecv.argtypes = [ctypes.POINTER(HcclSendRecvItem), u32, vp, vp]
    L.HcclCommInitAll.argtypes = [u32, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(vp)]
    L.HcclGetRootInfo.argtypes = [vp]
    L.HcclCommInitRootInfo.argtypes = [u32, vp, u32, ctypes.POINTER(vp)]
    L.HcclCommDestroy.argtypes = [vp]
    L.HcclGetRankSize.argtypes = [vp, ctypes.POINTER(u32)]
    L.HcclGetRankId.argtypes = [vp, ctypes.POINTER(u32)]
    L.HcclGetCommName.argtypes = [vp, ctypes.c_char_p]
    L.HcclGetErrorString.argtypes = [i32]
    L.HcclGetErrorString.restype = ctypes.c_char_p
    L.HcclGroupStart.argtypes = []
    L.HcclGroupEnd.argtypes = []
    L.HcclAmdSetAlgo.argtypes = [vp, i32, i32]
    L.HcclAmdGetAlgo.argtypes = [vp, i32, ctypes.POINTER(i32)]
    L.HcclAmdGetFoldProgram.argtypes = [i32, i32, u32, u32, vp, u32, ctypes.POINTER(u32), ctypes.POINTER(u32)]
    L.HcclAmdGetFoldProgramTwoLevel.argtypes = [i32, i32, u32, u32, u32, vp, u32, ctypes.POINTER(u32), ctypes.POINTER(u32)]
    L.HcclAmdGetFoldProgramLevels.argtypes = [i32, i32, u32, u32, u32, u32, vp, u32, ctypes.POINTER(u32),
                                              ctypes.POINTER(u32)]
    L.HcclAmdSetLevel0RankSize.argtypes = [vp, u32]
    L.HcclAmdSetLevel1GroupSize.argtypes = [vp, u32]
    L.HcclAmdGetLevel1GroupSize.argtypes = [vp, ctypes.POINTER(u32)]
    L.HcclAmdGetLevel0RankSize.argtypes = [vp, ctypes.POINTER(u32)]
    L.HcclAmdSelectFromHcclAlgo.argtypes = [ctypes.c_char_p, i32, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(i32),
                                            ctypes.POINTER(ctypes.c_int32), ctypes.c_char_p, u32]
    L.HcclAmdGetStuckCounters.argtypes = [vp, ctypes.POINTER(u64), ctypes.POINTER(u64)]
    L.HcclAmdSetCclBufferSize.argtypes = [vp, u64]
    L.HcclAmdGetCclBufferSize.argtypes = [vp, ctypes.POINTER(u64)]
    for name in ("HcclAllReduce", "HcclReduceScatter", "HcclAllGather", "HcclAllGatherV", "HcclAlltoAllV",
                 "HcclAlltoAll", "HcclAlltoAllVC", "HcclReduceScatterV", "HcclReduce", "HcclBroadcast", "HcclScatter",
                 "HcclSend", "HcclRecv", "HcclBatchSendRecv", "HcclBarrier",
                 "HcclCommInitAll", "HcclGetRootInfo", "HcclCommInitRootInfo", "HcclCommDestroy", "HcclGetRankSize",
                 "HcclGetRankId", "HcclGetCommName", "HcclGroupStart", "HcclGroupEnd", "HcclAmdSetAlgo", "HcclAmdGetAlgo",
                 "HcclAmdGetFoldProgram", "HcclAmdSetCclBufferSize", "HcclAmdGetCclBufferSize",
                 "HcclAmdAlltoAllVNoAlloc", "HcclAmdGetStuckCounters"):
        getattr(L, name).restype = ctypes.c_int
    return L


def error_string(code):
    return lib().HcclGetErrorString(int(code)).decode()


def check(code, where):
    if int(code) != 0:
        raise HcclError(code, where)
    return int(code)


def _as_ptr(buf):
    """Accepts None, an int address, a ctypes pointer, or anything with data_ptr() (torch tensors)."""
    if buf is None:
        return None
    if hasattr(buf, "data_ptr"):
        return ctypes.c_void_p(buf.data_ptr())
    if isinstance(buf, int):
        return ctypes.c_void_p(buf)
    return ctypes.cast(buf, ctypes.c_void_p)


def _as_stream(stream):
    if stream is None:
        return None
    if hasattr(stream, "cuda_stream"):
        return ctypes.c_void_p(stream.cuda_stream)
    return ctypes.c_void_p(int(stream))


def u64_array(values):
    """Builds the host uint64 array the V-collectives take; pass the result to skip per-call conversion."""
    vals = [int(v) for v in values]
    return (ctypes.c_uint64 * len(vals))(*vals)


def _u64_array(values, n):
    if isinstance(values, ctypes.Array) and values._type_ is ctypes.c_uint64:
        if len(values) != n:
            raise ValueError("expected %d entries, got %d" % (n, len(values)))
        return values
    vals = [int(v) for v in values]
    if len(vals) != n:
        raise ValueError("expected %d entries, got %d" % (n, len(vals)))
    return (ctypes.c_uint64 * n)(*vals)


# ---- lifecycle ------------------------------------------------------------------------------------
def comm_init_all(ndev, devices=None):
    """Creates the ``ndev`` communicators of one loopback world; element r has rank r."""
    comms = (ctypes.c_void_p * ndev)()
    dev = None
    if devices is not None:
        dev = (ctypes.c_int32 * ndev)(*devices)
    check(lib().HcclCommInitAll(ndev, dev, comms), "HcclCommInitAll")
    return [ctypes.c_void_p(c) for c in comms]


def get_root_info():
    buf = ctypes.create_string_buffer(4108)
    check(lib().HcclGetRootInfo(buf), "HcclGetRootInfo")
    return buf


def comm_init_root_info(n_ranks, root_info, rank):
    comm = ctypes.c_void_p()
    check(lib().HcclCommInitRootInfo(n_ranks, root_info, rank, ctypes.byref(comm)), "HcclCommInitRootInfo")
    return comm


def comm_destroy(hccl_comm):
    return check(lib().HcclCommDestroy(hccl_comm), "HcclCommDestroy")


def get_rank_size(hccl_comm):
    v = ctypes.c_uint32()
    check(lib().HcclGetRankSize(hccl_comm, ctypes.byref(v)), "HcclGetRankSize")
    return v.value


def get_rank_id(hccl_comm):
    v = ctypes.c_uint32()
    check(lib().HcclGetRankId(hccl_comm, ctypes.byref(v)), "HcclGetRankId")
    return v.value


def get_comm_name(hccl_comm):
    """The world's name: the same for every rank of a world, different between worlds."""
    buf = ctypes.create_string_buffer(128)
    check(lib().HcclGetCommName(hccl_comm, buf), "HcclGetCommName")
    return buf.value.decode()


def group_start():
    return check(lib().HcclGroupStart(), "HcclGroupStart")


def group_end():
    return check(lib().HcclGroupEnd(), "HcclGroupEnd")


class group:
    """``with hccl_amd.group():`` -- queue the per-rank calls of one host thread without blocking."""

    def __enter__(self):
        group_start()
        return self

    def __exit__(self, *exc):
        group_end()
        return False


def set_algo(hccl_comm, op_kind, algo):
    return check(lib().HcclAmdSetAlgo(hccl_comm, int(op_kind), int(algo)), "HcclAmdSetAlgo")


def get_algo(hccl_comm, op_kind):
    v = ctypes.c_int()
    check(lib().HcclAmdGetAlgo(hccl_comm, int(op_kind), ctypes.byref(v)), "HcclAmdGetAlgo")
    return Algo(v.value)


def set_ccl_buffer_size(hccl_comm, nbytes):
    """Size of the staging buffer whose loops NHR / RHD AllReduce reproduce; 0 = one loop."""
    return check(lib().HcclAmdSetCclBufferSize(hccl_comm, ctypes.c_uint64(nbytes)), "HcclAmdSetCclBufferSize")


def get_ccl_buffer_size(hccl_comm):
    v = ctypes.c_uint64()
    check(lib().HcclAmdGetCclBufferSize(hccl_comm, ctypes.byref(v)), "HcclAmdGetCclBufferSize")
    return v.value


def get_stuck_counters(hccl_comm):
    """(head, tail): numbers of the last collective of the world whose kernels have started / finished; needs
    HCCL_AMD_STUCK_COUNTERS=1 when the communicators are created."""
    head, tail = ctypes.c_uint64(), ctypes.c_uint64()
    check(lib().HcclAmdGetStuckCounters(hccl_comm, ctypes.byref(head), ctypes.byref(tail)), "HcclAmdGetStuckCounters")
    return head.value, tail.value


def fold_programs(op_kind, algo, rank_size, level0=1, level1=0):
    """Host-only: the byte programs (one per segment) that fix the reduction order; level0 > 1: the two-level
    AllReduce, ReduceScatter or Reduce over groups of level0 consecutive ranks with `algo` between the groups;
    level1 > 0: the three-level one, level1 consecutive groups forming a level-1 group."""
    L = lib()
    out = []
    seg, count = 0, 1
    while seg < count:
        buf = (ctypes.c_uint8 * 512)()
        ln, cnt = ctypes.c_uint32(), ctypes.c_uint32()
        check(L.HcclAmdGetFoldProgramLevels(int(op_kind), int(algo), rank_size, level0, level1, seg, buf, 512,
                                            ctypes.byref(ln), ctypes.byref(cnt)), "HcclAmdGetFoldProgramLevels")
        count = cnt.value
        out.append(bytes(buf[:ln.value]))
        seg += 1
    return out


def set_level0_rank_size(hccl_comm, ranks_per_group):
    """Groups of consecutive ranks (servers) for the two-level AllReduce of the world hccl_comm belongs to."""
    return check(lib().HcclAmdSetLevel0RankSize(hccl_comm, ctypes.c_uint32(ranks_per_group)), "HcclAmdSetLevel0RankSize")


def get_level0_rank_size(hccl_comm):
    v = ctypes.c_uint32()
    check(lib().HcclAmdGetLevel0RankSize(hccl_comm, ctypes.byref(v)), "HcclAmdGetLevel0RankSize")
    return v.value


def set_level1_group_size(hccl_comm, groups_per_level1_group):
    """How many consecutive level-0 groups form a level-1 group (a pod of servers) in the world hccl_comm belongs
    to; 0: all of them, which leaves two levels."""
    return check(lib().HcclAmdSetLevel1GroupSize(hccl_comm, ctypes.c_uint32(groups_per_level1_group)),
                 "HcclAmdSetLevel1GroupSize")


def get_level1_group_size(hccl_comm):
    v = ctypes.c_uint32()
    check(lib().HcclAmdGetLevel1GroupSize(hccl_comm, ctypes.byref(v)), "HcclAmdGetLevel1GroupSize")
    return v.value


def select_from_hccl_algo(config, op_kind):
    """How the library reads an HCCL_ALGO value for op_kind: (canonical text, Algo or None, two_level).  Raises
    HcclError(HCCL_E_PARA) for a string the reference's parser rejects."""
    sel, algo, two = ctypes.c_int32(), ctypes.c_int(), ctypes.c_int32()
    text = ctypes.create_string_buffer(4096)
    check(lib().HcclAmdSelectFromHcclAlgo(config.encode(), int(op_kind), ctypes.byref(sel), ctypes.byref(algo),
                                          ctypes.byref(two), text, 4096), "HcclAmdSelectFromHcclAlgo")
    return text.value.decode(), (Algo(algo.value) if sel.value else None), bool(two.value)


# ---- collectives (names and argument order of hccl4py.ops) ----------------------------------------
def all_reduce(hccl_comm, send_buf, recv_buf, count, data_type=HcclDataType.FP32, reduce_op=HcclReduceOp.SUM,
               stream=None):
    code = lib().HcclAllReduce(_as_ptr(send_buf), _as_ptr(recv_buf), ctypes.c_uint64(count), int(data_type),
                               int(reduce_op), hccl_comm, _as_stream(stream))
    return check(code, "HcclAllReduce")


def prepared_group(calls):
    """One collective of a host thread that drives all ranks, for loops that repeat it: `calls` is a list of
    (entry point name, argument tuple) with the arguments as the mirror functions would pass them (buffers, counts,
    enums, communicator, stream); they are converted to their C types once, and the function returned issues
    HcclGroupStart, the calls and HcclGroupEnd.  Saves the per-call conversions, which cost more than the library's
    own host work when a collective runs for a few microseconds."""
    library = lib()
    start, end = library.HcclGroupStart, library.HcclGroupEnd
    bound = []
    for name, args in calls:
        fn = getattr(library, name)
        conv = []
        for a, ctype in zip(args, fn.argtypes):
            if ctype is ctypes.c_void_p:
                conv.append(_as_ptr(a) if not hasattr(a, "cuda_stream") else _as_stream(a))
            elif isinstance(a, enum.IntEnum):
                conv.append(int(a))
            elif isinstance(a, int):
                conv.append(ctype(a))
            else:
                conv.append(a)
        bound.append((fn, tuple(conv), name))

    def run():
        start()
        for fn, conv, name in bound:
            code = fn(*conv)
            if code:
                end()
                check(code, name)
        return check(end(), "HcclGroupEnd")
    return run


def reduce_scatter(hccl_comm, send_buf, recv_buf, recv_count, data_type=HcclDataType.FP32,
                   reduce_op=HcclReduceOp.SUM, stream=None):
    code = lib().HcclReduceScatter(_as_ptr(send_buf), _as_ptr(recv_buf), ctypes.c_uint64(recv_count), int(data_type),
                                   int(reduce_op), hccl_comm, _as_stream(stream))
    return check(code, "HcclReduceScatter")


def all_gather(hccl_comm, send_buf, recv_buf, send_count, data_type=HcclDataType.FP32, stream=None):
    code = lib().HcclAllGather(_as_ptr(send_buf), _as_ptr(recv_buf), ctypes.c_uint64(send_count), int(data_type),
                               hccl_comm, _as_stream(stream))
    return check(code, "HcclAllGather")


def all_gather_v(hccl_comm, send_buf, send_count, recv_buf, recv_counts, recv_displs,
                 data_type=HcclDataType.FP32, stream=None):
    n = get_rank_size(hccl_comm)
    counts = _u64_array(recv_counts, n)
    displs = _u64_array(recv_displs, n)
    code = lib().HcclAllGatherV(_as_ptr(send_buf), ctypes.c_uint64(send_count), _as_ptr(recv_buf), counts, displs,
                                int(data_type), hccl_comm, _as_stream(stream))
    return check(code, "HcclAllGatherV")


def all_to_all_v(hccl_comm, send_buf, send_counts, sdispls, send_type, recv_buf, recv_counts, rdispls, recv_type,
                 stream=None):
    n = get_rank_size(hccl_comm)
    code = lib().HcclAlltoAllV(_as_ptr(send_buf), _u64_array(send_counts, n), _u64_array(sdispls, n), int(send_type),
                               _as_ptr(recv_buf), _u64_array(recv_counts, n), _u64_array(rdispls, n), int(recv_type),
                               hccl_comm, _as_stream(stream))
    return check(code, "HcclAlltoAllV")


def all_to_all_v_no_alloc(hccl_comm, send_buf, send_counts, sdispls, send_type, recv_buf, recv_counts, rdispls,
                          recv_type, stream=None):
    """all_to_all_v for callers that cannot allocate device memory (HcclAmdAlltoAllVNoAlloc)."""
    n = get_rank_size(hccl_comm)
    code = lib().HcclAmdAlltoAllVNoAlloc(_as_ptr(send_buf), _u64_array(send_counts, n), _u64_array(sdispls, n),
                                         int(send_type), _as_ptr(recv_buf), _u64_array(recv_counts, n),
                                         _u64_array(rdispls, n), int(recv_type), hccl_comm, _as_stream(stream))
    return check(code, "HcclAmdAlltoAllVNoAlloc")


def all_to_all(hccl_comm, send_buf, send_count, send_type, recv_buf, recv_count, recv_type, stream=None):
    code = lib().HcclAlltoAll(_as_ptr(send_buf), ctypes.c_uint64(send_count), int(send_type), _as_ptr(recv_buf),
                              ctypes.c_uint64(recv_count), int(recv_type), hccl_comm, _as_stream(stream))
    return check(code, "HcclAlltoAll")


def all_to_all_vc(hccl_comm, send_buf, send_count_matrix, send_type, recv_buf, recv_type, stream=None):
    """send_count_matrix: rankSize x rankSize element counts, row = sender, column = receiver (flat or nested)."""
    n = get_rank_size(hccl_comm)
    flat = send_count_matrix
    if not isinstance(flat, ctypes.Array):
        flat = [int(v) for row in send_count_matrix for v in (row if hasattr(row, "__len__") else [row])]
    code = lib().HcclAlltoAllVC(_as_ptr(send_buf), _u64_array(flat, n * n), int(send_type), _as_ptr(recv_buf),
                                int(recv_type), hccl_comm, _as_stream(stream))
    return check(code, "HcclAlltoAllVC")


def reduce_scatter_v(hccl_comm, send_buf, send_counts, send_displs, recv_buf, recv_count,
                     data_type=HcclDataType.FP32, reduce_op=HcclReduceOp.SUM, stream=None):
    n = get_rank_size(hccl_comm)
    code = lib().HcclReduceScatterV(_as_ptr(send_buf), _u64_array(send_counts, n), _u64_array(send_displs, n),
                                    _as_ptr(recv_buf), ctypes.c_uint64(recv_count), int(data_type), int(reduce_op),
                                    hccl_comm, _as_stream(stream))
    return check(code, "HcclReduceScatterV")


def reduce(hccl_comm, send_buf, recv_buf, count, data_type=HcclDataType.FP32, reduce_op=HcclReduceOp.SUM, root=0,
           stream=None):
    code = lib().HcclReduce(_as_ptr(send_buf), _as_ptr(recv_buf), ctypes.c_uint64(count), int(data_type),
                            int(reduce_op), ctypes.c_uint32(root), hccl_comm, _as_stream(stream))
    return check(code, "HcclReduce")


def broadcast(hccl_comm, buf, count, data_type=HcclDataType.FP32, root=0, stream=None):
    code = lib().HcclBroadcast(_as_ptr(buf), ctypes.c_uint64(count), int(data_type), ctypes.c_uint32(root), hccl_comm,
                               _as_stream(stream))
    return check(code, "HcclBroadcast")


def barrier(hccl_comm, stream=None):
    return check(lib().HcclBarrier(hccl_comm, _as_stream(stream)), "HcclBarrier")


def send(hccl_comm, send_buf, count, data_type=HcclDataType.FP32, dest_rank=0, stream=None):
    code = lib().HcclSend(_as_ptr(send_buf), ctypes.c_uint64(count), int(data_type), ctypes.c_uint32(dest_rank),
                          hccl_comm, _as_stream(stream))
    return check(code, "HcclSend")


def recv(hccl_comm, recv_buf, count, data_type=HcclDataType.FP32, src_rank=0, stream=None):
    code = lib().HcclRecv(_as_ptr(recv_buf), ctypes.c_uint64(count), int(data_type), ctypes.c_uint32(src_rank),
                          hccl_comm, _as_stream(stream))
    return check(code, "HcclRecv")


def make_send_recv_item(send_recv_type, buf, count, data_type, remote_rank):
    """One HcclSendRecvItem for batch_send_recv (reference hccl4py/ops.py:485-498)."""
    item = HcclSendRecvItem()
    item.sendRecvType = int(send_recv_type)
    ptr = _as_ptr(buf)
    item.buf = ptr.value if ptr is not None else None
    item.count = int(count)
    item.dataType = int(data_type)
    item.remoteRank = int(remote_rank)
    return item


def batch_send_recv(hccl_comm, items, stream=None):
    """items: a sequence of HcclSendRecvItem or a prebuilt (HcclSendRecvItem * n) array
    (reference hccl4py/ops.py:450-482)."""
    if items is None:
        raise TypeError("items must be a sequence of HcclSendRecvItem")
    if isinstance(items, ctypes.Array) and getattr(items, "_type_", None) is HcclSendRecvItem:
        arr = items
    else:
        for i, item in enumerate(items):
            if not isinstance(item, HcclSendRecvItem):
                raise TypeError("items[%d] must be HcclSendRecvItem, got %s" % (i, type(item).__name__))
        arr = (HcclSendRecvItem * len(items))(*items)
    code = lib().HcclBatchSendRecv(arr, ctypes.c_uint32(len(arr)), hccl_comm, _as_stream(stream))
    return check(code, "HcclBatchSendRecv")


def scatter(hccl_comm, send_buf, recv_buf, recv_count, data_type=HcclDataType.FP32, root=0, stream=None):
    code = lib().HcclScatter(_as_ptr(send_buf), _as_ptr(recv_buf), ctypes.c_uint64(recv_count), int(data_type),
                             ctypes.c_uint32(root), hccl_comm, _as_stream(stream))
    return check(code, "HcclScatter")
