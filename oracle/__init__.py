"""ctypes binding of the CPU oracle (``oracle/hccl_oracle.c``).  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this module.  The shipped package (``hccl_amd``) never does.

Buffers are numpy arrays.  Reduction dtypes that numpy lacks (bf16) travel as ``uint16`` bit
patterns together with the HCCL dtype code.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

INT8, INT16, INT32, FP16, FP32, INT64, UINT64, UINT8, UINT16, UINT32, FP64, BF16 = range(12)
SUM, PROD, MAX, MIN = range(4)
ACC_STEP, ACC_FP32 = 0, 1
INVALID_RANK = 0xFFFFFFFF

DTYPE_SIZE = {INT8: 1, INT16: 2, INT32: 4, FP16: 2, FP32: 4, INT64: 8, UINT64: 8, UINT8: 1, UINT16: 2,
              UINT32: 4, FP64: 8, BF16: 2}
# numpy carrier of each HCCL dtype (bit-exact container, not necessarily the arithmetic type)
NP_CARRIER = {INT8: np.int8, INT16: np.int16, INT32: np.int32, FP16: np.uint16, FP32: np.float32,
              INT64: np.int64, UINT64: np.uint64, UINT8: np.uint8, UINT16: np.uint16, UINT32: np.uint32,
              FP64: np.float64, BF16: np.uint16}


def build(force=False):
    """Compiles liboracle.so with the committed Makefile."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _LIB_PATH


_lib = None


class RhdPart1(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint32) for n in (
        "r", "effectiveRankSize", "virtualRank", "inPart1", "isRepresentative", "pairedAlgRank", "unitStart",
        "unitCount", "isPowerOfTwo")]


class RhdStep(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint32) for n in (
        "step", "peer", "nSlices", "txSegStart", "txSegEnd", "rxSegStart", "rxSegEnd")]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.orc_fp16_to_fp32.restype = ctypes.c_float
        L.orc_fp16_to_fp32.argtypes = [ctypes.c_uint16]
        L.orc_fp32_to_fp16.restype = ctypes.c_uint16
        L.orc_fp32_to_fp16.argtypes = [ctypes.c_float]
        L.orc_bf16_to_fp32.restype = ctypes.c_float
        L.orc_bf16_to_fp32.argtypes = [ctypes.c_uint16]
        L.orc_fp32_to_bf16.restype = ctypes.c_uint16
        L.orc_fp32_to_bf16.argtypes = [ctypes.c_float]
        L.orc_dtype_size.restype = ctypes.c_size_t
        L.orc_round_up.restype = ctypes.c_uint64
        L.orc_round_up.argtypes = [ctypes.c_uint64, ctypes.c_uint64]
        L.orc_rhd_select_loop_count.restype = ctypes.c_uint64
        L.orc_rhd_select_loop_count.argtypes = [ctypes.c_uint64] * 3
        for name in ("orc_nhr_step_num", "orc_rhd_step_num"):
            getattr(L, name).restype = ctypes.c_uint32
            getattr(L, name).argtypes = [ctypes.c_uint32]
        for name in ("orc_rhd_unit_start_of_rank", "orc_rhd_owner_of_unit"):
            getattr(L, name).restype = ctypes.c_uint32
            getattr(L, name).argtypes = [ctypes.c_uint32, ctypes.c_uint32]
        L.orc_rhd_alg_rank_of_virtual.restype = ctypes.c_uint32
        L.orc_rhd_alg_rank_of_virtual.argtypes = [ctypes.c_uint32] * 3
        L.orc_local_copy_slices.restype = ctypes.c_uint32
        L.orc_ccl_buffer_available_size.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_uint64)]
        L.orc_sole_max_count_per_loop.restype = ctypes.c_uint64
        L.orc_sole_max_count_per_loop.argtypes = [ctypes.c_uint64] * 3
        L.orc_rhd_prepare_tail_workspace.argtypes = [ctypes.c_uint64] * 3 + [ctypes.POINTER(ctypes.c_uint64)] * 3
        L.orc_rhd_max_count_per_loop.argtypes = [ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint64,
                                                 ctypes.POINTER(ctypes.c_uint64)]
        _lib = L
    return _lib


def _vp(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _ptr_array(arrs):
    return (ctypes.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])


def _u64(a):
    a = np.ascontiguousarray(a, dtype=np.uint64)
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint64))


# ---- conversions ---------------------------------------------------------------------------
def _convert(name, src, src_dt, dst_dt):
    a = np.ascontiguousarray(src, dtype=src_dt).ravel()
    out = np.empty(a.size, dtype=dst_dt)
    getattr(lib(), name)(_vp(a), _vp(out), ctypes.c_uint64(a.size))
    return out


def fp16_to_fp32_bits(h_bits):
    """uint16 array -> uint32 array of the fp32 bit patterns the oracle produces."""
    return _convert("orc_fp16_to_fp32_n", h_bits, np.uint16, np.float32).view(np.uint32)


def fp32_to_fp16_bits(f32_bits):
    """uint32 array of fp32 bit patterns -> uint16 array of fp16 bit patterns."""
    return _convert("orc_fp32_to_fp16_n", np.asarray(f32_bits, dtype=np.uint32).view(np.float32), np.float32,
                    np.uint16)


def fp32_to_bf16_bits(f32_bits):
    return _convert("orc_fp32_to_bf16_n", np.asarray(f32_bits, dtype=np.uint32).view(np.float32), np.float32,
                    np.uint16)


def np_fp32_to_bf16_bits(f32):
    """Vectorised numpy mirror of orc_fp32_to_bf16 for generating large inputs."""
    u = np.ascontiguousarray(f32, dtype=np.float32).view(np.uint32)
    nan = ((u & 0x7F800000) == 0x7F800000) & ((u & 0x007FFFFF) != 0)
    rounded = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    hi = (u >> 16).astype(np.uint16)
    return np.where(nan, np.where((hi & 0x7F) != 0, hi, hi | 1), rounded)


def bf16_bits_to_fp32(h_bits):
    return (np.asarray(h_bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ---- pairwise ------------------------------------------------------------------------------
def pair_reduce(dst, src, dtype, op):
    """dst[i] = src[i] (+) dst[i] in place (extended type set)."""
    assert dst.nbytes == src.nbytes
    return lib().orc_pair_reduce(_vp(dst), _vp(src), ctypes.c_uint64(dst.nbytes // DTYPE_SIZE[dtype]), dtype, op)


def aicpu_reduce(dst, src, dtype, op, dst_bytes=None, src_bytes=None):
    db = dst.nbytes if dst_bytes is None else dst_bytes
    sb = src.nbytes if src_bytes is None else src_bytes
    return lib().orc_aicpu_reduce(_vp(dst), ctypes.c_uint64(db), _vp(src), ctypes.c_uint64(sb), dtype, op)


# ---- geometry ------------------------------------------------------------------------------
def rhd_part1(p, alg_rank, root=INVALID_RANK):
    info = RhdPart1()
    rc = lib().orc_rhd_part1(ctypes.c_uint32(p), ctypes.c_uint32(alg_rank), ctypes.c_uint32(root),
                             ctypes.byref(info))
    return rc, info


def _steps(fn, info):
    steps = (RhdStep * 32)()
    n = ctypes.c_uint32(0)
    rc = fn(ctypes.byref(info), steps, ctypes.byref(n))
    return rc, [steps[i] for i in range(n.value)]


def rhd_rs_steps(info):
    return _steps(lib().orc_rhd_rs_steps, info)


def rhd_ag_steps(info):
    return _steps(lib().orc_rhd_ag_steps, info)


def rhd_prepost(info, pre_full, post_full):
    pre, post = RhdStep(), RhdStep()
    rc = lib().orc_rhd_prepost(ctypes.byref(info), ctypes.byref(pre), ctypes.byref(post), int(pre_full),
                               int(post_full))
    return rc, pre, post


def rhd_seg_bytes_uniform(us, ue, slice_size, tail_size, tail_unit):
    off, ln = ctypes.c_uint64(0), ctypes.c_uint64(0)
    lib().orc_rhd_seg_bytes_uniform(ctypes.c_uint32(us), ctypes.c_uint32(ue), ctypes.c_uint64(slice_size),
                                    ctypes.c_uint64(tail_size), ctypes.c_uint32(tail_unit), ctypes.byref(off),
                                    ctypes.byref(ln))
    return off.value, ln.value


def nhr_step_info(n, rank, step):
    to, frm, cnt = ctypes.c_uint32(0), ctypes.c_uint32(0), ctypes.c_uint32(0)
    tx = (ctypes.c_uint32 * max(n, 1))()
    rx = (ctypes.c_uint32 * max(n, 1))()
    rc = lib().orc_nhr_step_info(ctypes.c_uint32(n), ctypes.c_uint32(rank), ctypes.c_uint32(step),
                                 ctypes.byref(to), ctypes.byref(frm), ctypes.byref(cnt), tx, rx)
    return rc, to.value, frm.value, list(tx[:cnt.value]), list(rx[:cnt.value])


def mesh_chunk_segments(length, n, elem_size, align4k):
    """Element counts of the n - 1 segments of a slice."""
    out = (ctypes.c_uint64 * max(n - 1, 1))()
    lib().orc_mesh_chunk_segments(ctypes.c_uint64(length), ctypes.c_uint32(n), ctypes.c_uint32(elem_size),
                                  int(align4k), out)
    return list(out[:max(n - 1, 0)])


def ccl_buffer_available_size(env_value):
    """(rc, bytes) for a HCCL_BUFFSIZE string, None = unset."""
    out = ctypes.c_uint64(0)
    rc = lib().orc_ccl_buffer_available_size(None if env_value is None else env_value.encode(), ctypes.byref(out))
    return rc, out.value


def sole_max_count_per_loop(ccl_bytes, scratch_multiple, elem_size):
    return lib().orc_sole_max_count_per_loop(ccl_bytes, scratch_multiple, elem_size)


def rhd_prepare_tail_workspace(count, rank_align, elem_size, workspace_bytes):
    """(rc, workspace bytes left, input tile offset, output tile offset)."""
    ws, i, o = ctypes.c_uint64(workspace_bytes), ctypes.c_uint64(0), ctypes.c_uint64(0)
    rc = lib().orc_rhd_prepare_tail_workspace(count, rank_align, elem_size, ctypes.byref(ws), ctypes.byref(i),
                                              ctypes.byref(o))
    return rc, ws.value, i.value, o.value


def rhd_max_count_per_loop(ccl_bytes, count, p, elem_size):
    out = ctypes.c_uint64(0)
    rc = lib().orc_rhd_max_count_per_loop(ccl_bytes, count, p, elem_size, ctypes.byref(out))
    return rc, out.value


def local_copy_slices(src_off, dst_off, sizes):
    n = len(sizes)
    s, sp = _u64(src_off)
    d, dp = _u64(dst_off)
    z, zp = _u64(sizes)
    out = np.zeros(3 * max(n, 1), dtype=np.uint64)
    k = lib().orc_local_copy_slices(ctypes.c_uint32(n), sp, dp, zp,
                                    out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint64)))
    return [tuple(int(v) for v in out[3 * i:3 * i + 3]) for i in range(k)]


# ---- collectives ---------------------------------------------------------------------------
def _reduce_call(name, ins, outs, count, dtype, op, acc, *extra):
    fn = getattr(lib(), name)
    return fn(ctypes.c_uint32(len(ins)), _ptr_array(ins), _ptr_array(outs), ctypes.c_uint64(count), dtype, op, acc,
              *extra)


def all_reduce(ins, outs, count, dtype, op, acc=ACC_FP32, algo="mesh", max_count_per_loop=0):
    if algo in ("mesh", "ring"):
        return _reduce_call("orc_all_reduce_mesh", ins, outs, count, dtype, op, acc)
    if algo == "two_shot":
        return _reduce_call("orc_all_reduce_two_shot", ins, outs, count, dtype, op, acc)
    if algo == "mesh_symmetric":
        return _reduce_call("orc_all_reduce_two_shot_symmetric", ins, outs, count, dtype, op, acc)
    if algo == "rhd":
        return _reduce_call("orc_all_reduce_rhd", ins, outs, count, dtype, op, acc,
                            ctypes.c_uint64(max_count_per_loop))
    if algo == "nhr":
        return _reduce_call("orc_all_reduce_nhr_looped", ins, outs, count, dtype, op, acc,
                            ctypes.c_uint64(max_count_per_loop))
    if algo == "order_preserved":
        return _reduce_call("orc_all_reduce_order_preserved", ins, outs, count, dtype, op, acc)
    if algo == "mesh_chunk":
        return _reduce_call("orc_all_reduce_mesh_chunk", ins, outs, count, dtype, op, acc,
                            ctypes.c_uint64(max_count_per_loop))
    if algo == "mesh_concur":
        return _reduce_call("orc_all_reduce_mesh_concur", ins, outs, count, dtype, op, acc,
                            ctypes.c_uint64(max_count_per_loop))
    raise ValueError(algo)


L1_RHD, L1_NHR, L1_MESH = 0, 1, 2


def all_reduce_two_level(ins, outs, count, dtype, op, level0, level1_algo, acc=ACC_FP32, max_count_per_loop=0):
    """AllReduce over groups of `level0` consecutive ranks; level1_algo: "rhd", "nhr" or "mesh" (the own-first fold of
    the host-reduce template) between the groups."""
    code = {"rhd": L1_RHD, "nhr": L1_NHR, "mesh": L1_MESH}[level1_algo]
    return lib().orc_all_reduce_two_level(ctypes.c_uint32(len(ins)), ctypes.c_uint32(level0), code, _ptr_array(ins),
                                          _ptr_array(outs), ctypes.c_uint64(count), dtype, op, acc,
                                          ctypes.c_uint64(max_count_per_loop))


def reduce_scatter_two_level(ins, outs, recv_count, dtype, op, level0, level1_algo, acc=ACC_FP32):
    """ReduceScatter over groups of `level0` consecutive ranks; level1_algo as for all_reduce_two_level."""
    code = {"rhd": L1_RHD, "nhr": L1_NHR, "mesh": L1_MESH}[level1_algo]
    return lib().orc_reduce_scatter_two_level(ctypes.c_uint32(len(ins)), ctypes.c_uint32(level0), code, _ptr_array(ins),
                                              _ptr_array(outs), ctypes.c_uint64(recv_count), dtype, op, acc)


def all_reduce_three_level(ins, outs, count, dtype, op, level0, level1, algo, acc=ACC_FP32, ccl_bytes=0):
    """AllReduce over boxes of `level0` consecutive ranks and pods of `level1` consecutive boxes; algo "rhd" or "nhr"
    between the boxes of a pod and between the pods; ccl_bytes: the staging buffer whose loops show, 0 = one loop."""
    code = {"rhd": L1_RHD, "nhr": L1_NHR}[algo]
    return lib().orc_all_reduce_three_level(ctypes.c_uint32(len(ins)), ctypes.c_uint32(level0), ctypes.c_uint32(level1),
                                            code, _ptr_array(ins), _ptr_array(outs), ctypes.c_uint64(count), dtype, op,
                                            acc, ctypes.c_uint64(ccl_bytes))


def reduce_scatter_three_level(ins, outs, recv_count, dtype, op, level0, level1, algo, acc=ACC_FP32):
    code = {"rhd": L1_RHD, "nhr": L1_NHR}[algo]
    return lib().orc_reduce_scatter_three_level(ctypes.c_uint32(len(ins)), ctypes.c_uint32(level0),
                                                ctypes.c_uint32(level1), code, _ptr_array(ins), _ptr_array(outs),
                                                ctypes.c_uint64(recv_count), dtype, op, acc)


def reduce_levels(ins, outs, count, dtype, op, root, level0, level1, algo, acc=ACC_FP32, ccl_bytes=0):
    """Reduce over two (level1 = number of boxes) or three levels; algo "rhd", "nhr", or with two levels "mesh" (the
    host-reduce fold).  Only outs[root] is written."""
    code = {"rhd": L1_RHD, "nhr": L1_NHR, "mesh": L1_MESH}[algo]
    return lib().orc_reduce_levels(ctypes.c_uint32(len(ins)), ctypes.c_uint32(level0), ctypes.c_uint32(level1), code,
                                   _ptr_array(ins), _ptr_array(outs), ctypes.c_uint64(count), dtype, op,
                                   ctypes.c_uint32(root), acc, ctypes.c_uint64(ccl_bytes))


def sequence_max_count_per_loop(ccl_bytes, count, level0, total, esz, align, rhd_tail):
    """(elements per loop, elements of the result slice) of the three-level sequence executors; None when nothing fits."""
    m, e = ctypes.c_uint64(), ctypes.c_uint64()
    rc = lib().orc_sequence_max_count_per_loop(ctypes.c_uint64(ccl_bytes), ctypes.c_uint64(count),
                                               ctypes.c_uint32(level0), ctypes.c_uint32(total), ctypes.c_uint64(esz),
                                               ctypes.c_uint64(align), int(rhd_tail), ctypes.byref(m), ctypes.byref(e))
    return (m.value, e.value) if rc == 0 else None


def sequence_select_loop_count(remaining, max_count_per_loop, level0, result_elems):
    f = lib().orc_sequence_select_loop_count
    f.restype = ctypes.c_uint64
    return f(ctypes.c_uint64(remaining), ctypes.c_uint64(max_count_per_loop), ctypes.c_uint32(level0),
             ctypes.c_uint64(result_elems))


def reduce_scatter(ins, outs, recv_count, dtype, op, acc=ACC_FP32, algo="mesh", max_count_per_loop=0):
    if algo == "mesh_chunk":
        return _reduce_call("orc_reduce_scatter_mesh_chunk", ins, outs, recv_count, dtype, op, acc,
                            ctypes.c_uint64(max_count_per_loop))
    name = {"mesh": "orc_reduce_scatter_mesh", "mesh_symmetric": "orc_reduce_scatter_mesh", "nhr": "orc_reduce_scatter_nhr", "ring": "orc_reduce_scatter_nhr",
            "rhd": "orc_reduce_scatter_rhd", "order_preserved": "orc_reduce_scatter_order_preserved",
            "aiv_mesh": "orc_reduce_scatter_aiv_mesh"}[algo]
    return _reduce_call(name, ins, outs, recv_count, dtype, op, acc)


def reduce_scatter_mt(ins, outs, recv_count, dtype, op, acc, threads):
    return _reduce_call("orc_reduce_scatter_mesh_mt", ins, outs, recv_count, dtype, op, acc,
                        ctypes.c_uint32(threads))


def all_reduce_mt(ins, outs, count, dtype, op, acc, threads):
    return _reduce_call("orc_all_reduce_mesh_mt", ins, outs, count, dtype, op, acc, ctypes.c_uint32(threads))


def all_gather(ins, outs, send_count, dtype):
    return lib().orc_all_gather(ctypes.c_uint32(len(ins)), _ptr_array(ins), _ptr_array(outs),
                                ctypes.c_uint64(send_count), dtype)


def all_gather_v(ins, outs, counts, displs, dtype):
    c, cp = _u64(counts)
    d, dp = _u64(displs)
    return lib().orc_all_gather_v(ctypes.c_uint32(len(ins)), _ptr_array(ins), _ptr_array(outs), cp, dp, dtype)


def all_to_all_v(ins, outs, send_counts, sdispls, recv_counts, rdispls, dtype):
    """The four tables are (n, n) arrays, row r = rank r's argument array."""
    sc, scp = _u64(send_counts)
    sd, sdp = _u64(sdispls)
    rcn, rcp = _u64(recv_counts)
    rd, rdp = _u64(rdispls)
    return lib().orc_all_to_all_v(ctypes.c_uint32(len(ins)), _ptr_array(ins), _ptr_array(outs), scp, sdp, rcp, rdp,
                                  dtype)


def all_to_all(ins, outs, count, dtype):
    return lib().orc_all_to_all(ctypes.c_uint32(len(ins)), _ptr_array(ins), _ptr_array(outs), ctypes.c_uint64(count),
                                dtype)


def all_to_all_vc_params(n, rank, matrix):
    """(sendCounts, recvCounts, sdispls, rdispls) that the reference derives for `rank` from the n x n matrix."""
    m, mp = _u64(matrix)
    outs = [np.zeros(max(n, 1), dtype=np.uint64) for _ in range(4)]
    lib().orc_all_to_all_vc_params(ctypes.c_uint32(n), ctypes.c_uint32(rank), mp,
                                   *[o.ctypes.data_as(ctypes.POINTER(ctypes.c_uint64)) for o in outs])
    return tuple(o[:n] for o in outs)


def all_to_all_vc(ins, outs, matrix, dtype):
    m, mp = _u64(matrix)
    return lib().orc_all_to_all_vc(ctypes.c_uint32(len(ins)), _ptr_array(ins), _ptr_array(outs), mp, dtype)


def reduce_scatter_v(ins, outs, counts, displs, dtype, op, acc=ACC_FP32, algo="mesh"):
    c, cp = _u64(counts)
    d, dp = _u64(displs)
    fn = {"mesh": "orc_reduce_scatter_v_mesh", "mesh_chunk": "orc_reduce_scatter_v_mesh_chunk"}[algo]
    return getattr(lib(), fn)(ctypes.c_uint32(len(ins)), _ptr_array(ins), _ptr_array(outs), cp, dp, dtype, op, acc)


def reduce(ins, outs, count, dtype, op, root, acc=ACC_FP32, algo="mesh", max_count_per_loop=0):
    """Only outs[root] is written."""
    if algo == "mesh_two_shot":
        return lib().orc_reduce_two_shot(ctypes.c_uint32(len(ins)), _ptr_array(ins), _ptr_array(outs),
                                         ctypes.c_uint64(count), dtype, op, acc, ctypes.c_uint32(root),
                                         ctypes.c_uint64(max_count_per_loop))
    if algo == "nhr":
        return lib().orc_reduce_nhr(ctypes.c_uint32(len(ins)), _ptr_array(ins), _ptr_array(outs),
                                    ctypes.c_uint64(count), dtype, op, acc, ctypes.c_uint32(root),
                                    ctypes.c_uint64(max_count_per_loop))
    return lib().orc_reduce_mesh(ctypes.c_uint32(len(ins)), _ptr_array(ins), _ptr_array(outs),
                                 ctypes.c_uint64(count), dtype, op, acc, ctypes.c_uint32(root))


def broadcast(bufs, count, dtype, root):
    return lib().orc_broadcast(ctypes.c_uint32(len(bufs)), _ptr_array(bufs), ctypes.c_uint64(count), dtype,
                               ctypes.c_uint32(root))


def scatter(ins, outs, recv_count, dtype, root):
    return lib().orc_scatter(ctypes.c_uint32(len(ins)), _ptr_array(ins), _ptr_array(outs),
                             ctypes.c_uint64(recv_count), dtype, ctypes.c_uint32(root))


# ---- point to point --------------------------------------------------------------------------
class SendRecvItem(ctypes.Structure):
    _fields_ = [("sendRecvType", ctypes.c_int), ("buf", ctypes.c_void_p), ("count", ctypes.c_uint64),
                ("dataType", ctypes.c_int), ("remoteRank", ctypes.c_uint32)]


def batch_send_recv(items_per_rank):
    """items_per_rank[r] = [(0 send / 1 recv, numpy array, count, dtype, remote rank), ...]; receive arrays are
    written in place."""
    n = len(items_per_rank)
    arrays = []
    for items in items_per_rank:
        arr = (SendRecvItem * max(len(items), 1))()
        for i, (kind, buf, count, dtype, remote) in enumerate(items):
            arr[i].sendRecvType, arr[i].count, arr[i].dataType, arr[i].remoteRank = kind, count, dtype, remote
            arr[i].buf = None if buf is None else buf.ctypes.data
        arrays.append(arr)
    ptrs = (ctypes.POINTER(SendRecvItem) * n)(*[ctypes.cast(a, ctypes.POINTER(SendRecvItem)) for a in arrays])
    nums = (ctypes.c_uint32 * n)(*[len(items) for items in items_per_rank])
    return lib().orc_batch_send_recv(ctypes.c_uint32(n), ptrs, nums)
