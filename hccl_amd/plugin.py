"""ctypes view of libhccl_amd_plugin_broker.so: the algorithm-plugin function table a maintainer points the
reference's plugin manager at (reference src/algo_plugin/hccl_algo_plugin_mgr.cc loads the library named by its
plugin-path environment variable and calls GetHcclAlgoPlugin).  Used by the tests; a C caller includes
include/hccl_algo_plugin.h instead."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
BROKER_PATH = os.path.join(_HERE, "libhccl_amd_plugin_broker.so")

PARAM_MAGIC = 0x48415050
STRUCT_VERSION = 1
API_VERSION = 1


class HcclAlgoPluginParam(ctypes.Structure):
    """Field order and widths of reference src/algo_plugin/inc/hccl_algo_plugin_common.h:74-101."""
    _fields_ = [
        ("version", ctypes.c_uint32), ("magic", ctypes.c_uint32), ("structSize", ctypes.c_uint32),
        ("opType", ctypes.c_int), ("opName", ctypes.c_char * 32), ("count", ctypes.c_uint64),
        ("root", ctypes.c_uint32), ("topoType", ctypes.c_int), ("topoName", ctypes.c_char * 32),
        ("rankNum", ctypes.c_uint32), ("serverNum", ctypes.c_uint32), ("sendBuf", ctypes.c_void_p),
        ("recvBuf", ctypes.c_void_p), ("stream", ctypes.c_void_p), ("dataType", ctypes.c_int),
        ("reduceOp", ctypes.c_int), ("remoteRank", ctypes.c_uint32), ("deviceNumPerModule", ctypes.c_uint32),
        ("moduleNum", ctypes.c_uint32), ("superPodNum", ctypes.c_uint32), ("serverNumPerSuperPod", ctypes.c_uint32),
        ("isAsymmetricTopo", ctypes.c_bool), ("reserved", ctypes.c_uint32 * 7),
    ]


_PARAM_P = ctypes.POINTER(HcclAlgoPluginParam)


class HcclAlgoPluginTable(ctypes.Structure):
    """reference src/algo_plugin/inc/hccl_algo_plugin_broker_api.h:24-49."""
    _fields_ = [
        ("version", ctypes.c_uint32),
        ("IsReady", ctypes.CFUNCTYPE(ctypes.c_bool)),
        ("FetchContext", ctypes.CFUNCTYPE(ctypes.c_void_p)),
        ("SelectAlg", ctypes.CFUNCTYPE(ctypes.c_bool, ctypes.c_void_p, _PARAM_P, ctypes.c_char_p, ctypes.c_size_t)),
        ("ExecuteAlg", ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p, _PARAM_P,
                                        ctypes.c_void_p)),
        ("QueryAlgs", ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p,
                                       ctypes.c_size_t)),
    ]


ALG_DIR = os.path.join(_HERE, "plugin_algs")     # what a maintainer points HCCL_PLUGIN_ALG_DIR at
ENTRY_MAGIC = 0x48415045


class HcclAlgoPluginAlgEntry(ctypes.Structure):
    """reference src/algo_plugin/inc/hccl_algo_plugin_common.h:104-115."""
    _fields_ = [("version", ctypes.c_uint32), ("magic", ctypes.c_uint32), ("structSize", ctypes.c_uint32),
                ("algName", ctypes.c_char * 128), ("soPath", ctypes.c_char * 512), ("fnSymbol", ctypes.c_char * 128)]


def selector_path(op_name):
    """<ALG_DIR>/<Op>/libhccl_plugin_<op>_selector.so, the name the reference's broker derives
    (reference experimental/eco_system/algo_plugin/hccl_algo_plugin/plugin_broker/src/plugin_broker.cc:192)."""
    return os.path.join(ALG_DIR, op_name, "libhccl_plugin_%s_selector.so" % op_name.lower())


def load_selector(op_name):
    """dlopen-s a selector library the way the reference's broker does and types its two exports."""
    path = selector_path(op_name)
    if not os.path.exists(path):
        raise ImportError("%s is missing: run `make -C hccl_amd/csrc` first" % path)
    lib = ctypes.CDLL(path)
    lib.HcclAlgoPluginQueryEntries.restype = ctypes.POINTER(HcclAlgoPluginAlgEntry)
    lib.HcclAlgoPluginQueryEntries.argtypes = [ctypes.POINTER(ctypes.c_int)]
    lib.Select.restype = ctypes.c_bool
    lib.Select.argtypes = [_PARAM_P, ctypes.c_char_p, ctypes.c_size_t]
    return lib


_table = None


def table():
    """Loads the broker (raises if it has not been built) and returns its function table."""
    global _table
    if _table is None:
        if not os.path.exists(BROKER_PATH):
            raise ImportError("%s is missing: run `make -C hccl_amd/csrc` first" % BROKER_PATH)
        lib = ctypes.CDLL(BROKER_PATH)
        lib.GetHcclAlgoPlugin.restype = ctypes.POINTER(HcclAlgoPluginTable)
        _table = (lib, lib.GetHcclAlgoPlugin().contents)
    return _table[1]


def make_param(op_name, count=0, data_type=4, reduce_op=0, root=0, send_buf=None, recv_buf=None, stream=None,
               rank_num=0, remote_rank=0):
    p = HcclAlgoPluginParam()
    p.version, p.magic, p.structSize = STRUCT_VERSION, PARAM_MAGIC, ctypes.sizeof(HcclAlgoPluginParam)
    p.opName = op_name.encode()
    p.count, p.dataType, p.reduceOp, p.root, p.rankNum = count, int(data_type), int(reduce_op), root, rank_num
    p.remoteRank = remote_rank
    p.sendBuf = send_buf
    p.recvBuf = recv_buf
    p.stream = stream
    return p
