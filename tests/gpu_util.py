"""Helpers for the GPU parity tests: a loopback world whose per-rank buffers are separate HBM
allocations, driven through the C ABI exactly as a single-threaded caller would (one call per rank
inside a group, all on one non-default stream)."""
import ctypes
import os

import numpy as np

import hccl_amd
from hccl_amd import Algo, OpKind

# HCCL_AMD_TEST_EMU=1 (set by tests/test_emulated_kernels.py for the pytest run it starts, never on the GPU box):
# the same tests drive the CPU emulation build of the library (tests/emu) with host buffers, so that the kernels'
# index arithmetic runs where AddressSanitizer and a debugger can see it.  conftest.py has then replaced the
# library the Python mirror calls.
EMU = os.environ.get("HCCL_AMD_TEST_EMU") == "1"
_libc = ctypes.CDLL(None)
_libc.malloc.restype = ctypes.c_void_p
_libc.malloc.argtypes = [ctypes.c_size_t]
_libc.free.argtypes = [ctypes.c_void_p]


class HostBuf:
    """A malloc'ed block of the bytes asked for, rounded up to whole 16-byte granules (so that the sanitizer's red zone
    starts with the first granule behind the payload), or a byte range of one; stands in for a torch device tensor in
    the emulation run.  Whole granules because the irregular copy path loads the aligned 16-byte vectors that cover
    its source bytes: it may read, never use, the rest of the first and last granule, which on the GPU cannot leave
    the allocation (or its page) either."""

    class _Block:
        def __init__(self, nbytes):
            self.ptr = _libc.malloc(max((nbytes + 15) & ~15, 16))
            assert self.ptr and self.ptr % 16 == 0, "out of memory"

        def __del__(self):
            _libc.free(self.ptr)

    def __init__(self, nbytes, block=None, offset=0):
        self.block = block if block is not None else HostBuf._Block(nbytes)
        self.offset = offset
        self.nbytes = nbytes

    def data_ptr(self):
        return self.block.ptr + self.offset

    def numel(self):
        return self.nbytes

    def bytes(self):
        return (ctypes.c_uint8 * self.nbytes).from_address(self.data_ptr())

    def __getitem__(self, key):
        start, stop, step = key.indices(self.nbytes)
        assert step == 1
        return HostBuf(max(stop - start, 0), self.block, self.offset + start)

    def fill(self, value):
        ctypes.memset(self.data_ptr(), value, self.nbytes)

    def write(self, raw):
        if raw.size:
            ctypes.memmove(self.data_ptr(), raw.ctypes.data, raw.size)

    def read(self):
        return np.frombuffer(self.bytes(), dtype=np.uint8).copy() if self.nbytes else np.zeros(0, np.uint8)


class _EmuStream:
    cuda_stream = 0x1000   # any non-null handle: the emulation runs every launch to completion

    def synchronize(self):
        pass

ALGO_BY_NAME = {"mesh": Algo.MESH, "ring": Algo.RING, "rhd": Algo.RHD, "nhr": Algo.NHR,
                "order_preserved": Algo.ORDER_PRESERVED, "aiv_mesh": Algo.AIV_MESH, "mesh_symmetric": Algo.MESH_SYMMETRIC,
                "mesh_chunk": Algo.MESH_CHUNK, "mesh_two_shot": Algo.MESH_TWO_SHOT, "mesh_concur": Algo.MESH_CONCUR}


def require_library_on_gpu():
    """The GPU tests are meaningless without the native library: fail, never skip."""
    if EMU:
        assert "emu" in os.path.basename(hccl_amd.lib()._name), "the emulation run must not load the GPU library"
        return
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    hccl_amd.lib()


def to_dev(arr, pad_front=0):
    """Uploads a numpy array as raw bytes.  pad_front shifts the payload to break 16-byte alignment."""
    raw = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
    if EMU:
        t = HostBuf(raw.size + pad_front)
        view = t[pad_front:pad_front + raw.size]
        view.write(raw)
        return view
    import torch
    t = torch.empty(raw.size + pad_front + 64, dtype=torch.uint8, device="cuda")
    view = t[pad_front:pad_front + raw.size]
    if raw.size:
        view.copy_(torch.from_numpy(raw.copy()))
    return view


def dev_zeros(nbytes, pad_front=0, fill=0xAB):
    if EMU:
        t = HostBuf(nbytes + pad_front)
        t.fill(fill)
        return t[pad_front:pad_front + nbytes]
    import torch
    t = torch.full((nbytes + pad_front + 64,), fill, dtype=torch.uint8, device="cuda")
    return t[pad_front:pad_front + nbytes]


def to_host(t, np_dtype):
    if EMU:
        return t.read().view(np_dtype).copy()
    return t.cpu().numpy().view(np_dtype).copy()


class World:
    def __init__(self, n):
        self.n = n
        self.comms = hccl_amd.comm_init_all(n)
        if EMU:
            self.stream = _EmuStream()
        else:
            import torch
            self.stream = torch.cuda.Stream()

    def close(self):
        if not EMU:
            import torch
            torch.cuda.synchronize()
        for c in self.comms:
            hccl_amd.comm_destroy(c)

    def set_algo(self, kind, name):
        hccl_amd.set_algo(self.comms[0], kind, ALGO_BY_NAME[name])

    def set_ccl_buffer_size(self, nbytes):
        hccl_amd.set_ccl_buffer_size(self.comms[0], nbytes)

    def inputs_ready(self):
        """Inputs are produced on torch's default stream; the collective runs on self.stream."""
        if EMU:
            return
        import torch
        torch.cuda.current_stream().synchronize()

    def sync(self):
        self.stream.synchronize()

    def all_reduce(self, sends, recvs, count, dtype, op, algo="mesh"):
        self.set_algo(OpKind.ALL_REDUCE, algo)
        self.inputs_ready()
        with hccl_amd.group():
            for r in range(self.n):
                hccl_amd.all_reduce(self.comms[r], sends[r], recvs[r], count, dtype, op, self.stream)
        self.sync()

    def reduce_scatter(self, sends, recvs, recv_count, dtype, op, algo="mesh"):
        self.set_algo(OpKind.REDUCE_SCATTER, algo)
        self.inputs_ready()
        with hccl_amd.group():
            for r in range(self.n):
                hccl_amd.reduce_scatter(self.comms[r], sends[r], recvs[r], recv_count, dtype, op, self.stream)
        self.sync()

    def all_gather(self, sends, recvs, send_count, dtype):
        self.inputs_ready()
        with hccl_amd.group():
            for r in range(self.n):
                hccl_amd.all_gather(self.comms[r], sends[r], recvs[r], send_count, dtype, self.stream)
        self.sync()

    def all_gather_v(self, sends, recvs, counts, displs, dtype):
        self.inputs_ready()
        with hccl_amd.group():
            for r in range(self.n):
                hccl_amd.all_gather_v(self.comms[r], sends[r], int(counts[r]), recvs[r], counts, displs, dtype,
                                      self.stream)
        self.sync()

    def all_to_all_v(self, sends, send_counts, sdispls, recvs, recv_counts, rdispls, dtype):
        self.inputs_ready()
        with hccl_amd.group():
            for r in range(self.n):
                hccl_amd.all_to_all_v(self.comms[r], sends[r], send_counts[r], sdispls[r], dtype, recvs[r],
                                      recv_counts[r], rdispls[r], dtype, self.stream)
        self.sync()

    def all_to_all(self, sends, recvs, count, dtype):
        self.inputs_ready()
        with hccl_amd.group():
            for r in range(self.n):
                hccl_amd.all_to_all(self.comms[r], sends[r], count, dtype, recvs[r], count, dtype, self.stream)
        self.sync()

    def all_to_all_vc(self, sends, recvs, matrix, dtype):
        self.inputs_ready()
        flat = hccl_amd.u64_array(np.asarray(matrix).reshape(-1))
        with hccl_amd.group():
            for r in range(self.n):
                hccl_amd.all_to_all_vc(self.comms[r], sends[r], flat, dtype, recvs[r], dtype, self.stream)
        self.sync()

    def reduce_scatter_v(self, sends, recvs, counts, displs, dtype, op, algo="mesh"):
        self.set_algo(OpKind.REDUCE_SCATTER, algo)
        self.inputs_ready()
        with hccl_amd.group():
            for r in range(self.n):
                hccl_amd.reduce_scatter_v(self.comms[r], sends[r], counts, displs, recvs[r], int(counts[r]), dtype, op,
                                          self.stream)
        self.sync()

    def reduce(self, sends, recvs, count, dtype, op, root, algo="mesh"):
        self.set_algo(OpKind.REDUCE, algo)
        self.inputs_ready()
        with hccl_amd.group():
            for r in range(self.n):
                hccl_amd.reduce(self.comms[r], sends[r], recvs[r], count, dtype, op, root, self.stream)
        self.sync()

    def broadcast(self, bufs, count, dtype, root):
        self.inputs_ready()
        with hccl_amd.group():
            for r in range(self.n):
                hccl_amd.broadcast(self.comms[r], bufs[r], count, dtype, root, self.stream)
        self.sync()

    def scatter(self, sends, recvs, recv_count, dtype, root):
        self.inputs_ready()
        with hccl_amd.group():
            for r in range(self.n):
                hccl_amd.scatter(self.comms[r], sends[r], recvs[r], recv_count, dtype, root, self.stream)
        self.sync()


def same_bits_nan_class(got, want, float_view=None):
    """Bit equality; where float_view is given, positions that are NaN on both sides only need to be NaN."""
    if float_view is None:
        return np.array_equal(got, want)
    g, w = float_view(got), float_view(want)
    both = np.isnan(g) & np.isnan(w)
    return np.array_equal(got[~both], want[~both]) and np.array_equal(np.isnan(g), np.isnan(w))


def rand_bytes(rng, nbytes):
    return rng.integers(0, 256, nbytes, dtype=np.uint8)


# A random AlltoAllV case: counts up to max_count with some empty segments; unless `aligned`, displacements are
# shuffled and leave gaps, so sources and destinations sit at arbitrary element offsets.
def a2a_case(rng, n, esz, max_count, aligned):
    send_counts = rng.integers(0, max_count, size=(n, n)).astype(np.uint64)
    send_counts[rng.random((n, n)) < 0.15] = 0
    if aligned:
        send_counts = (send_counts // (16 // esz)) * (16 // esz)
    recv_counts = send_counts.T.copy()
    sdispls = np.zeros((n, n), dtype=np.uint64)
    rdispls = np.zeros((n, n), dtype=np.uint64)
    for r in range(n):
        for tab, cnts in ((sdispls, send_counts), (rdispls, recv_counts)):
            off = 0
            for j in (range(n) if aligned else rng.permutation(n)):
                tab[r, j] = off
                off += int(cnts[r, j]) + (0 if aligned else int(rng.integers(0, 4)))
    in_sz = int((sdispls + send_counts).max()) + 1
    out_sz = int((rdispls + recv_counts).max()) + 1
    return send_counts, sdispls, recv_counts, rdispls, in_sz, out_sz
