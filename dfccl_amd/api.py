"""Host-side mirror of the ofccl interface (src/nccl.h.in:202-378 in the
reference) over the C ABI.  Method names and argument meaning follow the C
entry points one to one; buffers are torch tensors that live on the GPU."""
import ctypes
import threading

import torch

from . import _lib
from ._lib import CALLBACK, CollGeometry, Stats, UniqueId

ncclSum, ncclProd, ncclMax, ncclMin, ncclAvg = 0, 1, 2, 3, 4
(ncclInt8, ncclUint8, ncclInt32, ncclUint32, ncclInt64, ncclUint64, ncclFloat16, ncclFloat32, ncclFloat64,
 ncclBfloat16) = range(10)
ncclScalarDevice, ncclScalarHostImmediate = 0, 1

DTYPE_OF = {torch.int8: ncclInt8, torch.uint8: ncclUint8, torch.int32: ncclInt32, torch.int64: ncclInt64,
            torch.float16: ncclFloat16, torch.float32: ncclFloat32, torch.float64: ncclFloat64,
            torch.bfloat16: ncclBfloat16}
for _name, _code in (("uint32", ncclUint32), ("uint64", ncclUint64)):  # (newer torch versions have these)
    if hasattr(torch, _name):
        DTYPE_OF[getattr(torch, _name)] = _code


class NcclError(RuntimeError):
    def __init__(self, code, what):
        msg = _lib.load().ncclGetErrorString(code) if hasattr(_lib.load(), "ncclGetErrorString") else b""
        super().__init__(f"{what}: ncclResult_t {code} ({(msg or b'').decode()})")
        self.code = code


def check(code, what="dfccl"):
    if code != 0:
        raise NcclError(code, what)


def nccl_dtype(t):
    try:
        return DTYPE_OF[t.dtype]
    except KeyError:
        raise TypeError(f"dtype {t.dtype} is not on this path") from None


def _dev_ptr(t):
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("buffers must live on the GPU")
    if not t.is_contiguous():
        raise ValueError("buffers must be contiguous")
    return ctypes.c_void_p(t.data_ptr())


def reduce_copy(srcs, dst, op=ncclSum, chunk_bytes=0, stream=None, dtype=None):
    """dst = srcs[0] (op) srcs[1] (op) ... folded left to right (dfcclReduceCopy). Asynchronous on `stream`
    (default: torch's current stream).  `dtype` overrides the ncclDataType_t taken from the tensors (for element
    types torch has no tensor type for, held in tensors of the same width)."""
    lib = _lib.load()
    n = dst.numel()
    for s in srcs:
        if s.dtype != dst.dtype or s.numel() != n:
            raise ValueError("sources and destination must agree in dtype and length")
    arr = (ctypes.c_void_p * len(srcs))(*[s.data_ptr() for s in srcs])
    if stream is None:
        stream = torch.cuda.current_stream(dst.device)
    check(lib.dfcclReduceCopy(arr, len(srcs), _dev_ptr(dst), n, nccl_dtype(dst) if dtype is None else dtype, op,
                              chunk_bytes, ctypes.c_void_p(stream.cuda_stream)), "dfcclReduceCopy")


class VirtualComm:
    """One virtual rank's handle on a communicator (ncclCommInitRank)."""

    def __init__(self, nranks, unique_id, rank):
        self.handle = ctypes.c_void_p()
        check(_lib.load().ncclCommInitRank(ctypes.byref(self.handle), nranks, unique_id, rank), "ncclCommInitRank")
        self.nranks, self.rank = nranks, rank

    @staticmethod
    def unique_id():
        uid = UniqueId()
        check(_lib.load().ncclGetUniqueId(ctypes.byref(uid)), "ncclGetUniqueId")
        return uid

    @classmethod
    def create_all(cls, nranks):
        """The nranks handles of one fresh communicator, index = rank."""
        uid = cls.unique_id()
        return [cls(nranks, uid, r) for r in range(nranks)]

    def create_premul_sum(self, dtype, scalar_bytes=None, device_ptr=None):
        """ncclRedOpCreatePreMulSum; returns the op value.  The scalar is given as the bytes of one element
        (ncclScalarHostImmediate), or as the device address it is to be read from whenever an instance starts
        (ncclScalarDevice)."""
        op = ctypes.c_int()
        if device_ptr is not None:
            check(_lib.load().ncclRedOpCreatePreMulSum(ctypes.byref(op), ctypes.c_void_p(device_ptr), dtype,
                                                       ncclScalarDevice, self.handle), "ncclRedOpCreatePreMulSum")
            return op.value
        buf = ctypes.create_string_buffer(bytes(scalar_bytes).ljust(8, b"\0"), 8)
        check(_lib.load().ncclRedOpCreatePreMulSum(ctypes.byref(op), ctypes.cast(buf, ctypes.c_void_p), dtype,
                                                   ncclScalarHostImmediate, self.handle), "ncclRedOpCreatePreMulSum")
        return op.value

    def destroy_op(self, op):
        check(_lib.load().ncclRedOpDestroy(op, self.handle), "ncclRedOpDestroy")

    def destroy(self):
        if self.handle:
            check(_lib.load().ncclCommDestroy(self.handle), "ncclCommDestroy")
            self.handle = ctypes.c_void_p()


class RankCtx:
    """ofcclRankCtx_t for one virtual rank: prepare*, finalize, run*, destroy."""

    def __init__(self, rank):
        self.lib = _lib.load()
        self.rank = rank
        self.handle = ctypes.c_void_p()
        check(self.lib.ofcclInitRankCtx(ctypes.byref(self.handle), rank), "ofcclInitRankCtx")
        self._keep = {}  # collId -> ctypes callback object, kept alive while in flight
        self._lock = threading.Lock()

    # -- prepare ------------------------------------------------------------
    def prepare_all_reduce(self, count, dtype, op, comm, coll_id):
        check(self.lib.ofcclPrepareAllReduce(count, dtype, op, comm.handle, coll_id, self.handle),
              "ofcclPrepareAllReduce")

    def prepare_reduce_scatter(self, recvcount, dtype, op, comm, coll_id):
        check(self.lib.ofcclPrepareReduceScatter(recvcount, dtype, op, comm.handle, coll_id, self.handle),
              "ofcclPrepareReduceScatter")

    def prepare_all_gather(self, sendcount, dtype, comm, coll_id):
        check(self.lib.ofcclPrepareAllGather(sendcount, dtype, comm.handle, coll_id, self.handle),
              "ofcclPrepareAllGather")

    def prepare_reduce(self, count, dtype, op, root, comm, coll_id):
        check(self.lib.ofcclPrepareReduce(count, dtype, op, root, comm.handle, coll_id, self.handle),
              "ofcclPrepareReduce")

    def prepare_broadcast(self, count, dtype, root, comm, coll_id):
        check(self.lib.ofcclPrepareBroadcast(count, dtype, root, comm.handle, coll_id, self.handle),
              "ofcclPrepareBroadcast")

    def prepare_bcast(self, count, dtype, root, comm, coll_id):
        check(self.lib.ofcclPrepareBcast(count, dtype, root, comm.handle, coll_id, self.handle), "ofcclPrepareBcast")

    def finalize(self):
        check(self.lib.ofcclFinalizeRankCtx7StartHostThrds(self.handle), "ofcclFinalizeRankCtx7StartHostThrds")

    def prepare_done(self):
        check(self.lib.ofcclPrepareDone(self.handle), "ofcclPrepareDone")

    # -- run ----------------------------------------------------------------
    def _callback(self, coll_id, fn):
        def tramp(cid, _args):
            try:
                if fn is not None:
                    fn(cid)
            except Exception:  # never let an exception cross the C boundary
                import traceback
                traceback.print_exc()
            return 0
        cb = CALLBACK(tramp)
        with self._lock:
            self._keep[coll_id] = cb
        return cb

    def _run(self, name, coll_id, fn, *bufs):
        cb = self._callback(coll_id, fn)
        check(getattr(self.lib, name)(*[_dev_ptr(b) for b in bufs], coll_id, cb, None, self.handle), name)

    def run_all_reduce(self, send, recv, coll_id, callback=None):
        self._run("ofcclRunAllReduce", coll_id, callback, send, recv)

    def run_reduce_scatter(self, send, recv, coll_id, callback=None):
        self._run("ofcclRunReduceScatter", coll_id, callback, send, recv)

    def run_all_gather(self, send, recv, coll_id, callback=None):
        self._run("ofcclRunAllGather", coll_id, callback, send, recv)

    def run_reduce(self, send, recv, coll_id, callback=None):
        self._run("ofcclRunReduce", coll_id, callback, send, recv)

    def run_broadcast(self, send, recv, coll_id, callback=None):
        self._run("ofcclRunBroadcast", coll_id, callback, send, recv)

    def run_bcast(self, buf, coll_id, callback=None):
        self._run("ofcclRunBcast", coll_id, callback, buf)

    # -- introspection --------------------------------------------------------
    def dump_state(self):
        """What the host knows about the daemon, printed to stderr (a diagnosis aid when a collective hangs)."""
        check(self.lib.dfcclDumpState(self.handle), "dfcclDumpState")

    def stats(self):
        s = Stats()
        s.structBytes = ctypes.sizeof(Stats)
        check(self.lib.dfcclGetStats(self.handle, ctypes.byref(s)), "dfcclGetStats")
        return {n: getattr(s, n) for n, _ in Stats._fields_}

    def timing_ns(self, coll_id):
        """(submit, complete) steady-clock ns of coll_id's last instance, taken inside the library."""
        a, b = ctypes.c_uint64(), ctypes.c_uint64()
        check(self.lib.dfcclGetCollTiming(self.handle, coll_id, ctypes.byref(a), ctypes.byref(b)), "dfcclGetCollTiming")
        return a.value, b.value

    def geometry(self, coll_id):
        g = CollGeometry()
        check(self.lib.dfcclGetCollGeometry(self.handle, coll_id, ctypes.byref(g)), "dfcclGetCollGeometry")
        return g

    def destroy(self):
        if self.handle:
            check(self.lib.ofcclDestroy(self.handle), "ofcclDestroy")
            self.handle = ctypes.c_void_p()
            self._keep.clear()
