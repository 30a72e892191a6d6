"""Loads libdfccl.so (the HIP kernels + C++ host runtime) through ctypes.

There is no fallback: if the library has not been built, or cannot be loaded,
every entry point raises.  Build it with `make -C dfccl_amd/csrc` (or
`__graft_entry__.build()`).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdfccl.so")

CALLBACK = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_int, ctypes.c_void_p)


class UniqueId(ctypes.Structure):
    _fields_ = [("internal", ctypes.c_char * 128)]


class Stats(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint64) for n in
                ("structBytes", "sqesRead", "cqesWritten", "ctxSaves", "ctxLoads", "voluntaryQuits", "daemonLaunches",
                 "forcedQuits", "slicesMoved", "sqFullWaits")]


class CollGeometry(ctypes.Structure):
    _fields_ = [("nRanks", ctypes.c_int), ("nChannels", ctypes.c_int), ("chunkElems", ctypes.c_int64),
                ("alignElems", ctypes.c_int64), ("sliceElems", ctypes.c_int64), ("slicesPerChunk", ctypes.c_int),
                ("fifoSlots", ctypes.c_int), ("protocol", ctypes.c_int)]


# every symbol include/ofccl.h declares: name -> (restype, argtypes)
_vp, _sz, _int = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
SIGNATURES = {
    "ncclGetUniqueId": (_int, [ctypes.POINTER(UniqueId)]),
    "ncclCommInitRank": (_int, [ctypes.POINTER(_vp), _int, UniqueId, _int]),
    "ncclCommDestroy": (_int, [_vp]),
    "ncclCommCount": (_int, [_vp, ctypes.POINTER(_int)]),
    "ncclCommUserRank": (_int, [_vp, ctypes.POINTER(_int)]),
    "ncclGetErrorString": (ctypes.c_char_p, [_int]),
    "ncclRedOpCreatePreMulSum": (_int, [ctypes.POINTER(_int), _vp, _int, _int, _vp]),
    "ncclRedOpDestroy": (_int, [_int, _vp]),
    "ofcclInitRankCtx": (_int, [ctypes.POINTER(_vp), _int]),
    "ofcclFinalizeRankCtx7StartHostThrds": (_int, [_vp]),
    "ofcclPrepareDone": (_int, [_vp]),
    "ofcclDestroy": (_int, [_vp]),
    "ofcclPrepareReduce": (_int, [_sz, _int, _int, _int, _vp, _int, _vp]),
    "ofcclPrepareBcast": (_int, [_sz, _int, _int, _vp, _int, _vp]),
    "ofcclPrepareBroadcast": (_int, [_sz, _int, _int, _vp, _int, _vp]),
    "ofcclPrepareAllReduce": (_int, [_sz, _int, _int, _vp, _int, _vp]),
    "ofcclPrepareReduceScatter": (_int, [_sz, _int, _int, _vp, _int, _vp]),
    "ofcclPrepareAllGather": (_int, [_sz, _int, _vp, _int, _vp]),
    "ofcclRunReduce": (_int, [_vp, _vp, _int, CALLBACK, _vp, _vp]),
    "ofcclRunBcast": (_int, [_vp, _int, CALLBACK, _vp, _vp]),
    "ofcclRunBroadcast": (_int, [_vp, _vp, _int, CALLBACK, _vp, _vp]),
    "ofcclRunAllReduce": (_int, [_vp, _vp, _int, CALLBACK, _vp, _vp]),
    "ofcclRunReduceScatter": (_int, [_vp, _vp, _int, CALLBACK, _vp, _vp]),
    "ofcclRunAllGather": (_int, [_vp, _vp, _int, CALLBACK, _vp, _vp]),
    "dfcclReduceCopy": (_int, [ctypes.POINTER(_vp), _int, _vp, _sz, _int, _int, _sz, _vp]),
    "dfcclGetStats": (_int, [_vp, ctypes.POINTER(Stats)]),
    "dfcclDumpState": (_int, [_vp]),
    "dfcclGetCollTiming": (_int, [_vp, _int, ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64)]),
    "dfcclGetCollGeometry": (_int, [_vp, _int, ctypes.POINTER(CollGeometry)]),
}

_lib = None


def load():
    """Returns the loaded library with argument types set; raises if it is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C dfccl_amd/csrc`. "
                "dfccl_amd has no fallback path.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the ABI lost a symbol
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib
