"""ctypes binding of the CPU oracle (test infrastructure only).

Only tests/, the smoke test and the benchmark's cpu_baseline leg import this
module; the shipped package never does.  Arrays are numpy; bf16 and fp16 travel
as uint16 bit patterns so that no float conversion happens on the way.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdfccl_oracle.so")

I8, U8, I32, U32, I64, U64, F16, F32, F64, BF16 = range(10)
SUM, PROD, MAX, MIN, AVG, PREMULSUM = 0, 1, 2, 3, 4, 5
DTYPES = (I8, I32, F16, F32, BF16)          # the five types of the headline configurations
ALL_DTYPES = tuple(range(10))               # every ncclDataType_t
OPS = (SUM, PROD, MAX, MIN)
FLOAT_DTYPES = (F16, F32, F64, BF16)
TYPE_SIZE = {I8: 1, U8: 1, I32: 4, U32: 4, I64: 8, U64: 8, F16: 2, F32: 4, F64: 8, BF16: 2}
NP_STORAGE = {I8: np.int8, U8: np.uint8, I32: np.int32, U32: np.uint32, I64: np.int64, U64: np.uint64,
              F16: np.uint16, F32: np.float32, F64: np.float64, BF16: np.uint16}


def build(force=False):
    """Compile the oracle with gcc. Building the checker is not using it."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-B", "-C", _HERE, "libdfccl_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class Geom(ctypes.Structure):
    _fields_ = [("n_ranks", ctypes.c_int), ("n_channels", ctypes.c_int),
                ("chunk_elems", ctypes.c_int64), ("align_elems", ctypes.c_int64)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, vpp = ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)
        L.orc_type_size.argtypes = [ctypes.c_int]
        L.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        L.orc_f32_to_bf16.restype = ctypes.c_uint16
        L.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_bf16_to_f32.restype = ctypes.c_float
        L.orc_f32_to_f16.argtypes = [ctypes.c_float]
        L.orc_f32_to_f16.restype = ctypes.c_uint16
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f16_to_f32.restype = ctypes.c_float
        L.orc_reduce_copy.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, vpp, vp, ctypes.c_size_t]
        L.orc_reduce_copy_mt.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, vpp, vp, ctypes.c_size_t,
                                         ctypes.c_int]
        u64 = ctypes.c_uint64
        L.orc_reduce_copy_x.argtypes = [ctypes.c_int, ctypes.c_int, u64, ctypes.c_int, vpp, vp, ctypes.c_size_t]
        L.orc_avg_scalar.argtypes = [ctypes.c_int, ctypes.c_int]
        L.orc_avg_scalar.restype = u64
        L.orc_real_chunk.argtypes = [ctypes.c_int64] * 4
        L.orc_real_chunk.restype = ctypes.c_int64
        gp = ctypes.POINTER(Geom)
        L.orc_all_reduce.argtypes = [ctypes.c_int, ctypes.c_int, gp, ctypes.c_int64, vpp, vpp]
        L.orc_reduce_scatter.argtypes = [ctypes.c_int, ctypes.c_int, gp, ctypes.c_int64, vpp, vpp]
        L.orc_all_gather.argtypes = [ctypes.c_int, gp, ctypes.c_int64, vpp, vpp]
        L.orc_reduce.argtypes = [ctypes.c_int, ctypes.c_int, gp, ctypes.c_int64, ctypes.c_int, vpp, vpp]
        L.orc_broadcast.argtypes = [ctypes.c_int, gp, ctypes.c_int64, ctypes.c_int, vpp, vpp]
        L.orc_all_reduce_x.argtypes = [ctypes.c_int, ctypes.c_int, u64, gp, ctypes.c_int64, vpp, vpp]
        L.orc_reduce_scatter_x.argtypes = [ctypes.c_int, ctypes.c_int, u64, gp, ctypes.c_int64, vpp, vpp]
        L.orc_reduce_x.argtypes = [ctypes.c_int, ctypes.c_int, u64, gp, ctypes.c_int64, ctypes.c_int, vpp, vpp]
        u64p = ctypes.POINTER(u64)
        L.orc_all_reduce_xr.argtypes = [ctypes.c_int, ctypes.c_int, u64p, gp, ctypes.c_int64, vpp, vpp]
        L.orc_reduce_scatter_xr.argtypes = [ctypes.c_int, ctypes.c_int, u64p, gp, ctypes.c_int64, vpp, vpp]
        L.orc_reduce_xr.argtypes = [ctypes.c_int, ctypes.c_int, u64p, gp, ctypes.c_int64, ctypes.c_int, vpp, vpp]
        L.orc_all_reduce_owner.argtypes = [gp, ctypes.c_int64, ctypes.c_int64]
        L.orc_cqe_encode.argtypes = [ctypes.c_uint, ctypes.c_uint, ctypes.c_uint]
        L.orc_cqe_encode.restype = ctypes.c_uint64
        L.orc_cqe_decode.argtypes = [ctypes.c_uint64] + [ctypes.POINTER(ctypes.c_uint)] * 3
        L.orc_sq_full.argtypes = [ctypes.c_uint64] * 3
        L.orc_sq_empty.argtypes = [ctypes.c_uint64] * 2
        _lib = L
    return _lib


def _ptrs(arrays):
    arr = (ctypes.c_void_p * len(arrays))()
    for i, a in enumerate(arrays):
        assert a.flags["C_CONTIGUOUS"]
        arr[i] = a.ctypes.data
    return arr


def _check(dtype, arrays):
    for a in arrays:
        assert a.dtype == NP_STORAGE[dtype], (a.dtype, dtype)


def reduce_copy(dtype, op, srcs, nthreads=1, scalar=0):
    """Fold srcs left to right with op; returns the destination array.  op may be AVG (over the len(srcs)
    sources) or PREMULSUM with `scalar` = the bits of one element."""
    _check(dtype, srcs)
    dst = np.empty_like(srcs[0])
    if nthreads > 1 and scalar == 0:
        rc = lib().orc_reduce_copy_mt(dtype, op, len(srcs), _ptrs(srcs), dst.ctypes.data, srcs[0].size, nthreads)
    else:
        rc = lib().orc_reduce_copy_x(dtype, op, scalar, len(srcs), _ptrs(srcs), dst.ctypes.data, srcs[0].size)
    assert rc == 0
    return dst


def avg_scalar(dtype, n):
    """What ncclAvg turns into for a group of n: n (integer types) or the bits of 1/n in the element type."""
    return lib().orc_avg_scalar(dtype, n)


def scalar_bits(dtype, value):
    """Bits of one element of `dtype` holding `value` (for PREMULSUM)."""
    if dtype == F16:
        return int(f32_to_f16_bits(np.array([value], dtype=np.float32))[0])
    if dtype == BF16:
        return int(f32_to_bf16_bits(np.array([value], dtype=np.float32))[0])
    a = np.array([value]).astype(NP_STORAGE[dtype])
    return int(np.frombuffer(a.tobytes().ljust(8, b"\0"), dtype=np.uint64)[0])


def _scalars(scalar, n):
    """`scalar` of the reducing collectives: the bits of one element for every rank, or a sequence with one per
    rank (every rank's own PreMulSum operator)."""
    vals = list(scalar) if isinstance(scalar, (list, tuple)) else [scalar] * n
    assert len(vals) == n
    return (ctypes.c_uint64 * n)(*[int(v) for v in vals])


def all_reduce(dtype, op, geom, sends, scalar=0):
    _check(dtype, sends)
    recvs = [np.zeros_like(s) for s in sends]
    rc = lib().orc_all_reduce_xr(dtype, op, _scalars(scalar, len(sends)), ctypes.byref(geom), sends[0].size,
                                 _ptrs(sends), _ptrs(recvs))
    assert rc == 0
    return recvs


def reduce_scatter(dtype, op, geom, sends, scalar=0):
    _check(dtype, sends)
    n = geom.n_ranks
    recvcount = sends[0].size // n
    recvs = [np.zeros(recvcount, dtype=s.dtype) for s in sends]
    rc = lib().orc_reduce_scatter_xr(dtype, op, _scalars(scalar, len(sends)), ctypes.byref(geom), recvcount,
                                     _ptrs(sends), _ptrs(recvs))
    assert rc == 0
    return recvs


def all_gather(dtype, geom, sends):
    _check(dtype, sends)
    n = geom.n_ranks
    recvs = [np.zeros(s.size * n, dtype=s.dtype) for s in sends]
    rc = lib().orc_all_gather(dtype, ctypes.byref(geom), sends[0].size, _ptrs(sends), _ptrs(recvs))
    assert rc == 0
    return recvs


def reduce(dtype, op, geom, root, sends, scalar=0):
    _check(dtype, sends)
    recvs = [np.zeros_like(s) for s in sends]
    rc = lib().orc_reduce_xr(dtype, op, _scalars(scalar, len(sends)), ctypes.byref(geom), sends[0].size, root,
                             _ptrs(sends), _ptrs(recvs))
    assert rc == 0
    return recvs


def broadcast(dtype, geom, root, sends):
    _check(dtype, sends)
    recvs = [np.zeros_like(s) for s in sends]
    rc = lib().orc_broadcast(dtype, ctypes.byref(geom), sends[0].size, root, _ptrs(sends), _ptrs(recvs))
    assert rc == 0
    return recvs


def all_reduce_owner(geom, count, i):
    return lib().orc_all_reduce_owner(ctypes.byref(geom), count, i)


# ---- bit-pattern helpers shared by the tests -------------------------------

def f32_to_bf16_bits(x):
    """Round-to-nearest-even float32 -> bfloat16 bit patterns (numpy, vectorised)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    return ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (b.astype(np.uint32) << 16).view(np.float32)


def f32_to_f16_bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def f16_bits_to_f32(b):
    return b.view(np.float16).astype(np.float32)
