"""dfccl_amd: MI355X-native DFCCL data path (daemon kernel, SQ/CQ, ring
reduce-copy collectives) behind the reference's ofccl C API.

The Python layer is a thin ctypes mirror of include/ofccl.h used by the tests
and the benchmark; torch is only used for device memory and streams.
"""
from .api import (  # noqa: F401
    DTYPE_OF, NcclError, RankCtx, UniqueId, VirtualComm, check, nccl_dtype, reduce_copy,
    ncclSum, ncclProd, ncclMax, ncclMin, ncclAvg, ncclInt8, ncclUint8, ncclInt32, ncclUint32, ncclInt64, ncclUint64,
    ncclFloat16, ncclFloat32, ncclFloat64, ncclBfloat16,
)
