"""Helpers shared by the GPU parity tests: numpy storage arrays <-> torch tensors
on the GPU without any value conversion."""
import numpy as np
import torch

import dfccl_oracle as orc

# where the tests' buffers live; the suite's emulation mode (see conftest.py) puts them in host memory
DEVICE = "cuda:0"
EMULATED = False  # the daemon runs as host threads: few channels, and timing-dependent tests do not apply

# torch tensor type that holds each element type (uint32 / uint64 travel in signed tensors of the same width:
# only the bits matter, the library is told the ncclDataType_t separately)
TORCH_OF = {orc.I8: torch.int8, orc.U8: torch.uint8, orc.I32: torch.int32, orc.U32: torch.int32, orc.I64: torch.int64,
            orc.U64: torch.int64, orc.F16: torch.float16, orc.F32: torch.float32, orc.F64: torch.float64,
            orc.BF16: torch.bfloat16}
_NP_SIGNED = {orc.F16: np.int16, orc.BF16: np.int16, orc.U32: np.int32, orc.U64: np.int64}
_TORCH_SIGNED = {orc.F16: torch.int16, orc.BF16: torch.int16, orc.U32: torch.int32, orc.U64: torch.int64}


def to_gpu(dtype, arr):
    """Oracle storage array (bf16 / fp16 as uint16 bits) -> torch tensor on cuda:0, same bits."""
    if dtype in _NP_SIGNED:
        t = torch.from_numpy(arr.view(_NP_SIGNED[dtype]).copy()).view(TORCH_OF[dtype])
    else:
        t = torch.from_numpy(arr.copy())
    return t.to(DEVICE)


def to_np(dtype, t):
    """Torch tensor on the GPU -> oracle storage array, same bits."""
    c = t.detach().cpu()
    if dtype in _NP_SIGNED:
        return c.view(_TORCH_SIGNED[dtype]).numpy().view(orc.NP_STORAGE[dtype]).copy()
    return c.numpy().copy()


def geom_of(ring, coll_id):
    g = ring.ctxs[0].geometry(coll_id)
    return orc.Geom(g.nRanks, g.nChannels, g.chunkElems, g.alignElems)
