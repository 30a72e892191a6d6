"""Helpers shared by the GPU parity tests: numpy storage arrays <-> torch tensors
on the GPU without any value conversion."""
import numpy as np
import torch

import dfccl_oracle as orc

# where the tests' buffers live; the suite's emulation mode (see conftest.py) puts them in host memory
DEVICE = "cuda:0"
EMULATED = False  # the daemon runs as host threads: few channels, and timing-dependent tests do not apply

TORCH_OF = {orc.I8: torch.int8, orc.I32: torch.int32, orc.F16: torch.float16, orc.F32: torch.float32,
            orc.BF16: torch.bfloat16}


def to_gpu(dtype, arr):
    """Oracle storage array (bf16 / fp16 as uint16 bits) -> torch tensor on cuda:0, same bits."""
    if dtype in (orc.F16, orc.BF16):
        t = torch.from_numpy(arr.view(np.int16).copy()).view(TORCH_OF[dtype])
    else:
        t = torch.from_numpy(arr.copy())
    return t.to(DEVICE)


def to_np(dtype, t):
    """Torch tensor on the GPU -> oracle storage array, same bits."""
    c = t.detach().cpu()
    if dtype in (orc.F16, orc.BF16):
        return c.view(torch.int16).numpy().view(np.uint16).copy()
    return c.numpy().copy()


def geom_of(ring, coll_id):
    g = ring.ctxs[0].geometry(coll_id)
    return orc.Geom(g.nRanks, g.nChannels, g.chunkElems, g.alignElems)
