"""Pins the torch restatement of the ring-order all-reduce (tests/torch_ring.py), which the GPU suite uses as the
expected result at the benchmark configurations' full sizes, against the CPU oracle at sizes the oracle covers:
ragged counts, a last loop with its own chunk size, 2..8 ranks, several channels, every float storage type."""
import types

import numpy as np
import pytest
import torch

import datagen
import dfccl_oracle as orc
import torch_ring

TORCH_OF = {orc.I32: torch.int32, orc.F16: torch.float16, orc.F32: torch.float32, orc.BF16: torch.bfloat16}
OP_NAME = {orc.SUM: "sum", orc.PROD: "prod", orc.MAX: "max", orc.MIN: "min"}


def to_torch(dtype, arr):
    if dtype in (orc.F16, orc.BF16):
        return torch.from_numpy(arr.view(np.int16).copy()).view(TORCH_OF[dtype])
    return torch.from_numpy(arr.copy())


def to_np(dtype, t):
    if dtype in (orc.F16, orc.BF16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


GEOMS = [  # ranks, channels, chunk, align, count
    (2, 1, 512, 256, 1000),
    (3, 2, 512, 256, 7013),
    (4, 1, 4096, 512, 100003),
    (4, 4, 2048, 512, 300001),
    (8, 2, 1024, 512, 150000),
    (8, 1, 4096, 512, 5),
    (5, 3, 512, 256, 512 * 15 * 2),
]


@pytest.mark.parametrize("n,channels,chunk,align,count", GEOMS)
def test_owner_map_matches_the_oracle(n, channels, chunk, align, count):
    g = orc.Geom(n, channels, chunk, align)
    owner = torch_ring.all_reduce_owner_map(count, n, channels, chunk, align, "cpu").numpy()
    for i in list(range(0, count, max(1, count // 997))) + [count - 1]:
        assert owner[i] == orc.all_reduce_owner(g, count, i), i


@pytest.mark.parametrize("dtype", [orc.BF16, orc.F16, orc.F32, orc.I32])
@pytest.mark.parametrize("op", [orc.SUM, orc.PROD, orc.MAX])
@pytest.mark.parametrize("n,channels,chunk,align,count", GEOMS[:5])
def test_fold_matches_the_oracle(dtype, op, n, channels, chunk, align, count):
    g = orc.Geom(n, channels, chunk, align)
    sends_np = [datagen.make(dtype, 77 + r, count) for r in range(n)]
    want = orc.all_reduce(dtype, op, g, sends_np)[0]
    geom = types.SimpleNamespace(nRanks=n, nChannels=channels, chunkElems=chunk, alignElems=align)
    got = torch_ring.all_reduce_expected([to_torch(dtype, s) for s in sends_np], geom, OP_NAME[op])
    assert np.array_equal(to_np(dtype, got), want)


def test_a_wrong_rank_order_would_be_noticed():
    # bf16 sums depend on the order: the restatement with the owner shifted by one must differ from the oracle
    n, channels, chunk, align, count = 4, 1, 4096, 512, 100003
    g = orc.Geom(n, channels, chunk, align)
    sends_np = [datagen.make(orc.BF16, 5 + r, count) for r in range(n)]
    want = orc.all_reduce(orc.BF16, orc.SUM, g, sends_np)[0]
    sends = [to_torch(orc.BF16, s) for s in sends_np]
    owner = torch_ring.all_reduce_owner_map(count, n, channels, chunk, align, "cpu")
    wrong = torch_ring.fold_in_ring_order(sends, (owner + 1) % n, "sum")
    assert not np.array_equal(to_np(orc.BF16, wrong), want)
