"""Golden vectors (tests/golden/ring_cases.npz, written by tests/golden/make_golden.py from the CPU oracle):
the oracle must keep reproducing them (CPU), and the HIP path must match them (GPU).  The chunk geometry of
each case is part of the fixture, so on the GPU only the cases whose geometry the library's planner also
chooses for that size are compared bit for bit in float; integer and Min/Max cases do not depend on it."""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import dfccl_oracle as orc  # noqa: E402
from make_golden import CASES, PREMUL_CASES, run_case, run_premul_case  # noqa: E402

DATA = np.load(os.path.join(HERE, "golden", "ring_cases.npz"), allow_pickle=False)


def case_arrays(idx, n, kind):
    sends = [DATA[f"c{idx}_in{r}"] for r in range(n)]
    nout = 1 if kind == "reduce_copy" else n
    outs = [DATA[f"c{idx}_out{r}"] for r in range(nout)]
    return sends, outs


@pytest.mark.parametrize("idx", range(len(CASES)))
def test_oracle_reproduces_golden(idx):
    kind, dtype, op, n, count, root, geom = CASES[idx]
    sends, outs = case_arrays(idx, n, kind)
    got = run_case(kind, dtype, op, n, count, root, geom, [s.copy() for s in sends])
    for r in range(len(outs)):
        assert np.array_equal(got[r], outs[r]), (idx, r)


def order_independent(dtype, op):
    return dtype not in orc.FLOAT_DTYPES or op in (orc.MAX, orc.MIN)


@pytest.mark.gpu
@pytest.mark.parametrize("idx", range(len(CASES)))
def test_hip_path_matches_golden(idx, monkeypatch):
    import torch
    import dfccl_amd
    from dfccl_amd.ring import VirtualRing
    import gpu_util
    from gpu_util import TORCH_OF, to_gpu, to_np
    kind, dtype, op, n, count, root, geom = CASES[idx]
    sends_np, outs = case_arrays(idx, n, kind)
    sends = [to_gpu(dtype, s) for s in sends_np]
    if kind == "reduce_copy":
        dst = torch.zeros(count, dtype=TORCH_OF[dtype], device=gpu_util.DEVICE)
        dfccl_amd.reduce_copy(sends, dst, op, dtype=dtype)
        torch.cuda.current_stream().synchronize()
        assert np.array_equal(to_np(dtype, dst), outs[0])
        return
    monkeypatch.setenv("DFCCL_DAEMON_MAX_MS", "10000")
    recv_len = count * n if kind == "all_gather" else count
    recvs = [torch.zeros(recv_len, dtype=TORCH_OF[dtype], device=gpu_util.DEVICE) for _ in range(n)]
    torch.cuda.current_stream().synchronize()
    with VirtualRing(n) as ring:
        ring.prepare(0, kind, count, dtype, op, root)
        ring.finalize()
        g = ring.ctxs[0].geometry(0)
        same_geometry = (g.nChannels, g.chunkElems, g.alignElems) == geom
        ring.run(0, sends, recvs, timeout=30)
        copy_kind = kind in ("all_gather", "broadcast")
        if not (copy_kind or order_independent(dtype, op) or same_geometry or kind in ("reduce_scatter", "reduce")):
            pytest.skip("float all-reduce planned with another chunk geometry than the fixture's")
        for r in range(n):
            if kind == "reduce" and r != root:
                continue
            assert np.array_equal(to_np(dtype, recvs[r]), outs[r]), (idx, r)


# ---- PreMulSum with a scalar per rank ------------------------------------------------------------------------

def premul_arrays(idx, n):
    return [DATA[f"p{idx}_in{r}"] for r in range(n)], [DATA[f"p{idx}_out{r}"] for r in range(n)]


@pytest.mark.parametrize("idx", range(len(PREMUL_CASES)))
def test_oracle_reproduces_golden_premul_sum(idx):
    kind, dtype, values, n, count, root, geom = PREMUL_CASES[idx]
    sends, outs = premul_arrays(idx, n)
    got = run_premul_case(kind, dtype, values, n, count, root, geom, [s.copy() for s in sends])
    for r in range(n):
        assert np.array_equal(got[r], outs[r]), (idx, r)


@pytest.mark.gpu
@pytest.mark.parametrize("idx", range(len(PREMUL_CASES)))
def test_hip_path_matches_golden_premul_sum(idx, monkeypatch):
    import torch
    from dfccl_amd.ring import VirtualRing
    import gpu_util
    from gpu_util import TORCH_OF, to_gpu, to_np
    kind, dtype, values, n, count, root, geom = PREMUL_CASES[idx]
    sends_np, outs = premul_arrays(idx, n)
    sends = [to_gpu(dtype, s) for s in sends_np]
    monkeypatch.setenv("DFCCL_DAEMON_MAX_MS", "10000")
    recvs = [torch.zeros(count, dtype=TORCH_OF[dtype], device=gpu_util.DEVICE) for _ in range(n)]
    torch.cuda.current_stream().synchronize()
    es = orc.TYPE_SIZE[dtype]
    premul = [int(orc.scalar_bits(dtype, v)).to_bytes(8, "little")[:es] for v in values]
    with VirtualRing(n) as ring:
        ring.prepare(0, kind, count, dtype, root=root, premul=premul)
        ring.finalize()
        g = ring.ctxs[0].geometry(0)
        same_geometry = (g.nChannels, g.chunkElems, g.alignElems) == geom
        ring.run(0, sends, recvs, timeout=30)
        if kind == "all_reduce" and dtype in orc.FLOAT_DTYPES and not same_geometry:
            pytest.skip("float all-reduce planned with another chunk geometry than the fixture's")
        for r in range(n):
            if kind == "reduce" and r != root:
                continue
            assert np.array_equal(to_np(dtype, recvs[r]), outs[r]), (idx, r)
