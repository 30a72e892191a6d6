"""Parity of the one-shot reduce-copy kernel (dfcclReduceCopy through the C ABI)
against the CPU oracle: bit-exact for every dtype / op, ragged and misaligned
lengths included."""
import numpy as np
import pytest
import torch

import datagen
import dfccl_oracle as orc
import gpu_util
from gpu_util import TORCH_OF, to_gpu, to_np

pytestmark = pytest.mark.gpu


def _run(dtype, op, srcs_np, chunk_bytes=0, offset_elems=0):
    import dfccl_amd
    srcs = [to_gpu(dtype, s) for s in srcs_np]
    n = srcs_np[0].size - offset_elems
    dst = torch.zeros(srcs_np[0].size, dtype=TORCH_OF[dtype], device=gpu_util.DEVICE)
    dfccl_amd.reduce_copy([s[offset_elems:] for s in srcs], dst[offset_elems:], op, chunk_bytes, dtype=dtype)
    torch.cuda.current_stream().synchronize()
    out = to_np(dtype, dst)
    assert not out[:offset_elems].any()  # nothing before the start was touched
    return out[offset_elems:], n


@pytest.mark.parametrize("dtype", orc.ALL_DTYPES)
@pytest.mark.parametrize("op", orc.OPS + (orc.AVG,))
def test_reduce_copy_two_sources_bit_exact(dtype, op):
    n = 1 << 20 if dtype not in (orc.I8, orc.U8) else 1 << 22
    if gpu_util.EMULATED:
        n >>= 4
    small = op == orc.PROD
    srcs = [datagen.make(dtype, 1000 + 10 * dtype + r, n, small_ints=small) for r in range(2)]
    got, _ = _run(dtype, op, srcs)
    want = orc.reduce_copy(dtype, op, srcs, nthreads=8)
    assert np.array_equal(got, want)


def test_config1_fp32_sum_two_ranks_chunk_128k():
    # fp32 Sum of 2 virtual-rank inputs, 1,048,576 elements, uniform[-1,1), chunk 128 KiB,
    # against a scalar host loop accumulating in rank order
    n = 1 << 20
    srcs = [datagen.uniform(1 + r, n) for r in range(2)]
    got, _ = _run(orc.F32, orc.SUM, srcs, chunk_bytes=128 << 10)
    assert np.array_equal(got.view(np.uint32), (srcs[0] + srcs[1]).view(np.uint32))
    assert np.array_equal(got, orc.reduce_copy(orc.F32, orc.SUM, srcs))


@pytest.mark.parametrize("k", [1, 3, 4, 5, 8])
@pytest.mark.parametrize("dtype,op", [(orc.F32, orc.SUM), (orc.BF16, orc.SUM), (orc.I32, orc.MAX), (orc.F16, orc.PROD),
                                      (orc.F64, orc.SUM), (orc.U64, orc.MIN), (orc.BF16, orc.AVG), (orc.I8, orc.AVG),
                                      (orc.F64, orc.AVG), (orc.U32, orc.AVG)])
def test_reduce_copy_k_sources_fold_order(k, dtype, op):
    # more than four sources take several launches that fold into the destination; an average multiplies only
    # the caller's sources (never the running value) and divides in the launch that finishes the sum
    n = 300000 if not gpu_util.EMULATED else 30000
    srcs = [datagen.make(dtype, 2000 + r, n) for r in range(k)]
    got, _ = _run(dtype, op, srcs)
    assert np.array_equal(got, orc.reduce_copy(dtype, op, srcs, nthreads=4))


def _nan_inputs(dtype, n):
    """Three sources with NaNs at every 3rd, 4th and 6th element: all-NaN at multiples of 12."""
    srcs = [datagen.make(dtype, 5000 + r, n) for r in range(3)]
    for x, every in zip(srcs, (3, 4, 6)):
        x[::every] = {orc.F16: 0x7e00, orc.BF16: 0x7fc0}.get(dtype, np.nan)
    return srcs


def _nan_mask(dtype, x):
    if dtype == orc.F16:
        return np.isnan(x.view(np.float16))
    if dtype == orc.BF16:
        return np.isnan(orc.bf16_bits_to_f32(x))
    return np.isnan(x)


@pytest.mark.parametrize("dtype", orc.FLOAT_DTYPES)
@pytest.mark.parametrize("op", [orc.MAX, orc.MIN])
def test_reduce_copy_max_min_with_nan_operands(dtype, op):
    # fmaxf / fminf (src/include/reduce_kernel.h:344-362,442-469) return the operand that is a number; a NaN comes
    # out only where every source holds one.  Equal to the oracle wherever the result is a number, NaN where it is
    # NaN (which NaN is not compared).
    n = 48000
    srcs = _nan_inputs(dtype, n)
    got, _ = _run(dtype, op, srcs)
    want = orc.reduce_copy(dtype, op, srcs)
    nan = _nan_mask(dtype, want)
    assert nan[::12].all() and not nan[1::12].any()
    assert np.array_equal(_nan_mask(dtype, got), nan)
    assert np.array_equal(got[~nan], want[~nan])


@pytest.mark.parametrize("n", [0, 1, 3, 15, 16, 17, 255, 1023, 1025, 65537, 262144 + 5])
@pytest.mark.parametrize("dtype", [orc.I8, orc.BF16, orc.F32])
def test_reduce_copy_ragged_lengths(n, dtype):
    srcs = [datagen.make(dtype, 3000 + r, max(n, 1))[:n] for r in range(2)]
    if n == 0:
        import dfccl_amd
        e = torch.empty(0, dtype=TORCH_OF[dtype], device=gpu_util.DEVICE)
        dfccl_amd.reduce_copy([e, e], e)  # a no-op, must not fault
        return
    got, _ = _run(dtype, orc.SUM, srcs, chunk_bytes=4096)
    assert np.array_equal(got, orc.reduce_copy(dtype, orc.SUM, srcs))


@pytest.mark.parametrize("offset", [1, 3, 7])
@pytest.mark.parametrize("dtype", [orc.I8, orc.F16, orc.I32])
def test_reduce_copy_misaligned_pointers(offset, dtype):
    # operands that are not 16-byte aligned take the element path
    n = 100000 + offset
    srcs = [datagen.make(dtype, 4000 + r, n) for r in range(2)]
    got, m = _run(dtype, orc.MIN, srcs, offset_elems=offset)
    want = orc.reduce_copy(dtype, orc.MIN, [s[offset:].copy() for s in srcs])
    assert m == n - offset and np.array_equal(got, want)


@pytest.mark.skipif(gpu_util.EMULATED, reason="256 MiB buffers are for the GPU")
def test_reduce_copy_full_size_linearity_property():
    # 256 MiB per buffer (the benchmark's size): too big for a bit-by-bit host check in
    # seconds, so check size-independent properties: int32 Sum equals torch's wrapped add,
    # and copy (k = 1) round-trips.
    import dfccl_amd
    n = (256 << 20) // 4
    g = torch.Generator(device="cuda:0").manual_seed(7)
    a = torch.randint(-(1 << 30), 1 << 30, (n,), dtype=torch.int32, device="cuda:0", generator=g)
    b = torch.randint(-(1 << 30), 1 << 30, (n,), dtype=torch.int32, device="cuda:0", generator=g)
    d = torch.empty_like(a)
    dfccl_amd.reduce_copy([a, b], d, dfccl_amd.ncclSum)
    torch.cuda.current_stream().synchronize()
    assert torch.equal(d, a + b)
    dfccl_amd.reduce_copy([a], d)
    torch.cuda.current_stream().synchronize()
    assert torch.equal(d, a)
    fa, fb = a.view(torch.float32).abs().clamp(max=1e30).nan_to_num(0.0), b.view(torch.float32).abs().clamp(max=1e30).nan_to_num(0.0)
    fd = torch.empty_like(fa)
    dfccl_amd.reduce_copy([fa, fb], fd, dfccl_amd.ncclMax)
    torch.cuda.current_stream().synchronize()
    assert torch.equal(fd, torch.maximum(fa, fb))


def test_reduce_copy_rejects_bad_arguments():
    import ctypes
    from dfccl_amd import _lib
    lib = _lib.load()
    a = torch.zeros(16, device=gpu_util.DEVICE)
    arr = (ctypes.c_void_p * 1)(a.data_ptr())
    assert lib.dfcclReduceCopy(arr, 1, a.data_ptr(), 16, 10, 0, 0, None) == 4  # no such datatype
    assert lib.dfcclReduceCopy(arr, 1, a.data_ptr(), 16, 7, 5, 0, None) == 4   # no such op (user operators belong to communicators)
    assert lib.dfcclReduceCopy(arr, 9, a.data_ptr(), 16, 7, 0, 0, None) == 4   # too many sources
    assert lib.dfcclReduceCopy(arr, 1, None, 16, 7, 0, 0, None) == 4
