"""Pins the oracle's remaining element types (uint8, uint32, int64, uint64, fp64), its scaled sums (ncclAvg:
SumPostDiv on integers, PreMulSum on floats; PreMulSum with a caller's scalar) and the NaN rule of Max / Min
against independent arithmetic: exact Python integers, numpy float64 / float32 / float16, torch bfloat16."""
import numpy as np
import pytest
import torch

import datagen
import dfccl_oracle as orc
from test_oracle import GEOMS, py_owner

INT_BITS = {orc.I8: (8, True), orc.U8: (8, False), orc.I32: (32, True), orc.U32: (32, False), orc.I64: (64, True),
            orc.U64: (64, False)}


def wrap(v, bits, signed):
    m = 1 << bits
    v %= m
    return v - m if signed and v >= m // 2 else v


@pytest.mark.parametrize("dtype", [orc.U8, orc.U32, orc.I64, orc.U64])
@pytest.mark.parametrize("op", orc.OPS)
def test_remaining_integer_types_match_python_integers(dtype, op):
    bits, signed = INT_BITS[dtype]
    a, b = datagen.make(dtype, 61, 20000), datagen.make(dtype, 62, 20000)
    f = {orc.SUM: lambda x, y: x + y, orc.PROD: lambda x, y: x * y, orc.MAX: max, orc.MIN: min}[op]
    want = np.array([wrap(f(int(x), int(y)), bits, signed) for x, y in zip(a, b)], dtype=a.dtype)
    assert np.array_equal(orc.reduce_copy(dtype, op, [a, b]), want)


@pytest.mark.parametrize("op", orc.OPS)
def test_fp64_ops_match_numpy(op):
    a, b = datagen.make(orc.F64, 71, 50000), datagen.make(orc.F64, 72, 50000, sigma=1e-3)
    want = {orc.SUM: a + b, orc.PROD: a * b, orc.MAX: np.fmax(a, b), orc.MIN: np.fmin(a, b)}[op]
    assert np.array_equal(orc.reduce_copy(orc.F64, op, [a, b]).view(np.uint64), want.view(np.uint64))
    # three sources fold left to right
    c = datagen.make(orc.F64, 73, 50000, sigma=1e6)
    want3 = {orc.SUM: (a + b) + c, orc.PROD: (a * b) * c, orc.MAX: np.fmax(np.fmax(a, b), c),
             orc.MIN: np.fmin(np.fmin(a, b), c)}[op]
    assert np.array_equal(orc.reduce_copy(orc.F64, op, [a, b, c]).view(np.uint64), want3.view(np.uint64))


# ---- ncclAvg on integers: the wrapped sum, then C++'s truncating division by the group size ----------------

def c_div(x, n):
    q = abs(x) // n
    return q if x >= 0 else -q


@pytest.mark.parametrize("dtype", list(INT_BITS))
@pytest.mark.parametrize("k", [2, 3, 7])
def test_avg_of_integers_is_wrapped_sum_then_truncating_division(dtype, k):
    bits, signed = INT_BITS[dtype]
    srcs = [datagen.make(dtype, 80 + i, 5000) for i in range(k)]
    want = np.array([wrap(c_div(wrap(sum(int(s[i]) for s in srcs), bits, signed), k), bits, signed)
                     for i in range(5000)], dtype=srcs[0].dtype)
    assert np.array_equal(orc.reduce_copy(dtype, orc.AVG, srcs), want)
    assert orc.avg_scalar(dtype, k) == k


def test_avg_of_negative_sums_truncates_towards_zero():
    srcs = [np.array([-7, -1, 5, -128], np.int8), np.array([0, 0, 0, -128], np.int8), np.array([0, -1, 0, 0], np.int8)]
    # sums -7, -2, 5, and -256 wrapped to 0; divided by 3 towards zero
    assert orc.reduce_copy(orc.I8, orc.AVG, srcs).tolist() == [-2, 0, 1, 0]


# ---- PreMulSum / ncclAvg on floats: every input times the scalar (one rounding in the type), then the sum ----

def np_mul(dtype, a, scalar_bits):
    """a * scalar in the storage type, by numpy / torch arithmetic."""
    if dtype == orc.F64:
        return a * np.array([scalar_bits], np.uint64).view(np.float64)[0]
    if dtype == orc.F32:
        return a * np.array([scalar_bits], np.uint32).view(np.float32)[0]
    if dtype == orc.F16:
        with np.errstate(over="ignore"):
            return (a.view(np.float16) * np.array([scalar_bits], np.uint16).view(np.float16)[0]).view(np.uint16)
    ta = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    ts = torch.from_numpy(np.array([scalar_bits], np.uint16).view(np.int16)).view(torch.bfloat16)
    return (ta * ts).view(torch.int16).numpy().view(np.uint16)


def np_add(dtype, a, b):
    if dtype in (orc.F64, orc.F32):
        return a + b
    if dtype == orc.F16:
        with np.errstate(over="ignore"):
            return (a.view(np.float16) + b.view(np.float16)).view(np.uint16)
    ta = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    tb = torch.from_numpy(b.view(np.int16).copy()).view(torch.bfloat16)
    return (ta + tb).view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("dtype", orc.FLOAT_DTYPES)
def test_avg_scalar_of_floats_is_one_over_n_in_the_type(dtype):
    for n in (2, 3, 4, 7, 8):
        bits = orc.avg_scalar(dtype, n)
        if dtype == orc.F64:
            assert bits == int(np.array([1.0 / n]).view(np.uint64)[0])
        elif dtype == orc.F32:
            assert bits == int(np.array([np.float32(1.0 / n)]).view(np.uint32)[0])
        elif dtype == orc.F16:
            assert bits == int(np.array([np.float32(1.0 / n)]).astype(np.float16).view(np.uint16)[0])
        else:
            assert bits == int(torch.tensor([1.0 / n], dtype=torch.float32).to(torch.bfloat16).view(torch.int16)[0]) & 0xffff


@pytest.mark.parametrize("dtype", orc.FLOAT_DTYPES)
@pytest.mark.parametrize("n,C,chunk,align,count", GEOMS[:6])
def test_avg_all_reduce_of_floats_scales_inputs_then_sums_in_ring_order(dtype, n, C, chunk, align, count):
    g = orc.Geom(n, C, chunk, align)
    sends = [datagen.make(dtype, 900 + r, count) for r in range(n)]
    scaled = [np_mul(dtype, s, orc.avg_scalar(dtype, n)) for s in sends]
    owner = py_owner(n, C, chunk, align, count)
    want = np.empty_like(sends[0])
    for c in range(n):
        sel = owner == c
        acc = scaled[(c + 1) % n][sel]
        for j in range(2, n + 1):
            acc = np_add(dtype, scaled[(c + j) % n][sel], acc)
        want[sel] = acc
    for got in orc.all_reduce(dtype, orc.AVG, g, sends):
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    # the same through PREMULSUM with the scalar given explicitly
    for got in orc.all_reduce(dtype, orc.PREMULSUM, g, sends, scalar=orc.avg_scalar(dtype, n)):
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


@pytest.mark.parametrize("dtype", list(INT_BITS))
@pytest.mark.parametrize("n,C,chunk,align,count", GEOMS[:6])
def test_avg_ring_collectives_of_integers(dtype, n, C, chunk, align, count):
    bits, signed = INT_BITS[dtype]
    g = orc.Geom(n, C, chunk, align)
    sends = [datagen.make(dtype, 950 + r, count * n) for r in range(n)]
    exact = [wrap(c_div(wrap(sum(int(s[i]) for s in sends), bits, signed), n), bits, signed) for i in range(count * n)]
    want = np.array(exact, dtype=sends[0].dtype)
    for got in orc.all_reduce(dtype, orc.AVG, g, sends):
        assert np.array_equal(got, want)
    for r, got in enumerate(orc.reduce_scatter(dtype, orc.AVG, g, sends)):
        assert np.array_equal(got, want[r * count:(r + 1) * count])
    root = n - 1
    assert np.array_equal(orc.reduce(dtype, orc.AVG, g, root, sends)[root], want)


def test_premulsum_of_integers_multiplies_with_wrap():
    srcs = [datagen.make(orc.I32, 990 + i, 3000) for i in range(3)]
    k = 1_000_003
    want = np.array([wrap(sum(wrap(int(s[i]) * k, 32, True) for s in srcs), 32, True) for i in range(3000)], np.int32)
    assert np.array_equal(orc.reduce_copy(orc.I32, orc.PREMULSUM, srcs, scalar=orc.scalar_bits(orc.I32, k)), want)


def test_reduce_scatter_and_reduce_premulsum_floats():
    n, C, chunk, align, count = 4, 2, 64, 16, 1000
    g = orc.Geom(n, C, chunk, align)
    s = orc.scalar_bits(orc.F32, 0.3)
    sends = [datagen.make(orc.F32, 1000 + r, count * n) for r in range(n)]
    scaled = [np_mul(orc.F32, x, s) for x in sends]
    for d, got in enumerate(orc.reduce_scatter(orc.F32, orc.PREMULSUM, g, sends, scalar=s)):
        blocks = [x[d * count:(d + 1) * count] for x in scaled]
        acc = blocks[(d + 1) % n]
        for j in range(2, n + 1):
            acc = blocks[(d + j) % n] + acc
        assert np.array_equal(got, acc)
    root = 1
    acc = scaled[(root + 1) % n]
    for j in range(2, n + 1):
        acc = scaled[(root + j) % n] + acc
    assert np.array_equal(orc.reduce(orc.F32, orc.PREMULSUM, g, root, sends, scalar=s)[root], acc)


# ---- PreMulSum with every rank's own scalar: input r enters the sum multiplied by rank r's scalar ------------
# (every rank makes its own operator, src/enqueue.cc:1443-1475, and applies it to the input it reads itself,
# src/collectives_ofccl/device/ofccl_prims_simple.h:405-411)

PER_RANK_VALUES = [0.5, -1.25, 3.0, 0.0625, 1.5, -0.75, 2.0, 0.3]


@pytest.mark.parametrize("dtype", orc.FLOAT_DTYPES)
@pytest.mark.parametrize("n,C,chunk,align,count", GEOMS[:6])
def test_premulsum_all_reduce_with_a_scalar_per_rank(dtype, n, C, chunk, align, count):
    g = orc.Geom(n, C, chunk, align)
    sends = [datagen.make(dtype, 1100 + r, count) for r in range(n)]
    scalars = [orc.scalar_bits(dtype, PER_RANK_VALUES[r % 8] * (1 + r // 8)) for r in range(n)]
    assert len(set(scalars)) == n  # all different: a scalar applied to the wrong rank's input would be noticed
    scaled = [np_mul(dtype, sends[r], scalars[r]) for r in range(n)]
    owner = py_owner(n, C, chunk, align, count)
    want = np.empty_like(sends[0])
    for c in range(n):
        sel = owner == c
        acc = scaled[(c + 1) % n][sel]
        for j in range(2, n + 1):
            acc = np_add(dtype, scaled[(c + j) % n][sel], acc)
        want[sel] = acc
    for got in orc.all_reduce(dtype, orc.PREMULSUM, g, sends, scalar=scalars):
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    # rotating the scalars by one rank gives something else
    rotated = scalars[1:] + scalars[:1]
    assert not np.array_equal(orc.all_reduce(dtype, orc.PREMULSUM, g, sends, scalar=rotated)[0].view(np.uint8),
                              want.view(np.uint8))


def test_premulsum_per_rank_scalars_integers_reduce_scatter_and_reduce():
    n, C, chunk, align, count = 3, 2, 64, 16, 500
    g = orc.Geom(n, C, chunk, align)
    ks = [7, -3, 1_000_003]
    sends = [datagen.make(orc.I32, 1200 + r, count * n) for r in range(n)]
    exact = np.array([wrap(sum(wrap(int(sends[r][i]) * ks[r], 32, True) for r in range(n)), 32, True)
                      for i in range(count * n)], np.int32)
    scalars = [orc.scalar_bits(orc.I32, k) for k in ks]
    for r, got in enumerate(orc.reduce_scatter(orc.I32, orc.PREMULSUM, g, sends, scalar=scalars)):
        assert np.array_equal(got, exact[r * count:(r + 1) * count])
    root = 2
    assert np.array_equal(orc.reduce(orc.I32, orc.PREMULSUM, g, root, sends, scalar=scalars)[root], exact)
    for got in orc.all_reduce(orc.I32, orc.PREMULSUM, g, sends, scalar=scalars):
        assert np.array_equal(got, exact)


def test_premulsum_per_rank_scalars_floats_reduce_scatter_and_reduce():
    n, C, chunk, align, count = 4, 2, 64, 16, 1000
    g = orc.Geom(n, C, chunk, align)
    scalars = [orc.scalar_bits(orc.F32, v) for v in (0.3, -1.7, 2.5, 0.01)]
    sends = [datagen.make(orc.F32, 1300 + r, count * n) for r in range(n)]
    scaled = [np_mul(orc.F32, sends[r], scalars[r]) for r in range(n)]
    for d, got in enumerate(orc.reduce_scatter(orc.F32, orc.PREMULSUM, g, sends, scalar=scalars)):
        blocks = [x[d * count:(d + 1) * count] for x in scaled]
        acc = blocks[(d + 1) % n]
        for j in range(2, n + 1):
            acc = blocks[(d + j) % n] + acc
        assert np.array_equal(got, acc)
    root = 1
    acc = scaled[(root + 1) % n]
    for j in range(2, n + 1):
        acc = scaled[(root + j) % n] + acc
    assert np.array_equal(orc.reduce(orc.F32, orc.PREMULSUM, g, root, sends, scalar=scalars)[root], acc)


# ---- Max / Min with NaN operands: fmaxf / fminf return the operand that is a number -------------------------
# (src/include/reduce_kernel.h:442-469; fp16 goes through float, :344-362,393-411).  A NaN comes out only where
# every operand is a NaN.  Which of two zeros of different sign comes out is not fixed by fmax / fmin and stays
# unpinned.

def _with_nans(dtype, seed, n, every):
    x = datagen.make(dtype, seed, n)
    nan = {orc.F16: 0x7e00, orc.BF16: 0x7fc0}.get(dtype)
    if nan is None:
        x[::every] = np.nan
    else:
        x[::every] = nan
    return x


def _is_nan(dtype, x):
    if dtype == orc.F16:
        return np.isnan(x.view(np.float16))
    if dtype == orc.BF16:
        return np.isnan(orc.bf16_bits_to_f32(x))
    return np.isnan(x)


@pytest.mark.parametrize("dtype", orc.FLOAT_DTYPES)
@pytest.mark.parametrize("op", [orc.MAX, orc.MIN])
def test_max_min_return_the_operand_that_is_a_number(dtype, op):
    n = 6000
    a, b, c = _with_nans(dtype, 1, n, 3), _with_nans(dtype, 2, n, 4), _with_nans(dtype, 3, n, 6)
    clean = [datagen.make(dtype, s, n) for s in (1, 2, 3)]
    got = orc.reduce_copy(dtype, op, [a, b, c])
    nan_a, nan_b, nan_c = _is_nan(dtype, a), _is_nan(dtype, b), _is_nan(dtype, c)
    all_nan = nan_a & nan_b & nan_c
    assert all_nan.any() and (~all_nan).any()
    assert np.array_equal(_is_nan(dtype, got), all_nan)
    # expected: the extreme over the operands that are numbers, computed on float64 copies
    def f64(dtype, x):
        if dtype == orc.F16:
            return x.view(np.float16).astype(np.float64)
        if dtype == orc.BF16:
            return orc.bf16_bits_to_f32(x).astype(np.float64)
        return x.astype(np.float64)
    fill = -np.inf if op == orc.MAX else np.inf
    vals = np.stack([np.where(m, fill, f64(dtype, x)) for m, x in ((nan_a, clean[0]), (nan_b, clean[1]), (nan_c, clean[2]))])
    want = vals.max(0) if op == orc.MAX else vals.min(0)
    ok = ~all_nan
    assert np.array_equal(f64(dtype, got)[ok], want[ok])
