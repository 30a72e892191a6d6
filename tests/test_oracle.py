"""Pins the CPU oracle against independent arithmetic (numpy float16, torch
bfloat16, two's-complement closed forms) and against a per-element closed form
of the ring accumulation order.  No GPU, no product code."""
import ctypes

import numpy as np
import pytest
import torch

import datagen
import dfccl_oracle as orc


# ---------------------------------------------------------------- soft float

def test_f16_decode_all_patterns_match_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    L = orc.lib()
    got = np.array([L.orc_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def _edge_floats():
    vals = [0.0, -0.0, 1.0, -1.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, 2.0 ** -14, 2.0 ** -24, 2.0 ** -25,
            2.0 ** -25 * 1.0000001, 2.0 ** -26, 6.1e-5, 5.96e-8, 3.0e-8, 2.98e-8, 1.00048828125, 1.000244140625,
            1.0009765625 + 2.0 ** -11, 0.33333334, 3.4e38, 1e-40, 2.0 ** -126]
    # exact ties between neighbouring halves / bfloat16s, both parities
    for k in range(1, 40):
        vals.append(1.0 + (2 * k + 1) * 2.0 ** -11)
        vals.append(1.0 + (2 * k + 1) * 2.0 ** -8)
        vals.append((2 * k + 1) * 2.0 ** -25)
    return np.array(vals + [-v for v in vals], dtype=np.float32)


def test_f32_to_f16_matches_numpy():
    x = np.concatenate([_edge_floats(), datagen.normal(11, 20000), datagen.normal(12, 20000, 1e-4),
                        datagen.normal(13, 20000, 3e4), datagen.normal(14, 5000, 1e-7)])
    want = x.astype(np.float16).view(np.uint16)
    L = orc.lib()
    got = np.array([L.orc_f32_to_f16(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_f32_to_bf16_matches_torch():
    x = np.concatenate([_edge_floats(), datagen.normal(21, 20000), datagen.normal(22, 20000, 1e-20),
                        datagen.normal(23, 20000, 1e30)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    L = orc.lib()
    got = np.array([L.orc_f32_to_bf16(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(orc.f32_to_bf16_bits(x), want)  # the numpy helper used by the tests


# ------------------------------------------------------------- element ops

def _two(dtype, n, seed, **kw):
    return datagen.make(dtype, seed, n, **kw), datagen.make(dtype, seed + 1, n, **kw)


@pytest.mark.parametrize("op", orc.OPS)
def test_fp16_ops_match_numpy_float16(op):
    a, b = _two(orc.F16, 50000, 31)
    fa, fb = a.view(np.float16), b.view(np.float16)
    with np.errstate(over="ignore"):
        want = {orc.SUM: fa + fb, orc.PROD: fa * fb, orc.MAX: np.maximum(fa, fb), orc.MIN: np.minimum(fa, fb)}[op]
    got = orc.reduce_copy(orc.F16, op, [a, b])
    assert np.array_equal(got, want.view(np.uint16))


@pytest.mark.parametrize("op", orc.OPS)
def test_bf16_ops_match_torch_bfloat16(op):
    a, b = _two(orc.BF16, 50000, 41)
    ta = torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)
    tb = torch.from_numpy(b.view(np.int16)).view(torch.bfloat16)
    want = {orc.SUM: ta + tb, orc.PROD: ta * tb, orc.MAX: torch.maximum(ta, tb), orc.MIN: torch.minimum(ta, tb)}[op]
    got = orc.reduce_copy(orc.BF16, op, [a, b])
    assert np.array_equal(got, want.view(torch.int16).numpy().view(np.uint16))


@pytest.mark.parametrize("op", orc.OPS)
def test_fp32_ops_match_numpy(op):
    a, b = _two(orc.F32, 50000, 51)
    want = {orc.SUM: a + b, orc.PROD: a * b, orc.MAX: np.maximum(a, b), orc.MIN: np.minimum(a, b)}[op]
    got = orc.reduce_copy(orc.F32, op, [a, b])
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("dtype,bits", [(orc.I8, 8), (orc.I32, 32)])
@pytest.mark.parametrize("op", orc.OPS)
def test_integer_ops_wrap_mod_2n(dtype, bits, op):
    a, b = _two(dtype, 50000, 61)
    if dtype == orc.I32:  # cover the whole 32-bit range so Sum/Prod really wrap
        a = (datagen.splitmix64(62, a.size) & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.int32)
        b = (datagen.splitmix64(63, a.size) & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.int32)
    A, B = a.astype(object), b.astype(object)  # exact Python integers
    if op == orc.SUM:
        exact = A + B
    elif op == orc.PROD:
        exact = A * B
    elif op == orc.MAX:
        exact = np.maximum(A, B)
    else:
        exact = np.minimum(A, B)
    m = 1 << bits
    want = np.array([((int(v) + m // 2) % m) - m // 2 for v in exact], dtype=a.dtype)
    got = orc.reduce_copy(dtype, op, [a, b])
    assert np.array_equal(got, want)


def test_reduce_copy_folds_left_to_right():
    # values chosen so that (a+b)+c != a+(b+c) in float32
    a = np.full(1000, 1e8, np.float32)
    b = np.full(1000, -1e8, np.float32)
    c = datagen.uniform(71, 1000)
    got = orc.reduce_copy(orc.F32, orc.SUM, [a, b, c])
    assert np.array_equal(got, c)                 # (a+b)+c == c exactly
    assert not np.array_equal((a + (b + c)), c)   # the other association differs
    # k = 1 is a copy; k = 4 matches a numpy fold with per-step rounding
    assert np.array_equal(orc.reduce_copy(orc.F32, orc.SUM, [c]), c)
    xs = [datagen.make(orc.BF16, 80 + i, 4097) for i in range(4)]
    acc = orc.bf16_bits_to_f32(xs[0])
    for x in xs[1:]:
        acc = orc.bf16_bits_to_f32(orc.f32_to_bf16_bits(acc + orc.bf16_bits_to_f32(x)))
    assert np.array_equal(orc.reduce_copy(orc.BF16, orc.SUM, xs), orc.f32_to_bf16_bits(acc))


def test_reduce_copy_mt_equals_single_thread():
    srcs = [datagen.make(orc.F32, 90 + i, 100003, kind="uniform") for i in range(3)]
    assert np.array_equal(orc.reduce_copy(orc.F32, orc.SUM, srcs, nthreads=1),
                          orc.reduce_copy(orc.F32, orc.SUM, srcs, nthreads=5))


# ------------------------------------------------------------ ring schedule

def np_op(dtype, op, a, b):
    """One reduction step on storage arrays with independent numpy/torch arithmetic."""
    if dtype in (orc.I8, orc.I32):
        with np.errstate(over="ignore"):
            return {orc.SUM: a + b, orc.PROD: a * b, orc.MAX: np.maximum(a, b), orc.MIN: np.minimum(a, b)}[op]
    if dtype == orc.F32:
        return {orc.SUM: a + b, orc.PROD: a * b, orc.MAX: np.maximum(a, b), orc.MIN: np.minimum(a, b)}[op]
    if dtype == orc.F16:
        fa, fb = a.view(np.float16), b.view(np.float16)
        with np.errstate(over="ignore"):
            r = {orc.SUM: fa + fb, orc.PROD: fa * fb, orc.MAX: np.maximum(fa, fb), orc.MIN: np.minimum(fa, fb)}[op]
        return r.view(np.uint16)
    fa, fb = orc.bf16_bits_to_f32(a), orc.bf16_bits_to_f32(b)
    r = {orc.SUM: fa + fb, orc.PROD: fa * fb, orc.MAX: np.maximum(fa, fb), orc.MIN: np.minimum(fa, fb)}[op]
    return orc.f32_to_bf16_bits(r)


def ring_order_reduce(dtype, op, sends, owner):
    """Closed form: the chunk owned by ring position c accumulates
    in[c+1], in[c+2], ..., in[c+n-1], and finally in[c]."""
    n = len(sends)
    out = np.empty_like(sends[0])
    for c in range(n):
        sel = owner == c
        if not sel.any():
            continue
        acc = sends[(c + 1) % n][sel]
        for j in range(2, n + 1):
            acc = np_op(dtype, op, sends[(c + j) % n][sel], acc)
        out[sel] = acc
    return out


def py_owner(n, C, chunk, align, count):
    """Owner ring position of every element, restated in numpy from the chunk geometry."""
    i = np.arange(count, dtype=np.int64)
    loop = C * n * chunk
    grid = (i // loop) * loop
    real = np.minimum(chunk, -(-(count - grid) // (C * n)))
    real = -(-real // align) * align
    rel = i - grid
    bid = rel // (n * real)
    return ((rel - bid * n * real) // real).astype(np.int64)


GEOMS = [  # n, C, chunk, align, count
    (2, 1, 64, 16, 1000), (3, 2, 64, 16, 1000), (4, 1, 128, 32, 37), (4, 3, 32, 8, 5000),
    (8, 2, 64, 64, 4096), (8, 4, 256, 64, 100003), (5, 1, 16, 16, 3), (2, 2, 512, 128, 513),
]


@pytest.mark.parametrize("n,C,chunk,align,count", GEOMS)
@pytest.mark.parametrize("dtype,op", [(orc.F32, orc.SUM), (orc.BF16, orc.SUM), (orc.F16, orc.SUM), (orc.F32, orc.PROD),
                                      (orc.I32, orc.SUM), (orc.I8, orc.MIN), (orc.F32, orc.MAX), (orc.BF16, orc.PROD)])
def test_all_reduce_matches_ring_order_closed_form(n, C, chunk, align, count, dtype, op):
    g = orc.Geom(n, C, chunk, align)
    sends = [datagen.make(dtype, 100 + r, count) for r in range(n)]
    recvs = orc.all_reduce(dtype, op, g, sends)
    owner = py_owner(n, C, chunk, align, count)
    assert all(orc.all_reduce_owner(g, count, int(i)) == owner[i] for i in range(0, count, max(1, count // 97)))
    want = ring_order_reduce(dtype, op, sends, owner)
    for r in range(n):
        assert np.array_equal(recvs[r], want), r


def test_all_reduce_order_is_observable_in_float():
    # the test above would not notice a wrong rank order if float addition were associative here
    n, count = 4, 4096
    g = orc.Geom(n, 1, 256, 64)
    sends = [datagen.make(orc.F32, 200 + r, count) for r in range(n)]
    got = orc.all_reduce(orc.F32, orc.SUM, g, sends)[0]
    natural = ((sends[0] + sends[1]) + sends[2]) + sends[3]
    assert not np.array_equal(got, natural)
    assert np.allclose(got, natural, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("n,C,chunk,align,count", GEOMS)
def test_all_reduce_in_place(n, C, chunk, align, count):
    g = orc.Geom(n, C, chunk, align)
    sends = [datagen.make(orc.I32, 300 + r, count) for r in range(n)]
    want = orc.all_reduce(orc.I32, orc.SUM, g, sends)
    bufs = [s.copy() for s in sends]
    ptrs = orc._ptrs(bufs)
    assert orc.lib().orc_all_reduce(orc.I32, orc.SUM, ctypes.byref(g), count, ptrs, ptrs) == 0
    for r in range(n):
        assert np.array_equal(bufs[r], want[r])
        assert np.array_equal(bufs[r], sum(s.astype(np.int64) for s in sends).astype(np.int32))


@pytest.mark.parametrize("n,C,chunk,align,count", GEOMS)
@pytest.mark.parametrize("dtype,op", [(orc.F32, orc.SUM), (orc.BF16, orc.SUM), (orc.I8, orc.SUM), (orc.F16, orc.MAX)])
def test_reduce_scatter_closed_form(n, C, chunk, align, count, dtype, op):
    g = orc.Geom(n, C, chunk, align)
    sends = [datagen.make(dtype, 400 + r, count * n) for r in range(n)]
    recvs = orc.reduce_scatter(dtype, op, g, sends)
    for d in range(n):  # block d starts at the ring successor of d and ends at d
        blocks = [s[d * count:(d + 1) * count] for s in sends]
        acc = blocks[(d + 1) % n]
        for j in range(2, n + 1):
            acc = np_op(dtype, op, blocks[(d + j) % n], acc)
        assert np.array_equal(recvs[d], acc), d


@pytest.mark.parametrize("n,C,chunk,align,count", GEOMS)
@pytest.mark.parametrize("dtype", [orc.I8, orc.F16, orc.F32])
def test_all_gather_is_concatenation(n, C, chunk, align, count, dtype):
    g = orc.Geom(n, C, chunk, align)
    sends = [datagen.make(dtype, 500 + r, count) for r in range(n)]
    recvs = orc.all_gather(dtype, g, sends)
    want = np.concatenate(sends)
    for r in range(n):
        assert np.array_equal(recvs[r], want)
    # in place: rank r's send buffer is its own slot of the receive buffer
    bufs = [np.zeros(count * n, dtype=sends[0].dtype) for _ in range(n)]
    for r in range(n):
        bufs[r][r * count:(r + 1) * count] = sends[r]
    sp = orc._ptrs([bufs[r][r * count:(r + 1) * count] for r in range(n)])
    assert orc.lib().orc_all_gather(dtype, ctypes.byref(g), count, sp, orc._ptrs(bufs)) == 0
    for r in range(n):
        assert np.array_equal(bufs[r], want)


@pytest.mark.parametrize("n,C,chunk,align,count", GEOMS)
@pytest.mark.parametrize("dtype,op", [(orc.F32, orc.SUM), (orc.BF16, orc.SUM), (orc.I32, orc.PROD)])
def test_reduce_chain_closed_form(n, C, chunk, align, count, dtype, op):
    g = orc.Geom(n, C, chunk, align)
    for root in {0, n - 1, n // 2}:
        sends = [datagen.make(dtype, 600 + r, count, small_ints=True) for r in range(n)]
        recvs = orc.reduce(dtype, op, g, root, sends)
        acc = sends[(root + 1) % n]
        for j in range(2, n + 1):
            acc = np_op(dtype, op, sends[(root + j) % n], acc)
        assert np.array_equal(recvs[root], acc)
        for r in range(n):
            if r != root:
                assert not recvs[r].any()  # non-root receive buffers are untouched


@pytest.mark.parametrize("n,C,chunk,align,count", GEOMS)
def test_broadcast_copies_root(n, C, chunk, align, count):
    g = orc.Geom(n, C, chunk, align)
    for root in {0, n - 1}:
        sends = [datagen.make(orc.F16, 700 + r, count) for r in range(n)]
        recvs = orc.broadcast(orc.F16, g, root, sends)
        for r in range(n):
            assert np.array_equal(recvs[r], sends[root])


def test_real_chunk_formula():
    L = orc.lib()
    assert L.orc_real_chunk(1048576, 33554432, 8 * 4, 512) == 1048576
    assert L.orc_real_chunk(1048576, 2048, 4, 512) == 512
    assert L.orc_real_chunk(1048576, 2049, 4, 512) == 1024
    assert L.orc_real_chunk(64, 1, 8, 16) == 16


# ------------------------------------------------------------------ queues

def test_cqe_slot_encoding_round_trip():
    L = orc.lib()
    for blk, cnt, coll in [(0, 0, 0), (255, 0xFFFFFF, 1999), (7, 123456, 42), (31, 1, 0xFFFFFFFF)]:
        v = L.orc_cqe_encode(blk, cnt, coll)
        assert v == (blk << 56) | (cnt << 32) | coll
        b, c, i = ctypes.c_uint(), ctypes.c_uint(), ctypes.c_uint()
        L.orc_cqe_decode(v, ctypes.byref(b), ctypes.byref(c), ctypes.byref(i))
        assert (b.value, c.value, i.value) == (blk, cnt, coll)
    assert L.orc_cqe_encode(255, 0xFFFFFF, 0xFFFFFFFF) == 0xFFFFFFFFFFFFFFFF  # the "empty slot" value is reserved
    assert L.orc_cqe_encode(0, 0x1000000, 5) == 5  # the count wraps at 24 bits


def test_sq_ring_model():
    L = orc.lib()
    length = 5  # capacity 4
    head = tail = 0
    assert L.orc_sq_empty(head, tail)
    for _ in range(4):
        assert not L.orc_sq_full(head, tail, length)
        tail += 1
    assert L.orc_sq_full(head, tail, length)
    head += 1
    assert not L.orc_sq_full(head, tail, length)
    assert not L.orc_sq_empty(head, tail)
