"""Parity of the collectives run through the daemon kernel (ofccl C ABI) against
the CPU oracle, plus the scheduler's invariants: preemption and resume are
bit-exact, out-of-order submission completes, the kernel leaves when idle and is
relaunched, contexts can be destroyed and recreated.

Bit-exact everywhere: integer ops by nature, float ops because the oracle
reproduces the ring's per-chunk rank order from the geometry the library reports."""
import os
import threading
import time

import numpy as np
import pytest
import torch

import datagen
import dfccl_oracle as orc
import gpu_util
from gpu_util import TORCH_OF, geom_of, to_gpu, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["direct", "fifo"])
def proto(request, monkeypatch):
    """Every test runs under both data protocols: `direct` (up to 8 ranks read and write each other's buffers in
    place) and `fifo` (the reference's staged ring)."""
    monkeypatch.setenv("DFCCL_PROTO", request.param)
    # a daemon that would otherwise stay resident leaves (and is relaunched on demand) every 10 s
    monkeypatch.setenv("DFCCL_DAEMON_MAX_MS", "10000")
    yield request.param


def oracle_run(kind, dtype, op, g, root, sends):
    if kind == "all_reduce":
        return orc.all_reduce(dtype, op, g, sends)
    if kind == "reduce_scatter":
        return orc.reduce_scatter(dtype, op, g, sends)
    if kind == "all_gather":
        return orc.all_gather(dtype, g, sends)
    if kind == "reduce":
        return orc.reduce(dtype, op, g, root, sends)
    return orc.broadcast(dtype, g, root, sends)


def make_buffers(kind, dtype, n, count, seed, **kw):
    send_len = count * n if kind == "reduce_scatter" else count
    recv_len = count * n if kind == "all_gather" else count
    sends_np = [datagen.make(dtype, seed + r, send_len, **kw) for r in range(n)]
    sends = [to_gpu(dtype, s) for s in sends_np]
    recvs = [torch.zeros(recv_len, dtype=TORCH_OF[dtype], device=gpu_util.DEVICE) for _ in range(n)]
    torch.cuda.current_stream().synchronize()
    return sends_np, sends, recvs


def check(kind, dtype, op, n, count, root=0, seed=100, reps=1, **kw):
    from dfccl_amd.ring import VirtualRing
    with VirtualRing(n) as ring:
        ring.prepare(0, kind, count, dtype, op, root)
        ring.finalize()
        want_proto = 1 if (os.environ.get("DFCCL_PROTO") == "direct" and 2 <= n <= 8) else 0
        assert ring.ctxs[0].geometry(0).protocol == want_proto
        sends_np, sends, recvs = make_buffers(kind, dtype, n, count, seed, **kw)
        want = oracle_run(kind, dtype, op, geom_of(ring, 0), root, sends_np)
        for _ in range(reps):
            ring.run(0, sends, recvs, timeout=30)
            for r in range(n):
                if kind == "reduce" and r != root:
                    continue
                assert np.array_equal(to_np(dtype, recvs[r]), want[r]), f"rank {r}"
            for t in recvs:
                t.zero_()
            torch.cuda.current_stream().synchronize()
        return ring.stats()


@pytest.mark.parametrize("n", [2, 3, 4, 8])
@pytest.mark.parametrize("count", [1, 37, 2048, 100003, 1 << 20])
def test_all_reduce_fp32_sum_sizes_and_ranks(n, count):
    check("all_reduce", orc.F32, orc.SUM, n, count, reps=2)


@pytest.mark.parametrize("dtype", orc.ALL_DTYPES)
@pytest.mark.parametrize("op", orc.OPS + (orc.AVG,))
def test_all_reduce_every_dtype_and_op(dtype, op):
    # the whole ncclDataType_t x {Sum, Prod, Max, Min, Avg} table; Avg is a sum divided afterwards (integers) or
    # of inputs multiplied by 1/4 first (floats)
    check("all_reduce", dtype, op, 4, 300001, small_ints=(op == orc.PROD), seed=200 + dtype)


@pytest.mark.parametrize("dtype", orc.FLOAT_DTYPES)
@pytest.mark.parametrize("op", [orc.MAX, orc.MIN])
def test_all_reduce_max_min_with_nan_operands(dtype, op):
    # fmaxf / fminf semantics (src/include/reduce_kernel.h:344-362,442-469): the operand that is a number wins;
    # NaN only where all four ranks hold one.  The values are compared where the oracle's result is a number.
    from dfccl_amd.ring import VirtualRing
    n, count = 4, 40000
    nan_bits = {orc.F16: 0x7e00, orc.BF16: 0x7fc0}.get(dtype, np.nan)

    def is_nan(x):
        if dtype == orc.F16:
            return np.isnan(x.view(np.float16))
        if dtype == orc.BF16:
            return np.isnan(orc.bf16_bits_to_f32(x))
        return np.isnan(x)

    with VirtualRing(n) as ring:
        ring.prepare(0, "all_reduce", count, dtype, op)
        ring.finalize()
        sends_np = [datagen.make(dtype, 700 + r, count) for r in range(n)]
        for x, every in zip(sends_np, (2, 3, 4, 6)):
            x[::every] = nan_bits
        sends = [to_gpu(dtype, x) for x in sends_np]
        recvs = [torch.zeros(count, dtype=TORCH_OF[dtype], device=gpu_util.DEVICE) for _ in range(n)]
        torch.cuda.current_stream().synchronize()
        want = orc.all_reduce(dtype, op, geom_of(ring, 0), sends_np)
        ring.run(0, sends, recvs, timeout=30)
        nan = is_nan(want[0])
        assert nan[::12].all() and not nan[1::12].any()
        for r in range(n):
            got = to_np(dtype, recvs[r])
            assert np.array_equal(is_nan(got), nan), r
            assert np.array_equal(got[~nan], want[r][~nan]), r


@pytest.mark.parametrize("kind", ["reduce_scatter", "reduce"])
@pytest.mark.parametrize("dtype", [orc.U8, orc.I64, orc.F64, orc.BF16, orc.F16])
def test_avg_on_the_other_reducing_collectives(kind, dtype):
    check(kind, dtype, orc.AVG, 3, 50021, root=2, seed=250 + dtype)


@pytest.mark.parametrize("n,count", [(2, 1000), (8, 4099), (5, 100000)])
def test_avg_small_and_ragged(n, count):
    # 2 and 8 ranks on sizes that wave 0 folds alone, 5 ranks on 7 (odd) bytes per element boundary cases
    check("all_reduce", orc.F32, orc.AVG, n, count, seed=260)
    check("all_reduce", orc.I8, orc.AVG, n, count, seed=261)


PREMUL_VALUES = {orc.F32: [0.3, -1.7, 2.5, 0.01, 1.0, -0.5, 3.25, 0.125], orc.BF16: [-1.5, 0.5, 2.0, -0.25, 1.0, 3.0, -2.0, 0.75],
                 orc.F64: [1e-3, -2.5, 0.3, 7.0, 1.0, -1.0, 0.5, 2.0], orc.F16: [0.5, -1.25, 2.0, 0.1, 1.0, -3.0, 0.25, 1.5],
                 orc.I32: [1000003, -3, 7, 2, 1, -1, 5, 11], orc.U8: [3, 2, 5, 1, 7, 4, 6, 9],
                 orc.I64: [-1000000007, 3, 2, 5, 1, -1, 7, 11]}


def scalar_bytes_of(dtype, value):
    return int(orc.scalar_bits(dtype, value)).to_bytes(8, "little")[:orc.TYPE_SIZE[dtype]]


@pytest.mark.parametrize("per_rank", [False, True], ids=["one-scalar", "scalar-per-rank"])
@pytest.mark.parametrize("dtype", [orc.F32, orc.BF16, orc.F64, orc.I32, orc.U8])
def test_premul_sum_operator(dtype, per_rank):
    # operators made by ncclRedOpCreatePreMulSum, one per rank: every rank's input times that rank's scalar (one
    # rounding in the type), summed in the ring's order; all three reducing collectives
    from dfccl_amd.ring import VirtualRing
    n, count, root = 4, (9001 if gpu_util.EMULATED else 70001), 2
    values = PREMUL_VALUES[dtype][:n] if per_rank else [PREMUL_VALUES[dtype][0]] * n
    bits = [orc.scalar_bits(dtype, v) for v in values]
    premul = [scalar_bytes_of(dtype, v) for v in values]
    with VirtualRing(n) as ring:
        ring.prepare(0, "all_reduce", count, dtype, premul=premul)
        ring.prepare(1, "reduce_scatter", count // n, dtype, premul=premul)
        ring.prepare(2, "reduce", count, dtype, root=root, premul=premul)
        ring.finalize()
        sends_np, sends, recvs = make_buffers("all_reduce", dtype, n, count, 270)
        want = orc.all_reduce(dtype, orc.PREMULSUM, geom_of(ring, 0), sends_np, scalar=bits)
        ring.run(0, sends, recvs, timeout=30)
        for r in range(n):
            assert np.array_equal(to_np(dtype, recvs[r]), want[r]), r
        rs_np, rs_send, rs_recv = make_buffers("reduce_scatter", dtype, n, count // n, 280)
        want = orc.reduce_scatter(dtype, orc.PREMULSUM, geom_of(ring, 1), rs_np, scalar=bits)
        ring.run(1, rs_send, rs_recv, timeout=30)
        for r in range(n):
            assert np.array_equal(to_np(dtype, rs_recv[r]), want[r]), r
        rd_np, rd_send, rd_recv = make_buffers("reduce", dtype, n, count, 290)
        want = orc.reduce(dtype, orc.PREMULSUM, geom_of(ring, 2), root, rd_np, scalar=bits)
        ring.run(2, rd_send, rd_recv, timeout=30)
        assert np.array_equal(to_np(dtype, rd_recv[root]), want[root])


@pytest.mark.parametrize("n,count", [(2, 1000), (8, 4099), (3, 200003), (10, 5003)])
def test_premul_sum_scalar_per_rank_small_and_large(n, count):
    # sizes that wave 0 folds alone (2 and 8 ranks), one that takes several channels, and more ranks than the direct
    # protocol folds in one pass (the FIFO ring then, whatever protocol was asked for)
    from dfccl_amd.ring import VirtualRing
    if gpu_util.EMULATED:
        count = min(count, 40003)
    for dtype in (orc.F16, orc.I64):
        values = [PREMUL_VALUES[dtype][r % 8] * (1 + r // 8) for r in range(n)]
        bits = [orc.scalar_bits(dtype, v) for v in values]
        with VirtualRing(n) as ring:
            ring.prepare(0, "all_reduce", count, dtype, premul=[scalar_bytes_of(dtype, v) for v in values])
            ring.finalize()
            sends_np, sends, recvs = make_buffers("all_reduce", dtype, n, count, 275)
            want = orc.all_reduce(dtype, orc.PREMULSUM, geom_of(ring, 0), sends_np, scalar=bits)
            for rep in range(2):
                ring.run(0, sends, recvs, timeout=30)
                for r in range(n):
                    assert np.array_equal(to_np(dtype, recvs[r]), want[r]), (dtype, rep, r)


@pytest.mark.parametrize("dtype", [orc.F32, orc.BF16, orc.I32, orc.F64, orc.U8])
def test_premul_sum_scalar_in_device_memory(dtype):
    # ncclScalarDevice: every rank's scalar lives in device memory and is read whenever an instance starts, so a
    # value written between two runs takes effect with the second (src/collectives/device/common.h:117-136)
    from dfccl_amd.ring import VirtualRing
    n, count = 4, 30011
    es = orc.TYPE_SIZE[dtype]
    first, second = PREMUL_VALUES[dtype][:n], PREMUL_VALUES[dtype][n:2 * n]
    # one element of the type per rank, 16 bytes apart
    slots = torch.zeros(n * 16, dtype=torch.uint8, device=gpu_util.DEVICE)

    def write(values):
        host = np.zeros(n * 16, np.uint8)
        for r, v in enumerate(values):
            host[r * 16:r * 16 + es] = np.frombuffer(scalar_bytes_of(dtype, v), np.uint8)
        slots.copy_(torch.from_numpy(host))
        torch.cuda.current_stream().synchronize()

    write(first)
    with VirtualRing(n) as ring:
        ring.prepare(0, "all_reduce", count, dtype, premul_device=[slots.data_ptr() + 16 * r for r in range(n)])
        ring.prepare(1, "reduce_scatter", count // n, dtype,
                     premul_device=[slots.data_ptr() + 16 * r for r in range(n)])
        ring.finalize()
        sends_np, sends, recvs = make_buffers("all_reduce", dtype, n, count, 295)
        rs_np, rs_send, rs_recv = make_buffers("reduce_scatter", dtype, n, count // n, 296)
        for values in (first, second):
            write(values)
            bits = [orc.scalar_bits(dtype, v) for v in values]
            want = orc.all_reduce(dtype, orc.PREMULSUM, geom_of(ring, 0), sends_np, scalar=bits)
            ring.run(0, sends, recvs, timeout=30)
            for r in range(n):
                assert np.array_equal(to_np(dtype, recvs[r]), want[r]), r
            want = orc.reduce_scatter(dtype, orc.PREMULSUM, geom_of(ring, 1), rs_np, scalar=bits)
            ring.run(1, rs_send, rs_recv, timeout=30)
            for r in range(n):
                assert np.array_equal(to_np(dtype, rs_recv[r]), want[r]), r


def test_premul_sum_ranks_mix_host_and_device_scalars():
    # even ranks give their scalar by value, odd ranks leave it in device memory
    import dfccl_amd
    from dfccl_amd import api
    from dfccl_amd.ring import VirtualRing
    dtype, n, count = orc.F32, 4, 20011
    values = PREMUL_VALUES[dtype][:n]
    slots = torch.zeros(n * 4, dtype=torch.float32, device=gpu_util.DEVICE)
    slots.copy_(torch.tensor([v for v in values for _ in range(4)], dtype=torch.float32))
    torch.cuda.current_stream().synchronize()
    with VirtualRing(n) as ring:
        comms = api.VirtualComm.create_all(n)
        for r, ctx in enumerate(ring.ctxs):
            if r % 2 == 0:
                op = comms[r].create_premul_sum(dtype, scalar_bytes_of(dtype, values[r]))
            else:
                op = comms[r].create_premul_sum(dtype, device_ptr=slots.data_ptr() + 16 * r)
            ctx.prepare_all_reduce(count, dtype, op, comms[r], 0)
            ring.done[(r, 0)] = threading.Event()
        ring.comms[0] = comms
        ring.kinds[0] = "all_reduce"
        ring.finalize()
        sends_np, sends, recvs = make_buffers("all_reduce", dtype, n, count, 298)
        want = orc.all_reduce(dtype, orc.PREMULSUM, geom_of(ring, 0), sends_np,
                              scalar=[orc.scalar_bits(dtype, v) for v in values])
        for rep in range(2):
            ring.run(0, sends, recvs, timeout=30)
            for r in range(n):
                assert np.array_equal(to_np(dtype, recvs[r]), want[r]), (rep, r)


def test_premul_sum_on_a_communicator_of_one_rank():
    # a sum of one term is still multiplied, out of place and in place
    from dfccl_amd.ring import VirtualRing
    dtype, count = orc.F32, 5003
    bits = orc.scalar_bits(dtype, 0.3)
    with VirtualRing(1) as ring:
        ring.prepare(0, "all_reduce", count, dtype, premul=scalar_bytes_of(dtype, 0.3))
        ring.finalize()
        sends_np, sends, recvs = make_buffers("all_reduce", dtype, 1, count, 297)
        want = orc.all_reduce(dtype, orc.PREMULSUM, geom_of(ring, 0), sends_np, scalar=bits)
        ring.run(0, sends, recvs, timeout=30)
        assert np.array_equal(to_np(dtype, recvs[0]), want[0])
        ring.run(0, sends, sends, timeout=30)
        assert np.array_equal(to_np(dtype, sends[0]), want[0])


def test_premul_sum_operator_errors():
    import dfccl_amd
    from dfccl_amd import api
    comms = api.VirtualComm.create_all(2)
    ctxs = [api.RankCtx(r) for r in range(2)]
    try:
        half = np.array([0.5], np.float32).tobytes()
        op0 = comms[0].create_premul_sum(dfccl_amd.ncclFloat32, half)
        assert op0 >= 5
        # an operator is tied to its datatype
        with pytest.raises(api.NcclError) as e:
            ctxs[0].prepare_all_reduce(100, dfccl_amd.ncclFloat16, op0, comms[0], 0)
        assert e.value.code == 4
        # an unknown operator value
        with pytest.raises(api.NcclError):
            ctxs[0].prepare_all_reduce(100, dfccl_amd.ncclFloat32, op0 + 17, comms[0], 0)
        ctxs[0].prepare_all_reduce(100, dfccl_amd.ncclFloat32, op0, comms[0], 0)
        # the ranks of a communicator have to agree on the kind of operator (a scalar of their own is fine) ...
        with pytest.raises(api.NcclError) as e:
            ctxs[1].prepare_all_reduce(100, dfccl_amd.ncclFloat32, dfccl_amd.ncclSum, comms[1], 0)
        assert e.value.code == 4
        # ... and a scalar in device memory has to be aligned to its type
        with pytest.raises(api.NcclError) as e:
            comms[1].create_premul_sum(dfccl_amd.ncclFloat32, device_ptr=0x7f0000000002)
        assert e.value.code == 4
        op1 = comms[1].create_premul_sum(dfccl_amd.ncclFloat32, np.array([0.25], np.float32).tobytes())
        ctxs[1].prepare_all_reduce(100, dfccl_amd.ncclFloat32, op1, comms[1], 0)
        comms[0].destroy_op(op0)
        with pytest.raises(api.NcclError):
            comms[0].destroy_op(op0)
        with pytest.raises(api.NcclError):
            comms[0].destroy_op(dfccl_amd.ncclSum)
    finally:
        for c in ctxs:
            c.destroy()
        for c in comms:
            c.destroy()


@pytest.mark.parametrize("kind", ["reduce_scatter", "all_gather", "reduce", "broadcast"])
@pytest.mark.parametrize("n,count", [(2, 1000), (4, 65537), (8, 1 << 18), (3, 5)])
def test_other_collectives_bf16(kind, n, count):
    check(kind, orc.BF16, orc.SUM, n, count, root=n - 1, seed=300)


@pytest.mark.parametrize("kind", ["reduce_scatter", "reduce"])
@pytest.mark.parametrize("dtype,op", [(orc.I8, orc.MIN), (orc.I32, orc.SUM), (orc.F16, orc.MAX), (orc.F32, orc.PROD)])
def test_reducing_collectives_dtypes(kind, dtype, op):
    check(kind, dtype, op, 4, 70001, root=1, seed=400)


@pytest.mark.parametrize("chunk_bytes", [524288, None])
def test_config2_geometry_ring_all_reduce_8_ranks_bf16(proto, chunk_bytes, monkeypatch):
    # 8 virtual ranks, bf16 Sum, 512 KiB chunks (262,144 elements), normal(0,1); 4 Mi elements per
    # rank here so that the host oracle finishes in seconds (the full 64 MiB shape is in the benchmark).
    # chunk_bytes None: the library's own grain for the direct protocol (the FIFO default is 512 KiB).
    from dfccl_amd.ring import VirtualRing
    n, count = 8, 4 << 20
    if chunk_bytes is not None:
        monkeypatch.setenv("DFCCL_DIRECT_CHUNK_BYTES", str(chunk_bytes))
    with VirtualRing(n) as ring:
        ring.prepare(0, "all_reduce", count, orc.BF16, orc.SUM)
        ring.finalize()
        g = ring.ctxs[0].geometry(0)
        # 8 ranks share the 256 workgroup slots less a headroom of 8: 31 channels each
        assert (g.nChannels == 31 or gpu_util.EMULATED) and g.protocol == (1 if proto == "direct" else 0)
        if chunk_bytes is not None or proto == "fifo":
            assert g.chunkElems == 262144
        sends_np, sends, recvs = make_buffers("all_reduce", orc.BF16, n, count, 2)
        want = orc.all_reduce(orc.BF16, orc.SUM, geom_of(ring, 0), sends_np)
        ring.run(0, sends, recvs, timeout=30)
        for r in range(n):
            assert np.array_equal(to_np(orc.BF16, recvs[r]), want[r])
        # and within 1 bf16 ulp (2^-8 relative) per accumulated term of the exact sum, the ulp taken at the
        # largest magnitude a partial sum can reach
        exact = sum(orc.bf16_bits_to_f32(s).astype(np.float64) for s in sends_np)
        bound = sum(np.abs(orc.bf16_bits_to_f32(s).astype(np.float64)) for s in sends_np)
        got = orc.bf16_bits_to_f32(to_np(orc.BF16, recvs[0])).astype(np.float64)
        assert np.all(np.abs(got - exact) <= (n - 1) * 2.0 ** -8 * bound + 1e-30)


def test_in_place_all_reduce_and_bcast():
    from dfccl_amd.ring import VirtualRing
    n, count = 4, 50000
    with VirtualRing(n) as ring:
        ring.prepare(0, "all_reduce", count, orc.I32, orc.SUM)
        ring.prepare(1, "broadcast", count, orc.I32, root=2)
        ring.finalize()
        sends_np, bufs, _ = make_buffers("all_reduce", orc.I32, n, count, 500)
        ring.run(0, bufs, bufs, timeout=30)
        want = sum(s.astype(np.int64) for s in sends_np).astype(np.int32)
        for r in range(n):
            assert np.array_equal(to_np(orc.I32, bufs[r]), want)
        sends_np, bufs, _ = make_buffers("broadcast", orc.I32, n, count, 510)
        ring.run(1, bufs, bufs, timeout=30)
        for r in range(n):
            assert np.array_equal(to_np(orc.I32, bufs[r]), sends_np[2])


def test_forced_preemption_is_bit_exact(monkeypatch):
    # force a context save after every slice: the resumed run must reproduce the
    # un-preempted result bit for bit, for a float op whose result depends on order
    plain = check("all_reduce", orc.F32, orc.SUM, 4, 3_000_001, seed=600)
    assert plain["forcedQuits"] == 0
    monkeypatch.setenv("DFCCL_FORCE_QUIT_EVERY", "1")
    forced = check("all_reduce", orc.F32, orc.SUM, 4, 3_000_001, seed=600)
    assert forced["forcedQuits"] > 0 and forced["ctxSaves"] >= forced["forcedQuits"]
    # a context that is still resident in LDS when its collective is visited again is not loaded again,
    # so loads only have to cover the first visit of every workgroup
    assert forced["ctxLoads"] >= 1
    monkeypatch.setenv("DFCCL_FORCE_QUIT_EVERY", "3")
    check("reduce_scatter", orc.BF16, orc.SUM, 8, 400_000, seed=610)
    check("all_gather", orc.I8, orc.SUM, 3, 1_000_003, seed=620)
    check("reduce", orc.F16, orc.SUM, 4, 900_001, root=3, seed=630)


def test_tiny_spin_budget_preempts_and_still_completes(monkeypatch):
    monkeypatch.setenv("BASE_CTX_SWITCH_THRESHOLD", "1")
    monkeypatch.setenv("NUM_TRY_TASKQ_HEAD", "1")
    monkeypatch.setenv("RECV_SUCCESS_FACTOR", "0")
    stats = check("all_reduce", orc.I32, orc.SUM, 8, 2_000_000, seed=700, reps=2)
    assert stats["ctxSaves"] > 0


def test_disordered_submission_completes_and_is_correct():
    # every rank submits the same set of collectives in its own random order: a blocking
    # library would deadlock; here every collective must complete with the right result
    from dfccl_amd.ring import VirtualRing
    n, ncoll = 4, 24
    rng = np.random.RandomState(3)
    counts = [int(c) for c in np.exp(rng.uniform(np.log(2048), np.log(1 << 20), ncoll)).astype(np.int64) // 8 * 8]
    with VirtualRing(n) as ring:
        for cid in range(ncoll):
            ring.prepare(cid, "all_reduce", counts[cid], orc.F16, orc.SUM)
        ring.finalize()
        data = {}
        for cid in range(ncoll):
            data[cid] = make_buffers("all_reduce", orc.F16, n, counts[cid], 300 + cid * 4)
        orders = [np.random.RandomState(30 + r).permutation(ncoll) for r in range(n)]
        for i in range(ncoll):
            for r in range(n):
                cid = int(orders[r][i])
                ring.submit(r, cid, data[cid][1][r], data[cid][2][r])
        ring.wait([(r, cid) for r in range(n) for cid in range(ncoll)], timeout=40)
        for cid in range(ncoll):
            want = orc.all_reduce(orc.F16, orc.SUM, geom_of(ring, cid), data[cid][0])
            for r in range(n):
                assert np.array_equal(to_np(orc.F16, data[cid][2][r]), want[r]), (cid, r)
        s = ring.stats()
        assert s["cqesWritten"] == n * ncoll


def test_rank_by_rank_submission_needs_preemption():
    # rank 0 submits everything, then rank 1, ...: the first ranks' collectives cannot finish
    # until the last rank has submitted, in reverse order
    from dfccl_amd.ring import VirtualRing
    n, ncoll, count = 3, 6, 40000
    with VirtualRing(n) as ring:
        for cid in range(ncoll):
            ring.prepare(cid, "all_reduce", count, orc.I32, orc.SUM)
        ring.finalize()
        data = {cid: make_buffers("all_reduce", orc.I32, n, count, 800 + cid * 3) for cid in range(ncoll)}
        for r in range(n):
            order = range(ncoll) if r % 2 == 0 else reversed(range(ncoll))
            for cid in order:
                ring.submit(r, cid, data[cid][1][r], data[cid][2][r])
            time.sleep(0.02)
        ring.wait([(r, cid) for r in range(n) for cid in range(ncoll)], timeout=40)
        for cid in range(ncoll):
            want = sum(s.astype(np.int64) for s in data[cid][0]).astype(np.int32)
            for r in range(n):
                assert np.array_equal(to_np(orc.I32, data[cid][2][r]), want)
        assert ring.stats()["ctxSaves"] > 0


def test_idle_daemon_leaves_and_is_relaunched(monkeypatch):
    from dfccl_amd.ring import VirtualRing
    # (on the host emulation a scheduler round takes milliseconds)
    monkeypatch.setenv("TOLERANT_UNPROGRESSED_CNT", "100" if gpu_util.EMULATED else "2000")
    n, count = 2, 10000
    with VirtualRing(n) as ring:
        ring.prepare(0, "all_reduce", count, orc.I32, orc.SUM)
        ring.finalize()
        sends_np, sends, recvs = make_buffers("all_reduce", orc.I32, n, count, 900)
        want = (sends_np[0].astype(np.int64) + sends_np[1]).astype(np.int32)
        ring.run(0, sends, recvs, timeout=30)
        time.sleep(4.0 if gpu_util.EMULATED else 0.5)  # long enough for every workgroup to give up polling
        torch.cuda.synchronize()  # returns only if the daemon really left the GPU
        s1 = ring.stats()
        assert s1["voluntaryQuits"] >= n
        for t in recvs:
            t.zero_()
        torch.cuda.current_stream().synchronize()
        ring.run(0, sends, recvs, timeout=30)
        assert np.array_equal(to_np(orc.I32, recvs[1]), want)
        assert ring.stats()["daemonLaunches"] >= s1["daemonLaunches"] + 1


def test_voluntary_quit_with_collectives_in_flight(monkeypatch):
    # rank 1 submits late: rank 0's workgroups give up, save their task queue, and pick the
    # collective up again after the relaunch
    from dfccl_amd.ring import VirtualRing
    monkeypatch.setenv("TOLERANT_UNPROGRESSED_CNT", "60" if gpu_util.EMULATED else "300")
    n, count = 2, 200000
    with VirtualRing(n) as ring:
        ring.prepare(0, "all_reduce", count, orc.F32, orc.SUM)
        ring.finalize()
        sends_np, sends, recvs = make_buffers("all_reduce", orc.F32, n, count, 910)
        ring.submit(0, 0, sends[0], recvs[0])
        time.sleep(4.0 if gpu_util.EMULATED else 0.3)
        ring.submit(1, 0, sends[1], recvs[1])
        ring.wait([(0, 0), (1, 0)], timeout=30)
        want = orc.all_reduce(orc.F32, orc.SUM, geom_of(ring, 0), sends_np)
        for r in range(n):
            assert np.array_equal(to_np(orc.F32, recvs[r]), want[r])
        s = ring.stats()
        assert s["voluntaryQuits"] > 0 and s["daemonLaunches"] > 1


def test_contexts_can_be_destroyed_and_recreated():
    for i in range(3):
        check("all_reduce", orc.I32, orc.SUM, 2 + i, 10000 + i, seed=950 + i)


def test_second_ring_joins_a_running_daemon():
    from dfccl_amd.ring import VirtualRing
    count = 30000
    with VirtualRing(2) as a:
        a.prepare(0, "all_reduce", count, orc.I32, orc.SUM)
        a.finalize()
        sa_np, sa, ra = make_buffers("all_reduce", orc.I32, 2, count, 960)
        a.run(0, sa, ra, timeout=30)
        with VirtualRing(3) as b:  # attaches while a's daemon is resident
            b.prepare(5, "all_reduce", count, orc.I32, orc.MAX)
            b.finalize()
            sb_np, sb, rb = make_buffers("all_reduce", orc.I32, 3, count, 970)
            b.run(5, sb, rb, timeout=30)
            a.run(0, sa, ra, timeout=30)
            assert np.array_equal(to_np(orc.I32, rb[2]), np.maximum(np.maximum(sb_np[0], sb_np[1]), sb_np[2]))
        a.run(0, sa, ra, timeout=30)
        assert np.array_equal(to_np(orc.I32, ra[0]), (sa_np[0].astype(np.int64) + sa_np[1]).astype(np.int32))


def test_callback_gets_coll_id_and_args_on_poller_thread():
    import ctypes
    from dfccl_amd import _lib, api
    lib = _lib.load()
    n, count = 2, 4096
    comms = api.VirtualComm.create_all(n)
    ctxs = [api.RankCtx(r) for r in range(n)]
    try:
        for r in range(n):
            ctxs[r].prepare_all_reduce(count, api.ncclFloat32, api.ncclSum, comms[r], 7)
            ctxs[r].finalize()
        seen = []
        done = threading.Event()

        @_lib.CALLBACK
        def cb(coll_id, args):
            seen.append((coll_id, args, threading.get_ident()))
            if len(seen) == n:
                done.set()
            return 0

        bufs = [torch.ones(count, device=gpu_util.DEVICE) for _ in range(n)]
        torch.cuda.current_stream().synchronize()
        for r in range(n):
            assert lib.ofcclRunAllReduce(bufs[r].data_ptr(), bufs[r].data_ptr(), 7, cb, ctypes.c_void_p(0x1000 + r),
                                         ctxs[r].handle) == 0
        assert done.wait(30)
        assert sorted(a for _, a, _ in seen) == [0x1000, 0x1001]
        assert all(c == 7 for c, _, _ in seen)
        assert all(t != threading.get_ident() for _, _, t in seen)
        assert torch.equal(bufs[0], torch.full((count,), 2.0, device=gpu_util.DEVICE))
    finally:
        for c in ctxs:
            c.destroy()
        for c in comms:
            c.destroy()


@pytest.mark.parametrize("capacity,sleep_ms", [("6", 0), ("2000", 2)])
def test_queue_back_pressure_every_submission_gets_one_callback(capacity, sleep_ms, monkeypatch):
    # Two submitting threads per rank push 24 small all-reduces three times each as fast as Run takes them (a second
    # Run of a collective waits for the first inside the library), the last rank starting late so that the others
    # pile up parked collectives.  With a submission queue of 6 entries the full-queue path of Run (sqWrite
    # returning "full", src/enqueue_ofccl.cc:623-627) and the lazily published queue head are exercised; with the
    # full-size queue the callback sleeps on the poller thread (src/enqueue_ofccl.cc:908-965) instead.
    import ctypes
    import time
    from dfccl_amd import _lib, api
    monkeypatch.setenv("DFCCL_SQ_CAPACITY", capacity)
    lib = _lib.load()
    n, ncolls, rounds, count = 3, 24, 3, 600
    comms = [api.VirtualComm.create_all(n) for _ in range(ncolls)]
    ctxs = [api.RankCtx(r) for r in range(n)]
    calls = [[0] * ncolls for _ in range(n)]
    lock = threading.Lock()
    try:
        for c in range(ncolls):
            for r in range(n):
                ctxs[r].prepare_all_reduce(count, api.ncclInt32, api.ncclSum, comms[c][r], c)
        for r in range(n):
            ctxs[r].finalize()

        @_lib.CALLBACK
        def cb(coll_id, args):
            if sleep_ms:
                time.sleep(sleep_ms / 1000.0)
            with lock:
                calls[int(args or 0)][coll_id] += 1
            return 0

        send = [[(torch.arange(count, dtype=torch.int32) + 3 * r + 7 * c).to(gpu_util.DEVICE) for r in range(n)]
                for c in range(ncolls)]
        recv = [[torch.full((count,), -1, dtype=torch.int32, device=gpu_util.DEVICE) for r in range(n)]
                for c in range(ncolls)]
        torch.cuda.current_stream().synchronize()
        failures = []

        def submitter(r, half):
            if r == n - 1:
                time.sleep(0.2)
            for _ in range(rounds):
                for c in range(half, ncolls, 2):
                    rc = lib.ofcclRunAllReduce(send[c][r].data_ptr(), recv[c][r].data_ptr(), c, cb,
                                               ctypes.c_void_p(r) if r else None, ctxs[r].handle)
                    if rc != 0:
                        failures.append((r, c, rc))

        threads = [threading.Thread(target=submitter, args=(r, h)) for r in range(n) for h in (0, 1)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(120)
        assert not any(t.is_alive() for t in threads) and not failures
        deadline = time.monotonic() + 60
        while time.monotonic() < deadline and any(v < rounds for row in calls for v in row):
            time.sleep(0.005)
        time.sleep(0.05)  # a callback too many would show up now
        assert all(v == rounds for row in calls for v in row), calls
        for c in range(ncolls):
            want = sum(torch.arange(count, dtype=torch.int32) + 3 * q + 7 * c for q in range(n))
            for r in range(n):
                assert torch.equal(recv[c][r].cpu(), want), (c, r)
        stats = [ctx.stats() for ctx in ctxs]
        assert sum(s["cqesWritten"] for s in stats) == n * ncolls * rounds
        if int(capacity) < ncolls // 2 and gpu_util.EMULATED:
            # the queue really was found full.  (Only asserted where the daemon is slow enough to make that
            # certain: a GPU empties a queue of 6 faster than Python threads fill it, except while the kernel is
            # being launched; there the run still checks that nothing is lost or duplicated.)
            assert sum(s["sqFullWaits"] for s in stats) > 0
    finally:
        for c in ctxs:
            c.destroy()
        for cs in comms:
            for c in cs:
                c.destroy()


def test_prepare_validation_follows_the_reference():
    from dfccl_amd import api
    comms = api.VirtualComm.create_all(2)
    other = api.VirtualComm.create_all(2)
    ctx = api.RankCtx(0)
    try:
        with pytest.raises(api.NcclError) as e:
            ctx.prepare_all_reduce(16, api.ncclFloat32, api.ncclSum, comms[0], 2000)  # collId out of range
        assert e.value.code == 5
        with pytest.raises(api.NcclError) as e:
            ctx.prepare_reduce(16, api.ncclFloat32, api.ncclSum, 2, comms[0], 1)  # root out of range
        assert e.value.code == 4
        with pytest.raises(api.NcclError) as e:
            ctx.prepare_all_reduce(16, 10, api.ncclSum, comms[0], 1)  # dtype out of range
        assert e.value.code == 4
        with pytest.raises(api.NcclError) as e:
            ctx.prepare_all_reduce(16, api.ncclFloat32, 5, comms[0], 1)  # no operator with that value was created
        assert e.value.code == 4
        with pytest.raises(api.NcclError) as e:
            ctx.prepare_all_reduce(16, api.ncclFloat32, -1, comms[0], 1)
        assert e.value.code == 4
        with pytest.raises(api.NcclError) as e:
            ctx.prepare_broadcast(16, 11, 0, comms[0], 1)  # dtype out of range on a copy collective
        assert e.value.code == 4
        ctx.prepare_all_reduce(16, api.ncclFloat32, api.ncclSum, comms[0], 1)
        with pytest.raises(api.NcclError) as e:
            ctx.prepare_all_reduce(16, api.ncclFloat32, api.ncclSum, comms[0], 2)  # communicator reuse
        assert e.value.code == 5
        with pytest.raises(api.NcclError) as e:
            ctx.prepare_all_reduce(16, api.ncclFloat32, api.ncclSum, other[0], 1)  # collId reuse
        assert e.value.code == 5
        with pytest.raises(api.NcclError) as e:
            ctx.prepare_all_reduce(16, api.ncclFloat32, api.ncclSum, other[1], 3)  # handle of another rank
        assert e.value.code == 4
    finally:
        ctx.destroy()
        for c in comms + other:
            c.destroy()


@pytest.mark.parametrize("dtype,op", [(orc.F16, orc.SUM), (orc.BF16, orc.SUM), (orc.F32, orc.PROD), (orc.I8, orc.MAX)])
@pytest.mark.parametrize("n,count", [(4, 2048), (2, 1), (8, 16384 // 4), (3, 1000), (5, 8191)])
def test_small_all_reduce_and_in_place(dtype, op, n, count, proto):
    # small messages (some ranks own no chunk at all), out of place and in place
    from dfccl_amd.ring import VirtualRing
    with VirtualRing(n) as ring:
        ring.prepare(0, "all_reduce", count, dtype, op)
        ring.finalize()
        sends_np, sends, recvs = make_buffers("all_reduce", dtype, n, count, 1100, small_ints=(op == orc.PROD))
        want = orc.all_reduce(dtype, op, geom_of(ring, 0), sends_np)
        for rep in range(3):
            ring.run(0, sends, recvs, timeout=30)
            for r in range(n):
                assert np.array_equal(to_np(dtype, recvs[r]), want[r]), (rep, r)
        bufs = [s.clone() for s in sends]
        torch.cuda.current_stream().synchronize()
        ring.run(0, bufs, bufs, timeout=30)  # in place
        for r in range(n):
            assert np.array_equal(to_np(dtype, bufs[r]), want[r]), ("in place", r)


def test_small_all_reduce_under_forced_preemption(monkeypatch):
    monkeypatch.setenv("DFCCL_FORCE_QUIT_EVERY", "1")
    check("all_reduce", orc.F32, orc.SUM, 4, 1024, seed=1200, reps=3)
    monkeypatch.setenv("BASE_CTX_SWITCH_THRESHOLD", "1")
    monkeypatch.setenv("NUM_TRY_TASKQ_HEAD", "1")
    monkeypatch.setenv("RECV_SUCCESS_FACTOR", "0")
    check("all_reduce", orc.BF16, orc.SUM, 8, 2000, seed=1210, reps=3)


def test_many_ranks_fall_back_to_fifo():
    # more ranks than one workgroup folds in a pass: the collective runs over FIFOs
    stats = check("all_reduce", orc.I32, orc.SUM, 12, 50000, seed=1300)
    assert stats["cqesWritten"] == 12


def test_in_place_and_absent_buffers_of_the_other_collectives():
    # in place as NCCL defines it: reduce-scatter receives into block `rank` of its send buffer, all-gather sends
    # from block `rank` of its receive buffer, reduce at the root; ranks that are not the root of a reduce pass no
    # receive buffer, ranks that are not the root of a broadcast no send buffer
    from dfccl_amd.ring import VirtualRing
    n, count, root = 4, 30011, 1
    with VirtualRing(n) as ring:
        ring.prepare(0, "reduce_scatter", count, orc.F32, orc.SUM)
        ring.prepare(1, "all_gather", count, orc.F16)
        ring.prepare(2, "reduce", count, orc.BF16, orc.SUM, root)
        ring.prepare(3, "broadcast", count, orc.I8, root=root)
        ring.finalize()
        # reduce-scatter
        sends_np, sends, _ = make_buffers("reduce_scatter", orc.F32, n, count, 2100)
        want = orc.reduce_scatter(orc.F32, orc.SUM, geom_of(ring, 0), sends_np)
        ring.run(0, sends, [sends[r][r * count:(r + 1) * count] for r in range(n)], timeout=30)
        for r in range(n):
            assert np.array_equal(to_np(orc.F32, sends[r][r * count:(r + 1) * count]), want[r]), ("reduce_scatter", r)
        # all-gather
        sends_np, _, recvs = make_buffers("all_gather", orc.F16, n, count, 2200)
        for r in range(n):
            recvs[r][r * count:(r + 1) * count].copy_(to_gpu(orc.F16, sends_np[r]))
        torch.cuda.current_stream().synchronize()
        want = orc.all_gather(orc.F16, geom_of(ring, 1), sends_np)
        ring.run(1, [recvs[r][r * count:(r + 1) * count] for r in range(n)], recvs, timeout=30)
        for r in range(n):
            assert np.array_equal(to_np(orc.F16, recvs[r]), want[r]), ("all_gather", r)
        # reduce: in place at the root, no receive buffer elsewhere
        sends_np, sends, _ = make_buffers("reduce", orc.BF16, n, count, 2300)
        want = orc.reduce(orc.BF16, orc.SUM, geom_of(ring, 2), root, sends_np)
        ring.run(2, sends, [sends[r] if r == root else None for r in range(n)], timeout=30)
        assert np.array_equal(to_np(orc.BF16, sends[root]), want[root])
        for r in range(n):
            if r != root:  # the other ranks' send buffers are untouched
                assert np.array_equal(to_np(orc.BF16, sends[r]), sends_np[r])
        # broadcast: no send buffer except at the root
        sends_np, sends, recvs = make_buffers("broadcast", orc.I8, n, count, 2400)
        ring.run(3, [sends[r] if r == root else None for r in range(n)], recvs, timeout=30)
        for r in range(n):
            assert np.array_equal(to_np(orc.I8, recvs[r]), sends_np[root]), ("broadcast", r)


@pytest.mark.parametrize("kind,dtype,op", [("reduce_scatter", orc.F16, orc.SUM), ("reduce", orc.F32, orc.SUM),
                                           ("reduce", orc.BF16, orc.PROD), ("all_gather", orc.I8, orc.SUM),
                                           ("broadcast", orc.F16, orc.SUM)])
@pytest.mark.parametrize("n,count", [(8, 3_000_017), (5, 999_999), (2, 12_345_678)])
def test_other_collectives_large_and_ragged(kind, dtype, op, n, count):
    # several channels and loops, sizes that are no multiple of anything (all-gather then writes at offsets that
    # rule out 128-bit accesses), a root in the middle
    if kind in ("all_gather", "reduce_scatter"):
        count //= n
    check(kind, dtype, op, n, count, root=n // 2, seed=2500 + n, small_ints=(op == orc.PROD))


def test_other_collectives_disordered_submission(proto):
    # the four other collectives registered side by side, every rank submitting them in its own order
    from dfccl_amd.ring import VirtualRing
    n, count = 4, 70_001
    kinds = ["reduce_scatter", "all_gather", "reduce", "broadcast", "all_reduce"] * 3
    rng = np.random.default_rng(26)
    with VirtualRing(n) as ring:
        for cid, kind in enumerate(kinds):
            ring.prepare(cid, kind, count, orc.F32, orc.SUM, root=cid % n)
        ring.finalize()
        bufs, wants = [], []
        for cid, kind in enumerate(kinds):
            sends_np, sends, recvs = make_buffers(kind, orc.F32, n, count, 2600 + 10 * cid)
            bufs.append((sends, recvs))
            wants.append(oracle_run(kind, orc.F32, orc.SUM, geom_of(ring, cid), cid % n, sends_np))
        for r in range(n):
            for cid in rng.permutation(len(kinds)):
                ring.submit(r, int(cid), bufs[cid][0][r], bufs[cid][1][r])
        ring.wait([(r, cid) for r in range(n) for cid in range(len(kinds))], timeout=40)
        for cid, kind in enumerate(kinds):
            for r in range(n):
                if kind == "reduce" and r != cid % n:
                    continue
                assert np.array_equal(to_np(orc.F32, bufs[cid][1][r]), wants[cid][r]), (cid, kind, r)


@pytest.mark.parametrize("seed", range(int(os.environ.get("DFCCL_RANDOM_SEEDS", "8"))))  # (more for a longer campaign)
def test_random_collectives_every_type_and_op_disordered(seed):
    # random ranks, kinds, element types, ops (Avg included), sizes (from a few elements to several tiles, mostly
    # ragged) and roots, registered side by side and submitted by every rank in its own order, twice
    from dfccl_amd.ring import VirtualRing
    rng = np.random.default_rng(9000 + seed)
    n = int(rng.integers(2, 9))
    ncolls = int(rng.integers(3, 8))
    specs = []
    for cid in range(ncolls):
        kind = ["all_reduce", "reduce_scatter", "all_gather", "reduce", "broadcast"][int(rng.integers(5))]
        dtype = int(rng.integers(10))
        op = int(rng.integers(5))
        shape = int(rng.integers(4))
        count = [int(rng.integers(1, 17)), int(rng.integers(1, 3000)), 256 * int(rng.integers(1, 40)),
                 int(rng.integers(1, 120000))][shape]
        if gpu_util.EMULATED:
            count = min(count, 30000)
        specs.append((kind, dtype, op, count, int(rng.integers(n))))
    with VirtualRing(n) as ring:
        for cid, (kind, dtype, op, count, root) in enumerate(specs):
            ring.prepare(cid, kind, count, dtype, op, root)
        ring.finalize()
        for rep in range(2):
            bufs, wants = [], []
            for cid, (kind, dtype, op, count, root) in enumerate(specs):
                sends_np, sends, recvs = make_buffers(kind, dtype, n, count, 9100 + 100 * seed + 10 * cid + rep,
                                                      small_ints=(op == orc.PROD))
                bufs.append((sends, recvs))
                wants.append(oracle_run(kind, dtype, op, geom_of(ring, cid), root, sends_np))
            for r in range(n):
                for cid in rng.permutation(ncolls):
                    ring.submit(r, int(cid), bufs[cid][0][r], bufs[cid][1][r])
            ring.wait([(r, cid) for r in range(n) for cid in range(ncolls)], timeout=60)
            for cid, (kind, dtype, op, count, root) in enumerate(specs):
                for r in range(n):
                    if kind == "reduce" and r != root:
                        continue
                    assert np.array_equal(to_np(dtype, bufs[cid][1][r]), wants[cid][r]), (seed, rep, cid, specs[cid], r)


@pytest.mark.parametrize("knobs", [{"BASE_CTX_SWITCH_THRESHOLD": "1", "NUM_TRY_TASKQ_HEAD": "1", "RECV_SUCCESS_FACTOR": "0"},
                                   {}, {"DFCCL_IDLE_POLL_ROUNDS": "0"}])
def test_small_all_reduce_repeated_and_fallbacks(knobs, monkeypatch):
    # the same small collectives over and over: each rank's share is one tile of 2 KiB / 3 KiB, which wave 0 of the
    # workgroup runs on its own (waits, fold, release, final wait without a workgroup barrier in between); with a
    # spin budget of one poll most visits run out at one of the two waits and park the collective, because the
    # ranks are submitted one after the other from this thread
    from dfccl_amd.ring import VirtualRing
    for k, v in knobs.items():
        monkeypatch.setenv(k, v)
    n, count = 4, 2048
    with VirtualRing(n) as ring:
        ring.prepare(0, "all_reduce", count, orc.F32, orc.SUM)
        ring.prepare(1, "all_reduce", 3 * count, orc.BF16, orc.MAX)
        ring.finalize()
        for rep in range(40):
            cid = rep % 3 // 2  # 0, 0, 1, 0, 0, 1, ...: the resident context changes now and then
            dtype, op, cnt = (orc.F32, orc.SUM, count) if cid == 0 else (orc.BF16, orc.MAX, 3 * count)
            sends_np, sends, recvs = make_buffers("all_reduce", dtype, n, cnt, 3000 + rep)
            want = orc.all_reduce(dtype, op, geom_of(ring, cid), sends_np)
            ring.run(cid, sends, recvs, timeout=30)
            for r in range(n):
                assert np.array_equal(to_np(dtype, recvs[r]), want[r]), (rep, r)
        stats = ring.stats()
        assert stats["cqesWritten"] == 40 * n


def test_empty_collectives_complete_and_touch_nothing():
    # count 0 (NCCL accepts it: nothing moves): every kind completes with a callback, twice in a row, and the
    # one-element buffers that are passed keep their contents; a real collective registered beside them still works
    from dfccl_amd.ring import VirtualRing
    n = 3
    with VirtualRing(n) as ring:
        for cid, kind in enumerate(("all_reduce", "reduce_scatter", "all_gather", "reduce", "broadcast")):
            ring.prepare(cid, kind, 0, orc.F32, orc.SUM, root=1)
        ring.prepare(5, "all_reduce", 1000, orc.I32, orc.SUM)
        ring.finalize()
        marks = [torch.full((4,), 7.0, device=gpu_util.DEVICE) for _ in range(n)]
        outs = [torch.full((4,), 9.0, device=gpu_util.DEVICE) for _ in range(n)]
        sends_np, sends, recvs = make_buffers("all_reduce", orc.I32, n, 1000, 2500)
        torch.cuda.current_stream().synchronize()
        for rep in range(2):
            for r in range(n):
                for cid in range(5):
                    ring.submit(r, cid, marks[r], outs[r])
                ring.submit(r, 5, sends[r], recvs[r])
            ring.wait([(r, cid) for r in range(n) for cid in range(6)], timeout=30)
        want = orc.all_reduce(orc.I32, orc.SUM, geom_of(ring, 5), sends_np)
        for r in range(n):
            assert bool((marks[r] == 7.0).all()) and bool((outs[r] == 9.0).all()), r
            assert np.array_equal(to_np(orc.I32, recvs[r]), want[r]), r
