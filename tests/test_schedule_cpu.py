"""CPU checks of the host logic that the daemon kernel shares with the host
(ring_schedule.h): the per-step roles, slice sizing, FIFO flow control and the
completion-entry encoding, interpreted on the host and compared with the oracle."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

import datagen
import dfccl_oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
KIND = {"all_reduce": 0, "reduce_scatter": 1, "all_gather": 2, "reduce": 3, "broadcast": 4}


@pytest.fixture(scope="module")
def sim(tmp_path_factory):
    orc.build()
    tmp = tmp_path_factory.mktemp("sim")
    out, obj = str(tmp / "libschedule_sim.so"), str(tmp / "dfccl_oracle.o")
    subprocess.check_call(["gcc", "-O2", "-std=c11", "-fPIC", "-ffp-contract=off", "-c",
                           os.path.join(ROOT, "oracle", "dfccl_oracle.c"), "-o", obj])
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-o", out,
                           os.path.join(HERE, "schedule_sim.cc"), obj, "-lm", "-lpthread"])
    lib = ctypes.CDLL(out)
    vpp = ctypes.POINTER(ctypes.c_void_p)
    lib.sim_collective.argtypes = [ctypes.c_int] * 5 + [ctypes.c_int64] * 3 + [ctypes.c_int] * 2 + \
        [ctypes.c_int64, ctypes.c_int, vpp, vpp, ctypes.POINTER(ctypes.c_int64)]
    lib.sim_direct.argtypes = [ctypes.c_int] * 5 + [ctypes.c_int64] * 3 + [ctypes.c_int, vpp, vpp, ctypes.c_uint64]
    lib.sim_direct.restype = ctypes.c_int64
    lib.sim_plan_channels.argtypes = [ctypes.c_int64, ctypes.c_int, ctypes.c_int64]
    lib.sim_cqe_encode.argtypes = [ctypes.c_uint] * 3
    lib.sim_cqe_encode.restype = ctypes.c_uint64
    lib.sim_cqe_decode.argtypes = [ctypes.c_uint64] + [ctypes.POINTER(ctypes.c_uint)] * 3
    return lib


def run_sim(sim, kind, dtype, op, n, C, chunk, align, slice_, spc, slots, count, root, sends, recvs):
    seen = ctypes.c_int64()
    rc = sim.sim_collective(KIND[kind], dtype, op, n, C, chunk, align, slice_, spc, slots, count, root,
                            orc._ptrs(sends), orc._ptrs(recvs), ctypes.byref(seen))
    assert rc == 0, f"schedule interpreter failed with {rc}"
    return seen.value


# n, C, chunk, align, count  (slice = chunk / slices-per-chunk)
CASES = [(2, 1, 64, 16, 1000), (3, 2, 64, 16, 1000), (4, 1, 128, 32, 37), (4, 3, 32, 16, 5000), (8, 2, 64, 64, 4096),
         (8, 4, 256, 64, 100003), (5, 1, 16, 16, 3), (2, 2, 512, 128, 513), (1, 2, 64, 16, 300), (4, 1, 2048, 512, 2048)]


@pytest.mark.parametrize("n,C,chunk,align,count", CASES)
@pytest.mark.parametrize("dtype,op", [(orc.F32, orc.SUM), (orc.BF16, orc.SUM), (orc.I8, orc.MAX), (orc.F16, orc.PROD),
                                      (orc.BF16, orc.AVG), (orc.I32, orc.AVG), (orc.F64, orc.AVG), (orc.U8, orc.AVG),
                                      (orc.U64, orc.MAX)])
def test_all_reduce_schedule_matches_oracle(sim, n, C, chunk, align, count, dtype, op):
    g = orc.Geom(n, C, chunk, align)
    sends = [datagen.make(dtype, 10 + r, count) for r in range(n)]
    want = orc.all_reduce(dtype, op, g, sends)
    recvs = [np.zeros_like(s) for s in sends]
    seen = run_sim(sim, "all_reduce", dtype, op, n, C, chunk, align, chunk // 2, 2, 4, count, 0, sends, recvs)
    for r in range(n):
        assert np.array_equal(recvs[r], want[r]), r
    assert seen <= max(chunk // 2, 16)
    # in place
    bufs = [s.copy() for s in sends]
    run_sim(sim, "all_reduce", dtype, op, n, C, chunk, align, chunk // 2, 2, 4, count, 0, bufs, bufs)
    for r in range(n):
        assert np.array_equal(bufs[r], want[r]), r


@pytest.mark.parametrize("n,C,chunk,align,count", CASES)
@pytest.mark.parametrize("dtype,op", [(orc.F32, orc.SUM), (orc.BF16, orc.MIN), (orc.I32, orc.SUM), (orc.F16, orc.AVG),
                                      (orc.I64, orc.AVG)])
def test_reduce_scatter_schedule_matches_oracle(sim, n, C, chunk, align, count, dtype, op):
    g = orc.Geom(n, C, chunk, align)
    sends = [datagen.make(dtype, 20 + r, count * n) for r in range(n)]
    want = orc.reduce_scatter(dtype, op, g, sends)
    recvs = [np.zeros(count, dtype=s.dtype) for s in sends]
    run_sim(sim, "reduce_scatter", dtype, op, n, C, chunk, align, chunk // 2, 2, 4, count, 0, sends, recvs)
    for r in range(n):
        assert np.array_equal(recvs[r], want[r]), r


@pytest.mark.parametrize("n,C,chunk,align,count", CASES)
@pytest.mark.parametrize("dtype", [orc.I8, orc.F16, orc.F32])
def test_all_gather_schedule_matches_oracle(sim, n, C, chunk, align, count, dtype):
    sends = [datagen.make(dtype, 30 + r, count) for r in range(n)]
    want = np.concatenate(sends)
    recvs = [np.zeros(count * n, dtype=sends[0].dtype) for _ in range(n)]
    # chunk / align are in bytes for the copy collectives
    run_sim(sim, "all_gather", dtype, 0, n, C, chunk, align, chunk // 2, 2, 4, count, 0, sends, recvs)
    for r in range(n):
        assert np.array_equal(recvs[r], want), r
    bufs = [np.zeros(count * n, dtype=sends[0].dtype) for _ in range(n)]
    for r in range(n):
        bufs[r][r * count:(r + 1) * count] = sends[r]
    run_sim(sim, "all_gather", dtype, 0, n, C, chunk, align, chunk // 2, 2, 4, count, 0,
            [bufs[r][r * count:(r + 1) * count] for r in range(n)], bufs)
    for r in range(n):
        assert np.array_equal(bufs[r], want), r


@pytest.mark.parametrize("n,C,chunk,align,count", CASES)
def test_reduce_and_broadcast_schedules_match_oracle(sim, n, C, chunk, align, count):
    g = orc.Geom(n, C, chunk, align)
    for root in {0, n - 1, n // 2}:
        sends = [datagen.make(orc.BF16, 40 + r, count) for r in range(n)]
        want = orc.reduce(orc.BF16, orc.SUM, g, root, sends)
        recvs = [np.zeros_like(s) for s in sends]
        run_sim(sim, "reduce", orc.BF16, orc.SUM, n, C, chunk, align, chunk, 1, 8, count, root, sends, recvs)
        for r in range(n):
            assert np.array_equal(recvs[r], want[r]), (root, r)
        for dtype in (orc.F32, orc.I8):  # an average: inputs scaled where the chain reads them, or the root divides
            isends = [datagen.make(dtype, 45 + r, count) for r in range(n)]
            want = orc.reduce(dtype, orc.AVG, g, root, isends)
            recvs = [np.zeros_like(s) for s in isends]
            run_sim(sim, "reduce", dtype, orc.AVG, n, C, chunk, align, chunk, 1, 8, count, root, isends, recvs)
            assert np.array_equal(recvs[root], want[root]), (dtype, root)
        recvs = [np.zeros_like(s) for s in sends]
        run_sim(sim, "broadcast", orc.F16, 0, n, C, chunk, align, chunk, 1, 8, count, root, sends, recvs)
        for r in range(n):
            assert np.array_equal(recvs[r], sends[root]), (root, r)
        bufs = [s.copy() for s in sends]  # in place (Bcast)
        run_sim(sim, "broadcast", orc.F16, 0, n, C, chunk, align, chunk, 1, 8, count, root, bufs, bufs)
        for r in range(n):
            assert np.array_equal(bufs[r], sends[root]), (root, r)


def test_channel_planning_rule(sim):
    per = 512 * 64
    assert sim.sim_plan_channels(4096, 32, per) == 1
    assert sim.sim_plan_channels(per * 2, 32, per) == 2
    assert sim.sim_plan_channels(per * 2 - 1, 32, per) == 1
    assert sim.sim_plan_channels(64 << 20, 32, per) == 32
    assert sim.sim_plan_channels(0, 32, per) == 1


def test_cqe_encoding_equals_oracle(sim):
    L = orc.lib()
    for blk, cnt, coll in [(0, 1, 0), (63, 0xFFFFFF, 1999), (5, 4097, 77)]:
        v = sim.sim_cqe_encode(blk, cnt, coll)
        assert v == L.orc_cqe_encode(blk, cnt, coll)
        b, c, i = ctypes.c_uint(), ctypes.c_uint(), ctypes.c_uint()
        sim.sim_cqe_decode(v, ctypes.byref(b), ctypes.byref(c), ctypes.byref(i))
        assert (b.value, c.value, i.value) == (blk, cnt, coll)


# ---- direct protocol: roles and tile geometry of ring_schedule.h against the oracle ---------------------------

def run_direct(sim, kind, dtype, op, n, C, chunk, align, count, root, sends, recvs, order):
    return sim.sim_direct(KIND[kind], dtype, op, n, C, chunk, align, count, root, orc._ptrs(sends), orc._ptrs(recvs),
                          order)


def kind_buffers(kind, dtype, n, count, seed, **kw):
    send_len = count * n if kind == "reduce_scatter" else count
    recv_len = count * n if kind == "all_gather" else count
    sends = [datagen.make(dtype, seed + r, send_len, **kw) for r in range(n)]
    recvs = [np.zeros(recv_len, dtype=sends[0].dtype) for _ in range(n)]
    return sends, recvs


def oracle_kind(kind, dtype, op, g, root, sends):
    if kind == "all_reduce":
        return orc.all_reduce(dtype, op, g, sends)
    if kind == "reduce_scatter":
        return orc.reduce_scatter(dtype, op, g, sends)
    if kind == "all_gather":
        return orc.all_gather(dtype, g, sends)
    if kind == "reduce":
        return orc.reduce(dtype, op, g, root, sends)
    return orc.broadcast(dtype, g, root, sends)


DIRECT_CASES = [(2, 1, 64, 16, 1000), (3, 2, 64, 16, 1000), (4, 1, 128, 32, 37), (4, 3, 32, 16, 5000),
                (8, 2, 64, 64, 4096), (8, 4, 256, 64, 100003), (5, 1, 16, 16, 3), (2, 2, 512, 128, 513),
                (4, 64, 4096, 512, 1 << 20), (7, 5, 48, 16, 12345)]


@pytest.mark.parametrize("kind", list(KIND))
@pytest.mark.parametrize("n,C,chunk,align,count", DIRECT_CASES)
@pytest.mark.parametrize("dtype,op", [(orc.F32, orc.SUM), (orc.BF16, orc.SUM), (orc.I8, orc.MIN), (orc.F16, orc.AVG),
                                      (orc.U32, orc.AVG)])
def test_direct_protocol_roles_and_tiles_match_oracle(sim, kind, n, C, chunk, align, count, dtype, op):
    root = (n - 1) // 2
    if kind in ("reduce_scatter", "all_gather"):
        count = max(1, count // n)
    sends, recvs = kind_buffers(kind, dtype, n, count, 40)
    want = oracle_kind(kind, dtype, op, orc.Geom(n, C, chunk, align), root, sends)
    for order in (0, 7):  # two different orders in which the tiles are taken
        for t in recvs:
            t[...] = 0
        written = run_direct(sim, kind, dtype, op, n, C, chunk, align, count, root, sends, recvs, order)
        # every destination element is written exactly once
        expect = {"all_reduce": n * count, "reduce_scatter": n * count, "all_gather": n * n * count,
                  "reduce": count, "broadcast": n * count}[kind]
        if kind in ("all_gather", "broadcast"):
            expect *= orc.TYPE_SIZE[dtype]  # these run as bytes
        assert written == expect
        for r in range(n):
            if kind == "reduce" and r != root:
                assert not recvs[r].any()
                continue
            assert np.array_equal(recvs[r], want[r]), (kind, order, r)


@pytest.mark.parametrize("kind", ["all_reduce", "reduce_scatter", "all_gather", "reduce", "broadcast"])
def test_direct_protocol_in_place(sim, kind):
    n, C, chunk, align, count, root, dtype = 4, 2, 64, 16, 3000, 1, orc.F32
    sends, _ = kind_buffers(kind, dtype, n, count, 70)
    want = oracle_kind(kind, dtype, orc.SUM, orc.Geom(n, C, chunk, align), root, [s.copy() for s in sends])
    if kind == "reduce_scatter":
        bufs = [s.copy() for s in sends]
        recvs = [bufs[r][r * count:(r + 1) * count] for r in range(n)]
        run_direct(sim, kind, dtype, orc.SUM, n, C, chunk, align, count, root, bufs, recvs, 3)
    elif kind == "all_gather":
        recvs = [np.zeros(count * n, dtype=sends[0].dtype) for _ in range(n)]
        for r in range(n):
            recvs[r][r * count:(r + 1) * count] = sends[r]
        run_direct(sim, kind, dtype, orc.SUM, n, C, chunk, align, count, root,
                   [recvs[r][r * count:(r + 1) * count] for r in range(n)], recvs, 3)
    else:
        recvs = [s.copy() for s in sends]
        run_direct(sim, kind, dtype, orc.SUM, n, C, chunk, align, count, root, recvs, recvs, 3)
    for r in range(n):
        if kind == "reduce" and r != root:
            continue
        assert np.array_equal(recvs[r], want[r]), (kind, r)
