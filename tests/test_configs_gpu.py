"""The benchmark configurations at full size, checked through size-independent properties: exact sums of small
integers in every dtype (native driver, element-by-element verification on the host), zero deadlocks under
per-rank random submission order, and bit-exact Max / Min under forced preemption with a concurrent GEMM stream."""
import json
import os
import subprocess

import numpy as np
import pytest
import torch

import dfccl_oracle as orc

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "dfccl_amd", "dfccl_bench")


def native(args, env=None, timeout=240):
    # the driver gives up on its own after 20 s (30 s here for the disordered run) and then tears the daemon down
    # in order; the limit below is only a last resort (a killed driver would leave the daemon kernel resident)
    e = dict(os.environ, DFCCL_DAEMON_MAX_MS="20000")
    e.update(env or {})
    out = subprocess.run([DRIVER] + [str(a) for a in args], env=e, capture_output=True, text=True, timeout=timeout)
    assert out.returncode == 0, out.stderr[-2000:]
    return json.loads(out.stdout.strip().splitlines()[-1])


@pytest.mark.parametrize("proto", ["direct", "fifo"])
def test_config3_disordered_256_collectives_no_deadlock(proto):
    # 256 registered fp16 all-reduces over 4 virtual ranks, sizes log-uniform 4 KiB..4 MiB, every rank submits in
    # its own random permutation; every element of every result is verified (inputs are rank + 1, sum = 10)
    r = native(["disorder", "--ranks", 4, "--colls", 256, "--dtype", "fp16", "--timeout", 30], {"DFCCL_PROTO": proto})
    assert r["deadlocks"] == 0 and r["correct"] is True
    assert r["cqes"] == 4 * 256


def test_config3_disordered_with_a_submission_queue_of_four_entries():
    # the same 256 disordered all-reduces with DFCCL_SQ_CAPACITY=4: the four submitting threads (C++, a fraction
    # of a microsecond per Run) find the queue full over and over, wait as ofcclRun* does in the reference
    # (src/collectives_ofccl/ofccl_all_reduce.cc:29-33), and nothing is lost: every submission completes, every
    # result is right.  How often the queue was found full depends on timing, so the count is only reported here
    # (the emulation scenario `backpressure`, where it is certain, asserts that it is positive).
    r = native(["disorder", "--ranks", 4, "--colls", 256, "--dtype", "fp16", "--timeout", 30], {"DFCCL_SQ_CAPACITY": "4"})
    assert r["deadlocks"] == 0 and r["correct"] is True
    assert r["cqes"] == 4 * 256
    assert r["sq_full_waits"] >= 0
    print("submissions that found the queue full:", r["sq_full_waits"])


@pytest.mark.parametrize("dtype", ["bf16", "int32"])
def test_config4_gradient_buckets_full_size(dtype):
    # 4 virtual ranks, 40 buckets of 25,000,000 elements, all submitted at once; results verified element by element
    r = native(["buckets", "--ranks", 4, "--colls", 40, "--elems", 25000000, "--dtype", dtype, "--iters", 1])
    assert r["correct"] is True


def test_config2_full_size_all_reduce_8_ranks_bf16():
    for proto in ("direct", "fifo"):
        r = native(["allreduce", "--ranks", 8, "--bytes", 64 << 20, "--dtype", "bf16", "--iters", 2],
                   {"DFCCL_PROTO": proto})
        assert r["correct"] is True and r["protocol"] == proto


def test_latency_mode_small_collectives_correct():
    r = native(["latency", "--ranks", 4, "--bytes", 4096, "--dtype", "fp16", "--iters", 200])
    assert r["correct"] is True and r["p50_us"] > 0


@pytest.mark.parametrize("proto", ["direct", "fifo"])
def test_config5_preemption_under_gemm_contention(proto, monkeypatch):
    # 8 virtual ranks, fp32 Max over 128 MiB and int8 Min over 128 MiB per rank, a bf16 8192^3 GEMM loop on another
    # stream, forced quit / resume every 64 slices; results bit-exact against torch's own max / min and against
    # the un-preempted run
    from dfccl_amd.ring import VirtualRing
    import dfccl_amd
    n = 8
    nf, ni = (128 << 20) // 4, 128 << 20
    g = torch.Generator(device="cuda:0").manual_seed(5)
    fsend = [torch.randn(nf, device="cuda:0", generator=g) for _ in range(n)]
    isend = [torch.randint(-128, 128, (ni,), device="cuda:0", generator=g, dtype=torch.int8) for _ in range(n)]
    fwant, iwant = fsend[0], isend[0]
    for r in range(1, n):
        fwant = torch.maximum(fwant, fsend[r])
        iwant = torch.minimum(iwant, isend[r])
    a = torch.randn(8192, 8192, device="cuda:0", dtype=torch.bfloat16)
    b = torch.randn(8192, 8192, device="cuda:0", dtype=torch.bfloat16)
    torch.cuda.synchronize()  # no daemon is resident yet
    monkeypatch.setenv("DFCCL_PROTO", proto)
    monkeypatch.setenv("DFCCL_DAEMON_MAX_MS", "20000")
    results = {}
    # a workgroup moves dozens of slices per collective here (direct: one 8 KiB tile per loop of the sweep; FIFO:
    # 15 ring steps of 2 slices per loop): the hook fires every 8 slices, so every workgroup is preempted several
    # times
    forced = "8"
    for force in ("0", forced):
        monkeypatch.setenv("DFCCL_FORCE_QUIT_EVERY", force)
        frecv = [torch.zeros_like(t) for t in fsend]
        irecv = [torch.zeros_like(t) for t in isend]
        torch.cuda.current_stream().synchronize()
        with VirtualRing(n) as ring:
            ring.prepare(0, "all_reduce", nf, dfccl_amd.ncclFloat32, dfccl_amd.ncclMax)
            ring.prepare(1, "all_reduce", ni, dfccl_amd.ncclInt8, dfccl_amd.ncclMin)
            ring.finalize()
            side = torch.cuda.Stream()
            with torch.cuda.stream(side):
                for _ in range(60):
                    c = a @ b
            for rep in range(2):
                for r in range(n):
                    ring.submit(r, 0, fsend[r], frecv[r])
                    ring.submit(r, 1, isend[r], irecv[r])
                ring.wait([(r, cid) for r in range(n) for cid in (0, 1)], timeout=40)
            stats = ring.stats()
            side.synchronize()
        results[force] = (frecv, irecv, stats)
        for r in range(n):
            assert torch.equal(frecv[r], fwant), (force, r)
            assert torch.equal(irecv[r], iwant), (force, r)
        del c
    assert results["0"][2]["forcedQuits"] == 0
    s = results[forced][2]
    assert s["forcedQuits"] > 0 and s["ctxSaves"] >= s["forcedQuits"]
    for r in range(n):  # preempted run == un-preempted run, bit for bit
        assert torch.equal(results["0"][0][r], results[forced][0][r])
        assert torch.equal(results["0"][1][r], results[forced][1][r])


# ---- the configurations at full size on their stated distributions ------------------------------------------
# Expected results come from tests/torch_ring.py: the ring's chunk -> owner geometry restated in torch integer
# arithmetic and a per-step-rounded fold in the ring's order with torch's own operations on the GPU (pinned
# against the CPU oracle in tests/test_torch_ring_cpu.py).  Bit-exact comparison.

def _normal(gen, n, dtype, sigma=1.0):
    return (torch.randn(n, device="cuda:0", generator=gen) * sigma).to(dtype)


@pytest.mark.parametrize("proto", ["direct", "fifo"])
def test_config2_full_size_normal_inputs_ring_order(proto, monkeypatch):
    # 8 virtual ranks x 64 MiB bf16, values normal(0, 1), Sum
    import dfccl_amd
    import torch_ring
    from dfccl_amd.ring import VirtualRing
    monkeypatch.setenv("DFCCL_PROTO", proto)
    n, count = 8, (64 << 20) // 2
    sends = [_normal(torch.Generator(device="cuda:0").manual_seed(2 + r), count, torch.bfloat16) for r in range(n)]
    recvs = [torch.zeros_like(s) for s in sends]
    torch.cuda.current_stream().synchronize()
    with VirtualRing(n) as ring:
        ring.prepare(0, "all_reduce", count, dfccl_amd.ncclBfloat16, dfccl_amd.ncclSum)
        ring.finalize()
        geom = ring.ctxs[0].geometry(0)
        ring.run(0, sends, recvs, timeout=40)
    want = torch_ring.all_reduce_expected(sends, geom, "sum")
    for r in range(n):
        assert torch_ring.same_bits(recvs[r], want), (proto, r)
    # and the 1-ulp-per-term bound against an fp64 sum, as a check of the check
    exact = torch.stack([s.double() for s in sends]).sum(0)
    err = (want.double() - exact).abs()
    scale = torch.stack([s.double().abs() for s in sends]).sum(0)
    assert bool((err <= (n - 1) * scale * 2.0 ** -8 + 1e-30).all())


def test_config3_full_size_disordered_normal_inputs_ring_order():
    # 256 registered fp16 all-reduces over 4 virtual ranks, sizes log-uniform in [4 KiB, 4 MiB] (multiples of
    # 16 bytes, one list for all ranks), values normal(0, 1), every rank submitting in its own random permutation
    import dfccl_amd
    import torch_ring
    from dfccl_amd.ring import VirtualRing
    n, ncolls = 4, 256
    rng = np.random.default_rng(3)
    sizes = np.exp(rng.uniform(np.log(4096), np.log(4 << 20), ncolls)).astype(np.int64) // 16 * 16
    sizes[0], sizes[1] = 4096, 4 << 20
    counts = [int(b) // 2 for b in sizes]
    sends, recvs = {}, {}
    for cid, count in enumerate(counts):
        sends[cid] = [_normal(torch.Generator(device="cuda:0").manual_seed(300 + cid * 4 + r), count, torch.float16)
                      for r in range(n)]
        recvs[cid] = [torch.zeros_like(s) for s in sends[cid]]
    torch.cuda.current_stream().synchronize()
    orders = [np.random.default_rng(30 + r).permutation(ncolls) for r in range(n)]
    with VirtualRing(n) as ring:
        for cid, count in enumerate(counts):
            ring.prepare(cid, "all_reduce", count, dfccl_amd.ncclFloat16, dfccl_amd.ncclSum)
        ring.finalize()
        geoms = [ring.ctxs[0].geometry(cid) for cid in range(ncolls)]
        # the ranks' submissions interleaved at random, each rank in its own order
        pick = np.random.default_rng(33)
        nxt = [0] * n
        left = n * ncolls
        while left:
            r = int(pick.integers(n))
            if nxt[r] == ncolls:
                continue
            cid = int(orders[r][nxt[r]])
            nxt[r] += 1
            left -= 1
            ring.submit(r, cid, sends[cid][r], recvs[cid][r])
        ring.wait([(r, cid) for r in range(n) for cid in range(ncolls)], timeout=60)
        stats = ring.stats()
    assert stats["cqesWritten"] == n * ncolls
    for cid in range(ncolls):
        want = torch_ring.all_reduce_expected(sends[cid], geoms[cid], "sum")
        for r in range(n):
            assert torch_ring.same_bits(recvs[cid][r], want), (cid, counts[cid], r)


@pytest.mark.parametrize("dtype", ["bf16", "int32"])
def test_config4_full_size_buckets_stated_distributions(dtype):
    # 4 virtual ranks, 40 buckets of 25,000,000 elements submitted at once: bf16 Sum on normal(0, 1e-3) against
    # the ring-order result, int32 Sum on uniform integers in [-2^20, 2^20] against the exact sum
    import dfccl_amd
    import torch_ring
    from dfccl_amd.ring import VirtualRing
    n, nb, count = 4, 40, 25_000_000
    sends, recvs = {}, {}
    for b in range(nb):
        gens = [torch.Generator(device="cuda:0").manual_seed((4 if dtype == "bf16" else 40) * 1000 + b * n + r)
                for r in range(n)]
        if dtype == "bf16":
            sends[b] = [_normal(g, count, torch.bfloat16, 1e-3) for g in gens]
        else:
            sends[b] = [torch.randint(-(1 << 20), (1 << 20) + 1, (count,), device="cuda:0", generator=g,
                                      dtype=torch.int32) for g in gens]
        recvs[b] = [torch.zeros_like(s) for s in sends[b]]
    torch.cuda.current_stream().synchronize()
    nccl_dtype = dfccl_amd.ncclBfloat16 if dtype == "bf16" else dfccl_amd.ncclInt32
    with VirtualRing(n) as ring:
        for b in range(nb):
            ring.prepare(b, "all_reduce", count, nccl_dtype, dfccl_amd.ncclSum)
        ring.finalize()
        geoms = [ring.ctxs[0].geometry(b) for b in range(nb)]
        for r in range(n):
            for b in range(nb):
                ring.submit(r, b, sends[b][r], recvs[b][r])
        ring.wait([(r, b) for r in range(n) for b in range(nb)], timeout=60)
    for b in range(nb):
        if dtype == "bf16":
            want = torch_ring.all_reduce_expected(sends[b], geoms[b], "sum")
        else:
            want = sends[b][0] + sends[b][1] + sends[b][2] + sends[b][3]  # exact: |sum| < 2^23
        for r in range(n):
            assert torch_ring.same_bits(recvs[b][r], want), (dtype, b, r)
        del want
