#!/usr/bin/env python3
"""Benchmark of the DFCCL data path on one MI355X.

Headline (the JSON line's `value`): the reduce-copy primitive, fp32 Sum of 2
sources at 256 MiB per buffer, in GB/s on (k+1)*N*sizeof(T) algorithmic bytes,
with inputs resident in HBM.  One "step" is one launch over the whole buffer.
The kernel is timed with HIP events on the stream it is launched on; the same
figure feeds the `roofline` object (bound: HBM, peak 8 TB/s).

Also reported on the same line: the CPU oracle's reduce-copy timed on this
host's cores (`cpu_baseline`, a bounded sample), the 8-virtual-rank bf16 ring
all-reduce through the daemon kernel (64 MiB per rank), and the
submission-to-completion latency of 4 KiB all-reduces.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "oracle"))

HBM_PEAK_GBPS = 8000.0


def bench_reduce_copy(steps, warmup, nbytes=256 << 20, k=2):
    import torch
    import dfccl_amd
    n = nbytes // 4
    g = torch.Generator(device="cuda:0").manual_seed(1)
    srcs = [torch.rand(n, device="cuda:0", generator=g) * 2 - 1 for _ in range(k)]
    dst = torch.empty(n, device="cuda:0")
    stream = torch.cuda.current_stream()
    for _ in range(warmup):
        dfccl_amd.reduce_copy(srcs, dst, dfccl_amd.ncclSum)
    stream.synchronize()
    torch.cuda.synchronize()
    # whole timed region: wall clock around K launches, HIP events on the launch stream inside it
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for a, b in evs:
        a.record(stream)
        dfccl_amd.reduce_copy(srcs, dst, dfccl_amd.ncclSum)
        b.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kernel_ms = [a.elapsed_time(b) for a, b in evs]
    ok = bool(torch.equal(dst, srcs[0] + srcs[1])) if k == 2 else bool(torch.equal(dst, srcs[0]))
    alg_bytes = (k + 1) * nbytes
    return {"wall_s": wall, "kernel_ms_avg": sum(kernel_ms) / len(kernel_ms), "kernel_ms_min": min(kernel_ms),
            "alg_bytes": alg_bytes, "correct": ok}


def bench_cpu_baseline(budget_s=12.0, nbytes=256 << 20):
    """The oracle's reduce-copy (same fp32 Sum, k = 2, same buffer size) on this host's cores."""
    import numpy as np
    import dfccl_oracle as orc
    n = nbytes // 4
    rng = np.random.default_rng(1)
    srcs = [rng.random(n, dtype=np.float32) * 2 - 1 for _ in range(2)]
    cores = len(os.sched_getaffinity(0))
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)) or cores)
    alg = 3 * nbytes
    out = {}
    for label, threads in (("single", 1), ("all", cores)):
        orc.reduce_copy(orc.F32, orc.SUM, srcs, nthreads=threads)  # warm-up
        best, t_end, reps = None, time.perf_counter() + budget_s / 2, 0
        while reps < 5 or (time.perf_counter() < t_end and reps < 40):
            t0 = time.perf_counter()
            orc.reduce_copy(orc.F32, orc.SUM, srcs, nthreads=threads)
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
            reps += 1
            if time.perf_counter() > t_end and reps >= 5:
                break
        out[label] = (alg / best / 1e9, threads, reps)
    return {"value": round(out["all"][0], 2), "unit": "GB/s", "cores": out["all"][1], "kind": "port",
            "sample": (f"oracle reduce-copy, fp32 Sum, 2 sources x 256 MiB, best of {out['all'][2]} runs on "
                       f"{out['all'][1]} threads; single thread: {out['single'][0]:.2f} GB/s")}


def bench_daemon_all_reduce(iters=6, n=8, nbytes=64 << 20):
    """Config: ring all-reduce over 8 virtual ranks, bf16 Sum, 64 MiB per rank, through the daemon."""
    import torch
    import dfccl_amd
    from dfccl_amd.ring import VirtualRing
    count = nbytes // 2
    g = torch.Generator(device="cuda:0").manual_seed(2)
    sends = [torch.randn(count, device="cuda:0", generator=g).to(torch.bfloat16) for _ in range(n)]
    recvs = [torch.empty_like(s) for s in sends]
    torch.cuda.current_stream().synchronize()
    times = []
    with VirtualRing(n) as ring:
        ring.prepare(0, "all_reduce", count, dfccl_amd.ncclBfloat16, dfccl_amd.ncclSum)
        ring.finalize()
        geom = ring.ctxs[0].geometry(0)
        for i in range(iters + 2):
            t0 = time.perf_counter()
            ring.run(0, sends, recvs, timeout=60)
            dt = time.perf_counter() - t0
            if i >= 2:
                times.append(dt)
        stats = ring.stats()
    ref = sends[0].float()
    for s in sends[1:]:
        ref = ref + s.float()
    err = (recvs[0].float() - ref).abs().max().item()
    same = all(torch.equal(recvs[0], r) for r in recvs[1:])
    best = min(times)
    # bytes the ring schedule moves: per rank (6n-4)/n * N * s (FIFO write and read counted)
    sched_bytes = (6 * n - 4) / n * nbytes * n
    return {"workload": f"ring all-reduce, {n} virtual ranks x {nbytes >> 20} MiB bf16 Sum, "
                        f"{geom.chunkElems * 2 >> 10} KiB chunks, {geom.nChannels} channels/rank",
            "ms": round(best * 1e3, 3), "algbw_GBps": round(nbytes / best / 1e9, 1),
            "busbw_GBps": round(nbytes / best / 1e9 * 2 * (n - 1) / n, 1),
            "schedule_GBps": round(sched_bytes / best / 1e9, 1),
            "frac_of_hbm_peak": round(sched_bytes / best / 1e9 / HBM_PEAK_GBPS, 4),
            "ranks_agree": same, "max_abs_err_vs_fp32_sum": err, "ctx_saves": stats["ctxSaves"]}


def bench_latency(n=4, count=2048, iters=300):
    """Submission-to-completion time of 4 KiB fp16 all-reduces over 4 virtual ranks, measured around the
    Python submit / callback pair of the last-submitting rank (includes ctypes overhead)."""
    import torch
    import dfccl_amd
    from dfccl_amd.ring import VirtualRing
    sends = [torch.ones(count, device="cuda:0", dtype=torch.float16) for _ in range(n)]
    recvs = [torch.empty_like(s) for s in sends]
    torch.cuda.current_stream().synchronize()
    lat = []
    with VirtualRing(n) as ring:
        ring.prepare(0, "all_reduce", count, dfccl_amd.ncclFloat16, dfccl_amd.ncclSum)
        ring.finalize()
        for i in range(iters + 20):
            ring.run(0, sends, recvs, timeout=30)
            if i >= 20:
                last = (n - 1, 0)
                lat.append((ring.t_done[last] - ring.t_submit[last]) * 1e6)
    lat.sort()
    return {"workload": f"{n} virtual ranks, {count * 2} B fp16 all-reduce, last submitter's submit->callback",
            "p50_us": round(lat[len(lat) // 2], 2), "p90_us": round(lat[int(len(lat) * 0.9)], 2),
            "p99_us": round(lat[int(len(lat) * 0.99)], 2), "min_us": round(lat[0], 2)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--skip-daemon", action="store_true", help="skip the daemon legs")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch the 1-source copy kernel on the same buffers (known traffic: 2*N*sizeof), "
                         "used to scale the HBM byte counters of a profiler run")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; virtual ranks share it, so --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    os.environ.setdefault("DFCCL_DAEMON_MAX_MS", "20000")

    rc = bench_reduce_copy(args.steps, args.warmup)
    if args.copy_calibration:
        bench_reduce_copy(args.steps, 1, k=1)
    gbps_kernel = rc["alg_bytes"] / (rc["kernel_ms_avg"] * 1e-3) / 1e9
    gbps_wall = rc["alg_bytes"] * args.steps / rc["wall_s"] / 1e9
    line = {
        "metric": "reduce-copy GB/s at 256 MiB per buffer",
        "value": round(gbps_wall, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(rc["wall_s"] / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "reduce-copy fp32 Sum, 2 sources -> 1 destination, 67108864 elements "
                               "(256 MiB per buffer, 768 MiB algorithmic traffic per step)",
                   "bytes_counted": "(k+1)*N*sizeof(T)", "correct": rc["correct"]},
        "frac_of_hbm_peak": round(gbps_wall / HBM_PEAK_GBPS, 4),
        "roofline": {"bound": "hbm", "achieved": round(gbps_kernel, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps_kernel / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "reduceCopyKernel<f32,Sum,2>", "kernel_ms_avg": round(rc["kernel_ms_avg"], 5),
                     "kernel_ms_min": round(rc["kernel_ms_min"], 5)},
    }
    if not args.skip_daemon:
        line["daemon_all_reduce"] = bench_daemon_all_reduce()
        line["sqe_to_cqe_latency"] = bench_latency()
    if not args.skip_cpu:
        line["cpu_baseline"] = bench_cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
