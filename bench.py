#!/usr/bin/env python3
"""Benchmark of the DFCCL data path on one MI355X.

Headline (the JSON line's `value`): the reduce-copy primitive, fp32 Sum of 2
sources at 256 MiB per buffer, in GB/s on (k+1)*N*sizeof(T) algorithmic bytes,
with inputs resident in HBM.  One "step" is one launch over the whole buffer.
The kernel is timed with HIP events on the stream it is launched on; the same
figure feeds the `roofline` object (bound: HBM, peak 8 TB/s).

Also reported on the same line: the CPU oracle's reduce-copy timed on this
host's cores (`cpu_baseline`, a bounded sample), the 8-virtual-rank bf16 ring
all-reduce through the daemon kernel (64 MiB per rank), the
submission-to-completion latency of 4 KiB all-reduces, the disordered
small-collective workload and the gradient-bucket workload (all four through
the native driver dfccl_amd/dfccl_bench, one host thread per virtual rank).
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
PROFILE_SUMMARY = os.path.join(ROOT, "profiles", "reduce_copy_f32_sum_k2_256MiB.md")
DAEMON_PROFILE_SUMMARY = os.path.join(ROOT, "profiles", "daemon_all_reduce_8x64MiB_bf16_pmc.md")


def measured_traffic_bytes():
    """HBM bytes per launch of the headline kernel as the rocprofv3 --pmc runs measured them (FETCH_SIZE and
    WRITE_SIZE, each scaled by what the counter reads for a plain copy of known size): the figure the profile
    summary records on its `traffic_bytes_per_launch:` line.  None if the summary is not there."""
    import re
    try:
        with open(PROFILE_SUMMARY) as f:
            m = re.search(r"^traffic_bytes_per_launch:\s*(\d+)", f.read(), re.M)
        return int(m.group(1)) if m else None
    except OSError:
        return None


def measured_daemon_traffic_bytes(label):
    """HBM bytes one 8 x 64 MiB bf16 all-reduce moved through the daemon under rocprofv3 --pmc (line
    `traffic_bytes_per_all_reduce_<label>:` of the daemon's profile summary).  None if no such run is recorded."""
    import re
    try:
        with open(DAEMON_PROFILE_SUMMARY) as f:
            m = re.search(r"^traffic_bytes_per_all_reduce_%s:\s*(\d+)" % re.escape(label), f.read(), re.M)
        return int(m.group(1)) if m else None
    except OSError:
        return None


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
    # The timed region: wall clock around K back-to-back launches, and one pair of HIP events on the launch stream
    # around the same K launches (the kernel's average launch duration = that interval / K; it includes the gaps
    # between launches).  No events between the launches: an event record is a packet of its own on the queue and
    # costs the next kernel several microseconds.
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    first.record(stream)
    for _ in range(steps):
        dfccl_amd.reduce_copy(srcs, dst, dfccl_amd.ncclSum)
    last.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kernel_ms_avg = first.elapsed_time(last) / steps
    # outside the timed region: every launch bracketed by its own events, for the shortest single launch
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in evs:
        a.record(stream)
        dfccl_amd.reduce_copy(srcs, dst, dfccl_amd.ncclSum)
        b.record(stream)
    torch.cuda.synchronize()
    kernel_ms = [a.elapsed_time(b) for a, b in evs]
    ok = bool(torch.equal(dst, srcs[0] + srcs[1])) if k == 2 else bool(torch.equal(dst, srcs[0]))
    alg_bytes = (k + 1) * nbytes
    return {"wall_s": wall, "kernel_ms_avg": kernel_ms_avg, "kernel_ms_min": min(kernel_ms),
            "kernel_ms_avg_bracketed": sum(kernel_ms) / len(kernel_ms),
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


NATIVE_DRIVER = os.path.join(ROOT, "dfccl_amd", "dfccl_bench")


def run_native(args, env=None, timeout=180):
    """Runs one mode of the native driver (dfccl_amd/csrc/bench/dfccl_bench.cc: one host thread per virtual rank,
    public C ABI only) and returns its JSON object."""
    import subprocess
    if not os.path.exists(NATIVE_DRIVER):
        raise RuntimeError(f"{NATIVE_DRIVER} is missing: run __graft_entry__.build()")
    e = dict(os.environ)
    e.setdefault("DFCCL_DAEMON_MAX_MS", "20000")
    if env:
        e.update(env)
    out = subprocess.run([NATIVE_DRIVER] + [str(a) for a in args], env=e, capture_output=True, text=True,
                         timeout=timeout)
    if out.returncode != 0:
        raise RuntimeError(f"dfccl_bench {args} failed: {out.stderr[-500:]}")
    return json.loads(out.stdout.strip().splitlines()[-1])


def bench_daemon_all_reduce():
    """Ring all-reduce over 8 virtual ranks, bf16 Sum, 64 MiB per rank, through the daemon kernel: once with
    the library's defaults (direct protocol, 8 KiB tiles) and once as the FIFO ring with 512 KiB
    chunks. GB/s figures are on the bytes the respective schedule moves."""
    n, nbytes = 8, 64 << 20
    res = {}
    for label, env in (("direct", {"DFCCL_PROTO": "direct"}), ("fifo_512KiB_chunks", {"DFCCL_PROTO": "fifo"})):
        r = run_native(["allreduce", "--ranks", n, "--bytes", nbytes, "--dtype", "bf16", "--iters", 10], env)
        res[label] = {"ms": r["best_ms"], "median_ms": r["median_ms"], "algbw_GBps": r["algbw_GBps"],
                      "busbw_GBps": r["busbw_GBps"], "moved_GBps": r["moved_GBps"],
                      "frac_of_hbm_peak": round(r["moved_GBps"] / HBM_PEAK_GBPS, 4), "channels": r["channels"],
                      "chunk_bytes": r["chunk_bytes"], "correct": r["correct"], "ctx_saves": r["ctx_saves"]}
    res["workload"] = f"ring all-reduce, {n} virtual ranks x {nbytes >> 20} MiB bf16 Sum (time: submit on all ranks -> last callback)"
    return res


def daemon_roofline(ar):
    """The daemon's data movement against the HBM roofline, per protocol: algorithmic bytes of the schedule
    (direct: every input read once and every output written once, 2 * n * N * s; FIFO ring: (6n - 4) / n * N * s
    per rank), the best time from submission on all ranks to the last callback, and the fraction of the 8 TB/s
    peak that makes."""
    n, nbytes = 8, 64 << 20
    out = {"bound": "hbm", "peak": HBM_PEAK_GBPS, "unit": "GB/s", "kernel": "dfcclDaemonKernel"}
    for label, alg in (("direct", 2 * n * nbytes), ("fifo_512KiB_chunks", (6 * n - 4) * nbytes)):
        ms = ar[label]["ms"]
        gbps = alg / (ms * 1e-3) / 1e9
        out[label] = {"bytes": alg, "ms": ms, "achieved": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4),
                      "traffic": measured_daemon_traffic_bytes(label.split("_")[0])}
    return out


def bench_latency():
    """SQE->CQE interval of 4 KiB fp16 all-reduces over 4 virtual ranks (taken inside the library: entry
    written -> completion seen by the poller), all ranks submitting together."""
    r = run_native(["latency", "--ranks", 4, "--bytes", 4096, "--dtype", "fp16", "--iters", 2000])
    return {"workload": "4 virtual ranks, 4096 B fp16 Sum all-reduce, one host thread per rank",
            "p50_us": r["p50_us"], "p90_us": r["p90_us"], "p99_us": r["p99_us"], "min_us": r["min_us"],
            "correct": r["correct"]}


def bench_disordered():
    """256 registered fp16 all-reduces (4 KiB .. 4 MiB, log-uniform) over 4 virtual ranks, every rank submitting
    in its own random order."""
    r = run_native(["disorder", "--ranks", 4, "--colls", 256, "--dtype", "fp16"])
    return {"workload": "256 all-reduces, 4 virtual ranks, sizes log-uniform 4 KiB..4 MiB fp16, per-rank random order",
            "deadlocks": r["deadlocks"], "correct": r["correct"], "wall_ms": r["wall_ms"], "p50_us": r["p50_us"],
            "p99_us": r["p99_us"],
            # the latency this configuration is quoted on: SQE->CQE p50 of its smallest collectives (4..8 KiB),
            # submitted among all the others in every rank's own order
            "small_bucket_p50_us": r["small_bucket_p50_us"], "small_bucket_count": r["small_bucket_count"],
            "preemptions": r["preemptions_ctx_saves"], "completions": r["cqes"]}


def bench_buckets():
    """40 gradient buckets of 25M elements over 4 virtual ranks, all submitted at once: bf16 Sum, then int32 Sum."""
    out = {}
    for dt in ("bf16", "int32"):
        r = run_native(["buckets", "--ranks", 4, "--colls", 40, "--elems", 25000000, "--dtype", dt, "--iters", 3],
                       timeout=300)
        out[dt] = {"ms": r["best_ms"], "algbw_GBps": r["algbw_GBps"], "moved_GBps": r["moved_GBps"],
                   "correct": r["correct"], "ctx_saves": r["ctx_saves"], "protocol": r["protocol"]}
    return out


def bench_other_collectives():
    """Reduce-scatter, all-gather, reduce and broadcast over 8 virtual ranks (bf16; 8 MiB per rank block for the
    first two, 64 MiB messages for the other two) through the daemon, direct protocol. GB/s on the bytes the direct
    protocol moves (every input read once, every output written once)."""
    out = {}
    for kind in ("reduce_scatter", "all_gather", "reduce", "broadcast"):
        nbytes = (8 << 20) if kind in ("reduce_scatter", "all_gather") else (64 << 20)
        r = run_native(["collective", "--kind", kind, "--ranks", 8, "--bytes", nbytes, "--dtype", "bf16",
                        "--iters", 10])
        out[kind] = {"ms": r["best_ms"], "traffic_GBps": r["direct_traffic_GBps"], "protocol": r["protocol"],
                     "channels": r["channels"], "count_bytes": r["count_bytes"], "correct": r["correct"]}
    return out


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
                     "frac": round(gbps_kernel / HBM_PEAK_GBPS, 4), "traffic": measured_traffic_bytes(),
                     "kernel": "reduceCopyKernel<7,0,2,false> (fp32, Sum, 2 sources, unscaled)", "kernel_ms_avg": round(rc["kernel_ms_avg"], 5),
                     "kernel_ms_min": round(rc["kernel_ms_min"], 5),
                     "kernel_ms_avg_each_launch_bracketed_by_events": round(rc["kernel_ms_avg_bracketed"], 5)},
    }
    if not args.skip_daemon:
        # (a leg that fails is reported as such: the headline above does not depend on it)
        def leg(name, fn, *a):
            try:
                line[name] = fn(*a)
            except Exception as e:  # noqa: BLE001
                line[name] = {"error": f"{type(e).__name__}: {e}"[:500]}
                print(f"bench.py: {name} failed: {e}", file=sys.stderr)
        leg("daemon_all_reduce", bench_daemon_all_reduce)
        if "error" not in line["daemon_all_reduce"]:
            leg("daemon_roofline", daemon_roofline, line["daemon_all_reduce"])
        leg("sqe_to_cqe_latency", bench_latency)
        leg("disordered_small_collectives", bench_disordered)
        leg("gradient_buckets", bench_buckets)
        leg("other_collectives", bench_other_collectives)
    if not args.skip_cpu:
        line["cpu_baseline"] = bench_cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
