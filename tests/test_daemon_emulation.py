"""The daemon kernel's own source, compiled for the host and run with one OS thread per GPU thread
(tests/emul/): scheduling, preemption, both protocols and the relaunch path without a GPU.

What these runs can show that the GPU suite cannot show safely: a workgroup whose threads meet at different
__syncthreads() (reported with both source lines; on the GPU that is a hang), a run that stops moving (every
thread's position is printed) and, in the sanitizer builds (make -C tests/emul SAN=thread|address), races on LDS
and bad addresses.  Random delays after barriers (EMUL_JITTER) let waves drift apart as they do on the GPU."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EMUL = os.path.join(HERE, "emul")
CLANG = "/opt/rocm/lib/llvm/bin/clang++"

pytestmark = pytest.mark.skipif(not os.path.exists(CLANG) or shutil.which("make") is None,
                                reason="needs the ROCm clang++ and make to build the host emulation")


# EMUL_SAN=thread or EMUL_SAN=address runs the same scenarios in a sanitizer build (several times slower); any
# sanitizer report fails the scenario.
SAN = os.environ.get("EMUL_SAN", "none")
SLOW = 1 if SAN == "none" else 8


# Which sources the emulation has validated: when every test of this file has passed in one session, the hash of
# the kernel and runtime sources is recorded in tests/emul/validated_sources.stamp.  The GPU suite refuses to start
# on a real GPU while that record names other sources (tests/conftest.py): a persistent kernel that goes wrong hangs
# or faults the GPU, so no build of it goes there before it has run here.
STAMP = os.path.join(EMUL, "validated_sources.stamp")
PASSED = set()


def sources_hash():
    import hashlib
    csrc = os.path.join(os.path.dirname(HERE), "dfccl_amd", "csrc")
    files = sorted(os.path.join(csrc, f) for f in os.listdir(csrc) if f.endswith((".hip", ".h")))
    files.append(os.path.join(os.path.dirname(HERE), "include", "ofccl.h"))
    h = hashlib.sha256()
    for f in files:
        h.update(os.path.basename(f).encode() + b"\0")
        h.update(open(f, "rb").read())
    return h.hexdigest()


@pytest.fixture(scope="module")
def stress():
    r = subprocess.run(["make", "-C", EMUL, f"SAN={SAN}", "-j4"], capture_output=True, text=True, timeout=1800)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    return os.path.join(EMUL, "_build", SAN, "emul_stress")


def sanitizer_env(e, leaks=True):
    e["TSAN_OPTIONS"] = "halt_on_error=0 report_signal_unsafe=0"
    e["ASAN_OPTIONS"] = "detect_leaks=1" if leaks else "detect_leaks=0"
    return e


def no_sanitizer_report(r):
    out = r.stdout + r.stderr
    return "WARNING: ThreadSanitizer" not in out and "ERROR: AddressSanitizer" not in out and \
        "ERROR: LeakSanitizer" not in out


TINY = {"BASE_CTX_SWITCH_THRESHOLD": "1", "NUM_TRY_TASKQ_HEAD": "1", "RECV_SUCCESS_FACTOR": "0"}

SCENARIOS = [
    # the same small all-reduces over and over, ranks submitted in turn (one tile per rank: wave 0 runs them
    # alone), then with every bounded wait giving up after one look, then too large for a wave on its own
    ("repeat-default", {}, ["repeat", "4", "2048", "12", "2"]),
    ("repeat-tiny-budget", TINY, ["repeat", "4", "2048", "20", "2"]),
    ("repeat-whole-workgroup", {}, ["repeat", "4", "6000", "8", "2"]),
    ("repeat-tiny-budget-ragged", TINY, ["repeat", "3", "5000", "6", "2"]),
    ("repeat-8-ranks", {}, ["repeat", "8", "2048", "4", "1"]),
    ("repeat-several-channels", {"NCCL_MAX_NCHANNELS": "8"}, ["repeat", "2", "300000", "2", "1"]),
    # the traced build of the kernel (DFCCL_TRACE=1): same scheduler, with the timeline stamps compiled in
    ("repeat-traced", {"DFCCL_TRACE": "1", "DFCCL_TRACE_FILE": "/dev/null"}, ["repeat", "4", "2048", "6", "2"]),
    ("mixed-fifo-traced", {"DFCCL_TRACE": "1", "DFCCL_TRACE_FILE": "/dev/null", "DFCCL_PROTO": "fifo"}, ["mixed", "3", "1"]),
    # all five collectives side by side, ranks submit in different orders
    ("mixed-direct", {}, ["mixed", "4", "2"]),
    ("mixed-direct-tiny-budget", TINY, ["mixed", "4", "2"]),
    ("mixed-fifo", {"DFCCL_PROTO": "fifo"}, ["mixed", "3", "2"]),
    ("mixed-fifo-tiny-budget", dict(TINY, DFCCL_PROTO="fifo"), ["mixed", "3", "2"]),
    # FIFO links of two and of eight slices instead of the reference's four
    ("mixed-fifo-2-slots", {"DFCCL_PROTO": "fifo", "DFCCL_FIFO_SLOTS": "2"}, ["mixed", "3", "1"]),
    ("mixed-fifo-8-slots", {"DFCCL_PROTO": "fifo", "DFCCL_FIFO_SLOTS": "8"}, ["mixed", "3", "1"]),
    # forced preemption after every slice / tile
    ("forced-direct", {"DFCCL_FORCE_QUIT_EVERY": "1"}, ["repeat", "2", "40000", "2", "1"]),
    ("forced-fifo", {"DFCCL_FORCE_QUIT_EVERY": "2", "DFCCL_PROTO": "fifo"}, ["repeat", "3", "40000", "2", "1"]),
    # idle exit and relaunch, also with a collective parked
    ("relaunch", {"TOLERANT_UNPROGRESSED_CNT": "200"}, ["relaunch", "2"]),
    # a daemon that leaves every 50 ms, whatever it is doing, and is launched again: state saved and restored
    ("short-lifetime-direct", {"DFCCL_DAEMON_MAX_MS": "50"}, ["mixed", "4", "2"]),
    ("short-lifetime-fifo", {"DFCCL_DAEMON_MAX_MS": "50", "DFCCL_PROTO": "fifo"}, ["mixed", "3", "2"]),
    ("short-lifetime-small", {"DFCCL_DAEMON_MAX_MS": "50"}, ["repeat", "4", "2048", "20", "2"]),
    # random ranks, collectives, sizes, roots and submission orders (three rounds each)
    ("random-direct", {"NCCL_MAX_NCHANNELS": "2"}, ["fuzz", "1003", "3"]),
    ("random-fifo-short-lifetime", {"NCCL_MAX_NCHANNELS": "2", "DFCCL_PROTO": "fifo", "DFCCL_DAEMON_MAX_MS": "57"},
     ["fuzz", "1007", "3"]),
    ("random-tiny-budget", dict(TINY, NCCL_MAX_NCHANNELS="2"), ["fuzz", "1012", "3"]),
    # rank contexts destroyed and created again on the same daemon; a communicator that has run is refused
    ("reuse", {}, ["reuse", "3"]),
    # the queues' back-pressure: a submission queue of 4 entries under two submitting threads per rank and a late
    # rank (the full-queue path and the lazily published head), then the full-size queue with a callback that
    # sleeps 2 ms on the poller thread; every submission gets exactly one callback
    ("backpressure-small-queue", {"DFCCL_SQ_CAPACITY": "4"}, ["backpressure", "3", "24", "3", "0"]),
    ("backpressure-small-queue-channels", {"DFCCL_SQ_CAPACITY": "3", "NCCL_MAX_NCHANNELS": "2",
                                           "DFCCL_BYTES_PER_CHANNEL": "512"}, ["backpressure", "2", "16", "3", "0"]),
    ("backpressure-slow-callback", {}, ["backpressure", "2", "40", "2", "2000"]),
    # one ring busy, the other's workgroups gone for idleness: its next submission still gets through
    ("two-rings-idle-exit", {"TOLERANT_UNPROGRESSED_CNT": "300"}, ["tworings", "2"]),
]


@pytest.mark.parametrize("name,env,args", SCENARIOS, ids=[s[0] for s in SCENARIOS])
def test_emulated_daemon(stress, name, env, args):
    e = dict(os.environ)
    for k in ("DFCCL_PROTO", "DFCCL_FORCE_QUIT_EVERY", "BASE_CTX_SWITCH_THRESHOLD"):
        e.pop(k, None)
    e.update({"EMUL_JITTER": "30", "EMUL_WATCHDOG_S": "120", "DFCCL_DAEMON_MAX_MS": "100000"})
    e.update(env)
    r = subprocess.run([stress] + args, env=sanitizer_env(e), capture_output=True, text=True, timeout=300 * SLOW)
    assert r.returncode == 0, f"{name}: rc={r.returncode}\n{r.stdout[-2000:]}\n{r.stderr[-4000:]}"
    assert " ok" in r.stdout
    assert no_sanitizer_report(r), r.stderr[-6000:]
    PASSED.add(name)


def test_a_daemon_that_never_leaves_ends_the_process_with_a_report(stress):
    # the workgroups ignore every reason to leave (a host-side stand-in for a workgroup stuck at a barrier):
    # Destroy waits, aborts, waits again, then prints what it knows and ends the process instead of joining a
    # thread that waits for the kernel and freeing memory the kernel still uses
    e = dict(os.environ)
    e.update({"EMUL_JITTER": "30", "EMUL_WATCHDOG_S": "120", "EMUL_NEVER_LEAVE": "1", "DFCCL_DESTROY_WAIT_MS": "1500",
              "DFCCL_ABORT_WAIT_MS": "1500"})
    r = subprocess.run([stress, "stuck", "2"], env=sanitizer_env(e, leaks=False), capture_output=True, text=True,
                       timeout=120 * SLOW)
    assert r.returncode == 70, f"rc={r.returncode}\n{r.stdout[-2000:]}\n{r.stderr[-4000:]}"
    assert "still resident after an abort request" in r.stderr
    assert "ofcclDestroy returned" not in r.stdout
    PASSED.add("stuck")


DRIVER_ENV = {"disorder-small-queue": {"DFCCL_SQ_CAPACITY": "4"}}
DRIVER = [
    # the native driver of the timing workloads on the emulation: per-rank host threads submit in different
    # orders (disorder) or in bursts (buckets); the driver checks every result itself
    ("disorder", ["disorder", "--ranks", "4", "--colls", "16", "--min-bytes", "4096", "--max-bytes", "65536",
                  "--timeout", "250"]),
    ("disorder-small-queue", ["disorder", "--ranks", "3", "--colls", "24", "--min-bytes", "4096", "--max-bytes", "16384",
                              "--timeout", "250"]),
    ("buckets", ["buckets", "--ranks", "4", "--colls", "6", "--elems", "20000", "--dtype", "bf16", "--iters", "1",
                 "--warmup", "0", "--timeout", "250"]),
    ("latency-8-ranks", ["latency", "--ranks", "8", "--bytes", "4096", "--dtype", "fp16", "--iters", "3", "--warmup", "1",
                         "--timeout", "250"]),
]


@pytest.mark.parametrize("name,args", DRIVER, ids=[d[0] for d in DRIVER])
def test_emulated_daemon_under_the_native_driver(stress, name, args):
    import json
    e = dict(os.environ)
    e.update({"EMUL_JITTER": "30", "EMUL_WATCHDOG_S": "120", "DFCCL_DAEMON_MAX_MS": "100000"})
    e["DFCCL_STATS_WAIT_MS"] = "5000"  # emulated workgroups answer a request for their counters slowly
    e.update(DRIVER_ENV.get(name, {}))
    exe = os.path.join(os.path.dirname(stress), "dfccl_bench_emul")
    # (the benchmark driver leaves its buffers to the end of the process)
    r = subprocess.run([exe] + args, env=sanitizer_env(e, leaks=False), capture_output=True, text=True,
                       timeout=300 * SLOW)
    assert r.returncode == 0, f"{name}: rc={r.returncode}\n{r.stdout[-2000:]}\n{r.stderr[-4000:]}"
    assert no_sanitizer_report(r), r.stderr[-6000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert out["correct"] is True
    if name.startswith("disorder"):
        assert out["deadlocks"] == 0
    if name == "disorder-small-queue":
        assert out["sq_full_waits"] > 0 and out["cqes"] == 3 * 24
    PASSED.add("driver-" + name)


@pytest.mark.skipif(SAN != "none", reason="python cannot load a sanitizer build of the library without its runtime preloaded")
def test_parity_tests_on_the_emulation(stress):
    """A slice of the GPU parity suite (tests/test_daemon_gpu.py, tests/test_golden.py) with the emulated library
    in place of the GPU one and the buffers in host memory: same tests, same oracle, same bit-exact bar.  The
    whole of those two files runs this way in about five minutes:
        DFCCL_TESTS_ON_EMULATION=tests/emul/_build/none/libdfccl_emul.so python -m pytest tests/test_daemon_gpu.py
        tests/test_golden.py -m gpu"""
    import sys
    e = dict(os.environ)
    e.update({"DFCCL_TESTS_ON_EMULATION": os.path.join(os.path.dirname(stress), "libdfccl_emul.so"),
              "EMUL_JITTER": "30", "EMUL_WATCHDOG_S": "120"})
    pick = ("test_small_all_reduce_and_in_place or test_in_place_and_absent_buffers or golden or "
            "test_other_collectives_disordered or test_rank_by_rank or forced_preemption or avg_small_and_ragged or "
            "premul_sum or nan_operands or empty_collectives")
    r = subprocess.run([sys.executable, "-m", "pytest", os.path.join(HERE, "test_daemon_gpu.py"),
                        os.path.join(HERE, "test_golden.py"), "-q", "-m", "gpu", "-x", "-p", "no:cacheprovider",
                        "--timeout", "600", "-k", pick], env=e, capture_output=True, text=True, timeout=1200,
                       cwd=os.path.dirname(HERE))
    tail = r.stdout[-3000:] + r.stderr[-2000:]
    assert r.returncode == 0, tail
    assert " passed" in r.stdout and " failed" not in r.stdout, tail
    PASSED.add("parity")


def test_zz_record_the_sources_the_emulation_has_validated():
    """Last in this file: if every scenario above has passed in this session (none deselected), the sources they
    ran are recorded as validated."""
    want = {s[0] for s in SCENARIOS} | {"stuck"} | {"driver-" + d[0] for d in DRIVER}
    if SAN == "none":
        want.add("parity")
    missing = want - PASSED
    if missing:
        pytest.skip(f"not every scenario ran in this session (missing: {sorted(missing)[:4]}...): no record written")
    with open(STAMP, "w") as f:
        f.write(sources_hash() + "\n")
