"""The planner's default channel count (host logic of the runtime, src/enqueue_ofccl.cc:85-149 in the reference):
the workgroup slots of the device, less a residency headroom, shared among the ranks, such that the launch's
rounding to whole sets of 8 channels still fits.  Runs against the host build of the runtime (tests/emul): only
Prepare and dfcclGetCollGeometry are called, no kernel is launched."""
import ctypes
import os
import shutil
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EMUL = os.path.join(HERE, "emul")
CLANG = "/opt/rocm/lib/llvm/bin/clang++"

pytestmark = pytest.mark.skipif(not os.path.exists(CLANG) or shutil.which("make") is None,
                                reason="needs the ROCm clang++ and make to build the host emulation")

PROBE = r"""
import ctypes, os, sys
sys.path.insert(0, %(root)r)
import dfccl_amd._lib as L
L.LIB_PATH = %(lib)r
from dfccl_amd import api
n, count = int(sys.argv[1]), int(sys.argv[2])
ctxs = [api.RankCtx(r) for r in range(n)]
comms = api.VirtualComm.create_all(n)
for r in range(n):
    ctxs[r].prepare_all_reduce(count, api.ncclBfloat16, api.ncclSum, comms[r], 0)
print(ctxs[0].geometry(0).nChannels)
"""


@pytest.fixture(scope="module")
def probe(tmp_path_factory):
    r = subprocess.run(["make", "-C", EMUL, "SAN=none", "-j4"], capture_output=True, text=True, timeout=1800)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    lib = os.path.join(EMUL, "_build", "none", "libdfccl_emul.so")
    script = tmp_path_factory.mktemp("share") / "probe.py"
    script.write_text(PROBE % {"root": os.path.dirname(HERE), "lib": lib})

    def run(n, count, **env):
        e = dict(os.environ)
        for k in ("NCCL_MAX_NCHANNELS", "DFCCL_RESIDENCY_HEADROOM", "DFCCL_PROTO"):
            e.pop(k, None)
        e.update({k: str(v) for k, v in env.items()})
        out = subprocess.run([sys.executable, str(script), str(n), str(count)], env=e, capture_output=True, text=True,
                             timeout=120)
        assert out.returncode == 0, out.stderr[-2000:]
        return int(out.stdout.strip().splitlines()[-1])
    return run


BIG = (64 << 20) // 2  # 64 MiB of bf16 per rank: never limited by the bytes-per-channel rule


@pytest.mark.parametrize("n,want", [(8, 31), (4, 62), (2, 64), (5, 48), (6, 40), (7, 32), (3, 64), (16, 15)])
def test_default_share_leaves_eight_slots_and_fits_the_rounded_launch(probe, n, want):
    # 256 slots (the emulated device reports 256 compute units, one workgroup each), 8 left out, at most 64 per rank
    got = probe(n, BIG)
    assert got == want
    assert n * got <= 256 - 8 or got == 1
    assert n * ((got + 7) // 8 * 8) <= 256  # what the launch rounds it to


def test_headroom_and_channel_knobs(probe):
    assert probe(8, BIG, DFCCL_RESIDENCY_HEADROOM=0) == 32
    assert probe(8, BIG, DFCCL_RESIDENCY_HEADROOM=64) == 24
    assert probe(8, BIG, NCCL_MAX_NCHANNELS=4) == 4
    assert probe(4, 2048) == 1  # small messages: one channel (the thread-shrink rule, src/enqueue_ofccl.cc:133-137)
