"""Register and memory budget of the compiled kernels, from the compiler's own per-kernel remarks
(-Rpass-analysis=kernel-resource-usage, written to dfccl_amd/csrc/<source>.resources by the device compile).

The daemon is a persistent kernel whose workgroups wait for each other: every one of them has to be resident
(one 512-thread workgroup per compute unit), nothing may live in scratch memory (a persistent kernel that spills
vector registers holds its scratch for good, and private-memory traffic sits on the scheduler's serial path), and
builds with more vector registers than any build that has completed the GPU test suite do not go to a GPU before
that bound is raised here on purpose.  Scalar-register spills go to vector-register lanes (v_writelane /
v_readlane); they are recorded, and bounded so that growth is noticed."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "dfccl_amd", "csrc")

# Vector registers: the largest count of a build of this kernel that has completed the whole GPU suite.  (At 128
# or fewer, four waves per SIMD fit, i.e. a second workgroup per compute unit; the daemon places one per unit, so
# either side of that line is resident.)
DAEMON_MAX_VGPRS = 133
# Scalar spills, counted statically over every inlined variant of the data movers (one per element type,
# operator and source count: some 200 of them); a wave runs through the few that belong to the variant it
# executes.  The bound is there so that growth is noticed.
DAEMON_MAX_SGPR_SPILLS = 3000
# the traced build of the same file (DFCCL_TRACE=1 launches it) carries the timeline stamps and may be larger, but
# has to stay resident as a whole too
TRACED_MAX_VGPRS = 168


def resources(source, hip_file=None):
    """{kernel name: {field: value}} of one object (`source`.o, built from `hip_file`.hip, by default the file of
    the same name); compiles the object if its remarks are missing or stale."""
    src = os.path.join(CSRC, (hip_file or source) + ".hip")
    res = os.path.join(CSRC, source + ".resources")
    deps = [src] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    if not os.path.exists(res) or os.path.getmtime(res) < max(os.path.getmtime(d) for d in deps):
        subprocess.check_call(["make", "-B", "-C", CSRC, source + ".o"], stdout=subprocess.DEVNULL,
                              stderr=subprocess.DEVNULL)
    out, cur = {}, None
    for line in open(res):
        key, _, val = line.strip().partition(": ")
        if key == "Function Name":
            cur = out.setdefault(val, {})
        elif cur is not None:
            cur[key] = val
    return out


def test_daemon_kernel_fits_one_workgroup_per_cu_without_scratch(record_property):
    k = resources("daemon")["dfcclDaemonKernel"]
    for field in ("VGPRs", "AGPRs", "TotalSGPRs", "SGPRs Spill", "VGPRs Spill", "ScratchSize [bytes/lane]",
                  "Occupancy [waves/SIMD]", "LDS Size [bytes/block]"):
        record_property(field, k[field])
    print("dfcclDaemonKernel:", k)
    assert int(k["ScratchSize [bytes/lane]"]) == 0 and k["Dynamic Stack"] == "False"
    assert int(k["VGPRs Spill"]) == 0
    assert int(k["VGPRs"]) + int(k["AGPRs"]) <= DAEMON_MAX_VGPRS
    # 8 waves of a workgroup on 4 SIMDs: 2 waves per SIMD are needed for one workgroup per compute unit
    assert int(k["Occupancy [waves/SIMD]"]) >= 2
    assert int(k["LDS Size [bytes/block]"]) <= 64 * 1024
    assert int(k["SGPRs Spill"]) <= DAEMON_MAX_SGPR_SPILLS


def test_traced_daemon_kernel_stays_resident_too():
    k = resources("daemon_traced", "daemon")["dfcclDaemonKernelTraced"]
    print("dfcclDaemonKernelTraced:", k)
    assert int(k["ScratchSize [bytes/lane]"]) == 0 and k["Dynamic Stack"] == "False"
    assert int(k["VGPRs Spill"]) == 0
    assert int(k["VGPRs"]) + int(k["AGPRs"]) <= TRACED_MAX_VGPRS
    assert int(k["Occupancy [waves/SIMD]"]) >= 2


def test_reduce_copy_kernels_use_no_scratch_and_do_not_spill():
    ks = resources("reduce_copy")
    assert len(ks) >= 100  # every element type x operator x source count
    for name, k in ks.items():
        assert int(k["ScratchSize [bytes/lane]"]) == 0, name
        assert int(k["VGPRs Spill"]) == 0 and int(k["SGPRs Spill"]) == 0, name
        # two 512-thread workgroups per compute unit = 4 waves per SIMD
        assert int(k["Occupancy [waves/SIMD]"]) >= 4, name
