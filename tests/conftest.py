import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    if EMULATION_LIB:
        _enter_emulation()
    elif _have_gpu():
        _refuse_unvalidated_daemon_on_a_gpu(config)


# DFCCL_TESTS_ON_EMULATION=<path of libdfccl_emul.so> (see tests/emul): the tests marked `gpu` that go through the
# daemon then run against the host emulation of the kernel, with their buffers in host memory.  A way to put a
# change to the kernel through the parity suite on the CPU before it goes near a GPU; never the default, and
# nothing outside tests/ knows about it.
EMULATION_LIB = os.environ.get("DFCCL_TESTS_ON_EMULATION")


def _enter_emulation():
    import ctypes

    import torch

    import dfccl_amd._lib as lib
    import dfccl_amd.api as api
    import gpu_util

    lib.LIB_PATH = EMULATION_LIB
    os.environ.setdefault("NCCL_MAX_NCHANNELS", "2")  # every workgroup is a few hundred OS threads there
    os.environ.setdefault("DFCCL_STATS_WAIT_MS", "5000")  # and answers a request for its counters slowly
    os.environ.setdefault("DFCCL_RC_MAX_WGS", "3")        # the one-shot reduce-copy kernel: 3 workgroups of 512 OS threads
    gpu_util.EMULATED = True
    api._dev_ptr = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())  # host memory is device memory there
    gpu_util.DEVICE = "cpu"

    emul = ctypes.CDLL(EMULATION_LIB)

    class _NoStream:
        cuda_stream = 0

        def synchronize(self):
            emul.emulNullStreamSynchronize()  # kernels launched on the null stream run as threads of their own

    torch.cuda.current_stream = lambda *a, **k: _NoStream()
    torch.cuda.synchronize = lambda *a, **k: None


def _refuse_unvalidated_daemon_on_a_gpu(config):
    """On a real GPU: the sources of the daemon kernel must be the ones the host emulation last validated
    (tests/test_daemon_emulation.py records their hash when all its scenarios pass).  A record that names other
    sources ends the session before anything is launched; DFCCL_UNVALIDATED_DAEMON_OK=1 overrides, and a missing
    record (the CPU suite has not been run in this tree) only warns."""
    if EMULATION_LIB or os.environ.get("DFCCL_UNVALIDATED_DAEMON_OK") == "1":
        return
    markexpr = getattr(config.option, "markexpr", "") or ""
    if "gpu" not in markexpr or "not gpu" in markexpr:
        return
    stamp = os.path.join(ROOT, "tests", "emul", "validated_sources.stamp")
    if not os.path.exists(stamp):
        print("conftest: no record of an emulation run in this tree (tests/emul/validated_sources.stamp)", file=sys.stderr)
        return
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from test_daemon_emulation import sources_hash
    if open(stamp).read().strip() != sources_hash():
        pytest.exit("the daemon's sources have changed since the host emulation last passed on them: run "
                    "`python -m pytest tests/test_daemon_emulation.py` first (or set DFCCL_UNVALIDATED_DAEMON_OK=1)",
                    returncode=3)


def _have_gpu():
    if EMULATION_LIB:
        return True
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
