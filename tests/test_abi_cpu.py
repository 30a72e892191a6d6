"""The C-ABI library loads without a GPU and exports every symbol that
include/ofccl.h declares (no compute calls here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ofccl.h")
LIB = os.path.join(ROOT, "dfccl_amd", "libdfccl.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b((?:nccl|ofccl|dfccl)[A-Za-z0-9]+)\s*\(", text)
    return sorted(set(names))


def test_header_declares_the_reference_entry_points():
    names = declared_symbols()
    for required in ["ofcclInitRankCtx", "ofcclFinalizeRankCtx7StartHostThrds", "ofcclPrepareDone", "ofcclDestroy",
                     "ofcclPrepareAllReduce", "ofcclPrepareReduceScatter", "ofcclPrepareAllGather",
                     "ofcclPrepareReduce", "ofcclPrepareBroadcast", "ofcclPrepareBcast", "ofcclRunAllReduce",
                     "ofcclRunReduceScatter", "ofcclRunAllGather", "ofcclRunReduce", "ofcclRunBroadcast",
                     "ofcclRunBcast", "dfcclReduceCopy"]:
        assert required in names


@pytest.mark.skipif(not os.path.exists(LIB), reason="libdfccl.so not built (run __graft_entry__.build())")
def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(LIB)
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in ofccl.h but not exported"


@pytest.mark.skipif(not os.path.exists(LIB), reason="libdfccl.so not built (run __graft_entry__.build())")
def test_python_mirror_binds_every_declared_symbol():
    from dfccl_amd import _lib
    assert sorted(_lib.SIGNATURES) == declared_symbols()
    _lib.load()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from dfccl_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()


def test_error_strings_and_argument_checks_without_gpu():
    if not os.path.exists(LIB):
        pytest.skip("libdfccl.so not built")
    from dfccl_amd import _lib
    lib = _lib.load()
    assert lib.ncclGetErrorString(0) == b"no error"
    assert lib.ncclGetErrorString(4) == b"invalid argument"
    assert lib.ncclGetUniqueId(None) == 4
    assert lib.ofcclInitRankCtx(None, 0) == 4
    assert lib.ofcclDestroy(None) == 4
    assert lib.ofcclFinalizeRankCtx7StartHostThrds(None) == 4
    assert lib.dfcclReduceCopy(None, 2, None, 16, 7, 0, 0, None) == 4
