"""The shipped library loads without a GPU and exports exactly the C ABI that
include/w4_abi.h declares (no compute calls here)."""
import ctypes
import os
import re

import w4amd

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "w4_abi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(w4_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    capi = w4amd.capi()
    lib = ctypes.CDLL(capi.LIB_PATH)
    names = _declared()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in w4_abi.h but not exported"
    assert set(capi.SIGNATURES) == set(names), "the ctypes view and the header disagree"


def test_validation_runs_without_a_device():
    capi = w4amd.capi()
    v = capi.packed_view(2, 32, 7, 4, 1, 1, 1)
    try:
        capi.gemm(v, 1, 1, 1)
    except ValueError as e:
        assert "gs must be a multiple of 8" in str(e)
    else:
        raise AssertionError("a malformed view was accepted")
    assert capi.load().w4_dispatch_mma_min_m() >= 1
