"""The shipped library loads without a GPU and exports exactly the C ABI that
include/w4_abi.h declares (no compute calls here)."""
import ctypes
import os
import re

import pytest

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
    lib = capi.load()
    # one constant, lowered only for large matrices whose rows are not 16-byte aligned
    assert lib.w4_dispatch_mma_min_m_for(4096, 4096) == lib.w4_dispatch_mma_min_m()
    assert lib.w4_dispatch_mma_min_m_for(64, 4104) == lib.w4_dispatch_mma_min_m()
    assert lib.w4_dispatch_mma_min_m_for(11008, 4104) == 2
    assert lib.w4_dispatch_mma_min_m_for(4096, 11008) == 3
    assert lib.w4_dispatch_mma_min_m_for(4096, 4128) == 3
    assert lib.w4_dispatch_mma_min_m_for(4096, 6144) == 2
    assert lib.w4_dispatch_mma_min_m_for(11008, 4096) == 3
    assert lib.w4_dispatch_mma_min_m_for(8192, 4096) == lib.w4_dispatch_mma_min_m()
    assert lib.w4_dispatch_mma_min_m_for_gs(11008, 4096, 128) == 3
    assert lib.w4_dispatch_mma_min_m_for_gs(11008, 4096, 32) == 3
    assert lib.w4_dispatch_mma_min_m_for_gs(11008, 4096, 48) == lib.w4_dispatch_mma_min_m()
    assert lib.w4_dispatch_mma_min_m_for_gs(11008, 4104, 8) == 2
    assert lib.w4_dispatch_mma_min_m_for_mx(4096, 14336) == 2
    assert lib.w4_dispatch_mma_min_m_for_mx(4096, 8192) == 3
    assert lib.w4_dispatch_mma_min_m_for_mx(4096, 4096) == lib.w4_dispatch_mma_min_m()


def test_quantize_contracts():
    """Malformed calls are rejected before the device is touched (pack.hpp:64-72,
    mx.hpp:71-76, kvcache.hpp:60-68, kvfp8.hpp:70-79)."""
    c = w4amd.capi()
    one = 8  # any non-null address: nothing is dereferenced
    for view, text in [(c.packed_view(0, 32, 8, 4, 1, one, one), "bad dims"),
                       (c.packed_view(2, 32, 12, 3, 1, one, one), "multiple of 8"),
                       (c.packed_view(2, 32, 8, 5, 1, one, one), "G inconsistent"),
                       (c.packed_view(2, 32, 8, 4, 0, one, one, 0), "asymmetric without zeros"),
                       (c.packed_view(2, 32, 8, 4, 1, one, one, one), "symmetric carries no zeros"),
                       (c.packed_view(2, 32, 8, 4, 1, 0, one), "null pointer")]:
        with pytest.raises(ValueError, match=text):
            c.quantize(view, one, one)
    with pytest.raises(ValueError, match="null pointer"):
        c.quantize(c.packed_view(2, 32, 8, 4, 1, one, one), one, 0)
    with pytest.raises(ValueError, match="B inconsistent"):
        c.quantize_mx(c.packed_mx_view(2, 64, 3, one, one), one, one)
    with pytest.raises(ValueError, match="bad dims"):
        c.quantize_mx(c.packed_mx_view(2, 0, 0, one, one), one, one)
    with pytest.raises(ValueError, match="multiple of 8"):
        c.quantize_cache(c.kv_view(1, 1, 64, 20, 4, 1, one, one, 0, one, one, 0), one, one, one)
    with pytest.raises(ValueError, match="asymmetric without zeros"):
        c.quantize_cache(c.kv_view(1, 1, 64, 16, 4, 0, one, one, 0, one, one, 0), one, one, one)
    with pytest.raises(ValueError, match="null pointer"):
        c.quantize_cache_f8(c.kv_f8_view(1, 1, 64, 16, 4, one, one, one, one), 0, one, one)
    with pytest.raises(ValueError, match="G inconsistent"):
        c.quantize_cache_f8(c.kv_f8_view(1, 1, 64, 16, 3, one, one, one, one), one, one, one)
    # W4A4: both views checked, K must agree
    w, x = c.packed_mx_view(8, 64, 2, one, one), c.packed_mx_view(2, 32, 1, one, one)
    with pytest.raises(ValueError, match="disagree on K"):
        c.gemm_mx_w4a4(w, x, one)
    with pytest.raises(ValueError, match="null pointer"):
        c.gemm_mx_w4a4(w, c.packed_mx_view(2, 64, 2, one, one), 0)
    with pytest.raises(ValueError, match="B inconsistent"):
        c.gemm_mx_w4a4(w, c.packed_mx_view(2, 64, 3, one, one), one)
    with pytest.raises(ValueError, match="null pointer"):
        c.quantize_mx_f16(c.packed_mx_view(2, 64, 2, one, one), 0, one)
    # W4A8
    x8 = c.act_mx8_view(2, 64, 2, 16, one)
    with pytest.raises(ValueError, match="disagree on K"):
        c.gemm_mx_w4a8(c.packed_mx_view(8, 32, 1, one, one), x8, one)
    with pytest.raises(ValueError, match="multiple of 32"):
        c.gemm_mx_w4a8(c.packed_mx_view(8, 40, 2, one, one), c.act_mx8_view(2, 40, 2, 16, one), one)
    with pytest.raises(ValueError, match="16-byte aligned"):
        c.gemm_mx_w4a8(w, c.act_mx8_view(2, 64, 2, 8, one), one)
    with pytest.raises(ValueError, match="B inconsistent"):
        c.gemm_mx_w4a8(w, c.act_mx8_view(2, 64, 3, 16, one), one)
    with pytest.raises(ValueError, match="null pointer"):
        c.quantize_mx8_f16(x8, 0, one)


def test_noalloc_entry_contracts_without_a_device():
    """The entry point that allocates nothing validates like w4_attention_w4_flash_gqa
    and rejects partials beyond its built-in array before any device call."""
    c = w4amd.capi()
    one = 256
    with pytest.raises(ValueError, match="null pointer"):
        c.attention_w4_flash_noalloc(c.kv_view(1, 64, 128, 32, 4, 1, one, one, 0, one, one, 0), 0, one)
    with pytest.raises(ValueError, match="G inconsistent"):
        c.attention_w4_flash_noalloc(c.kv_view(1, 64, 128, 32, 3, 1, one, one, 0, one, one, 0), one, one)
    with pytest.raises(ValueError, match="bad query group"):
        c.attention_w4_flash_noalloc(c.kv_view(1, 64, 128, 32, 4, 1, one, one, 0, one, one, 0), one, one, group=65)
    # 512 splits x 64 query heads x 130 floats = 17 MB of partials
    with pytest.raises(ValueError, match="exceed the built-in scratch"):
        c.attention_w4_flash_noalloc(c.kv_view(1, 1 << 19, 128, 32, 4, 1, one, one, 0, one, one, 0), one, one, group=64)
