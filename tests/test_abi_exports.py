"""CPU-side checks of the product's boundary: the C-ABI library loads and exports every symbol that
include/mi_ccl_comp.h declares, and the pure-host entry points behave (no compute without a GPU)."""
import ctypes
import os
import re

import pytest

import oracle_lib as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mi_ccl_comp.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi_ccl_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    import oneccl_amd.comp as c
    if not os.path.exists(c.LIB_PATH):
        pytest.skip("libmi_ccl_comp.so not built (run __graft_entry__.build())")
    L = ctypes.CDLL(c.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 20
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing
    assert sorted(c.EXPORTS) == names


def test_host_only_entry_points():
    import oneccl_amd.comp as c
    if not os.path.exists(c.LIB_PATH):
        pytest.skip("libmi_ccl_comp.so not built")
    assert [c.datatype_size(i) for i in range(12)] == O.DTYPE_SIZE
    assert [c.datatype_name(i) for i in range(12)] == O.DTYPE_NAMES
    assert c.datatype_size(12) == 0 and c.datatype_name(-1) == ""
    assert [c.reduction_to_str(i) for i in range(6)] == ["sum", "prod", "min", "max", "custom", "unknown"]
    assert c.status_str(0) == "success" and c.status_str(2) == "invalid_arguments"
    assert c.kernel_name("Reduce_Local_Inplace_Kernel", c.FLOAT16, c.MAX) == "reduce_local_inplace_kernel_float16_max"
    offs, total = c.fusion_offsets([3, 5, 7], 2, 256)
    assert offs == [0, 256, 512] and total == 526
    offs, total = c.fusion_offsets([3, 5, 7], 2, 1)          # the reference's tight layout (fusion.cpp:314)
    assert offs == [0, 6, 16] and total == 30
    c.set_param("waves_per_cu", 8)
    assert c.get_param("waves_per_cu") == 8
    with pytest.raises(c.CclError):
        c.set_param("no_such_knob", 1)
    # count == 0 is a successful no-op before any argument is looked at (comp.cpp:132-134)
    L = c.lib()
    assert L.mi_ccl_comp_reduce(0, 0, None, 0, None, 2, 0, None) == 0
    assert L.mi_ccl_comp_copy(None, None, 0, 0, None) == 0
    # the entry point that allocates nothing refuses what its table cannot hold before it touches the GPU
    k = c.FUSION_STATIC_MAX_TENSORS + 1
    cnt = (ctypes.c_size_t * k)(*([1] * k))
    ptrs = (ctypes.c_void_p * k)(*([16] * k))
    assert L.mi_ccl_fusion_reduce_static(cnt, k, c.FLOAT32, 4, c.SUM, ptrs, None, 0, ptrs, 0, 2, 0, None) == c.OUT_OF_RESOURCE
    one = (ctypes.c_size_t * 1)((c.FUSION_STATIC_MAX_ITEMS + 1) * 4096)
    assert L.mi_ccl_fusion_reduce_static(one, 1, c.FLOAT32, 4, c.SUM, ptrs, None, 0, ptrs, 0, 2, 0, None) == c.OUT_OF_RESOURCE
    assert L.mi_ccl_fusion_reduce_static(one, 1, c.FLOAT32, 4, c.SUM, ptrs, None, 0, ptrs, 0, 2, 7, None) == c.INVALID_ARGUMENTS


def test_missing_library_fails_loudly(monkeypatch):
    import oneccl_amd.comp as c
    monkeypatch.setattr(c, "_lib", None)
    monkeypatch.setattr(c, "LIB_PATH", "/nonexistent/libmi_ccl_comp.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        c.lib()
