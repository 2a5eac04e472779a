"""CPU-only checks of the drop-in boundary: the C-ABI library loads and exports exactly the
symbols include/rg_hip.h declares (no compute calls are made here)."""
import ctypes
import os
import re

import pytest

from refactorgraph_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "rg_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rg_hip_\w+)\s*\(", text)))


def test_header_and_binding_list_the_same_symbols():
    assert declared_symbols() == sorted(abi.SIGNATURES)


def test_library_loads_and_exports_every_declared_symbol():
    if not os.path.exists(abi.LIB_PATH):
        pytest.fail(f"{abi.LIB_PATH} not built: run python -m refactorgraph_amd.build")
    L = ctypes.CDLL(abi.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(L, name), name


def test_missing_library_is_a_loud_error(monkeypatch):
    monkeypatch.setattr(abi, "_lib", None)
    monkeypatch.setattr(abi, "LIB_PATH", "/nonexistent/librg_hip.so")
    with pytest.raises(abi.RgHipError):
        abi.lib()


def test_error_strings_and_workspace_queries_need_no_gpu():
    L = abi.lib()
    assert b"no kernel" in L.rg_hip_error_string(-1)
    assert b"argument" in L.rg_hip_error_string(-2)
    # zero points are fused into the tile loads: no workspace (the reference needs m*k [+ k*n])
    assert L.rg_hip_matmul_integer_workspace(1, 4096, 4096, 4096, 3) == 0
    assert L.rg_hip_attention_kvcache_workspace(32, 32, 8, 1, 4096, 128) > 0


def test_product_package_does_not_touch_the_oracle():
    pkg = os.path.join(ROOT, "refactorgraph_amd")
    for dirpath, _, files in os.walk(pkg):
        if os.sep + "lib" in dirpath:
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cc")):
                src = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(import|from)\s+oracle\b", src, flags=re.M), f
                assert "liboracle" not in src and "oracle.h" not in src, f
