"""The C-ABI library loads and exports every symbol include/larql_hip.h declares
(no compute calls here: this runs without a GPU)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "larql_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(larql_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    syms = declared_symbols()
    assert len(syms) >= 45
    lib = ctypes.CDLL(os.path.join(ROOT, "larql_amd", "liblarql_hip.so"))
    for s in syms:
        assert hasattr(lib, s), f"{s} declared in include/larql_hip.h but not exported"
    from larql_amd import _lib
    assert sorted(_lib.SIGNATURES) == syms, set(_lib.SIGNATURES) ^ set(syms)


def test_no_device_is_an_error_not_a_fallback():
    # BackendSelectError::NoDevice (larql-compute/src/backend/factory.rs:164-173)
    if os.path.exists("/dev/kfd") and os.access("/dev/kfd", os.R_OK | os.W_OK):
        return
    import pytest
    import larql_amd
    with pytest.raises(RuntimeError):
        larql_amd.HipBackend()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "larql_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".hpp", ".cpp")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.lower(), f"{f} mentions the oracle"
