"""The C-ABI library loads and exports exactly what include/phyai_fp8.h declares.
No compute call is made here, so this runs without a GPU."""

from __future__ import annotations

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "phyai_fp8.h")


def declared_functions() -> list[str]:
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(phyai_fp8_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for required in ("phyai_fp8_quant_rowwise", "phyai_fp8_quant_static", "phyai_fp8_weight_quant_rowwise",
                     "phyai_fp8_gemm", "phyai_fp8_linear", "phyai_fp8_linear_workspace_bytes",
                     "phyai_fp8_abi_version", "phyai_fp8_last_error"):
        assert required in names


def test_library_exports_every_declared_symbol():
    from phyai_amd import _lib

    lib = _lib.load()
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == declared_functions()
    assert lib.phyai_fp8_abi_version() == _lib.ABI_VERSION


def test_workspace_query_and_argument_validation_without_gpu():
    """Size queries and argument checks run entirely on the host."""
    from phyai_amd import _lib

    lib = _lib.load()
    hdr = 16384
    assert lib.phyai_fp8_linear_workspace_bytes(50, 1024, 4096, 0) >= hdr + 50 * 4096
    assert lib.phyai_fp8_linear_workspace_bytes(0, 1024, 4096, 0) >= hdr
    # null pointers / bad shapes are rejected before anything is launched
    assert lib.phyai_fp8_quant_rowwise(None, 4, 64, 64, None, None, None) == -1
    assert lib.phyai_fp8_quant_rowwise(None, 0, 64, 64, None, None, None) == 0      # empty: nothing to do
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 4, 64, 60, 0, None, 0, None) == -2
    assert b"multiples of 16" in lib.phyai_fp8_last_error()
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 4, 64, 64, 9, None, 0, None) == -1
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 0, 64, 64, 0, None, 0, None) == 0
    buf = (ctypes.c_char * 64)()
    assert lib.phyai_fp8_linear(ctypes.addressof(buf), 64, None, None, None, None, 64, 4, 64, 64, 0, None, 0, None) == -3
    assert b"workspace" in lib.phyai_fp8_last_error()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from phyai_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.Fp8LibraryError, match="no non-HIP fallback"):
        _lib.load()


def test_product_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "phyai_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(base, f)).read()
                assert "oracle" not in text.replace("the oracle's", ""), f"{f} mentions the oracle"
