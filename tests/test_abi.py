"""The C-ABI library loads and exports exactly what include/mni_rocm.h
declares.  No device call is made, so this runs without a GPU."""
import ctypes
import os
import re

import pytest

from framework_amd import native

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "mni_rocm.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    names = re.findall(r"\b(mni_[a-z0-9_]+)\s*\(", text)
    return sorted(set(n for n in names if n not in ("mni_operand", "mni_gemm_desc")))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    assert "mni_rocm_sgemm" in names and "mni_matmul" in names and "mni_backward" in names
    assert len(names) >= 55


def test_library_exports_every_declared_symbol():
    if not os.path.exists(native.LIB_PATH):
        pytest.fail("libmni_rocm.so is not built: run `python -m framework_amd.build`")
    lib = ctypes.CDLL(native.LIB_PATH)
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, "declared in the header but not exported: %s" % missing


def test_binding_covers_every_declared_symbol():
    names = set(declared_functions())
    bound = set(native.SIGNATURES)
    assert names == bound, "header/binding mismatch: %s" % sorted(names ^ bound)


def test_struct_layout_matches_header():
    # mni_operand: pointer + 4 x int64; mni_gemm_desc as laid out in the header
    assert ctypes.sizeof(native.Operand) == 40
    assert ctypes.sizeof(native.GemmDesc) == 4 * 8 + 2 * 40 + 8 + 8 + 8 + 8 + 4 * 4 + 2 * 8
    assert native.GemmDesc.aux.offset == 160 and native.GemmDesc.colsum_part.offset == 168
    assert native.GemmDesc.A.offset == 32 and native.GemmDesc.B.offset == 72
    assert native.GemmDesc.C.offset == 112 and native.GemmDesc.bias.offset == 136


def test_last_error_is_callable_without_a_device():
    lib = native.load_library()
    assert isinstance(lib.mni_rocm_last_error(), bytes)


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    monkeypatch.setattr(native, "_lib", None)
    with pytest.raises(native.MniError, match="not found"):
        native.load_library(str(tmp_path / "libmni_rocm.so"))
    monkeypatch.setattr(native, "_lib", None)
