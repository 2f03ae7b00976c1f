"""The C-ABI library loads on a machine without a GPU and exports every symbol
that include/pfeife_hip.h declares; argument checking works without a device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "pfeife_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pf_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from pfeife_amd import hip

    lib = hip.load()
    names = declared_symbols()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), "libpfeife_hip.so does not export %s" % n
    # the binding declares exactly the header's entry points
    assert sorted(hip.EXPORTED_SYMBOLS) == names
    assert lib.pf_version() == hip.ABI_VERSION


def test_argument_errors_need_no_device():
    from pfeife_amd import hip

    lib = hip.load()
    assert lib.pf_gemm(None, None) == -1
    assert b"null descriptor" in lib.pf_last_error()
    d = hip.GemmDesc()
    d.in_dtype, d.c_dtype, d.M, d.N, d.K = 7, 0, 4, 4, 4
    assert lib.pf_gemm(ctypes.byref(d), None) == -1
    assert b"in_dtype" in lib.pf_last_error()
    assert lib.pf_colreduce_workspace(3152, 1024) >= 2 * 1024
    assert lib.pf_copy_strided(None, 0, None, None, 0, None, None, 9, 0, None) == -1


def test_missing_library_is_an_error_not_a_fallback(tmp_path, monkeypatch):
    from pfeife_amd import hip

    monkeypatch.setattr(hip, "_lib", None)
    with pytest.raises(RuntimeError, match="no fallback"):
        hip.load(str(tmp_path / "absent.so"))
