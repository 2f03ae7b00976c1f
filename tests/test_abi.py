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


def test_pinned_gemm_variant_that_cannot_run_the_product_is_refused():
    """pf_gemm_variant names the kernel a descriptor would run on; a pinned direct-to-LDS tile that
    cannot run the product (reduction shorter than a stage, ragged reduction with row-major
    operands, operands stored differently) is an error at naming time, for every tile id."""
    from pfeife_amd import hip

    lib = hip.load()
    name = ctypes.create_string_buffer(128)

    def desc(K, a_trans=0, b_trans=0, variant=0):
        d = hip.GemmDesc()
        d.in_dtype, d.c_dtype, d.M, d.N, d.K = hip.PF_F16, hip.PF_F16, 512, 512, K
        d.a_trans, d.b_trans, d.variant = a_trans, b_trans, variant
        d.lda = d.M if a_trans else K
        d.ldb = d.N if b_trans else K
        d.ldc, d.batch1, d.batch2, d.alpha = d.N, 1, 1, 1.0
        return d

    for v, bk in ((1, 32), (2, 64), (3, 64), (4, 32), (5, 32), (6, 32), (7, 32), (8, 64), (9, 64)):
        assert lib.pf_gemm_variant(ctypes.byref(desc(256, variant=v)), name, 128) == 0, v
        assert name.value.decode().startswith("gemm16x_kernel<1, "), name.value
        assert lib.pf_gemm_variant(ctypes.byref(desc(bk // 2, variant=v)), name, 128) == -1, v   # shorter than a stage
        assert b"variant" in lib.pf_last_error()
        assert lib.pf_gemm_variant(ctypes.byref(desc(bk * 4 + 8, variant=v)), name, 128) == -1, v  # ragged, row-major
        assert lib.pf_gemm_variant(ctypes.byref(desc(256, a_trans=1, variant=v)), name, 128) == -1, v  # mixed layouts
        assert lib.pf_gemm_variant(ctypes.byref(desc(256, b_trans=1, variant=v)), name, 128) == -1, v
    # the automatic choice never names a kernel that cannot run the product
    for K in (8, 24, 72, 256):
        for at, bt in ((0, 0), (1, 0), (0, 1), (1, 1)):
            assert lib.pf_gemm_variant(ctypes.byref(desc(K, at, bt)), name, 128) == 0, (K, at, bt)


def test_missing_library_is_an_error_not_a_fallback(tmp_path, monkeypatch):
    from pfeife_amd import hip

    monkeypatch.setattr(hip, "_lib", None)
    with pytest.raises(RuntimeError, match="no fallback"):
        hip.load(str(tmp_path / "absent.so"))
