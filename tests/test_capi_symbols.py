"""The C ABI library loads and exports every function include/sapphire_hip.h declares.
No compute entry point is called: this runs without a GPU."""
import ctypes
import os

import pytest

from sapphire_amd import capi


def test_header_declares_what_the_binding_binds():
    declared = set(capi.declared_symbols())
    bound = set(capi.SIGNATURES) | {"sph_last_error"}
    assert declared == bound, (declared ^ bound)


def test_library_exports_every_declared_symbol():
    assert os.path.exists(capi.LIB_PATH), "build with python -m sapphire_amd.build hip"
    lib = ctypes.CDLL(capi.LIB_PATH)
    for name in capi.declared_symbols():
        assert hasattr(lib, name), name


def test_last_error_starts_empty_and_statuses_carry_text():
    lib = capi.lib()
    # argument checks happen before any device call, so this is safe without a GPU
    rc = lib.sph_gemm_f32(None, None, None, 0, 4, 4, 1, 0, 0, 0)
    assert rc == 1
    assert b"non-zero" in lib.sph_last_error()
    rc = lib.sph_device_info(0, None)
    assert rc == 1 and b"null" in lib.sph_last_error()


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", "/nonexistent/libsapphire_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        capi.lib()
