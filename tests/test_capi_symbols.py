"""The native libraries load without a GPU and export every function that include/*.h declares (no compute calls)."""
import ctypes
import os
import re

import pytest

import fusedkernellibrary_amd as fk

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:fk|fkrt)_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def libs(native_build):
    rt_path, capi_path = fk.library_paths()
    assert os.path.exists(rt_path) and os.path.exists(capi_path), "native libraries are not built (python -m fusedkernellibrary_amd.build)"
    rt = ctypes.CDLL(rt_path, mode=ctypes.RTLD_GLOBAL)
    return rt, ctypes.CDLL(capi_path)


def test_runtime_abi_exports_every_declared_symbol(libs):
    names = declared_functions("fk_hip_rt.h")
    assert len(names) >= 20 and set(names) == set(fk.RUNTIME_SYMBOLS)
    for n in names:
        assert hasattr(libs[0], n), n


def test_chain_abi_exports_every_declared_symbol(libs):
    names = declared_functions("fk_capi.h")
    assert set(names) == set(fk.CAPI_SIGNATURES) | {"fk_last_error", "fk_interpolate_y1_from_x"}
    for n in names:
        assert hasattr(libs[1], n), n


def test_library_semantics_flags(libs):
    libs[1].fk_interpolate_y1_from_x.restype = ctypes.c_int
    assert libs[1].fk_interpolate_y1_from_x() == 0  # canonical build: bilinear row index from y
    libs[0].fkrt_max_kernarg_bytes.restype = ctypes.c_size_t
    assert libs[0].fkrt_max_kernarg_bytes() >= 4096


def test_argument_errors_are_reported_without_a_gpu(libs):
    capi = libs[1]
    capi.fk_last_error.restype = ctypes.c_char_p
    # null pointers are rejected before any runtime call
    rc = capi.fk_rgba2gray_u8c4(None, 4, 4, ctypes.c_size_t(16), None, ctypes.c_size_t(4), None)
    assert rc == 3 and b"null" in capi.fk_last_error()


def test_python_wrappers_fail_loudly_without_the_library(monkeypatch, tmp_path):
    monkeypatch.setattr(fk, "_libs", {})
    monkeypatch.setattr(fk, "_HERE", str(tmp_path))
    with pytest.raises(fk.FkError):
        fk.load()
