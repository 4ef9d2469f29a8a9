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


def test_literal_build_refuses_windows_whose_rows_do_not_exist(libs):
    """libfk_capi_literal.so takes the interpolation's row index from the x coordinate (the reference's host branch): over a
    window wider than the image has rows below the window's first row it would read past the image.  Its entry points
    refuse such windows before any GPU call (no GPU is needed here: the pointers are never used); the canonical library
    has no such limit in its arguments."""
    from fusedkernellibrary_amd import Rect, CAPI_SIGNATURES
    literal_path = os.path.join(os.path.dirname(fk.library_paths()[1]), "libfk_capi_literal.so")
    assert os.path.exists(literal_path), "the literal build is part of the native build"
    literal = ctypes.CDLL(literal_path)
    literal.fk_interpolate_y1_from_x.restype = ctypes.c_int
    assert literal.fk_interpolate_y1_from_x() == 1
    literal.fk_last_error.restype = ctypes.c_char_p
    for name in ("fk_crop_resize_muls_bgr_tensor", "fk_resize_crop_tiles", "fk_resize_mul_u8c4_f32c4", "fk_warp_u8c3_f32c3",
                 "fk_yuv_crop_resize_norm_split", "fk_conditional_resize_f32c3", "fk_batch_crop_resize_norm_split"):
        getattr(literal, name).argtypes = CAPI_SIGNATURES[name]
    fake = ctypes.c_void_p(0x1000)  # never dereferenced: the refusal comes first
    f3 = (ctypes.c_float * 3)(1, 1, 1)
    one = (Rect * 1)(Rect(0, 20, 64, 10))  # 64 columns from row 20 on, in an image of 48 rows: rows 20 .. 83 are asked for
    ptrs = (ctypes.c_void_p * 1)(0x1000)
    UNSUPPORTED = 1
    assert literal.fk_crop_resize_muls_bgr_tensor(fake, 64, 48, 192, one, 1, 8, 8, 1, f3, f3, f3, f3, fake, None) == UNSUPPORTED
    assert b"row index from the x coordinate" in literal.fk_last_error()
    assert literal.fk_batch_crop_resize_norm_split(ptrs, 64, 48, 192, one, 1, 8, 8, f3, f3, f3, fake, None) == UNSUPPORTED
    tile = (Rect * 1)(Rect(0, 0, 4, 4))
    assert literal.fk_resize_crop_tiles(fake, 64, 48, 192, 16, 12, tile, 1, 4, 4, f3, fake, None) == UNSUPPORTED
    assert literal.fk_resize_mul_u8c4_f32c4(fake, 64, 48, 256, 8, 8, 1.0, fake, 128, None) == UNSUPPORTED
    m = (ctypes.c_float * 9)(1, 0, 0, 0, 1, 0, 0, 0, 1)
    assert literal.fk_warp_u8c3_f32c3(0, m, fake, 64, 48, 192, 8, 8, fake, 96, None) == UNSUPPORTED
    assert literal.fk_yuv_crop_resize_norm_split(0, 1, 1, fake, 64, 64, 48, Rect(0, 20, 64, 10), 8, 8, 255.0, fake, None) == UNSUPPORTED
    assert literal.fk_conditional_resize_f32c3(ptrs, 64, 48, 192, 1, 1, f3, 8, 8, fake, None) == UNSUPPORTED
    # the canonical build checks the same arguments and finds nothing to refuse before it would launch: probe one that
    # fails later for another reason (an aspect-ratio mode that does not exist), which shows the window was accepted
    capi = libs[1]
    capi.fk_crop_resize_muls_bgr_tensor.argtypes = CAPI_SIGNATURES["fk_crop_resize_muls_bgr_tensor"]
    capi.fk_last_error.restype = ctypes.c_char_p
    assert capi.fk_crop_resize_muls_bgr_tensor(fake, 64, 48, 192, one, 1, 8, 8, 9, f3, f3, f3, f3, fake, None) == UNSUPPORTED
    assert b"aspect-ratio" in capi.fk_last_error()


def test_python_wrappers_fail_loudly_without_the_library(monkeypatch, tmp_path):
    monkeypatch.setattr(fk, "_libs", {})
    monkeypatch.setattr(fk, "_HERE", str(tmp_path))
    with pytest.raises(fk.FkError):
        fk.load()
