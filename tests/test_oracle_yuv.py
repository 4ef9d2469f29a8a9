"""Pins the YUV part of the oracle (oracle/fk_oracle_yuv.c), CPU only:

 1. ReadYUV against the known-answer vectors of the reference's own unit test for UYVY
    (utests/algorithm/image_processing/utest_color_conversion.h:226-324 of the reference), all three channels;
 2. every function against the committed vectors written by the reference's own headers
    (tests/golden/make_golden_yuv.py), and against that build directly on other seeds where it is present;
 3. what the layouts and the mathematics fix: hand-laid buffers whose every sample is distinct (a wrong plane offset,
    a swapped U/V or a wrong pair index reads a different number), write -> read round trips, the grey axis, the
    matrices evaluated in double precision, and the canonical (row index from y) resize against the composition of
    the separately pinned conversion and bilinear sample.
"""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
from oracle import binding as B  # noqa: E402
import make_golden_yuv as G  # noqa: E402

GOLD = np.load(os.path.join(HERE, "golden", "reference_yuv_vectors.npz"))
FORMATS = list(B.YUV_FORMATS)
MATRIX = {  # the reference's constants (color_conversion.h:137-171), rows R, G, B over (Y, Cb, Cr)
    (B.RANGE_FULL, B.BT601): [[1.164383562, 0.0, 1.596026786], [1.164383562, -0.39176229, -0.812967647], [1.164383562, 2.017232143, 0.0]],
    (B.RANGE_FULL, B.BT709): [[1.0, 0.0, 1.5748], [1.0, -0.1873, -0.4681], [1.0, 1.8556, 0.0]],
    (B.RANGE_LIMITED, B.BT709): [[1.0, 0.0, 1.402], [1.0, -0.34414, -0.71414], [1.0, 1.772, 0.0]],
    (B.RANGE_FULL, B.BT2020): [[1.0, 0.0, 1.4746], [1.0, -0.16455312684366, -0.57135312684366], [1.0, 1.8814, 0.0]],
}


def same_bits(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and a.tobytes() == b.tobytes()


# ---- 1. the reference's own known answers ------------------------------------------------------------------------------
def test_read_uyvy_known_answers(oracle):
    # case 1: a constant UYVY quad; case 2/3: bytes 0.. in U, Y0, V, Y1 order (values as listed in the reference's test)
    raw1 = np.tile(np.array([128, 254, 129, 255], np.uint8), (2, 2))
    exp1 = np.tile(np.array([[254, 128, 129], [255, 128, 129]], np.uint8), (2, 2, 1))
    assert same_bits(oracle.read_yuv(B.UYVY, raw1, 4, 2), exp1)
    raw2 = np.array([[0, 2, 1, 3, 4, 6, 5, 7], [8, 10, 9, 11, 12, 14, 13, 15]], np.uint8)
    exp2 = np.array([[[2, 0, 1], [3, 0, 1], [6, 4, 5], [7, 4, 5]], [[10, 8, 9], [11, 8, 9], [14, 12, 13], [15, 12, 13]]], np.uint8)
    assert same_bits(oracle.read_yuv(B.UYVY, raw2, 4, 2), exp2)
    two_rows = np.array([[0, 2, 1, 3, 4, 6, 5, 7, 8, 10, 9, 11, 12, 14, 13, 15],
                         [16, 18, 17, 19, 20, 22, 21, 23, 24, 26, 25, 27, 28, 30, 29, 31]], np.uint8)
    raw3 = np.tile(two_rows, (4, 1))
    exp_rows = np.array([[[2, 0, 1], [3, 0, 1], [6, 4, 5], [7, 4, 5], [10, 8, 9], [11, 8, 9], [14, 12, 13], [15, 12, 13]],
                         [[18, 16, 17], [19, 16, 17], [22, 20, 21], [23, 20, 21], [26, 24, 25], [27, 24, 25], [30, 28, 29], [31, 28, 29]]], np.uint8)
    assert same_bits(oracle.read_yuv(B.UYVY, raw3, 8, 8), np.tile(exp_rows, (4, 1, 1)))


# ---- 2. vectors written by the reference's own headers -------------------------------------------------------------------
@pytest.mark.parametrize("name", FORMATS)
def test_golden_read_write_convert(oracle, name):
    fmt, raw, pixels = G.yuv_case_input(oracle, name)
    assert same_bits(oracle.read_yuv(fmt, raw, *G.SIZE), GOLD[f"{name}_read"])
    assert same_bits(oracle.write_yuv(fmt, pixels), GOLD[f"{name}_write"])
    for rng, prim in B.YUV_MATRICES:
        for alpha in (0, 1):
            for float_out in (0, 1):
                got = oracle.yuv_to_rgb(fmt, rng, prim, alpha, float_out, raw, *G.SIZE)
                assert same_bits(got, GOLD[f"{name}_rgb_r{rng}p{prim}a{alpha}f{float_out}"]), (name, rng, prim, alpha, float_out)
        got = oracle.yuv_crop_resize_norm_split(fmt, rng, prim, raw, *G.SIZE, G.CROP, G.DST, G.DIV, quirk=1)
        assert same_bits(got, GOLD[f"{name}_chain_r{rng}p{prim}"]), (name, rng, prim)


@pytest.mark.parametrize("name", FORMATS)
def test_against_reference_build_other_seeds(oracle, reference, name):
    if reference.yuv is None:
        pytest.skip("oracle/_ref/libfkref_yuv.so not built")
    fmt = B.YUV_FORMATS[name]
    for seed, (w, h) in ((7, (2, 2)), (8, (34, 6)), (9, (64, 48))):
        rows, cols, dt = oracle.yuv_data_shape(fmt, w, h)
        raw = oracle.bytes(seed, (rows, cols * np.dtype(dt).itemsize)).view(dt)
        pixels = oracle.bytes(seed + 1, (h, w * 3 * np.dtype(dt).itemsize)).view(dt).reshape(h, w, 3)
        assert same_bits(oracle.read_yuv(fmt, raw, w, h), reference.read_yuv(fmt, raw, w, h))
        assert same_bits(oracle.write_yuv(fmt, pixels), reference.write_yuv(fmt, pixels))
        for rng, prim in B.YUV_MATRICES:
            for alpha, float_out in ((0, 0), (1, 0), (0, 1), (1, 1)):
                assert same_bits(oracle.yuv_to_rgb(fmt, rng, prim, alpha, float_out, raw, w, h),
                                 reference.yuv_to_rgb(fmt, rng, prim, alpha, float_out, raw, w, h))
        if w >= 34:  # a crop narrower than it is tall keeps the literal row index inside the image
            crop, dst = (4, 0, 5, 6), (13, 11)
            assert same_bits(oracle.yuv_crop_resize_norm_split(fmt, rng, prim, raw, w, h, crop, dst, 3.0, quirk=1),
                             reference.yuv_crop_resize_norm_split(fmt, rng, prim, raw, w, h, crop, dst, 3.0))


# ---- 3. what the layouts and the mathematics fix ---------------------------------------------------------------------------
def hand_laid(name, w, h):
    """A raw image whose samples are all distinct, laid out from the published definition of the format, and the
    {Y, U, V} image it encodes."""
    dt = np.uint16 if name in ("P010", "P210", "Y210") else np.uint8
    scale = 64 if dt == np.uint16 else 1  # 10-bit samples live in the high bits
    ys = (np.arange(h * w).reshape(h, w) % 200 + 1) * scale
    ch = h // 2 if name in ("NV12", "NV21", "P010") else h
    us = (np.arange(ch * (w // 2)).reshape(ch, w // 2) * 2 % 199 + 300 % 256) % 256 * scale
    vs = (np.arange(ch * (w // 2)).reshape(ch, w // 2) * 3 % 197 + 7) % 256 * scale
    if name in ("NV12", "NV21", "P010", "P210"):
        raw = np.zeros((h + ch, w), dt)
        raw[:h] = ys
        first, second = (vs, us) if name == "NV21" else (us, vs)
        raw[h:, 0::2] = first
        raw[h:, 1::2] = second
    else:
        raw = np.zeros((h, 2 * w), dt)
        if name == "UYVY":  # U Y0 V Y1
            raw[:, 0::4], raw[:, 1::4], raw[:, 2::4], raw[:, 3::4] = us, ys[:, 0::2], vs, ys[:, 1::2]
        else:               # Y210: Y0 U Y1 V
            raw[:, 0::4], raw[:, 1::4], raw[:, 2::4], raw[:, 3::4] = ys[:, 0::2], us, ys[:, 1::2], vs
    rep = 2 if ch != h else 1
    expect = np.stack([ys, np.repeat(np.repeat(us, rep, 0), 2, 1), np.repeat(np.repeat(vs, rep, 0), 2, 1)], -1).astype(dt)
    return raw, expect


@pytest.mark.parametrize("name", FORMATS)
def test_read_hand_laid_buffers(oracle, name):
    for w, h in ((2, 2), (6, 4), (16, 10)):
        raw, expect = hand_laid(name, w, h)
        assert same_bits(oracle.read_yuv(B.YUV_FORMATS[name], raw, w, h), expect)
    # a padded pitch moves the chroma plane with it
    raw, expect = hand_laid(name, 6, 4)
    padded = np.zeros((raw.shape[0], raw.shape[1] + 10), raw.dtype)
    padded[:, :raw.shape[1]] = raw
    assert same_bits(oracle.read_yuv(B.YUV_FORMATS[name], padded, 6, 4), expect)


@pytest.mark.parametrize("name", FORMATS)
def test_write_then_read_round_trip(oracle, name):
    fmt = B.YUV_FORMATS[name]
    raw, expect = hand_laid(name, 12, 6)  # chroma constant over each covered block, so nothing is lost
    assert same_bits(oracle.write_yuv(fmt, expect), raw)
    assert same_bits(oracle.read_yuv(fmt, oracle.write_yuv(fmt, expect), 12, 6), expect)


@pytest.mark.parametrize("name", FORMATS)
def test_conversion_grey_axis_and_double_precision(oracle, name):
    fmt = B.YUV_FORMATS[name]
    wide = name in ("P010", "P210", "Y210")
    shift, centre, luma_sub, top = (6, 512, 64, 65535) if wide else (0, 128, 16, 255)
    w, h = 16, 8
    _, expect = hand_laid(name, w, h)
    grey = expect.copy()
    grey[..., 1:] = centre << shift
    for (rng, prim), m in MATRIX.items():
        m = np.array(m)
        # neutral chroma: R = G = B = m00 * (Y - offset), rounded half up and saturated
        got = oracle.yuv_to_rgb(fmt, rng, prim, 0, 1, oracle.write_yuv(fmt, grey), w, h)
        y = (grey[..., 0] >> shift).astype(np.float64) - (luma_sub if prim == B.BT601 else 0)
        assert np.array_equal(got[..., 0], got[..., 1]) and np.array_equal(got[..., 1], got[..., 2])
        np.testing.assert_allclose(got[..., 0], y * m[0, 0] * (1 << shift), rtol=1e-6, atol=1e-3)
        # general pixels against a double-precision evaluation
        raw = oracle.write_yuv(fmt, expect)
        yuv = (oracle.read_yuv(fmt, raw, w, h) >> shift).astype(np.float64)
        yuv[..., 0] -= luma_sub if prim == B.BT601 else 0
        yuv[..., 1:] -= centre
        rgb = yuv @ m.T
        f = oracle.yuv_to_rgb(fmt, rng, prim, 1, 1, raw, w, h)
        np.testing.assert_allclose(f[..., :3], rgb * (1 << shift), rtol=1e-5, atol=2e-2 * (1 << shift))
        assert np.all(f[..., 3] == (1023 * 64 if wide else 255))
        i = oracle.yuv_to_rgb(fmt, rng, prim, 1, 0, raw, w, h).astype(np.int64)
        stored = np.floor(np.clip(rgb, 0, top) + 0.5)
        close = np.abs(rgb - np.floor(rgb) - 0.5) > 1e-3  # away from rounding ties the float path cannot differ
        want = (stored.astype(np.int64) << shift) & (0xFFFF if wide else 0xFF)
        assert np.array_equal(i[..., :3][close], want[close])
        assert np.all(i[..., 3] == ((1023 << 6) if wide else 255))


@pytest.mark.parametrize("name", ["NV12", "NV21", "UYVY"])
def test_canonical_chain_is_convert_crop_bilinear(oracle, name):
    """quirk = 0 differs from the reference-pinned quirk = 1 in the row index only; here it is rebuilt from pieces that
    are pinned on their own: the conversion (above) and fko_bilinear_u8 (tests/test_oracle_pinning.py)."""
    fmt = B.YUV_FORMATS[name]
    w, h = 20, 14
    rows, cols, dt = oracle.yuv_data_shape(fmt, w, h)
    raw = oracle.bytes(21, (rows, cols))
    crop, dst, div = (4, 2, 11, 9), (7, 13), 255.0
    for rng, prim in B.YUV_MATRICES:
        rgb = oracle.yuv_to_rgb(fmt, rng, prim, 0, 0, raw, w, h)
        p = oracle.resize_build(B.IGNORE_AR, crop[2], crop[3], *dst)
        want = np.empty((3, dst[1], dst[0]), np.float32)
        for y in range(dst[1]):
            for x in range(dst[0]):
                sx, sy = np.float32(x) * np.float32(p.fx), np.float32(y) * np.float32(p.fy)
                want[:, y, x] = oracle.bilinear_u8(rgb, (crop[0], crop[1]), (crop[2], crop[3]), sx, sy) / np.float32(div)
        got = oracle.yuv_crop_resize_norm_split(fmt, rng, prim, raw, w, h, crop, dst, div)
        assert same_bits(got, want)


@pytest.mark.parametrize("name", ["P010", "P210", "Y210"])
def test_canonical_chain_16bit_agrees_where_rows_coincide(oracle, name):
    """For the 16-bit formats the canonical chain is pinned on every element where both row rules give the same row
    (floor(sx) == floor(sy)) by the reference-pinned literal chain, and elsewhere by transposition-free symmetry:
    shifting the crop by whole rows shifts the output rows it reads."""
    fmt = B.YUV_FORMATS[name]
    w, h = 16, 16
    rows, cols, dt = oracle.yuv_data_shape(fmt, w, h)
    raw = oracle.bytes(33, (rows, cols * 2)).view(dt)
    crop, dst = (2, 2, 8, 8), (8, 8)  # unit scale: sx = x, sy = y, so the canonical result is the conversion itself
    for rng, prim in B.YUV_MATRICES:
        got = oracle.yuv_crop_resize_norm_split(fmt, rng, prim, raw, w, h, crop, dst, 1.0)
        lit = oracle.yuv_crop_resize_norm_split(fmt, rng, prim, raw, w, h, crop, dst, 1.0, quirk=1)
        diag = np.eye(8, dtype=bool)
        assert same_bits(got[:, diag], lit[:, diag])
        rgb = oracle.yuv_to_rgb(fmt, rng, prim, 0, 0, raw, w, h)[2:10, 2:10].astype(np.float32)
        assert same_bits(got, np.ascontiguousarray(rgb.transpose(2, 0, 1)))
    # a non-trivial scale: columns of the canonical result equal the literal result's where floor(sx) == floor(sy)
    dst = (12, 12)
    p = oracle.resize_build(B.IGNORE_AR, 8, 8, *dst)
    fl = np.floor(np.arange(12, dtype=np.float32) * np.float32(p.fx)).astype(int)
    agree = fl[None, :] == fl[:, None]
    got = oracle.yuv_crop_resize_norm_split(fmt, B.RANGE_FULL, B.BT709, raw, w, h, crop, dst, 7.0)
    lit = oracle.yuv_crop_resize_norm_split(fmt, B.RANGE_FULL, B.BT709, raw, w, h, crop, dst, 7.0, quirk=1)
    assert same_bits(got[:, agree], lit[:, agree]) and agree.sum() > 12
