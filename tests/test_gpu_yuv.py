"""GPU parity of the YUV front-end: ReadYUV / WriteYUV / ConvertYUVToRGB and the crop -> resize chain over a YUV source,
called through the C ABI on the MI355X, against the CPU oracle (oracle/fk_oracle_yuv.c) on the same seeded inputs,
against the vectors written by the reference's own headers, and against the reference's known answers for UYVY.
Bar: bit-exact, float outputs included."""
import os
import sys

import numpy as np
import pytest
import torch

from conftest import same_bits
from oracle import binding as B

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import make_golden_yuv as G  # noqa: E402

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_yuv_vectors.npz"))
FORMATS = list(B.YUV_FORMATS)


def dev(a, extra_cols=0):
    """numpy -> GPU; 16-bit data travels as int16 (same bits).  extra_cols pads every row, so the pitch exceeds the row."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        a = a.view(np.int16)
    t = torch.from_numpy(a).cuda()
    if extra_cols:
        shape = list(t.shape)
        shape[1] += extra_cols
        big = torch.zeros(shape, dtype=t.dtype, device="cuda")
        big[:, :t.shape[1]] = t
        t = big[:, :t.shape[1]]
    return t


def empty(shape, np_dtype, extra_cols=0):
    tdt = {np.uint8: torch.uint8, np.uint16: torch.int16, np.float32: torch.float32}[np_dtype]
    shape = list(shape)
    full = shape.copy()
    full[1] += extra_cols
    t = torch.zeros(full, dtype=tdt, device="cuda")
    t += 85 if tdt != torch.float32 else float("nan")  # a pattern the kernels never produce by leaving memory alone
    return t[:, :shape[1]]


def host(t, np_dtype):
    a = np.ascontiguousarray(t.cpu().numpy())
    return a.view(np.uint16) if np_dtype == np.uint16 else a


def random_raw(oracle, fmt, seed, w, h):
    rows, cols, dt = oracle.yuv_data_shape(fmt, w, h)
    return oracle.bytes(seed, (rows, cols * np.dtype(dt).itemsize)).view(dt), dt


def test_read_uyvy_known_answers(fk):
    raw = np.array([[0, 2, 1, 3, 4, 6, 5, 7], [8, 10, 9, 11, 12, 14, 13, 15]], np.uint8)
    want = np.array([[[2, 0, 1], [3, 0, 1], [6, 4, 5], [7, 4, 5]], [[10, 8, 9], [11, 8, 9], [14, 12, 13], [15, 12, 13]]], np.uint8)
    out = empty((2, 4, 3), np.uint8)
    fk.read_yuv(fk.UYVY, dev(raw), out)
    torch.cuda.synchronize()
    assert same_bits(host(out, np.uint8), want)


@pytest.mark.parametrize("name", FORMATS)
def test_reference_vectors(fk, oracle, name):
    fmt, raw, pixels = G.yuv_case_input(oracle, name)
    dt = raw.dtype.type
    w, h = G.SIZE
    d_raw = dev(raw)
    out = empty((h, w, 3), dt)
    fk.read_yuv(fmt, d_raw, out)
    assert same_bits(host(out, dt), GOLD[f"{name}_read"])
    d_written = dev(np.zeros_like(raw))
    fk.write_yuv(fmt, dev(pixels), d_written)
    assert same_bits(host(d_written, dt), GOLD[f"{name}_write"])
    for rng, prim in B.YUV_MATRICES:
        for alpha in (0, 1):
            for float_out in (0, 1):
                o = empty((h, w, 4 if alpha else 3), np.float32 if float_out else dt)
                fk.yuv_to_rgb(fmt, rng, prim, d_raw, o)
                assert same_bits(host(o, np.float32 if float_out else dt), GOLD[f"{name}_rgb_r{rng}p{prim}a{alpha}f{float_out}"]), (rng, prim, alpha, float_out)


@pytest.mark.parametrize("name", FORMATS)
def test_reference_chain_vectors_with_literal_build(oracle, name):
    """The crop -> resize chain of the reference's CPU backend takes its bilinear row index from the x coordinate; the
    library variant built the same way reproduces its vectors bit for bit."""
    import fusedkernellibrary_amd as lib
    fmt, raw, _ = G.yuv_case_input(oracle, name)
    lib.use_literal_interpolation(True)
    try:
        lib.load()
        for rng, prim in B.YUV_MATRICES:
            out = torch.full((3, G.DST[1], G.DST[0]), float("nan"), device="cuda")
            lib.yuv_crop_resize_norm_split(fmt, rng, prim, dev(raw), G.SIZE, G.CROP, out, G.DIV)
            torch.cuda.synchronize()
            assert same_bits(out.cpu().numpy(), GOLD[f"{name}_chain_r{rng}p{prim}"]), (rng, prim)
    finally:
        lib.use_literal_interpolation(False)
        lib.load()


@pytest.mark.parametrize("name", FORMATS)
@pytest.mark.parametrize("size,pad", [((2, 2), 0), ((70, 34), 0), ((130, 66), 6), ((1920, 1080), 0)])
def test_read_write_convert_vs_oracle(fk, oracle, name, size, pad):
    fmt = B.YUV_FORMATS[name]
    w, h = size
    raw, dt = random_raw(oracle, fmt, 40 + w, w, h)
    d_raw = dev(raw, pad)
    out = empty((h, w, 3), dt, pad)
    fk.read_yuv(fmt, d_raw, out)
    yuv = oracle.read_yuv(fmt, raw, w, h)
    assert same_bits(host(out, dt), yuv)
    # write: the pixels just read (chroma of a covered block equal) and arbitrary ones (the block's designated pixel wins)
    pixels = oracle.bytes(41 + w, (h, w * 3 * np.dtype(dt).itemsize)).view(dt).reshape(h, w, 3)
    for src in (yuv, pixels):
        d_written = dev(np.zeros_like(raw), pad)
        fk.write_yuv(fmt, dev(src, pad), d_written)
        assert same_bits(host(d_written, dt), oracle.write_yuv(fmt, src))
    for rng, prim in B.YUV_MATRICES:
        for alpha, float_out in ((0, 0), (1, 0), (0, 1), (1, 1)):
            odt = np.float32 if float_out else dt
            o = empty((h, w, 4 if alpha else 3), odt, pad)
            fk.yuv_to_rgb(fmt, rng, prim, d_raw, o)
            assert same_bits(host(o, odt), oracle.yuv_to_rgb(fmt, rng, prim, alpha, float_out, raw, w, h)), (rng, prim, alpha, float_out)


@pytest.mark.parametrize("name", FORMATS)
def test_crop_resize_chain_vs_oracle(fk, oracle, name):
    fmt = B.YUV_FORMATS[name]
    cases = [((64, 48), (10, 6, 40, 30), (224, 224), 255.0, 0),      # upscale
             ((1920, 1080), (300, 200, 1280, 720), (320, 180), 255.0, 0),  # 4x downscale of a crop
             ((130, 66), (1, 1, 127, 63), (127, 63), 1.0, 10),        # unit scale, odd origin, padded pitch
             ((34, 20), (0, 0, 34, 20), (5, 3), 65535.0, 0),          # whole image to a few pixels
             ((8, 8), (3, 2, 1, 1), (4, 4), 2.0, 0)]                  # one-pixel crop
    for i, (size, crop, dst, div, pad) in enumerate(cases):
        raw, _ = random_raw(oracle, fmt, 60 + i, *size)
        rng, prim = B.YUV_MATRICES[i % 4]
        out = torch.full((3, dst[1], dst[0]), float("nan"), device="cuda")
        fk.yuv_crop_resize_norm_split(fmt, rng, prim, dev(raw, pad), size, crop, out, div)
        torch.cuda.synchronize()
        want = oracle.yuv_crop_resize_norm_split(fmt, rng, prim, raw, *size, crop, dst, div)
        assert same_bits(out.cpu().numpy(), want), (size, crop, dst)


def test_write_then_read_is_identity_at_4k(fk, oracle):
    """Size-independent property at a full frame: pixels whose chroma is constant over each covered block survive
    write -> read unchanged, in every format."""
    w, h = 3840, 2160
    for name, fmt in B.YUV_FORMATS.items():
        raw, dt = random_raw(oracle, fmt, 77, w, h)
        d_raw = dev(raw)
        yuv = empty((h, w, 3), dt)
        fk.read_yuv(fmt, d_raw, yuv)
        again = dev(np.zeros_like(raw))
        fk.write_yuv(fmt, yuv, again)
        torch.cuda.synchronize()
        assert torch.equal(again, d_raw), name


def test_argument_errors(fk):
    raw = torch.zeros((12, 8), dtype=torch.uint8, device="cuda")
    out = torch.zeros((8, 8, 3), dtype=torch.uint8, device="cuda")
    with pytest.raises(fk.FkError, match="unsupported"):
        fk.read_yuv(9, raw, out)  # Y416: declared by the reference, but its read does not compile there
    with pytest.raises(fk.FkError, match="unsupported"):
        fk.yuv_to_rgb(fk.NV12, fk.RANGE_LIMITED, fk.BT601, raw, out)  # no matrix defined for this pair
    with pytest.raises(fk.FkError, match="argument"):
        fk.read_yuv(fk.NV12, raw, torch.zeros((7, 8, 3), dtype=torch.uint8, device="cuda"))  # odd height
    with pytest.raises(fk.FkError, match="argument"):
        fk.yuv_crop_resize_norm_split(fk.NV12, fk.RANGE_FULL, fk.BT709, raw, (8, 8), (4, 4, 8, 2),
                                      torch.zeros((3, 4, 4), device="cuda"), 1.0)  # crop leaves the image
