"""GPU parity of BorderReader and Warping chains, called through the C ABI on the MI355X, against the CPU oracle
(oracle/fk_oracle_border_warp.c) on the same seeded inputs and against the vectors written by the reference's own
headers.  Bar: bit-exact, float outputs included."""
import os
import sys

import numpy as np
import pytest
import torch

from conftest import same_bits
from oracle import binding as B

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import make_golden_border_warp as G  # noqa: E402

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_border_warp_vectors.npz"))


def dev(a, extra_cols=0):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    if extra_cols:
        shape = list(t.shape)
        shape[1] += extra_cols
        big = torch.zeros(shape, dtype=t.dtype, device="cuda")
        big[:, :t.shape[1]] = t
        t = big[:, :t.shape[1]]
    return t


def out_u8(w, h, extra_cols=0):
    return torch.full((h, w + extra_cols, 3), 85, dtype=torch.uint8, device="cuda")[:, :w]


def out_f32(w, h, extra_cols=0):
    return torch.full((h, w + extra_cols, 3), float("nan"), device="cuda")[:, :w]


def host(t):
    return np.ascontiguousarray(t.cpu().numpy())


@pytest.mark.parametrize("name", list(B.BORDER_TYPES))
def test_border_reference_vectors(fk, oracle, name):
    src = dev(oracle.bytes(G.SEED, G.SRC))
    for i, (left, top, dw, dh) in enumerate(G.WINDOWS):
        out = out_u8(dw, dh)
        fk.border_crop_u8c3(B.BORDER_TYPES[name], src, left, top, out, G.VALUE)
        assert same_bits(host(out), GOLD[f"border_{name}_{i}"]), i


@pytest.mark.parametrize("name", list(G.WARPS))
def test_warp_reference_vectors_with_literal_build(oracle, name):
    """The reference's CPU backend takes the bilinear row index from the x coordinate; the library variant built the
    same way reproduces its warp vectors bit for bit."""
    import fusedkernellibrary_amd as lib
    wt, m, dst = G.WARPS[name]
    lib.use_literal_interpolation(True)
    try:
        lib.load()
        out = out_f32(*dst)
        lib.warp_u8c3_f32c3(wt, m, dev(oracle.bytes(G.SEED, G.SRC)), out)
        torch.cuda.synchronize()
        assert same_bits(host(out), GOLD[f"warp_{name}"])
    finally:
        lib.use_literal_interpolation(False)
        lib.load()


@pytest.mark.parametrize("name", list(B.BORDER_TYPES))
def test_border_vs_oracle(fk, oracle, name):
    bt = B.BORDER_TYPES[name]
    cases = [((1, 1), 3, 2, (8, 5), 0), ((13, 11), 5, 5, (23, 21), 0), ((640, 360), 16, 9, (672, 378), 6),
             ((200, 120), -40, -30, (64, 48), 0), ((64, 48), 300, 200, (700, 500), 0), ((1920, 1080), 64, 64, (2048, 1208), 0)]
    for i, ((w, h), left, top, dst, pad) in enumerate(cases):
        src = oracle.bytes(30 + i, (h, w, 3))
        out = out_u8(*dst, pad)
        fk.border_crop_u8c3(bt, dev(src, pad), left, top, out, (11, 22, 33))
        assert same_bits(host(out), oracle.border_crop_u8c3(bt, src, left, top, dst, (11, 22, 33))), (w, h, left, top, dst)


def warp_matrices():
    rot = np.deg2rad(17.0)
    c, s = float(np.cos(rot)), float(np.sin(rot))
    return [(B.WARP_AFFINE, [[1, 0, 0], [0, 1, 0]]), (B.WARP_AFFINE, [[c, -s, 40.5], [s, c, -20.25]]),
            (B.WARP_AFFINE, [[2.5, 0, -3], [0, 1.75, 0.5]]), (B.WARP_AFFINE, [[0.31, 0, 0], [0, 0.29, 0]]),
            (B.WARP_PERSPECTIVE, [[0.9, 0.05, 1.0], [-0.02, 0.97, 2.0], [1e-4, -5e-5, 1.0]]),
            (B.WARP_PERSPECTIVE, [[1.2, 0.3, -40.0], [0.1, 1.4, -20.0], [8e-4, 6e-4, 1.0]])]


@pytest.mark.parametrize("size,dst,pad", [((1, 1), (3, 3), 0), ((33, 17), (40, 20), 0), ((640, 360), (320, 200), 4), ((1920, 1080), (1280, 720), 0)])
def test_warp_vs_oracle(fk, oracle, size, dst, pad):
    w, h = size
    src = oracle.bytes(50 + w, (h, w, 3))
    d_src = dev(src, pad)
    for wt, m in warp_matrices():
        out = out_f32(*dst, pad)
        fk.warp_u8c3_f32c3(wt, m, d_src, out)
        torch.cuda.synchronize()
        assert same_bits(host(out), oracle.warp_u8c3_f32c3(wt, m, src, dst)), (wt, m)


def test_full_frame_properties(fk, oracle):
    """At 4K: the identity warp returns the image; a wrapped window shifted by the image size returns the same window."""
    src = oracle.bytes(99, (2160, 3840, 3))
    d_src = dev(src)
    out = out_f32(3840, 2160)
    fk.warp_u8c3_f32c3(B.WARP_AFFINE, [[1, 0, 0], [0, 1, 0]], d_src, out)
    assert torch.equal(out, d_src.float())
    a, b = out_u8(3840, 2160), out_u8(3840, 2160)
    fk.border_crop_u8c3(B.BORDER_WRAP, d_src, 100, 50, a)
    fk.border_crop_u8c3(B.BORDER_WRAP, d_src, 100 + 3840, 50 - 2160, b)
    assert torch.equal(a, b) and torch.equal(a, torch.roll(d_src, shifts=(50, 100), dims=(0, 1)))
    c = out_u8(3840 + 64, 2160 + 64)
    fk.border_crop_u8c3(B.BORDER_REFLECT_101, d_src, 32, 32, c)
    assert torch.equal(c[32:-32, 32:-32], d_src) and torch.equal(c[:32, 32:-32], torch.flip(d_src[1:33], dims=(0,)))


def test_large_outputs_vs_oracle(fk, oracle):
    """Outputs of 4 M elements and more run four elements per thread: a rotation and a perspective map into 2601 x 1701
    (a width that is no multiple of the 256-element tile, rows padded) and a reflected border, element for element."""
    import math
    w, h = 1930, 1090
    src = oracle.bytes(123, (h, w, 3))
    d_src = dev(src, 5)
    dst = (2601, 1701)
    a = math.radians(7.0)
    maps = [(B.WARP_AFFINE, [[math.cos(a) * 0.7, -math.sin(a) * 0.7, 40.0], [math.sin(a) * 0.7, math.cos(a) * 0.7, -150.0]]),
            (B.WARP_PERSPECTIVE, [[0.8, 0.02, -30.0], [0.01, 0.7, 10.0], [1e-5, -2e-5, 1.0]])]
    for wt, m in maps:
        out = out_f32(*dst, 3)
        fk.warp_u8c3_f32c3(wt, m, d_src, out)
        torch.cuda.synchronize()
        assert same_bits(host(out), oracle.warp_u8c3_f32c3(wt, m, src, dst)), wt
    big = out_u8(w + 2 * 300, h + 2 * 300, 7)
    fk.border_crop_u8c3(B.BORDER_REFLECT, d_src, 300, 300, big)
    torch.cuda.synchronize()
    assert same_bits(host(big), oracle.border_crop_u8c3(B.BORDER_REFLECT, src, 300, 300, (w + 600, h + 600)))
    # rows that start at whole dwords (2532 * 3 bytes): a thread then packs four neighbouring pixels into three dwords;
    # the width is odd, so the last thread of a row holds one pixel
    for bt in (B.BORDER_REFLECT_101, B.BORDER_WRAP, B.BORDER_CONSTANT):
        packed = out_u8(w + 601, h + 600, 1)
        fk.border_crop_u8c3(bt, d_src, 300, 300, packed)
        torch.cuda.synchronize()
        assert same_bits(host(packed), oracle.border_crop_u8c3(bt, src, 300, 300, (w + 601, h + 600))), bt
        assert bool((packed._base[:, w + 601:] == 85).all()), "the padding of the rows was written"


def test_argument_errors(fk):
    src = torch.zeros((8, 8, 3), dtype=torch.uint8, device="cuda")
    with pytest.raises(fk.FkError, match="unsupported"):
        fk.border_crop_u8c3(5, src, 1, 1, out_u8(10, 10))  # TRANSPARENT_: declared by the reference, not implemented there
    with pytest.raises(fk.FkError, match="unsupported"):
        fk.warp_u8c3_f32c3(2, [[1, 0, 0], [0, 1, 0], [0, 0, 1]], src, out_f32(8, 8))


@pytest.mark.parametrize("kind,even", [(B.DEINTERLACE_BLEND, 1), (B.DEINTERLACE_INTER_LINEAR, 1), (B.DEINTERLACE_INTER_LINEAR, 0)])
def test_deinterlace(fk, oracle, kind, even):
    src = oracle.bytes(G.SEED, G.SRC)
    out = out_f32(G.SRC[1], G.SRC[0])
    fk.deinterlace_u8c3_f32c3(kind, even, dev(src), out)
    assert same_bits(host(out), GOLD[f"deinterlace_{kind}_{even}"])
    for i, ((w, h), pad) in enumerate((((1, 1), 0), ((8, 8), 0), ((33, 7), 3), ((1920, 1080), 0), ((720, 576), 4))):
        img = oracle.bytes(500 + i, (h, w, 3))
        out = out_f32(w, h, pad)
        fk.deinterlace_u8c3_f32c3(kind, even, dev(img, pad), out)
        torch.cuda.synchronize()
        assert same_bits(host(out), oracle.deinterlace_u8c3_f32c3(kind, even, img)), (w, h)
