"""Pins the BorderReader / Warping part of the oracle (oracle/fk_oracle_border_warp.c), CPU only:

 1. the border diagrams printed in the reference's own header (border_reader.h:26-33: `fedcba|abcdefgh|hgfedcb` ...);
 2. the committed vectors written by the reference's own headers (tests/golden/make_golden_border_warp.py), and that
    build directly on other seeds and windows where it is present;
 3. what the definitions fix: periodicity / symmetry of the index maps far outside the image, numpy.pad for one border
    width, and for warps: identity and integer translations, a pure scaling against the separately pinned bilinear
    sample of the resize path, agreement of the canonical row rule with the reference-pinned literal one wherever they
    pick the same row, and a double-precision evaluation.
"""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
from oracle import binding as B  # noqa: E402
import make_golden_border_warp as G  # noqa: E402

GOLD = np.load(os.path.join(HERE, "golden", "reference_border_warp_vectors.npz"))


def same_bits(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and a.tobytes() == b.tobytes()


# ---- 1. the diagrams of the reference's header ---------------------------------------------------------------------------
DIAGRAMS = {  # left of the image | the image abcdefgh | right of the image
    "REPLICATE": ("aaaaaa", "hhhhhhh"),
    "REFLECT": ("fedcba", "hgfedcb"),
    "WRAP": ("cdefgh", "abcdefg"),
    "REFLECT_101": ("gfedcb", "gfedcba"),
}


@pytest.mark.parametrize("name", list(DIAGRAMS))
def test_border_index_diagrams(oracle, name):
    left, right = DIAGRAMS[name]
    got = "".join("abcdefgh"[oracle.border_index(B.BORDER_TYPES[name], i, 8)] for i in range(-6, 15))
    assert got == left + "abcdefgh" + right
    assert [oracle.border_index(B.BORDER_CONSTANT, i, 8) for i in (-1, 0, 7, 8)] == [-1, 0, 7, -1]


# ---- 2. vectors written by the reference's own headers ---------------------------------------------------------------------
@pytest.mark.parametrize("name", list(B.BORDER_TYPES))
def test_golden_border(oracle, name):
    src = oracle.bytes(G.SEED, G.SRC)
    for i, (left, top, dw, dh) in enumerate(G.WINDOWS):
        assert same_bits(oracle.border_crop_u8c3(B.BORDER_TYPES[name], src, left, top, (dw, dh), G.VALUE), GOLD[f"border_{name}_{i}"]), i


@pytest.mark.parametrize("name", list(G.WARPS))
def test_golden_warp(oracle, name):
    src = oracle.bytes(G.SEED, G.SRC)
    wt, m, dst = G.WARPS[name]
    assert same_bits(oracle.warp_u8c3_f32c3(wt, m, src, dst, quirk=1), GOLD[f"warp_{name}"])
    coords = np.array([[oracle.warp_coords(wt, m, x, y) for x in range(0, dst[0], 5)] for y in range(0, dst[1], 5)], np.float32)
    assert same_bits(coords, GOLD[f"coords_{name}"])
    assert np.count_nonzero(GOLD[f"warp_{name}"]) > GOLD[f"warp_{name}"].size // 4  # the case does sample the image


def test_against_reference_build_other_inputs(oracle, reference):
    if reference.bw is None:
        pytest.skip("oracle/_ref/libfkref_border_warp.so not built")
    rng = np.random.RandomState(3)
    for seed, (h, w) in ((1, (1, 1)), (2, (7, 5)), (3, (64, 33))):
        src = oracle.bytes(seed, (h, w, 3))
        for bt in B.BORDER_TYPES.values():
            for _ in range(4):
                left, top = (int(v) for v in rng.randint(-2 * w - 3, 2 * w + 4, 2))
                dst = (int(rng.randint(1, 3 * w + 2)), int(rng.randint(1, 3 * h + 2)))
                assert same_bits(oracle.border_crop_u8c3(bt, src, left, top, dst, (1, 2, 3)), reference.border_crop_u8c3(bt, src, left, top, dst, (1, 2, 3)))
        if h >= w and w > 1:
            for _ in range(4):
                a = rng.uniform(-0.3, 0.3, (3, 3)) + np.eye(3)
                a[:2, 2] = rng.uniform(-3, 3, 2)
                a[2, :2] = rng.uniform(-2e-3, 2e-3, 2)
                a[2, 2] = 1.0
                assert same_bits(oracle.warp_u8c3_f32c3(B.WARP_AFFINE, a[:2], src, (w + 3, h + 2), quirk=1),
                                 reference.warp_u8c3_f32c3(B.WARP_AFFINE, a[:2], src, (w + 3, h + 2)))
                assert same_bits(oracle.warp_u8c3_f32c3(B.WARP_PERSPECTIVE, a, src, (w + 3, h + 2), quirk=1),
                                 reference.warp_u8c3_f32c3(B.WARP_PERSPECTIVE, a, src, (w + 3, h + 2)))


# ---- 3. what the definitions fix ---------------------------------------------------------------------------------------------
def test_border_index_identities(oracle):
    for n in (1, 2, 5, 8):
        for i in range(-4 * n, 5 * n):
            assert oracle.border_index(B.BORDER_WRAP, i, n) == i % n
            assert oracle.border_index(B.BORDER_REPLICATE, i, n) == min(max(i, 0), n - 1)
        for i in range(-n, 2 * n):  # one reflection on either side is what every definition of these borders agrees on
            refl = i if 0 <= i < n else (-i - 1 if i < 0 else 2 * n - 1 - i)
            assert oracle.border_index(B.BORDER_REFLECT, i, n) == refl
        for i in range(-(n - 1), 2 * n - 1):
            if n > 1:
                r101 = i if 0 <= i < n else (-i if i < 0 else 2 * (n - 1) - i)
                assert oracle.border_index(B.BORDER_REFLECT_101, i, n) == r101
        for bt in (B.BORDER_REFLECT, B.BORDER_REFLECT_101, B.BORDER_WRAP, B.BORDER_REPLICATE):
            assert all(0 <= oracle.border_index(bt, i, n) < n for i in range(-50, 60))


def test_border_crop_equals_numpy_pad(oracle):
    src = oracle.bytes(9, (11, 13, 3))
    pad = 5
    modes = {"REPLICATE": dict(mode="edge"), "REFLECT": dict(mode="symmetric"), "WRAP": dict(mode="wrap"), "REFLECT_101": dict(mode="reflect"),
             "CONSTANT": dict(mode="constant", constant_values=0)}
    for name, kw in modes.items():
        want = np.pad(src, ((pad, pad), (pad, pad), (0, 0)), **kw)
        got = oracle.border_crop_u8c3(B.BORDER_TYPES[name], src, pad, pad, (13 + 2 * pad, 11 + 2 * pad), (0, 0, 0))
        assert same_bits(got, want), name
    got = oracle.border_crop_u8c3(B.BORDER_CONSTANT, src, 2, 1, (17, 13), (200, 100, 50))
    assert tuple(got[0, 0]) == (200, 100, 50) and same_bits(got[1:12, 2:15], src)


def test_warp_identity_translation_and_scaling(oracle):
    src = oracle.bytes(4, (24, 20, 3))
    ident = [[1, 0, 0], [0, 1, 0]]
    assert same_bits(oracle.warp_u8c3_f32c3(B.WARP_AFFINE, ident, src, (20, 24)), src.astype(np.float32))
    assert same_bits(oracle.warp_u8c3_f32c3(B.WARP_PERSPECTIVE, ident + [[0, 0, 1]], src, (20, 24)), src.astype(np.float32))
    # integer translation: dst(x, y) = src(x + 3, y - 2), zero where that leaves the image
    moved = oracle.warp_u8c3_f32c3(B.WARP_AFFINE, [[1, 0, 3], [0, 1, -2]], src, (20, 24))
    want = np.zeros((24, 20, 3), np.float32)
    want[2:, :17] = src[:22, 3:]
    assert same_bits(moved, want)
    # a projective scale (all three rows doubled) is the same map
    assert same_bits(oracle.warp_u8c3_f32c3(B.WARP_PERSPECTIVE, [[2, 0, 6], [0, 2, -4], [0, 0, 2]], src, (20, 24)), want)
    # pure scaling = the resize path's sample at (x * sx, y * sy), pinned in tests/test_oracle_pinning.py
    sx, sy = np.float32(0.75), np.float32(1.5)
    got = oracle.warp_u8c3_f32c3(B.WARP_AFFINE, [[sx, 0, 0], [0, sy, 0]], src, (26, 16))
    for y in range(16):
        for x in range(26):
            cx, cy = np.float32(x) * sx, np.float32(y) * sy
            assert cx < 20 and cy < 24
            assert same_bits(got[y, x], oracle.bilinear_u8(src, (0, 0), (20, 24), cx, cy))


def test_warp_canonical_against_literal_and_double(oracle):
    src = oracle.bytes(G.SEED, G.SRC).astype(np.uint8)
    h, w, _ = src.shape
    for name, (wt, m, dst) in G.WARPS.items():
        can = oracle.warp_u8c3_f32c3(wt, m, src, dst)
        lit = oracle.warp_u8c3_f32c3(wt, m, src, dst, quirk=1)
        m64 = np.array(m, np.float64)
        checked = 0
        for y in range(dst[1]):
            for x in range(dst[0]):
                c = oracle.warp_coords(wt, m, x, y)
                inside = 0 <= c[0] < w and 0 <= c[1] < h
                if not inside:
                    assert not can[y, x].any()
                    continue
                if np.floor(c[0]) == np.floor(c[1]):
                    assert same_bits(can[y, x], lit[y, x])
                    checked += 1
                # double-precision bilinear at the double-precision coordinate
                v = m64 @ np.array([x, y, 1.0])
                cx, cy = (v[0] / v[2], v[1] / v[2]) if wt == B.WARP_PERSPECTIVE else (v[0], v[1])
                x1, y1 = int(np.floor(c[0])), int(np.floor(c[1]))
                if abs(cx - c[0]) > 1e-3 or abs(cy - c[1]) > 1e-3:
                    pytest.fail("coordinates drifted")
                x2, y2 = min(x1 + 1, w - 1), min(y1 + 1, h - 1)
                fx, fy = cx - x1, cy - y1
                ref = (src[y1, x1] * (1 - fx) * (1 - fy) + src[y1, x2] * fx * (1 - fy) + src[y2, x1] * (1 - fx) * fy + src[y2, x2] * fx * fy)
                np.testing.assert_allclose(can[y, x], ref, rtol=1e-4, atol=0.35)
        assert checked >= 3


# ---- Deinterlace --------------------------------------------------------------------------------------------------------------
def test_deinterlace_known_answers_and_golden(oracle):
    # the BLEND table of the reference's own unit test (utests/algorithm/image_processing/utest_deinterlace.h:24-45):
    # lines alternate (2, 4, 8) and (1, 1, 1); every line but the first becomes (2, 3, 5)
    src = np.empty((8, 8, 3), np.uint8)
    src[0::2] = (2, 4, 8)
    src[1::2] = (1, 1, 1)
    want = np.empty((8, 8, 3), np.float32)
    want[0] = (2, 4, 8)
    want[1:] = (2, 3, 5)
    assert same_bits(oracle.deinterlace_u8c3_f32c3(B.DEINTERLACE_BLEND, 1, src), want)
    # INTER_LINEAR on the same image, from the operation's code: kept lines unchanged, rebuilt lines (a + b + 1) * 0.5
    even = oracle.deinterlace_u8c3_f32c3(B.DEINTERLACE_INTER_LINEAR, 1, src)
    assert np.all(even[0::2] == (2, 4, 8)) and np.all(even[1:7:2] == (2.5, 4.5, 8.5)) and np.all(even[7] == (1, 1, 1))
    odd = oracle.deinterlace_u8c3_f32c3(B.DEINTERLACE_INTER_LINEAR, 0, src)
    assert np.all(odd[1::2] == (1, 1, 1)) and np.all(odd[2::2] == (1.5, 1.5, 1.5)) and np.all(odd[0] == (2, 4, 8))
    img = oracle.bytes(G.SEED, G.SRC)
    for kind, ev in ((B.DEINTERLACE_BLEND, 1), (B.DEINTERLACE_INTER_LINEAR, 1), (B.DEINTERLACE_INTER_LINEAR, 0)):
        assert same_bits(oracle.deinterlace_u8c3_f32c3(kind, ev, img), GOLD[f"deinterlace_{kind}_{ev}"])


def test_deinterlace_closed_forms_and_reference(oracle, reference):
    img = oracle.bytes(77, (12, 9, 3))
    i32 = img.astype(np.int32)
    blend = oracle.deinterlace_u8c3_f32c3(B.DEINTERLACE_BLEND, 1, img)
    assert same_bits(blend[0], img[0].astype(np.float32)) and same_bits(blend[1:], ((i32[1:] + i32[:-1] + 1) * np.float32(0.5)).astype(np.float32))
    even = oracle.deinterlace_u8c3_f32c3(B.DEINTERLACE_INTER_LINEAR, 1, img)
    assert same_bits(even[0::2], img[0::2].astype(np.float32)) and same_bits(even[11], img[11].astype(np.float32))
    assert same_bits(even[1:11:2], ((i32[0:10:2] + i32[2:12:2] + 1) * np.float32(0.5)).astype(np.float32))
    odd_h = oracle.bytes(78, (7, 5, 3))  # an odd number of lines: the last line passes through in both fields
    for ev in (0, 1):
        assert same_bits(oracle.deinterlace_u8c3_f32c3(B.DEINTERLACE_INTER_LINEAR, ev, odd_h)[6], odd_h[6].astype(np.float32))
    if reference.bw is not None:
        for seed, shape in ((1, (2, 1, 3)), (2, (10, 33, 3)), (3, (64, 64, 3))):
            a = oracle.bytes(seed, shape)
            for kind, ev in ((B.DEINTERLACE_BLEND, 1), (B.DEINTERLACE_INTER_LINEAR, 1), (B.DEINTERLACE_INTER_LINEAR, 0)):
                assert same_bits(oracle.deinterlace_u8c3_f32c3(kind, ev, a), reference.deinterlace_u8c3_f32c3(kind, ev, a))
