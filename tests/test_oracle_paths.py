"""Pins the oracle's restatement of the less common chain shapes (oracle/fk_oracle_paths.c): batch reads with
CONDITIONAL_WITH_DEFAULT, a write in the middle of a chain, a batch of output images, a tensor as the source.

Three kinds of pin, chosen so that a plausible mistake fails one of them (a default applied to the wrong planes or with
the comparison the wrong way round, the mid value taken after the addition, a crop offset dropped, channels swapped):
vectors written by the reference's own headers (committed), side-by-side runs against the reference build on other
seeds where it is present, and closed forms in numpy."""
import os
import sys

import numpy as np
import pytest

from conftest import same_bits

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_golden_paths as G  # noqa: E402  (the cases and their seeds)

GOLD = np.load(os.path.join(HERE, "golden", "reference_paths_vectors.npz"))


def test_reference_vectors_bit_for_bit(oracle):
    """The reference's CPU backend interpolates with its host rule (row index from x): the oracle with that rule
    reproduces every vector."""
    got = G.run(oracle, oracle, quirk=1)
    assert set(got) == set(GOLD.files) and len(got) == 18
    for name in GOLD.files:
        assert same_bits(got[name], GOLD[name]), name


def test_side_by_side_with_the_reference_build(oracle, reference):
    if reference.paths is None:
        pytest.skip("oracle/_ref/libfkref_paths.so not built")
    for seed in (101, 202):
        for n in (2, 3, 4, 8):
            srcs = [oracle.bytes(seed + i, (20 + n, 12, 3)) for i in range(n)]
            for used in (0, 1, n - 1, n, n + 3):
                assert same_bits(oracle.conditional_copy_u8c3(srcs, used, (1, 2, 3)), reference.conditional_copy_u8c3(srcs, used, (1, 2, 3)))
                assert same_bits(oracle.conditional_resize_f32c3(srcs, used, (9.5, 0.0, -1.0), (17, 9), quirk=1),
                                 reference.conditional_resize_f32c3(srcs, used, (9.5, 0.0, -1.0), (17, 9)))
            src = oracle.bytes(seed + 50, (64, 80, 3))
            rects = [(3 * i, 5 * i, 21, 17) for i in range(n)]
            for a, b in zip(oracle.batch_crop_cast_images(src, rects), reference.batch_crop_cast_images(src, rects)):
                assert same_bits(a, b)
            gray = oracle.bytes(seed + 70, (40, 90))
            windows = [(i, i, 31, 19) for i in range(n)]
            for ops in ((1.0, 1.0, 3.2), (0.37, -4.5, 0.003)):
                assert same_bits(oracle.batch_windows_saturate_muls_f32(gray, windows, *ops), reference.batch_windows_saturate_muls_f32(gray, windows, *ops))
        f = oracle.unit_floats(seed, 5 * 9 * 13 * 3).reshape(5, 9, 13, 3)
        assert same_bits(oracle.tensor_mul_f32c3(f, (3.0, 0.1, -7.0)), reference.tensor_mul_f32c3(f, (3.0, 0.1, -7.0)))
        for a, b in zip(oracle.muladd_midwrite_f32c3(f[0], 1.0001, 1e-4), reference.muladd_midwrite_f32c3(f[0], 1.0001, 1e-4)):
            assert same_bits(a, b)


def test_conditional_copy_closed_form(oracle):
    srcs = [oracle.bytes(300 + i, (6, 11, 3)) for i in range(5)]
    for used in range(-1, 8):
        got = oracle.conditional_copy_u8c3(srcs, used, (250, 0, 17))
        for z in range(5):
            want = srcs[z] if z < used else np.broadcast_to(np.array([250, 0, 17], np.uint8), (6, 11, 3))
            assert np.array_equal(got[z], want), (used, z)


def test_conditional_resize_is_the_pinned_resize_on_used_planes(oracle):
    """Used planes equal the pinned chain resize -> x1 -> -0 -> /1 of the README pipeline without channel swap (the
    resize of fk_oracle.c); the others hold the default exactly, also values no resize could produce."""
    srcs = [oracle.bytes(400 + i, (23, 31, 3)) for i in range(4)]
    default = (-1.5, 1000.0, float(np.float32(0.1)))
    for quirk in (0, 1):
        if quirk == 1:
            srcs = [oracle.bytes(400 + i, (40, 29, 3)) for i in range(4)]  # taller than wide for the host rule
        h, w, _ = srcs[0].shape
        got = oracle.conditional_resize_f32c3(srcs, 2, default, (19, 13), quirk=quirk)
        for z in range(2):
            # IGNORE_AR resize of the whole image through the README chain with neutral arithmetic; RGB2BGR undone
            from oracle import binding as B
            plane = oracle.crop_resize_muls_bgr_tensor(srcs[z], [(0, 0, w, h)], (19, 13), B.IGNORE_AR, (0, 0, 0), (1.0,) * 3, (0.0,) * 3, (1.0,) * 3, quirk=quirk)[0]
            assert same_bits(got[z], np.ascontiguousarray(plane[..., ::-1]))
        for z in (2, 3):
            assert same_bits(got[z], np.broadcast_to(np.array(default, np.float32), (13, 19, 3)).copy())


def test_midwrite_and_tensor_closed_forms(oracle):
    f = oracle.unit_floats(500, 7 * 9 * 3).reshape(7, 9, 3)
    mid, out = oracle.muladd_midwrite_f32c3(f, 2.5, 0.125)
    assert same_bits(mid, f * np.float32(2.5)) and same_bits(out, f * np.float32(2.5) + np.float32(0.125))
    assert not same_bits(mid, out)
    t = oracle.unit_floats(501, 2 * 4 * 5 * 3).reshape(2, 4, 5, 3)
    assert same_bits(oracle.tensor_mul_f32c3(t, (2.0, -3.0, 0.5)), t * np.array([2.0, -3.0, 0.5], np.float32))


def test_batch_images_closed_form(oracle):
    src = oracle.bytes(600, (30, 45, 3))
    rects = [(1, 2, 8, 6), (37, 24, 8, 6), (10, 10, 8, 6)]
    for (x, y, w, h), img in zip(rects, oracle.batch_crop_cast_images(src, rects)):
        assert same_bits(img, src[y:y + h, x:x + w].astype(np.float32))
    with pytest.raises(ValueError):
        oracle.batch_crop_cast_images(src, [(0, 0, 8, 6), (0, 0, 9, 6)])


def test_windows_chain_closed_form(oracle):
    """((float)v * mul - sub) / div with every step rounded to float, per window; the benchmark's own check: all elements of
    an image filled with 10 give (10 * 1 - 1) / 3.2."""
    src = oracle.bytes(400, (50, 64))
    rects = [(i, 2 * i, 20, 12) for i in range(9)]
    got = oracle.batch_windows_saturate_muls_f32(src, rects, 1.4, 0.5, 255.0)
    for z, (x, y, w, h) in enumerate(rects):
        want = (src[y:y + h, x:x + w].astype(np.float32) * np.float32(1.4) - np.float32(0.5)) / np.float32(255.0)
        assert same_bits(got[z], want.astype(np.float32)), z
    flat = np.full((130, 70), 10, np.uint8)
    got = oracle.batch_windows_saturate_muls_f32(flat, [(i, i, 60, 120) for i in range(10)], 1.0, 1.0, 3.2)
    assert np.all(got == np.float32(9.0) / np.float32(3.2))
