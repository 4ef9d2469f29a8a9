"""Oracle against the reference's own headers, run side by side on seeded inputs (only where oracle/_ref was built:
the build container).  Same literal host semantics on both sides (quirk_y1_from_x=1); resize inputs keep that branch
inside the image (crop.y + floor(sx_max) + 1 < image height)."""
import numpy as np
import pytest

from conftest import same_bits
from oracle import binding as B


@pytest.mark.parametrize("seed", [101, 102, 103])
def test_readme_chain_random_crops(oracle, reference, seed):
    h, w = 700, 320
    src = oracle.bytes(seed, (h, w, 3))
    n = 5
    ws = oracle.uniform_ints(seed + 1, 8, 300, n)
    hs = oracle.uniform_ints(seed + 2, 8, 200, n)
    rects = [(int((w - ww) * 0.3), 7 * i, int(ww), int(hh)) for i, (ww, hh) in enumerate(zip(ws, hs))]
    for aspect in (0, 1, 2, 3):
        args = (src, rects, (47, 31), aspect, (0.5, 1.5, -2.0), (1.4, 1.1, 0.9), (0.5, 0.25, 0.125), (255., 127., 3.))
        assert same_bits(oracle.crop_resize_muls_bgr_tensor(*args, quirk=1), reference.crop_resize_muls_bgr_tensor(*args))


@pytest.mark.parametrize("n", [1, 2, 3, 8])
def test_split_chain_batches(oracle, reference, n):
    srcs = [oracle.bytes(200 + i, (640, 200, 3)) for i in range(n)]
    rects = [(3 * i, 2 * i, 40 + 17 * i, 30 + 5 * i) for i in range(n)]
    args = (srcs, rects, (56, 40), (255.,) * 3, (.485, .456, .406), (.229, .224, .225))
    assert same_bits(oracle.batch_crop_resize_norm_split(*args, quirk=1), reference.batch_crop_resize_norm_split(*args))


def test_tiles_chain_32(oracle, reference):
    src = oracle.gradient_noise_u8c3(4, 120, 900)
    rects = [(4 * i, 6 * j, 8, 8) for j in range(4) for i in range(8)]
    args = (src, (40, 300), rects, (8, 8), (1 / 255.,) * 3)
    assert same_bits(oracle.resize_crop_tiles(*args, quirk=1), reference.resize_crop_tiles(*args))


def test_pointwise_chains_full_rows_and_pitch(oracle, reference):
    base = oracle.unit_floats(2, (37, 64, 3))
    view = base[:, :53]  # pitch larger than the row
    for d in (1, 2, 4, 8, 16):
        assert same_bits(oracle.muladd_chain_f32c3(view, d, 1.0001, 1e-4), reference.muladd_chain_f32c3(view, d, 1.0001, 1e-4))
    img = oracle.bytes(5, (130, 140, 4))
    v4 = img[:, :129]
    assert same_bits(oracle.rgba2gray_u8c4(v4), reference.rgba2gray_u8c4(v4))
    assert same_bits(oracle.rgba2bgr_sub_u8c4_f32c3(v4, 0.5), reference.rgba2bgr_sub_u8c4_f32c3(v4, 0.5))
    assert same_bits(oracle.crop_mul_saturate_u8c4(v4, (9, 11, 100, 64), 3), reference.crop_mul_saturate_u8c4(v4, (9, 11, 100, 64), 3))
    sq = img[:128, :128]
    assert same_bits(oracle.resize_mul_u8c4_f32c4(sq, (8, 8), 1 / 255., quirk=1), reference.resize_mul_u8c4_f32c4(sq, (8, 8), 1 / 255.))


def test_ragged_crops_exec_all_like_reference(oracle, reference):
    src = oracle.bytes(7, (90, 120, 3))
    rects = [(1, 2, 30, 20), (5, 5, 10, 25)]
    assert same_bits(oracle.batch_crop_cast_tensor(src, rects, (30, 25), exec_all=1), reference.batch_crop_cast_tensor(src, rects, (30, 25)))
