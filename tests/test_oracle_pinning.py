"""Pins the CPU oracle (oracle/fk_oracle.c) before anything is compared with it.

 1. against the committed golden vectors, written by the reference's own headers (tests/golden/make_golden.py),
    bit for bit, with the oracle in the reference's literal host semantics (quirk_y1_from_x=1);
 2. the canonical semantics (row index from y) differs from that by one token; it is pinned by the same reference
    vectors on every element whose floor(sx) == floor(sy), and by what the mathematics fixes: identity at scale 1,
    constant images, exact ramps, transposition symmetry, a double-precision brute force;
 3. against known answers that the reference's own unit tests hold (utests/algorithm/image_processing/
    utest_color_conversion.h:42-57,89-101,120-137; utests/.../utest_saturate.h:66-84) and the Resize parameters its
    README chain produces;
 4. the seeded generator against SplitMix64's published outputs.
"""
import json
import os

import numpy as np
import pytest

from conftest import same_bits
from oracle import binding as B

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = np.load(os.path.join(HERE, "golden", "reference_vectors.npz"))
CASES = json.load(open(os.path.join(HERE, "golden", "reference_cases.json")))


# ---- 4. generator -----------------------------------------------------------------------------------------------
def test_splitmix64_published_vector(oracle):
    # first outputs of SplitMix64 seeded with 1234567 (Vigna's splitmix64.c test values)
    want = [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431, 16408922859458223821]
    raw = oracle.bytes(1234567, (40,))
    got = np.frombuffer(raw.tobytes(), dtype="<u8").tolist()
    assert got == want


def test_generator_shapes(oracle):
    b = oracle.bytes(9, (13,))
    assert same_bits(b[:8], oracle.bytes(9, (8,)))  # ragged tail continues the same stream
    f = oracle.unit_floats(2, (1000,))
    assert f.min() >= 0.0 and f.max() < 1.0
    first = int(np.frombuffer(oracle.bytes(2, (8,)).tobytes(), "<u8")[0])
    assert f[0] == np.float32(first >> 40) * np.float32(2.0 ** -24)
    ints = oracle.uniform_ints(5, 16, 512, 2000)
    assert ints.min() >= 16 and ints.max() <= 512
    g = oracle.gradient_noise_u8c3(4, 64, 48)
    assert g.shape == (48, 64, 3) and abs(int(g[0, 0, 0]) - 0) <= 16 and abs(int(g[47, 63, 0]) - 255) <= 16


# ---- 3. known answers of the reference's unit tests ---------------------------------------------------------------
def test_rgb2gray_known_answers(oracle):
    assert oracle.c.fko_rgb2gray_u8(255, 0, 0) == 76
    assert oracle.c.fko_rgb2gray_u8(0, 255, 0) == 150
    assert oracle.c.fko_rgb2gray_u8(0, 0, 255) == 29
    assert oracle.c.fko_rgb2gray_u8(50, 100, 150) == int(np.rint(np.float32(50) * np.float32(.299) + np.float32(100) * np.float32(.587) + np.float32(150) * np.float32(.114)))
    ins, outs = GOLD["probe_gray_in"], GOLD["probe_gray_out"]
    assert [oracle.c.fko_rgb2gray_u8(int(a), int(b), int(c)) for a, b, c in ins] == outs.tolist()


def test_bgr_reorder_known_answer(oracle):
    # COLOR_BGR2RGB {100,150,200} -> {200,150,100}: the chain's reorder, seen through a 1x1 identity resize
    src = np.array([[[100, 150, 200]]], np.uint8)
    out = oracle.crop_resize_muls_bgr_tensor(src, [(0, 0, 1, 1)], (1, 1), B.IGNORE_AR, (0, 0, 0), (1,) * 3, (0,) * 3, (1,) * 3)
    assert out.reshape(3).tolist() == [200.0, 150.0, 100.0]


def test_saturate_and_round_known_answers(oracle):
    c = oracle.c
    # SaturateCast<float,uchar>: min / half / max of the input range, and the rounding of .5 away from zero
    assert [c.fko_saturate_float_to_u8(v) for v in (-1e30, 0.0, 127.5, 255.0, 1e30)] == [0, 0, 128, 255, 255]
    assert [c.fko_saturate_int_to_u8(v) for v in (-2 ** 31, -1, 0, 128, 255, 256, 2 ** 31 - 1)] == [0, 0, 0, 128, 255, 255, 255]
    assert [c.fko_saturate_float_to_u8(float(v)) for v in GOLD["probe_satf_in"]] == GOLD["probe_satf_out"].tolist()
    assert [c.fko_saturate_int_to_u8(int(v)) for v in GOLD["probe_sati_in"]] == GOLD["probe_sati_out"].tolist()
    got = np.array([c.fko_round(float(v)) for v in GOLD["probe_round_in"]], np.float32)
    assert same_bits(got, GOLD["probe_round_out"])
    assert c.fko_round(2.5) == 3.0 and c.fko_round(-2.5) == -3.0
    assert c.fko_round(0.49999997) == 1.0  # x + 0.5f rounds up to 1.0f before the truncation, as in the reference


def test_resize_parameters_of_the_readme_chain(oracle):
    # values read out of the reference for its README chain: region, conversion factors, source size per plane
    want = [((0, 8, 59, 51), 0.566666663, 0.568181813, (34, 25)),
            ((0, 23, 59, 35), 1.16666663, 1.15384614, (70, 15)),
            ((0, 0, 59, 58), 1.0, 1.0, (60, 59)),
            ((4, 0, 55, 59), 0.384615391, 0.383333325, (20, 23)),
            ((0, 2, 59, 56), 0.200000003, 0.200000003, (12, 11))]
    for rect, (roi, fx, fy, size) in zip(CASES["readme"]["rects"], want):
        p = oracle.resize_build(B.PRESERVE_AR, rect[2], rect[3], 60, 60)
        assert (p.x1, p.y1, p.x2, p.y2) == roi and (p.src_w, p.src_h) == size
        assert np.float32(p.fx) == np.float32(fx) and np.float32(p.fy) == np.float32(fy)


def test_resize_build_variants(oracle):
    p = oracle.resize_build(B.IGNORE_AR, 70, 15, 60, 60)
    assert np.float32(p.fx) == np.float32(1.0 / (60.0 / 70.0)) and np.float32(p.fy) == np.float32(1.0 / (60.0 / 15.0))
    left = oracle.resize_build(B.PRESERVE_AR_LEFT, 20, 23, 60, 60)
    assert (left.x1, left.x2) == (0, 51)
    even = oracle.resize_build(B.PRESERVE_AR_RN_EVEN, 21, 40, 60, 60)  # 31.5 -> 32 -> even 32
    assert (even.x2 - even.x1 + 1) % 2 == 0


# ---- 1. golden vectors from the reference's own headers -------------------------------------------------------------
def test_readme_chain_matches_reference_vectors(oracle):
    c = CASES["readme"]
    src = oracle.bytes(c["seed"], tuple(c["src"]))
    for aspect in (0, 1, 2, 3):
        got = oracle.crop_resize_muls_bgr_tensor(src, c["rects"], c["dst"], aspect, c["background"], c["mul"], c["sub"], c["div"], quirk=1)
        assert same_bits(got, GOLD[f"readme_ar{aspect}"]), aspect
    c = CASES["readme_small_bg"]
    src = oracle.bytes(c["seed"], tuple(c["src"]))
    for aspect in (0, 2, 3):
        got = oracle.crop_resize_muls_bgr_tensor(src, c["rects"], c["dst"], aspect, c["background"], c["mul"], c["sub"], c["div"], quirk=1)
        assert same_bits(got, GOLD[f"readme_small_bg_ar{aspect}"]), aspect


def test_other_chains_match_reference_vectors(oracle):
    c = CASES["split"]
    srcs = [oracle.bytes(c["seed"] + i, tuple(c["src"])) for i in range(c["n"])]
    assert same_bits(oracle.batch_crop_resize_norm_split(srcs, c["rects"], c["dst"], c["div1"], c["sub"], c["div2"], quirk=1), GOLD["split"])
    c = CASES["tiles"]
    src = oracle.gradient_noise_u8c3(c["seed"], c["src"][1], c["src"][0])
    assert same_bits(oracle.resize_crop_tiles(src, c["resized"], c["rects"], c["tile"], c["mul"], quirk=1), GOLD["tiles"])
    c = CASES["divergent"]
    src = oracle.bytes(c["seed"], tuple(c["src"]))
    assert same_bits(oracle.rgba2gray_u8c4(src), GOLD["div_gray"])
    assert same_bits(oracle.resize_mul_u8c4_f32c4(src, c["resized"], c["mul_b"], quirk=1), GOLD["div_resized"])
    assert same_bits(oracle.crop_mul_saturate_u8c4(src, c["rect_c"], c["mul_c"]), GOLD["div_crop"])
    assert same_bits(oracle.rgba2bgr_sub_u8c4_f32c3(src, c["sub_d"]), GOLD["div_bgr"])
    c = CASES["muladd"]
    src = oracle.unit_floats(c["seed"], tuple(c["src"]))
    for d in c["depths"]:
        assert same_bits(oracle.muladd_chain_f32c3(src, d, c["mul_v"], c["add_v"]), GOLD[f"muladd_{d}"]), d
    assert same_bits(oracle.single_op_f32c3(src, 0, c["mul_v"]), GOLD["single_mul"])
    assert same_bits(oracle.single_op_f32c3(src, 1, c["add_v"]), GOLD["single_add"])
    c = CASES["crops"]
    src = oracle.bytes(c["seed"], tuple(c["src"]))
    assert same_bits(oracle.batch_crop_cast_tensor(src, c["rects"], c["max_size"], exec_all=1), GOLD["crops"])


def test_deeper_chains_follow_from_shallower_ones(oracle):
    # depths beyond the reference-checked 16 are the same two operations repeated: chain(2k) == chain(k) o chain(k)
    src = oracle.unit_floats(2, (5, 7, 3))
    for d in (32, 64, 128):
        half = oracle.muladd_chain_f32c3(src, d // 2, 1.0001, 1e-4)
        assert same_bits(oracle.muladd_chain_f32c3(half, d // 2, 1.0001, 1e-4), oracle.muladd_chain_f32c3(src, d, 1.0001, 1e-4))


# ---- 2. canonical semantics (row index from y) ---------------------------------------------------------------------
def _where_rows_agree(rect, dst, aspect, oracle):
    """Mask of destination elements whose floor(sx) == floor(sy): there the reference's host branch and the canonical
    semantics read the same four source pixels with the same weights."""
    p = oracle.resize_build(aspect, rect[2], rect[3], dst[0], dst[1])
    ys, xs = np.mgrid[0:dst[1], 0:dst[0]]
    inside = (xs >= p.x1) & (xs <= p.x2) & (ys >= p.y1) & (ys <= p.y2)
    sx = (xs - p.x1).astype(np.float32) * np.float32(p.fx)
    sy = (ys - p.y1).astype(np.float32) * np.float32(p.fy)
    return ~inside | (np.floor(sx) == np.floor(sy))


def test_canonical_equals_reference_where_row_indices_agree(oracle):
    c = CASES["readme"]
    src = oracle.bytes(c["seed"], tuple(c["src"]))
    got = oracle.crop_resize_muls_bgr_tensor(src, c["rects"], c["dst"], 0, c["background"], c["mul"], c["sub"], c["div"], quirk=0)
    ref = GOLD["readme_ar0"]
    checked = 0
    for z, rect in enumerate(c["rects"]):
        m = _where_rows_agree(rect, c["dst"], 0, oracle)
        assert same_bits(got[z][m], ref[z][m])
        checked += int(m.sum())
    assert checked > 3000  # a real share of the 18000 elements, with non-trivial weights
    c = CASES["divergent"]
    src = oracle.bytes(c["seed"], tuple(c["src"]))
    got = oracle.resize_mul_u8c4_f32c4(src, c["resized"], c["mul_b"], quirk=0)
    m = _where_rows_agree((0, 0, 96, 96), c["resized"], B.IGNORE_AR, oracle)
    assert same_bits(got[m], GOLD["div_resized"][m]) and m.sum() >= 12


def test_canonical_transposition_symmetry(oracle):
    # bilinear(transposed image)(y, x) == bilinear(image)(x, y) up to the order of the two middle terms of the sum;
    # with the reference's literal host branch this symmetry does not hold
    img = oracle.bytes(21, (23, 37, 4))
    a = oracle.resize_mul_u8c4_f32c4(img, (50, 31), 1.0, quirk=0)
    b = oracle.resize_mul_u8c4_f32c4(np.ascontiguousarray(img.transpose(1, 0, 2)), (31, 50), 1.0, quirk=0)
    np.testing.assert_allclose(a, b.transpose(1, 0, 2), rtol=2e-6, atol=1e-4)
    lit = oracle.resize_mul_u8c4_f32c4(img[:23, :23], (40, 40), 1.0, quirk=1)
    lit_t = oracle.resize_mul_u8c4_f32c4(np.ascontiguousarray(img[:23, :23].transpose(1, 0, 2)), (40, 40), 1.0, quirk=1)
    assert np.abs(lit - lit_t.transpose(1, 0, 2)).max() > 1.0


def test_canonical_identity_constant_and_ramp(oracle):
    img = oracle.bytes(22, (19, 27, 4))
    assert same_bits(oracle.resize_mul_u8c4_f32c4(img, (27, 19), 1.0, quirk=0), img.astype(np.float32))  # scale 1: a copy
    const = np.full((9, 14, 4), 0, np.uint8)
    const[...] = (3, 1, 32, 200)
    out = oracle.resize_mul_u8c4_f32c4(const, (33, 20), 1.0, quirk=0)
    np.testing.assert_allclose(out, np.broadcast_to(np.array([3, 1, 32, 200], np.float32), out.shape), rtol=1e-6)
    assert np.all(out.astype(np.uint8)[..., :3] == np.array([3, 1, 32], np.uint8)) or np.all(np.rint(out)[..., :3] == [3, 1, 32])
    # ramp: channel 0 = x, channel 1 = y  ->  out = (x*fx, y*fy) exactly while no clamp applies
    h, w = 40, 60
    ramp = np.zeros((h, w, 4), np.uint8)
    ramp[..., 0] = np.arange(w)[None, :]
    ramp[..., 1] = np.arange(h)[:, None]
    dw, dh = 24, 16  # fx = fy = 2.5
    out = oracle.resize_mul_u8c4_f32c4(ramp, (dw, dh), 1.0, quirk=0)
    p = oracle.resize_build(B.IGNORE_AR, w, h, dw, dh)
    sx = np.arange(dw, dtype=np.float32) * np.float32(p.fx)
    sy = np.arange(dh, dtype=np.float32) * np.float32(p.fy)
    np.testing.assert_allclose(out[..., 0], np.broadcast_to(sx, (dh, dw)), rtol=1e-6)
    np.testing.assert_allclose(out[..., 1], np.broadcast_to(sy[:, None], (dh, dw)), rtol=1e-6)


def test_canonical_against_double_precision_brute_force(oracle):
    img = oracle.bytes(23, (11, 13, 4))
    for dst in ((29, 17), (5, 4), (13, 11)):
        out = oracle.resize_mul_u8c4_f32c4(img, dst, 1.0, quirk=0)
        p = oracle.resize_build(B.IGNORE_AR, 13, 11, dst[0], dst[1])
        for y in range(dst[1]):
            for x in range(dst[0]):
                sx = float(np.float32(x) * np.float32(p.fx))
                sy = float(np.float32(y) * np.float32(p.fy))
                x1, y1 = int(np.floor(sx)), int(np.floor(sy))
                x2r, y2r = min(x1 + 1, 12), min(y1 + 1, 10)
                a, b, c, d = (img[y1, x1].astype(np.float64), img[y1, x2r].astype(np.float64),
                              img[y2r, x1].astype(np.float64), img[y2r, x2r].astype(np.float64))
                want = (a * (x1 + 1 - sx) * (y1 + 1 - sy) + b * (sx - x1) * (y1 + 1 - sy) +
                        c * (x1 + 1 - sx) * (sy - y1) + d * (sx - x1) * (sy - y1))
                np.testing.assert_allclose(out[y, x], want, rtol=1e-5, atol=1e-4)


def test_preserve_ar_background_and_region(oracle):
    src = oracle.bytes(31, (50, 80, 3))
    out = oracle.crop_resize_muls_bgr_tensor(src, [(4, 5, 40, 10)], (32, 32), B.PRESERVE_AR, (9.0, 8.0, 7.0), (1,) * 3, (0,) * 3, (1,) * 3)
    p = oracle.resize_build(B.PRESERVE_AR, 40, 10, 32, 32)
    assert (p.x1, p.x2) == (0, 31) and p.y1 > 0 and p.y2 < 31
    assert np.all(out[0, :p.y1] == np.array([7.0, 8.0, 9.0], np.float32))  # background, channels swapped by RGB2BGR
    assert np.all(out[0, p.y2 + 1:] == np.array([7.0, 8.0, 9.0], np.float32))
    assert out[0, p.y1:p.y2 + 1].max() <= 255.0


def test_crop_reads_origin_shifted_pixels(oracle):
    # index-encoded image: a crop must return (x + rx, y + ry)
    h, w = 30, 40
    img = np.zeros((h, w, 3), np.uint8)
    img[..., 0] = np.arange(w)[None, :]
    img[..., 1] = np.arange(h)[:, None]
    out = oracle.batch_crop_cast_tensor(img, [(7, 3, 10, 6), (0, 20, 10, 6)], (10, 6), exec_all=1)
    assert np.all(out[0, :, :, 0] == np.arange(7, 17)) and np.all(out[0, :, :, 1] == np.arange(3, 9)[:, None])
    assert np.all(out[1, :, :, 0] == np.arange(0, 10)) and np.all(out[1, :, :, 1] == np.arange(20, 26)[:, None])
    part = oracle.batch_crop_cast_tensor(img, [(7, 3, 4, 2)], (10, 6), exec_all=0, fill=-1.0)
    assert np.all(part[0, 2:] == -1.0) and np.all(part[0, :2, 4:] == -1.0) and np.all(part[0, :2, :4, 0] == np.arange(7, 11))


def test_split_layout_is_n_c_h_w(oracle):
    src = oracle.bytes(41, (20, 30, 3))
    rect = (2, 3, 16, 12)
    split = oracle.batch_crop_resize_norm_split([src], [rect], (16, 12), (1,) * 3, (0,) * 3, (1,) * 3)
    packed = oracle.crop_resize_muls_bgr_tensor(src, [rect], (16, 12), B.IGNORE_AR, (0,) * 3, (1,) * 3, (0,) * 3, (1,) * 3)
    assert same_bits(split[0].transpose(1, 2, 0), packed[0])
