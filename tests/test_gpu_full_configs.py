"""GPU parity at the full shapes of the five benchmark configurations, through the C ABI, bit for bit against the CPU
oracle (the oracle is plain C and finishes each of these in well under a second or two), plus size-independent
properties on the largest ones."""
import numpy as np
import pytest
import torch

from conftest import same_bits
from oracle import binding as B

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_c2_vertical_fusion_full_size(fk, oracle):
    src = oracle.unit_floats(2, (2160, 3840, 3))
    d = dev(src)
    for depth in (1, 16, 128):
        out = torch.full((2160, 3840, 3), float("nan"), device="cuda")
        fk.muladd_chain_f32c3(d, out, depth, 1.0001, 1e-4)
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), oracle.muladd_chain_f32c3(src, depth, 1.0001, 1e-4)), depth
    # fused == the same operations as separate launches (ping-pong), whatever the depth
    a, b = d.clone(), torch.empty_like(d)
    for k in range(8):
        fk.single_op_f32c3(a, b, k % 2, 1e-4 if k % 2 else 1.0001)
        a, b = b, a
    fused = torch.empty_like(d)
    fk.muladd_chain_f32c3(d, fused, 8, 1.0001, 1e-4)
    torch.cuda.synchronize()
    assert torch.equal(a, fused)


def test_c3_horizontal_fusion_50_images(fk, oracle):
    n, w, h = 50, 1920, 1080
    srcs = [oracle.bytes(3 + i, (h, w, 3)) for i in range(n)]
    rects = []
    for i in range(n):
        cw, ch = (int(v) for v in oracle.uniform_ints(103 + i, 16, 512, 2))
        x = int(oracle.uniform_ints(203 + i, 0, w - cw, 1)[0])
        y = int(oracle.uniform_ints(303 + i, 0, h - ch, 1)[0])
        rects.append((x, y, cw, ch))
    args = ((255.,) * 3, (.485, .456, .406), (.229, .224, .225))
    want = oracle.batch_crop_resize_norm_split(srcs, rects, (224, 224), *args)
    out = torch.full((n, 3, 224, 224), float("nan"), device="cuda")
    fk.batch_crop_resize_norm_split([dev(s) for s in srcs], rects, out, *args)
    torch.cuda.synchronize()
    assert same_bits(out.cpu().numpy(), want)


def test_c4_backwards_vertical_fusion_full_size(fk, oracle):
    src = oracle.gradient_noise_u8c3(4, 3840, 2160)
    rects = [(160 * i, 180 * j, 128, 128) for j in range(4) for i in range(8)]
    want = oracle.resize_crop_tiles(src, (1280, 720), rects, (128, 128), (1 / 255.,) * 3)
    out = torch.full((32, 128, 128, 3), float("nan"), device="cuda")
    fk.resize_crop_tiles(dev(src), (1280, 720), rects, out, (1 / 255.,) * 3)
    torch.cuda.synchronize()
    assert same_bits(out.cpu().numpy(), want)
    assert 0.0 <= want.min() and want.max() <= 1.0


def test_c5_divergent_full_size(fk, oracle):
    size = 8192
    src = oracle.bytes(5, (size, size, 4))
    rect = (3584, 3584, 1024, 1024)
    gray = torch.zeros((size, size), dtype=torch.uint8, device="cuda")
    small = torch.full((512, 512, 4), float("nan"), device="cuda")
    crop = torch.zeros((1024, 1024, 4), dtype=torch.uint8, device="cuda")
    bgr = torch.full((size, size, 3), float("nan"), device="cuda")
    fk.divergent4_u8c4(dev(src), gray, small, 1 / 255., rect, 2, crop, 0.5, bgr)
    torch.cuda.synchronize()
    assert same_bits(gray.cpu().numpy(), oracle.rgba2gray_u8c4(src))
    assert same_bits(small.cpu().numpy(), oracle.resize_mul_u8c4_f32c4(src, (512, 512), 1 / 255.))
    assert same_bits(crop.cpu().numpy(), oracle.crop_mul_saturate_u8c4(src, rect, 2))
    got_bgr = bgr.cpu().numpy()
    del bgr
    assert same_bits(got_bgr, oracle.rgba2bgr_sub_u8c4_f32c3(src, 0.5))
    # size-independent properties: chain d is an exact, invertible recoding of the source; chain c saturates
    assert np.array_equal((got_bgr[..., ::-1] + 0.5).astype(np.uint8), src[..., :3])
    c = crop.cpu().numpy()
    window = src[3584:4608, 3584:4608].astype(np.int32) * 2
    assert np.array_equal(c, np.minimum(window, 255).astype(np.uint8))


README_ARGS = ((0, 0, 0), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)


@pytest.mark.parametrize("crop", [(1024, 768), (1024, 576)], ids=["4x3_with_bars", "16x9_no_bars"])
@pytest.mark.parametrize("aspect", [B.PRESERVE_AR, B.IGNORE_AR, B.PRESERVE_AR_RN_EVEN, B.PRESERVE_AR_LEFT])
def test_readme_pipeline_bandwidth_sized(fk, oracle, crop, aspect):
    """The README chain at the shapes its roofline figures are quoted on: five crops of a 4K frame -> 1920x1080 each.
    The 4:3 crops leave bars of background under PRESERVE_AR; the 16:9 crops resample every output pixel."""
    src = oracle.bytes(11, (2160, 3840, 3))
    cw, ch = crop
    rects = [(64 * i, 48 * i, cw, ch) for i in range(5)]
    want = oracle.crop_resize_muls_bgr_tensor(src, rects, (1920, 1080), aspect, *README_ARGS)
    out = torch.full((5, 1080, 1920, 3), float("nan"), device="cuda")
    fk.crop_resize_muls_bgr_tensor(dev(src), rects, out, aspect, *README_ARGS)
    torch.cuda.synchronize()
    assert same_bits(out.cpu().numpy(), want)


def test_c1_readme_matches_reference_vectors_where_defined(fk, oracle):
    """The committed vectors come from the reference's CPU backend, whose host branch takes the bilinear row from x;
    on every element where that equals the row from y the GPU must reproduce the reference's own bits."""
    import json
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    gold = np.load(os.path.join(here, "golden", "reference_vectors.npz"))
    case = json.load(open(os.path.join(here, "golden", "reference_cases.json")))["readme"]
    src = oracle.bytes(case["seed"], tuple(case["src"]))
    out = torch.full((5, 60, 60, 3), float("nan"), device="cuda")
    fk.crop_resize_muls_bgr_tensor(dev(src), case["rects"], out, B.PRESERVE_AR, case["background"], case["mul"], case["sub"], case["div"])
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    agree = 0
    for z, rect in enumerate(case["rects"]):
        p = oracle.resize_build(B.PRESERVE_AR, rect[2], rect[3], 60, 60)
        ys, xs = np.mgrid[0:60, 0:60]
        inside = (xs >= p.x1) & (xs <= p.x2) & (ys >= p.y1) & (ys <= p.y2)
        sx = (xs - p.x1).astype(np.float32) * np.float32(p.fx)
        sy = (ys - p.y1).astype(np.float32) * np.float32(p.fy)
        m = ~inside | (np.floor(sx) == np.floor(sy))
        assert same_bits(got[z][m], gold["readme_ar0"][z][m])
        agree += int(m.sum())
    assert agree > 3000
    # plane 2 is a 60x59 crop resized by exactly 1: a copy of the crop, normalised
    x, y, w, h = case["rects"][2]
    crop = src[y:y + h, x:x + w, ::-1].astype(np.float32)
    expect = ((crop * np.float32(1.4)) - np.float32(0.5)) / np.float32(255.0)
    assert same_bits(got[2, :59], expect.astype(np.float32))


def test_literal_build_reproduces_the_reference_cpu_backend(fk, oracle):
    """libfk_capi_literal.so takes the bilinear row index from x like the reference's host branch: its GPU output must
    equal the vectors written by the reference's own CPU backend, every element, for every chain with a resize."""
    import json
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    gold = np.load(os.path.join(here, "golden", "reference_vectors.npz"))
    cases = json.load(open(os.path.join(here, "golden", "reference_cases.json")))
    fk.use_literal_interpolation(True)
    try:
        _, capi = fk.load()
        assert capi.fk_interpolate_y1_from_x() == 1
        c = cases["readme"]
        src = dev(oracle.bytes(c["seed"], tuple(c["src"])))
        for aspect in (0, 1, 2, 3):
            out = torch.full((5, 60, 60, 3), float("nan"), device="cuda")
            fk.crop_resize_muls_bgr_tensor(src, c["rects"], out, aspect, c["background"], c["mul"], c["sub"], c["div"])
            torch.cuda.synchronize()
            assert same_bits(out.cpu().numpy(), gold[f"readme_ar{aspect}"]), aspect
        c = cases["split"]
        srcs = [dev(oracle.bytes(c["seed"] + i, tuple(c["src"]))) for i in range(c["n"])]
        out = torch.full((c["n"], 3, c["dst"][1], c["dst"][0]), float("nan"), device="cuda")
        fk.batch_crop_resize_norm_split(srcs, c["rects"], out, c["div1"], c["sub"], c["div2"])
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), gold["split"])
        c = cases["tiles"]
        src = dev(oracle.gradient_noise_u8c3(c["seed"], c["src"][1], c["src"][0]))
        out = torch.full((len(c["rects"]), c["tile"][1], c["tile"][0], 3), float("nan"), device="cuda")
        fk.resize_crop_tiles(src, c["resized"], c["rects"], out, c["mul"])
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), gold["tiles"])
        c = cases["divergent"]
        src = dev(oracle.bytes(c["seed"], tuple(c["src"])))
        out = torch.full((c["resized"][1], c["resized"][0], 4), float("nan"), device="cuda")
        fk.resize_mul_u8c4_f32c4(src, out, c["mul_b"])
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), gold["div_resized"])
    finally:
        fk.use_literal_interpolation(False)
        _, capi = fk.load()
        assert capi.fk_interpolate_y1_from_x() == 0
