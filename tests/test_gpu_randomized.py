"""Seeded random sweeps of every chain on the GPU against the oracle: image sizes, pitches, crop rectangles, scale
factors and batch sizes drawn from the repository's SplitMix64 generator, bit-exact on every case."""
import numpy as np
import pytest
import torch

from conftest import same_bits
from oracle import binding as B

pytestmark = pytest.mark.gpu


def dev(a, extra=0):
    if extra == 0:
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()
    h, w, c = a.shape
    buf = torch.zeros((h, w + extra, c), dtype=torch.from_numpy(a).dtype, device="cuda")
    buf[:, :w] = torch.from_numpy(a).cuda()
    return buf[:, :w]


class Draw:
    def __init__(self, oracle, seed):
        self.o, self.seed, self.k = oracle, seed, 0

    def __call__(self, lo, hi):
        self.k += 1
        return int(self.o.uniform_ints(self.seed * 1000 + self.k, lo, hi, 1)[0])


@pytest.mark.parametrize("seed", range(1, 13))
def test_random_readme_chains(fk, oracle, seed):
    d = Draw(oracle, seed)
    w, h = d(8, 700), d(8, 500)
    src = oracle.bytes(seed, (h, w, 3))
    n = (1, 2, 3, 5, 8)[d(0, 4)]
    rects = []
    for _ in range(n):
        cw, ch = d(1, w), d(1, h)
        rects.append((d(0, w - cw), d(0, h - ch), cw, ch))
    dst = (d(1, 400), d(1, 300))
    aspect = d(0, 3)
    args = (aspect, (d(0, 9) / 3.0, -1.0, 0.5), (1.4, d(1, 9) / 7.0, 2.0), (0.5, 0.1, d(0, 9) / 11.0), (255., 3., d(1, 9) / 5.0))
    want = oracle.crop_resize_muls_bgr_tensor(src, rects, dst, *args)
    out = torch.full((n, dst[1], dst[0], 3), float("nan"), device="cuda")
    fk.crop_resize_muls_bgr_tensor(dev(src, d(0, 3)), rects, out, *args)
    torch.cuda.synchronize()
    assert same_bits(out.cpu().numpy(), want), (w, h, rects, dst, aspect)


@pytest.mark.parametrize("seed", range(21, 29))
def test_random_split_and_tile_chains(fk, oracle, seed):
    d = Draw(oracle, seed)
    w, h = d(16, 600), d(16, 400)
    n = (1, 2, 3, 5, 8)[d(0, 4)]
    srcs = [oracle.bytes(seed * 10 + i, (h, w, 3)) for i in range(n)]
    rects = []
    for _ in range(n):
        cw, ch = d(1, w), d(1, h)
        rects.append((d(0, w - cw), d(0, h - ch), cw, ch))
    dst = (d(1, 300), d(1, 260))
    args = ((255.,) * 3, (.485, .456, .406), (.229, .224, .225))
    extra = d(0, 3)
    out = torch.full((n, 3, dst[1], dst[0]), float("nan"), device="cuda")
    fk.batch_crop_resize_norm_split([dev(s, extra) for s in srcs], rects, out, *args)
    torch.cuda.synchronize()
    assert same_bits(out.cpu().numpy(), oracle.batch_crop_resize_norm_split(srcs, rects, dst, *args)), (w, h, rects, dst)
    # resize first, then crop tiles out of the resized image
    rs = (d(8, 500), d(8, 400))
    tw, th = d(1, min(rs[0], 150)), d(1, min(rs[1], 150))
    tiles = [(d(0, rs[0] - tw), d(0, rs[1] - th), tw, th) for _ in range(n)]
    o2 = torch.full((n, th, tw, 3), float("nan"), device="cuda")
    fk.resize_crop_tiles(dev(srcs[0], extra), rs, tiles, o2, (1 / 255., 0.5, 2.0))
    torch.cuda.synchronize()
    assert same_bits(o2.cpu().numpy(), oracle.resize_crop_tiles(srcs[0], rs, tiles, (tw, th), (1 / 255., 0.5, 2.0))), (w, h, rs, tiles)


@pytest.mark.parametrize("seed", range(41, 49))
def test_random_uchar4_and_float3_chains(fk, oracle, seed):
    d = Draw(oracle, seed)
    w, h = d(1, 900), d(1, 300)
    src = oracle.bytes(seed, (h, w, 4))
    extra = d(0, 3)
    s = dev(src, extra)
    gray = torch.zeros((h, w), dtype=torch.uint8, device="cuda")
    fk.rgba2gray_u8c4(s, gray)
    bgr = torch.full((h, w, 3), float("nan"), device="cuda")
    fk.rgba2bgr_sub_u8c4_f32c3(s, bgr, 0.5)
    cw, ch = d(1, w), d(1, h)
    rect = (d(0, w - cw), d(0, h - ch), cw, ch)
    crop = torch.zeros((ch, cw, 4), dtype=torch.uint8, device="cuda")
    mul = d(1, 4)
    fk.crop_mul_saturate_u8c4(s, rect, crop, mul)
    dst = (d(1, 500), d(1, 200))
    small = torch.full((dst[1], dst[0], 4), float("nan"), device="cuda")
    fk.resize_mul_u8c4_f32c4(s, small, 1 / 255.)
    f = oracle.unit_floats(seed, (h, w, 3))
    depth = (1, 2, 4, 8, 16, 32)[d(0, 5)]
    fo = torch.full((h, w, 3), float("nan"), device="cuda")
    fk.muladd_chain_f32c3(dev(f, extra), fo, depth, 1.0001, 1e-4)
    torch.cuda.synchronize()
    assert same_bits(gray.cpu().numpy(), oracle.rgba2gray_u8c4(src))
    assert same_bits(bgr.cpu().numpy(), oracle.rgba2bgr_sub_u8c4_f32c3(src, 0.5))
    assert same_bits(small.cpu().numpy(), oracle.resize_mul_u8c4_f32c4(src, dst, 1 / 255.)), (w, h, dst)
    assert same_bits(fo.cpu().numpy(), oracle.muladd_chain_f32c3(f, depth, 1.0001, 1e-4)), (w, h, depth)
    assert same_bits(crop.cpu().numpy(), oracle.crop_mul_saturate_u8c4(src, rect, mul)), (w, h, rect, mul)
