"""GPU parity on seeded random shapes, through the C ABI and bit for bit against the CPU oracle: the four resize entry
points (README chain in all aspect modes, the planar batch, the conditional batch, the NV12 chain) with image sizes,
windows, output sizes and batch sizes drawn at random, so that tile edges, bars, staged and directly read source boxes,
one-pixel windows and planes narrower than a tile all occur in combinations that no hand-picked case names."""
import numpy as np
import pytest
import torch

from conftest import same_bits
from oracle import binding

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def windows(rng, n, w, h):
    out = []
    for _ in range(n):
        cw, ch = int(rng.integers(1, w + 1)), int(rng.integers(1, h + 1))
        out.append((int(rng.integers(0, w - cw + 1)), int(rng.integers(0, h - ch + 1)), cw, ch))
    return out


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_readme_chain(fk, oracle, seed):
    rng = np.random.default_rng(seed)
    for case in range(60):
        w, h = int(rng.integers(8, 700)), int(rng.integers(8, 500))
        src = oracle.bytes(int(rng.integers(1, 1 << 30)), (h, w, 3))
        n = int(rng.integers(1, 9))
        rects = windows(rng, n, w, h)
        dst = (int(rng.integers(1, 400)), int(rng.integers(1, 300)))
        args = (int(rng.integers(0, 4)), (1.0, 2.0, 3.0), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)
        out = torch.empty((n, dst[1], dst[0], 3), device="cuda")
        fk.crop_resize_muls_bgr_tensor(dev(src), rects, out, *args)
        assert same_bits(out.cpu().numpy(), oracle.crop_resize_muls_bgr_tensor(src, rects, dst, *args)), (seed, case, w, h, rects, dst, args[0])


@pytest.mark.parametrize("seed", [11, 12])
def test_readme_chain_large_outputs(fk, oracle, seed):
    """Launches of more than 1024 tiles, where the kernel takes 64x32 tiles and, for images whose rows are a whole number of
    dwords apart, fills them from aligned groups of four pixels: image widths that are and are not multiples of four, windows
    at any offset, up- and down-scaling, all aspect modes."""
    rng = np.random.default_rng(seed)
    for case in range(24):
        w, h = int(rng.integers(40, 900)), int(rng.integers(40, 600))
        if case % 3 != 2:
            w = (w + 3) & ~3
        src = oracle.bytes(int(rng.integers(1, 1 << 30)), (h, w, 3))
        n = int(rng.integers(2, 6))
        rects = windows(rng, n, w, h)
        if case % 2 == 0:  # windows of at least a third of the image: several tiles per source box row
            rects = [(x, y, max(cw, w // 3), max(ch, h // 3)) for x, y, cw, ch in rects]
            rects = [(min(x, w - cw), min(y, h - ch), cw, ch) for x, y, cw, ch in rects]
        dst = (int(rng.integers(640, 1400)), int(rng.integers(520, 900)))
        args = (int(rng.integers(0, 4)), (1.0, 2.0, 3.0), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)
        out = torch.empty((n, dst[1], dst[0], 3), device="cuda")
        fk.crop_resize_muls_bgr_tensor(dev(src), rects, out, *args)
        assert same_bits(out.cpu().numpy(), oracle.crop_resize_muls_bgr_tensor(src, rects, dst, *args)), (seed, case, w, h, rects, dst, args[0])


@pytest.mark.parametrize("seed", [4, 5])
def test_planar_batch(fk, oracle, seed):
    rng = np.random.default_rng(seed)
    norm = ((255.,) * 3, (.485, .456, .406), (.229, .224, .225))
    for case in range(50):
        w, h = int(rng.integers(8, 600)), int(rng.integers(8, 400))
        n = int(rng.integers(1, 7))
        srcs = [oracle.bytes(int(rng.integers(1, 1 << 30)), (h, w, 3)) for _ in range(n)]
        rects = windows(rng, n, w, h)
        dst = (int(rng.integers(1, 300)), int(rng.integers(1, 300)))
        out = torch.empty((n, 3, dst[1], dst[0]), device="cuda")
        fk.batch_crop_resize_norm_split([dev(s) for s in srcs], rects, out, *norm)
        assert same_bits(out.cpu().numpy(), oracle.batch_crop_resize_norm_split(srcs, rects, dst, *norm)), (seed, case, w, h, rects, dst)


@pytest.mark.parametrize("seed", [6, 7])
def test_conditional_batch(fk, oracle, seed):
    rng = np.random.default_rng(seed)
    default = (0.5, 0.25, 0.125)
    for case in range(50):
        w, h = int(rng.integers(8, 500)), int(rng.integers(8, 400))
        n = int(rng.integers(1, 9))
        used = int(rng.integers(0, n + 1))
        srcs = [oracle.bytes(int(rng.integers(1, 1 << 30)), (h, w, 3)) for _ in range(n)]
        dst = (int(rng.integers(1, 400)), int(rng.integers(1, 300)))
        out = torch.empty((n, dst[1], dst[0], 3), device="cuda")
        fk.conditional_resize_f32c3([dev(s) for s in srcs], used, default, out)
        assert same_bits(out.cpu().numpy(), oracle.conditional_resize_f32c3(srcs, used, default, dst)), (seed, case, w, h, n, used, dst)


@pytest.mark.parametrize("seed", [8, 9])
def test_nv12_chain(fk, oracle, seed):
    rng = np.random.default_rng(seed)
    for case in range(50):
        w, h = 2 * int(rng.integers(4, 300)), 2 * int(rng.integers(4, 200))
        raw = oracle.bytes(int(rng.integers(1, 1 << 30)), (h * 3 // 2, w))
        cw, ch = 2 * int(rng.integers(1, w // 2 + 1)), 2 * int(rng.integers(1, h // 2 + 1))
        crop = (2 * int(rng.integers(0, (w - cw) // 2 + 1)), 2 * int(rng.integers(0, (h - ch) // 2 + 1)), cw, ch)
        dst = (int(rng.integers(1, 400)), int(rng.integers(1, 300)))
        out = torch.empty((3, dst[1], dst[0]), device="cuda")
        fk.yuv_crop_resize_norm_split(fk.NV12, fk.RANGE_FULL, fk.BT709, dev(raw), (w, h), crop, out, 255.0)
        expect = oracle.yuv_crop_resize_norm_split(binding.NV12, binding.RANGE_FULL, binding.BT709, raw, w, h, crop, dst, 255.0)
        assert same_bits(out.cpu().numpy(), expect), (seed, case, w, h, crop, dst)
