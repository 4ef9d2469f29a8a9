"""The batch entry points take their number of planes at run time: any n >= 1, through the C ABI, bit for bit against the
CPU oracle.  7 fits the small plane table, 46 the large one (the last point of the reference's horizontal-fusion sweep,
benchmarks/fusion/benchmark_horizontal_fusion.h:27-31), 64 fills it, 65 and 120 ("Used 120 in the paper") take a second
launch."""
import numpy as np
import pytest
import torch

from conftest import same_bits
from oracle import binding as B

pytestmark = pytest.mark.gpu

SIZES = [1, 7, 46, 64, 65, 120]


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def crops(oracle, seed, n, w, h, lo, hi):
    out = []
    for i in range(n):
        cw, ch = (int(v) for v in oracle.uniform_ints(seed + i, lo, hi, 2))
        x = int(oracle.uniform_ints(seed + 1000 + i, 0, w - cw, 1)[0])
        y = int(oracle.uniform_ints(seed + 2000 + i, 0, h - ch, 1)[0])
        out.append((x, y, cw, ch))
    return out


@pytest.mark.parametrize("n", SIZES)
def test_readme_chain_any_batch(fk, oracle, n):
    src = oracle.bytes(500 + n, (200, 320, 3))
    rects = crops(oracle, 600 + n, n, 320, 200, 8, 120)
    for aspect in (B.PRESERVE_AR, B.IGNORE_AR):
        args = (aspect, (0.25, 0.5, 0.75), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)
        want = oracle.crop_resize_muls_bgr_tensor(src, rects, (60, 40), *args)
        out = torch.full((n, 40, 60, 3), float("nan"), device="cuda")
        fk.crop_resize_muls_bgr_tensor(dev(src), rects, out, *args)
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), want), (n, aspect)


@pytest.mark.parametrize("n", SIZES)
def test_split_chain_any_batch(fk, oracle, n):
    images = [oracle.bytes(700 + i, (90, 130, 3)) for i in range(min(n, 5))]
    srcs = [images[i % len(images)] for i in range(n)]
    devs = [dev(s) for s in images]
    rects = crops(oracle, 800 + n, n, 130, 90, 6, 80)
    args = ((255.,) * 3, (.485, .456, .406), (.229, .224, .225))
    want = oracle.batch_crop_resize_norm_split(srcs, rects, (48, 32), *args)
    out = torch.full((n, 3, 32, 48), float("nan"), device="cuda")
    fk.batch_crop_resize_norm_split([devs[i % len(devs)] for i in range(n)], rects, out, *args)
    torch.cuda.synchronize()
    assert same_bits(out.cpu().numpy(), want), n


@pytest.mark.parametrize("n", SIZES)
def test_tiles_and_ragged_crops_any_batch(fk, oracle, n):
    src = oracle.gradient_noise_u8c3(900 + n, 400, 260)
    tiles = [(int(v[0]), int(v[1]), 24, 16) for v in (oracle.uniform_ints(950 + i, 0, 100, 2) for i in range(n))]
    want = oracle.resize_crop_tiles(src, (160, 120), tiles, (24, 16), (1 / 255.,) * 3)
    out = torch.full((n, 16, 24, 3), float("nan"), device="cuda")
    fk.resize_crop_tiles(dev(src), (160, 120), tiles, out, (1 / 255.,) * 3)
    torch.cuda.synchronize()
    assert same_bits(out.cpu().numpy(), want), n
    # crops of different sizes without a resize: every plane's own rectangle is written
    rects = crops(oracle, 1000 + n, n, 400, 260, 1, 40)
    got = torch.full((n, 40, 40, 3), -1.0, device="cuda")
    fk.batch_crop_cast_tensor(dev(src), rects, got)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    for z, (x, y, w, h) in enumerate(rects):
        assert same_bits(got[z, :h, :w], src[y:y + h, x:x + w].astype(np.float32)), (n, z)
