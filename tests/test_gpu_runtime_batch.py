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
    # crops of different sizes without a resize: every plane receives the box of the largest width and height among ALL n
    # crops (the thread grid of the one batch, also where the entry point launches it in parts of 64 planes); origins are
    # drawn so that the box stays inside the image, where the oracle (exec_all=1) defines every element of it
    rects = crops(oracle, 1000 + n, n, 360, 220, 1, 40)
    box_w, box_h = max(r[2] for r in rects), max(r[3] for r in rects)
    got = torch.full((n, 40, 40, 3), -1.0, device="cuda")
    fk.batch_crop_cast_tensor(dev(src), rects, got)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    want = np.full((n, 40, 40, 3), -1.0, np.float32)
    want[:, :box_h, :box_w] = oracle.batch_crop_cast_tensor(src, rects, (box_w, box_h), exec_all=1)
    assert same_bits(got, want), n


def test_box_of_a_batch_launched_in_parts_is_the_whole_batch_s(fk, oracle):
    """70 crops whose tallest lies in the first 64 and whose widest lies in the last 6: both launches must cover the box of
    the largest width and the largest height of all 70."""
    src = oracle.bytes(77, (120, 160, 3))
    rects = [(i % 50, i % 30, 8, 6) for i in range(70)]
    rects[3] = (10, 10, 9, 37)
    rects[68] = (20, 5, 33, 4)
    got = torch.full((70, 40, 40, 3), -1.0, device="cuda")
    fk.batch_crop_cast_tensor(dev(src), rects, got)
    torch.cuda.synchronize()
    want = np.full((70, 40, 40, 3), -1.0, np.float32)
    want[:, :37, :33] = oracle.batch_crop_cast_tensor(src, rects, (33, 37), exec_all=1)
    assert same_bits(got.cpu().numpy(), want)


def test_one_row_window_in_a_ragged_batch_with_an_odd_padded_pitch(fk, oracle):
    """A window of one row batched with taller ones produces the rows of the largest: the wide (several pixels per thread)
    path may only be taken where the rows below the first are aligned too.  Source rows 3 * 41 + 5 = 128 bytes apart and
    131 bytes apart (odd)."""
    src = oracle.bytes(78, (60, 41, 3))
    rects = [(4, 7, 32, 1), (0, 0, 16, 9), (8, 20, 32, 5)]
    want = np.full((3, 12, 36, 3), -3.0, np.float32)
    want[:, :9, :32] = oracle.batch_crop_cast_tensor(src, rects, (32, 9), exec_all=1)
    for extra in (5, 8):
        padded = np.zeros((60, 41 * 3 + extra), np.uint8)
        padded[:, :41 * 3] = src.reshape(60, -1)
        view = torch.from_numpy(padded).cuda()[:, :41 * 3].view(60, 41, 3)
        out = torch.full((3, 12, 36, 3), -3.0, device="cuda")
        fk.batch_crop_cast_tensor(view, rects, out)
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), want), extra
