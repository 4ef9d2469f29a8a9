"""GPU parity: every chain of include/fk_capi.h, called through the C ABI on the MI355X, against the CPU oracle on the
same seeded inputs.  Bar: bit-exact, for float outputs too (both sides evaluate in the reference's order with FMA
contraction off); the north-star tolerance for floats is 1e-5 relative and is what `close` would enforce if a future
compiler broke bit-exactness."""
import numpy as np
import pytest
import torch

from conftest import same_bits
from oracle import binding as B

pytestmark = pytest.mark.gpu

README_RECTS = [(0, 0, 34, 25), (10, 10, 70, 15), (20, 20, 60, 59), (30, 30, 20, 23), (40, 40, 12, 11)]
REL_TOL = 1e-5


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def padded(a, extra):
    """Copy `a` (h, w, c) into a device buffer whose rows are `extra` pixels longer: pitch != width * pixel size."""
    h, w, c = a.shape
    buf = torch.zeros((h, w + extra, c), dtype=torch.from_numpy(a).dtype, device="cuda")
    buf[:, :w] = torch.from_numpy(a).cuda()
    return buf[:, :w]


def check(gpu, cpu):
    gpu = gpu.cpu().numpy()
    if gpu.dtype == np.float32 and not same_bits(gpu, cpu):
        diff = np.abs(gpu.astype(np.float64) - cpu.astype(np.float64))
        rel = diff / np.maximum(np.abs(cpu.astype(np.float64)), 1e-30)
        pytest.fail(f"not bit-exact: {np.count_nonzero(gpu != cpu)} elements differ, max rel {rel.max():.3e} (tolerance {REL_TOL})")
    assert same_bits(gpu, cpu)


@pytest.mark.parametrize("aspect", [B.PRESERVE_AR, B.IGNORE_AR, B.PRESERVE_AR_RN_EVEN, B.PRESERVE_AR_LEFT])
def test_readme_pipeline_full_size(fk, oracle, aspect):
    src = oracle.bytes(1, (2160, 3840, 3))
    args = ((60, 60), aspect, (0, 0, 0), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)
    want = oracle.crop_resize_muls_bgr_tensor(src, README_RECTS, *args)
    out = torch.full((5, 60, 60, 3), float("nan"), device="cuda")
    fk.crop_resize_muls_bgr_tensor(dev(src), README_RECTS, out, *args[1:])
    torch.cuda.synchronize()
    check(out, want)


@pytest.mark.parametrize("depth", [1, 2, 4, 8, 16, 32, 64, 128])
def test_muladd_chain(fk, oracle, depth):
    src = oracle.unit_floats(2, (270, 480, 3))
    want = oracle.muladd_chain_f32c3(src, depth, 1.0001, 1e-4)
    out = torch.full((270, 480, 3), float("nan"), device="cuda")
    fk.muladd_chain_f32c3(dev(src), out, depth, 1.0001, 1e-4)
    torch.cuda.synchronize()
    check(out, want)


def test_single_ops(fk, oracle):
    src = oracle.unit_floats(2, (33, 61, 3))
    for is_add, v in ((0, 1.0001), (1, 1e-4)):
        out = torch.full((33, 61, 3), float("nan"), device="cuda")
        fk.single_op_f32c3(dev(src), out, is_add, v)
        torch.cuda.synchronize()
        check(out, oracle.single_op_f32c3(src, is_add, v))


def test_batch_crop_resize_norm_split(fk, oracle):
    n = 5
    srcs = [oracle.bytes(3 + i, (270, 480, 3)) for i in range(n)]
    rects = [(5, 3, 100, 40), (0, 0, 16, 16), (100, 10, 200, 100), (17, 29, 33, 47), (50, 50, 250, 128)]
    args = ((255.,) * 3, (.485, .456, .406), (.229, .224, .225))
    want = oracle.batch_crop_resize_norm_split(srcs, rects, (224, 224), *args)
    out = torch.full((n, 3, 224, 224), float("nan"), device="cuda")
    fk.batch_crop_resize_norm_split([dev(s) for s in srcs], rects, out, *args)
    torch.cuda.synchronize()
    check(out, want)


def test_resize_crop_tiles(fk, oracle):
    src = oracle.gradient_noise_u8c3(4, 384, 216)
    rects = [(16 * i, 18 * j, 16, 16) for j in range(4) for i in range(8)]
    want = oracle.resize_crop_tiles(src, (128, 72), rects, (16, 16), (1 / 255.,) * 3)
    out = torch.full((32, 16, 16, 3), float("nan"), device="cuda")
    fk.resize_crop_tiles(dev(src), (128, 72), rects, out, (1 / 255.,) * 3)
    torch.cuda.synchronize()
    check(out, want)


def _divergent_inputs(oracle, size):
    src = oracle.bytes(5, (size, size, 4))
    c = size // 8
    rect = (size // 2 - c // 2, size // 2 - c // 2, c, c)
    return src, rect


def test_divergent_chains_separately(fk, oracle):
    src, rect = _divergent_inputs(oracle, 512)
    d = dev(src)
    gray = torch.zeros((512, 512), dtype=torch.uint8, device="cuda")
    fk.rgba2gray_u8c4(d, gray)
    small = torch.full((32, 32, 4), float("nan"), device="cuda")
    fk.resize_mul_u8c4_f32c4(d, small, 1 / 255.)
    crop = torch.zeros((rect[3], rect[2], 4), dtype=torch.uint8, device="cuda")
    fk.crop_mul_saturate_u8c4(d, rect, crop, 2)
    bgr = torch.full((512, 512, 3), float("nan"), device="cuda")
    fk.rgba2bgr_sub_u8c4_f32c3(d, bgr, 0.5)
    torch.cuda.synchronize()
    check(gray, oracle.rgba2gray_u8c4(src))
    check(small, oracle.resize_mul_u8c4_f32c4(src, (32, 32), 1 / 255.))
    check(crop, oracle.crop_mul_saturate_u8c4(src, rect, 2))
    check(bgr, oracle.rgba2bgr_sub_u8c4_f32c3(src, 0.5))


def test_divergent_one_launch(fk, oracle):
    src, rect = _divergent_inputs(oracle, 512)
    gray = torch.zeros((512, 512), dtype=torch.uint8, device="cuda")
    small = torch.full((32, 32, 4), float("nan"), device="cuda")
    crop = torch.zeros((rect[3], rect[2], 4), dtype=torch.uint8, device="cuda")
    bgr = torch.full((512, 512, 3), float("nan"), device="cuda")
    fk.divergent4_u8c4(dev(src), gray, small, 1 / 255., rect, 2, crop, 0.5, bgr)
    torch.cuda.synchronize()
    check(gray, oracle.rgba2gray_u8c4(src))
    check(small, oracle.resize_mul_u8c4_f32c4(src, (32, 32), 1 / 255.))
    check(crop, oracle.crop_mul_saturate_u8c4(src, rect, 2))
    check(bgr, oracle.rgba2bgr_sub_u8c4_f32c3(src, 0.5))


def test_ragged_crops_cover_the_largest_box_like_the_reference(fk, oracle):
    """Crops of different sizes: every plane receives the box of the largest width and height, as the reference's thread
    grid covers it (oracle with exec_all=1, pinned against the reference build); tensor elements beyond the box stay."""
    src = oracle.bytes(7, (120, 200, 3))
    rects = [(1, 2, 30, 20), (5, 5, 10, 25), (100, 60, 33, 7)]
    want = np.full((3, 27, 36, 3), -7.0, np.float32)
    want[:, :25, :33] = oracle.batch_crop_cast_tensor(src, rects, (33, 25), exec_all=1)
    for extra in (0, 1, 3):  # tight and padded source rows: the wide and the element-wise paths
        out = torch.full((3, 27, 36, 3), -7.0, device="cuda")
        fk.batch_crop_cast_tensor(padded(src, extra) if extra else dev(src), rects, out)
        torch.cuda.synchronize()
        check(out, want)


def test_ragged_crops_beyond_the_source_image_read_zero(fk, oracle):
    """Where the largest box leaves the source image the reference reads past it; here the source pixel is zero."""
    src = oracle.bytes(8, (40, 64, 3))
    rects = [(0, 0, 50, 6), (60, 36, 4, 4), (20, 10, 8, 30)]  # the second plane's 50 x 30 box leaves the image on both sides
    out = torch.full((3, 30, 50, 3), -7.0, device="cuda")
    fk.batch_crop_cast_tensor(dev(src), rects, out)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    big = np.zeros((40 + 30, 64 + 50, 3), np.uint8)
    big[:40, :64] = src
    for z, (x, y, _, _) in enumerate(rects):
        assert same_bits(got[z], big[y:y + 30, x:x + 50].astype(np.float32)), z
