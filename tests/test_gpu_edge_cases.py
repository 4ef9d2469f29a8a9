"""GPU parity on the awkward shapes: ragged and tiny inputs, odd widths, padded pitches, unaligned views, every tail
path of the vectorised kernels, large batches (kernel-argument blocks beyond 4 KiB) and argument errors."""
import numpy as np
import pytest
import torch

from conftest import same_bits
from oracle import binding as B

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def padded(a, extra):
    """Copy `a` (h, w, c) into a device buffer whose rows are `extra` pixels longer: pitch != width * pixel size."""
    h, w, c = a.shape
    buf = torch.zeros((h, w + extra, c), dtype=torch.from_numpy(a).dtype, device="cuda")
    buf[:, :w] = torch.from_numpy(a).cuda()
    return buf[:, :w]


@pytest.mark.parametrize("shape", [(1, 1), (1, 3), (3, 1), (7, 5), (1, 1023), (1, 1024), (1, 1025), (2, 4097), (33, 257), (64, 256)])
def test_pointwise_every_tail(fk, oracle, shape):
    h, w = shape
    src = oracle.unit_floats(2, (h, w, 3))
    out = torch.full((h, w, 3), float("nan"), device="cuda")
    fk.muladd_chain_f32c3(dev(src), out, 4, 1.0001, 1e-4)
    torch.cuda.synchronize()
    assert same_bits(out.cpu().numpy(), oracle.muladd_chain_f32c3(src, 4, 1.0001, 1e-4))


@pytest.mark.parametrize("extra", [1, 4, 13])
def test_pointwise_padded_and_unaligned_rows(fk, oracle, extra):
    src = oracle.unit_floats(2, (37, 1100, 3))
    want = oracle.muladd_chain_f32c3(src, 2, 1.0001, 1e-4)
    s = padded(src, extra)
    full = torch.full((37, 1100 + extra, 3), float("nan"), device="cuda")
    out = full[:, :1100]
    fk.muladd_chain_f32c3(s, out, 2, 1.0001, 1e-4)
    torch.cuda.synchronize()
    assert same_bits(out.cpu().numpy(), want)
    assert torch.isnan(full[:, 1100:]).all()  # nothing written past the row end
    # a view that starts 1 pixel (12 bytes) into the row: base no longer 16-byte aligned
    s2, o2 = s[:, 1:], out[:, 1:]
    fk.muladd_chain_f32c3(s2, o2, 2, 1.0001, 1e-4)
    torch.cuda.synchronize()
    assert same_bits(o2.cpu().numpy(), want[:, 1:])


def test_uchar4_chains_odd_sizes_and_pitch(fk, oracle):
    src = oracle.bytes(5, (61, 203, 4))
    s = padded(src, 3)
    gray_full = torch.zeros((61, 203 + 5), dtype=torch.uint8, device="cuda")
    fk.rgba2gray_u8c4(s, gray_full[:, :203])
    bgr = torch.full((61, 203, 3), float("nan"), device="cuda")
    fk.rgba2bgr_sub_u8c4_f32c3(s, bgr, 0.5)
    rect = (17, 9, 150, 40)
    crop = torch.zeros((40, 150, 4), dtype=torch.uint8, device="cuda")
    fk.crop_mul_saturate_u8c4(s, rect, crop, 3)
    small = torch.full((7, 11, 4), float("nan"), device="cuda")
    fk.resize_mul_u8c4_f32c4(s, small, 1 / 255.)
    up = torch.full((200, 333, 4), float("nan"), device="cuda")
    fk.resize_mul_u8c4_f32c4(s, up, 1.0)
    torch.cuda.synchronize()
    assert same_bits(gray_full[:, :203].cpu().numpy(), oracle.rgba2gray_u8c4(src)) and (gray_full[:, 203:] == 0).all()
    assert same_bits(bgr.cpu().numpy(), oracle.rgba2bgr_sub_u8c4_f32c3(src, 0.5))
    assert same_bits(crop.cpu().numpy(), oracle.crop_mul_saturate_u8c4(src, rect, 3))
    assert same_bits(small.cpu().numpy(), oracle.resize_mul_u8c4_f32c4(src, (11, 7), 1 / 255.))
    assert same_bits(up.cpu().numpy(), oracle.resize_mul_u8c4_f32c4(src, (333, 200), 1.0))


@pytest.mark.parametrize("aspect", [B.PRESERVE_AR, B.IGNORE_AR, B.PRESERVE_AR_RN_EVEN, B.PRESERVE_AR_LEFT])
@pytest.mark.parametrize("n", [1, 2, 3, 8])
def test_readme_chain_tiny_and_extreme_crops(fk, oracle, aspect, n):
    h, w = 97, 131
    src = oracle.bytes(40 + n, (h, w, 3))
    pool = [(0, 0, 1, 1), (130, 96, 1, 1), (0, 0, 131, 97), (5, 7, 2, 90), (3, 3, 120, 2), (64, 32, 33, 17), (1, 1, 129, 95), (100, 0, 31, 97)]
    rects = pool[:n]
    for dst in ((1, 1), (37, 53), (256, 9)):
        args = (aspect, (0.25, -1.0, 3.0), (1.4, 0.7, 2.0), (0.5, 0.1, -0.3), (255., 3., 0.5))
        want = oracle.crop_resize_muls_bgr_tensor(src, rects, dst, *args)
        out = torch.full((n, dst[1], dst[0], 3), float("nan"), device="cuda")
        fk.crop_resize_muls_bgr_tensor(padded(src, 1), rects, out, *args)
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), want), (dst, aspect, n)


def test_large_batches_exceed_four_kib_of_kernel_arguments(fk, oracle):
    for n in (32, 50):
        src = oracle.bytes(60, (200, 300, 3))
        rects = [((7 * i) % 200, (5 * i) % 120, 16 + (11 * i) % 80, 8 + (13 * i) % 70) for i in range(n)]
        args = (B.PRESERVE_AR, (0, 0, 0), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)
        want = oracle.crop_resize_muls_bgr_tensor(src, rects, (40, 24), *args)
        out = torch.full((n, 24, 40, 3), float("nan"), device="cuda")
        fk.crop_resize_muls_bgr_tensor(dev(src), rects, out, *args)
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), want), n


def test_split_and_tiles_small_batches(fk, oracle):
    for n in (1, 2, 3, 8):
        srcs = [oracle.bytes(70 + i, (90, 160, 3)) for i in range(n)]
        rects = [(3 * i, 2 * i, 20 + 15 * i, 11 + 9 * i) for i in range(n)]
        args = ((255.,) * 3, (.485, .456, .406), (.229, .224, .225))
        out = torch.full((n, 3, 30, 50), float("nan"), device="cuda")
        fk.batch_crop_resize_norm_split([dev(s) for s in srcs], rects, out, *args)
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), oracle.batch_crop_resize_norm_split(srcs, rects, (50, 30), *args)), n
        src = oracle.gradient_noise_u8c3(4, 200, 120)
        tiles = [(4 * i, 3 * i, 9, 7) for i in range(n)]
        o2 = torch.full((n, 7, 9, 3), float("nan"), device="cuda")
        fk.resize_crop_tiles(dev(src), (50, 40), tiles, o2, (1 / 255.,) * 3)
        torch.cuda.synchronize()
        assert same_bits(o2.cpu().numpy(), oracle.resize_crop_tiles(src, (50, 40), tiles, (9, 7), (1 / 255.,) * 3)), n


def test_upscale_of_crops_with_odd_byte_offsets(fk, oracle):
    # crops starting at every byte phase of a uchar3 row, tight and padded pitches: the LDS staging aligns rows itself
    src = oracle.bytes(80, (70, 101, 3))
    for extra in (0, 1, 2, 3):
        s = padded(src, extra) if extra else dev(src)
        rects = [(x, 3 + x, 37, 29) for x in (0, 1, 2, 3, 4)]
        out = torch.full((5, 120, 150, 3), float("nan"), device="cuda")
        args = (B.IGNORE_AR, (0, 0, 0), (1.0,) * 3, (0.0,) * 3, (1.0,) * 3)
        fk.crop_resize_muls_bgr_tensor(s, rects, out, *args)
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), oracle.crop_resize_muls_bgr_tensor(src, rects, (150, 120), *args)), extra


@pytest.mark.parametrize("case", ["behind", "shared", "mixed", "few_rows", "tall_boxes"])
def test_resize_lds_layouts(fk, oracle, case):
    """The resize kernel sizes its LDS from the planes' factors.  Packed outputs of 1 MB or more leave through LDS: behind
    the source tile when both fit 24 KiB ("behind": up-scaling, small boxes), in the tile's place after a block barrier when
    not ("shared": boxes above 12 KiB, down-scaling by 1.7); "mixed" has planes on both sides of that limit and one that is not staged at all in
    one launch; "few_rows" are boxes of two or three source rows (a wave stages four rows at a time and repeats the last);
    "tall_boxes" need more than one pass of four rows per wave."""
    src = oracle.bytes(91, (720, 1280, 3))
    rects, dst = {
        "behind": ([(10, 20, 320, 200), (301, 7, 200, 320)], (768, 480)),
        "shared": ([(0, 0, 1088, 626), (33, 11, 1090, 628)], (640, 368)),
        "mixed": ([(5, 5, 160, 90), (0, 0, 1088, 626), (100, 50, 640, 368), (0, 0, 1280, 720), (600, 300, 17, 400)], (640, 368)),
        "few_rows": ([(7, 300, 500, 3), (9, 100, 640, 2), (0, 0, 64, 1)], (1024, 512)),
        "tall_boxes": ([(3, 1, 300, 700), (640, 0, 200, 720)], (512, 400)),
    }[case]
    for aspect in (B.IGNORE_AR, B.PRESERVE_AR):
        args = (aspect, (0.5, 0.25, 0.125), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)
        out = torch.full((len(rects), dst[1], dst[0], 3), float("nan"), device="cuda")
        fk.crop_resize_muls_bgr_tensor(dev(src), rects, out, *args)
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), oracle.crop_resize_muls_bgr_tensor(src, rects, dst, *args)), (case, aspect)


@pytest.mark.parametrize("width", [100, 48])
def test_float_tiles_filled_from_groups_of_four_pixels(fk, oracle, width):
    """Up-scaled crops of an image whose rows are a whole number of dwords apart: the tiles of float taps are filled from
    aligned groups of four pixels of the parent image.  Windows that start at every phase of such a group, that end inside
    the parent (the pixel behind the window's last column exists in memory but must not be used: the tap clamps to the
    window) and at its last column and row (the last group of the last row ends at the end of the allocation).  The
    640x416 outputs make a launch of more than 1024 tiles of 64x32, which is where the kernel fills its tiles this way; the
    small ones take the fill of one pixel per thread on the same windows."""
    h = 61
    src = oracle.bytes(83 + width, (h, width, 3))
    rects = [(x, 2 + x, 31 + x, 23) for x in (0, 1, 2, 3, 5)]
    rects += [(width - 29, h - 19, 29, 19), (width - 1, h - 1, 1, 1), (width - 5, 0, 5, h), (0, h - 2, width, 2), (0, 0, width, h)]
    for dst in ((640, 416), (97, 131)):
        for aspect in (B.IGNORE_AR, B.PRESERVE_AR):
            args = (aspect, (0.5, 0.25, 0.125), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)
            out = torch.full((len(rects), dst[1], dst[0], 3), float("nan"), device="cuda")
            fk.crop_resize_muls_bgr_tensor(dev(src), rects, out, *args)
            torch.cuda.synchronize()
            assert same_bits(out.cpu().numpy(), oracle.crop_resize_muls_bgr_tensor(src, rects, dst, *args)), (width, dst, aspect)


def test_crop_at_the_last_row_and_column_of_the_buffer(fk, oracle):
    # the source window ends exactly at the end of the allocation: staging must not read past it
    src = oracle.bytes(81, (33, 47, 3))
    rects = [(20, 10, 27, 23), (46, 32, 1, 1)]
    out = torch.full((2, 64, 64, 3), float("nan"), device="cuda")
    args = (B.PRESERVE_AR, (1.0, 2.0, 3.0), (1.0,) * 3, (0.0,) * 3, (1.0,) * 3)
    fk.crop_resize_muls_bgr_tensor(dev(src), rects, out, *args)
    torch.cuda.synchronize()
    assert same_bits(out.cpu().numpy(), oracle.crop_resize_muls_bgr_tensor(src, rects, (64, 64), *args))


def test_argument_errors(fk, oracle):
    src = dev(oracle.bytes(1, (20, 30, 3)))
    out = torch.zeros((4, 8, 8, 3), device="cuda")
    with pytest.raises(fk.FkError, match="unsupported"):  # an aspect-ratio mode that does not exist
        fk.crop_resize_muls_bgr_tensor(src, [(0, 0, 4, 4)] * 4, out, 7, (0,) * 3, (1,) * 3, (0,) * 3, (1,) * 3)
    with pytest.raises(fk.FkError, match="no planes"):
        fk.crop_resize_muls_bgr_tensor(src, [], out[:0], 0, (0,) * 3, (1,) * 3, (0,) * 3, (1,) * 3)
    out = torch.zeros((1, 8, 8, 3), device="cuda")
    with pytest.raises(fk.FkError, match="outside"):
        fk.crop_resize_muls_bgr_tensor(src, [(25, 0, 10, 4)], out, 0, (0,) * 3, (1,) * 3, (0,) * 3, (1,) * 3)
    with pytest.raises(fk.FkError, match="unsupported"):
        f = torch.zeros((4, 4, 3), device="cuda")
        fk.muladd_chain_f32c3(f, f.clone(), 3, 1.0, 1.0)
    torch.cuda.synchronize()


def test_staged_parameter_block_path(oracle):
    """Jobs above the kernel-argument limit are staged through device memory; force that with a tiny limit (the limit is
    read once per process, hence the child process)."""
    import os
    import subprocess
    import sys
    code = (
        "import numpy as np, torch, fusedkernellibrary_amd as fk\n"
        "from oracle import binding as B\n"
        "o = B.oracle(); rt, _ = fk.load(); assert rt.fkrt_max_kernarg_bytes() == 256\n"
        "src = o.bytes(60, (200, 300, 3)); n = 32\n"
        "rects = [((7 * i) % 200, (5 * i) % 120, 16 + (11 * i) % 80, 8 + (13 * i) % 70) for i in range(n)]\n"
        "args = (B.PRESERVE_AR, (0, 0, 0), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)\n"
        "want = o.crop_resize_muls_bgr_tensor(src, rects, (40, 24), *args)\n"
        "out = torch.full((n, 24, 40, 3), float('nan'), device='cuda')\n"
        "for _ in range(3): fk.crop_resize_muls_bgr_tensor(torch.from_numpy(src).cuda(), rects, out, *args)\n"
        "torch.cuda.synchronize(); assert out.cpu().numpy().tobytes() == want.tobytes()\n"
        # more launches in flight than the staging ring has slots, different jobs in turn, on two streams
        "rects2 = [(r[0] // 2, r[1] // 2, r[2], r[3]) for r in rects]\n"
        "want2 = o.crop_resize_muls_bgr_tensor(src, rects2, (40, 24), *args)\n"
        "d_src = torch.from_numpy(src).cuda(); outs = [torch.full((n, 24, 40, 3), float('nan'), device='cuda') for _ in range(40)]\n"
        "side = torch.cuda.Stream(); torch.cuda.synchronize()\n"
        "for i, t in enumerate(outs):\n"
        "    fk.crop_resize_muls_bgr_tensor(d_src, rects2 if i % 2 else rects, t, *args, stream=side.cuda_stream if i % 4 >= 2 else None)\n"
        "torch.cuda.synchronize()\n"
        "for i, t in enumerate(outs): assert t.cpu().numpy().tobytes() == (want2 if i % 2 else want).tobytes(), i\n"
        "f = o.unit_floats(2, (64, 1024, 3)); d = torch.empty((64, 1024, 3), device='cuda')\n"
        "fk.muladd_chain_f32c3(torch.from_numpy(f).cuda(), d, 64, 1.0001, 1e-4); torch.cuda.synchronize()\n"
        "assert d.cpu().numpy().tobytes() == o.muladd_chain_f32c3(f, 64, 1.0001, 1e-4).tobytes()\n"
        "print('staged ok')\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, FK_MAX_KERNARG_BYTES="256", PYTHONPATH=root)
    proc = subprocess.run([sys.executable, "-c", code], env=env, cwd=root, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=150)
    assert proc.returncode == 0 and "staged ok" in proc.stdout, proc.stdout
