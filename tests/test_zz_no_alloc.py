"""The entry point that allocates nothing (fk_crop_resize_muls_bgr_tensor_noalloc) against the entry point it is a
variant of, through the C ABI, bit for bit: the chain's job lies in the library's fixed block of device memory instead of
the kernel arguments.  Two calls in a row, the second with a smaller input (fewer and smaller planes), so that what the
first call left in the block would show; then more planes than the block takes."""
import numpy as np
import pytest
import torch

from conftest import same_bits
from oracle import binding as B

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_no_alloc_entry_point_equals_the_allocating_one(fk, oracle):
    src = oracle.bytes(2001, (240, 400, 3))
    d = dev(src)
    calls = [
        # (rects, destination, aspect): a large call first, then a smaller one that leaves most of the block as it was
        ([((11 * i) % 200, (7 * i) % 120, 40 + (13 * i) % 150, 30 + (5 * i) % 100) for i in range(37)], (96, 64), B.PRESERVE_AR),
        ([(5, 9, 120, 80), (200, 100, 64, 64), (0, 0, 400, 240)], (50, 30), B.IGNORE_AR),
    ]
    for rects, dst, aspect in calls:
        args = (aspect, (0.5, 0.25, 0.125), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)
        want = torch.full((len(rects), dst[1], dst[0], 3), float("nan"), device="cuda")
        fk.crop_resize_muls_bgr_tensor(d, rects, want, *args)
        got = torch.full((len(rects), dst[1], dst[0], 3), float("nan"), device="cuda")
        fk.crop_resize_muls_bgr_tensor_noalloc(d, rects, got, *args)
        torch.cuda.synchronize()
        assert same_bits(got.cpu().numpy(), want.cpu().numpy()), (len(rects), dst)
        assert same_bits(got.cpu().numpy(), oracle.crop_resize_muls_bgr_tensor(src, rects, dst, *args))
    # what the entry point exists for: once warmed (the calls above), a call takes no device memory and gives none back
    rects, dst, aspect = calls[0]
    args = (aspect, (0.5, 0.25, 0.125), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)
    got = torch.empty((len(rects), dst[1], dst[0], 3), device="cuda")
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(20):
        fk.crop_resize_muls_bgr_tensor_noalloc(d, rects, got, *args)
    free_during = torch.cuda.mem_get_info()[0]
    torch.cuda.synchronize()
    assert free_during == free_before and torch.cuda.mem_get_info()[0] == free_before
    with pytest.raises(fk.FkError, match="at most 64 planes"):
        fk.crop_resize_muls_bgr_tensor_noalloc(d, [(0, 0, 8, 8)] * 65, torch.zeros((65, 4, 4, 3), device="cuda"), B.IGNORE_AR, (0,) * 3, (1,) * 3,
                                               (0,) * 3, (1,) * 3)
    torch.cuda.synchronize()
