"""GPU parity, through the C ABI and bit for bit against the CPU oracle, of the chains with the operator API's less common
shapes: batch reads with CONDITIONAL_WITH_DEFAULT (on the pointwise and the resize kernel), a write in the middle of a
chain, a batch of separate output images and a tensor as the source (the generic kernel)."""
import numpy as np
import pytest
import torch

from conftest import same_bits

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("n", [1, 3, 8, 9, 46, 64])
def test_conditional_copy(fk, oracle, n):
    srcs = [oracle.bytes(1100 + i, (37, 131, 3)) for i in range(min(n, 6))]
    srcs = [srcs[i % len(srcs)] for i in range(n)]
    devs = [dev(s) for s in srcs]
    for used in sorted({0, 1, n // 2, n - 1, n, n + 5}):
        out = torch.full((n, 37, 131, 3), 77, dtype=torch.uint8, device="cuda")
        fk.conditional_copy_u8c3(devs, used, (9, 250, 0), out)
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), oracle.conditional_copy_u8c3(srcs, used, (9, 250, 0))), (n, used)


@pytest.mark.parametrize("shape", [((45, 70), (200, 96)), ((300, 200), (64, 40)), ((64, 64), (64, 64))], ids=["up", "down", "same"])
@pytest.mark.parametrize("n", [2, 8, 17])
def test_conditional_resize(fk, oracle, n, shape):
    (h, w), dst = shape
    srcs = [oracle.bytes(1200 + i, (h, w, 3)) for i in range(min(n, 4))]
    srcs = [srcs[i % len(srcs)] for i in range(n)]
    devs = [dev(s) for s in srcs]
    default = (-3.5, 0.0, 1e6)
    for used in sorted({0, 1, n - 1, n}):
        out = torch.full((n, dst[1], dst[0], 3), float("nan"), device="cuda")
        fk.conditional_resize_f32c3(devs, used, default, out)
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), oracle.conditional_resize_f32c3(srcs, used, default, dst)), (n, used)


def test_conditional_batches_at_full_size(fk, oracle):
    """Eight 1080p frames, five in use: the planes that run their program go through the staged kernels' wide paths
    (streaming stores, LDS), the others receive the value."""
    srcs = [oracle.bytes(1300 + i, (1080, 1920, 3)) for i in range(3)]
    srcs = [srcs[i % 3] for i in range(8)]
    devs = [dev(s) for s in srcs[:3]]
    devs = [devs[i % 3] for i in range(8)]
    out = torch.zeros((8, 1080, 1920, 3), dtype=torch.uint8, device="cuda")
    fk.conditional_copy_u8c3(devs, 5, (1, 2, 3), out)
    torch.cuda.synchronize()
    assert same_bits(out.cpu().numpy(), oracle.conditional_copy_u8c3(srcs, 5, (1, 2, 3)))
    del out
    res = torch.full((8, 720, 1280, 3), float("nan"), device="cuda")
    fk.conditional_resize_f32c3(devs, 5, (0.25, 0.5, 0.75), res)
    torch.cuda.synchronize()
    assert same_bits(res.cpu().numpy(), oracle.conditional_resize_f32c3(srcs, 5, (0.25, 0.5, 0.75), (1280, 720)))


@pytest.mark.parametrize("shape", [(1, 1), (7, 13), (64, 257), (1080, 1920)])
def test_write_in_the_middle_of_a_chain(fk, oracle, shape):
    f = oracle.unit_floats(1400, shape[0] * shape[1] * 3).reshape(shape[0], shape[1], 3)
    mid = torch.full(f.shape, float("nan"), device="cuda")
    out = torch.full(f.shape, float("nan"), device="cuda")
    fk.muladd_midwrite_f32c3(dev(f), 1.0001, 1e-4, mid, out)
    torch.cuda.synchronize()
    want_mid, want_out = oracle.muladd_midwrite_f32c3(f, 1.0001, 1e-4)
    assert same_bits(mid.cpu().numpy(), want_mid) and same_bits(out.cpu().numpy(), want_out)


@pytest.mark.parametrize("n", [1, 5, 8, 23, 64])
def test_batch_of_output_images(fk, oracle, n):
    src = oracle.bytes(1500 + n, (240, 320, 3))
    rects = [((13 * i) % 250, (7 * i) % 180, 60, 45) for i in range(n)]
    outs = [torch.full((45, 60, 3), float("nan"), device="cuda") for _ in range(n)]
    fk.batch_crop_cast_images(dev(src), rects, outs)
    torch.cuda.synchronize()
    for got, want in zip(outs, oracle.batch_crop_cast_images(src, rects)):
        assert same_bits(got.cpu().numpy(), want)


@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 17, 33), (4, 270, 480), (2, 1080, 1920)])
def test_tensor_source(fk, oracle, shape):
    planes, h, w = shape
    t = oracle.unit_floats(1600, planes * h * w * 3).reshape(planes, h, w, 3)
    out = torch.full(t.shape, float("nan"), device="cuda")
    fk.tensor_mul_f32c3(dev(t), (2.0, -0.5, 1.0001), out)
    torch.cuda.synchronize()
    assert same_bits(out.cpu().numpy(), oracle.tensor_mul_f32c3(t, (2.0, -0.5, 1.0001)))


@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 17, 33), (5, 60, 60), (2, 1080, 1920)])
def test_set_to_fills_every_element_and_nothing_else(fk, shape):
    """fk::setTo on a float3 tensor: every element receives the value (a fill: the expectation is the value itself), and
    the elements of a larger allocation around the tensor keep theirs."""
    planes, h, w = shape
    around = torch.full((planes * h * w * 3 + 32,), -9.0, device="cuda")
    out = around[16:-16].view(planes, h, w, 3)
    fk.set_to_f32c3_tensor((1.5, -2.25, 1e-30), out)
    torch.cuda.synchronize()
    got = around.cpu().numpy()
    want = np.full(got.shape, -9.0, np.float32)
    want[16:-16] = np.tile(np.array([1.5, -2.25, 1e-30], np.float32), planes * h * w)
    assert same_bits(got, want)


def test_argument_errors_of_these_entry_points(fk, oracle):
    src = dev(oracle.bytes(1, (20, 30, 3)))
    with pytest.raises(fk.FkError, match="1 to 64"):
        fk.conditional_copy_u8c3([src] * 65, 3, (0, 0, 0), torch.zeros((65, 20, 30, 3), dtype=torch.uint8, device="cuda"))
    with pytest.raises(fk.FkError, match="size of the first"):
        fk.batch_crop_cast_images(src, [(0, 0, 5, 5), (1, 1, 6, 5)], [torch.zeros((5, 5, 3), device="cuda"), torch.zeros((5, 5, 3), device="cuda")])
    torch.cuda.synchronize()


@pytest.mark.parametrize("n", [1, 6, 46, 64, 65, 120])
def test_horizontal_fusion_benchmark_chain(fk, oracle, n):
    """The reference's horizontal-fusion benchmark through the C ABI at its batch sizes (1, 6, ... 46; "120 in the paper"):
    windows of 60 x 120 at (i, i) of one uchar image -> SaturateCast -> Mul -> Sub -> Div -> tensor; its constants and a
    set that rounds at every step."""
    src = oracle.bytes(1300 + n, (400, 500))
    rects = [(i, i, 60, 120) for i in range(n)]
    for ops in ((1.0, 1.0, 3.2), (1.4, 0.5, 255.0)):
        out = torch.full((n, 120, 60), float("nan"), device="cuda")
        fk.batch_windows_saturate_muls_f32(dev(src), rects, out, *ops)
        torch.cuda.synchronize()
        assert same_bits(out.cpu().numpy(), oracle.batch_windows_saturate_muls_f32(src, rects, *ops)), (n, ops)


def test_horizontal_fusion_benchmark_chain_argument_errors(fk):
    src = torch.zeros((50, 50), dtype=torch.uint8, device="cuda")
    out = torch.empty((2, 10, 10), device="cuda")
    with pytest.raises(fk.FkError):
        fk.batch_windows_saturate_muls_f32(src, [(45, 0, 10, 10), (0, 0, 10, 10)], out, 1.0, 1.0, 3.2)  # outside the image
    with pytest.raises(fk.FkError, match="size of the first"):
        fk.batch_windows_saturate_muls_f32(src, [(0, 0, 10, 10), (0, 0, 12, 10)], out, 1.0, 1.0, 3.2)  # the tensor has one plane size
