"""GPU parity of the tensor layouts, circular reads and CircularTensor::update, called through the C ABI on the MI355X,
against the CPU oracle (oracle/fk_oracle_circular.c) and the vectors written by the reference's own headers."""
import os
import sys

import numpy as np
import pytest
import torch

from conftest import same_bits
from oracle import binding as B

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import make_golden_circular as G  # noqa: E402

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_circular_vectors.npz"))


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_reference_vectors(fk, oracle):
    src = oracle.unit_floats(G.SEED, G.PLANES * G.H * G.W * 3)
    for mode in range(4):
        out = torch.full((src.size,), float("nan"), device="cuda")
        fk.tensor_relayout_f32c3(mode, dev(src), G.W, G.H, G.PLANES, out)
        assert same_bits(out.cpu().numpy(), GOLD[f"relayout_{mode}"]), mode
    ring = dev(src.reshape(G.PLANES, G.H, G.W, 3))
    for direction in (B.ASCENDENT, B.DESCENDENT):
        for first in range(G.PLANES):
            out = torch.full((G.PLANES, G.H, G.W, 3), float("nan"), device="cuda")
            fk.circular_tensor_read_f32c3(direction, first, ring, out)
            assert same_bits(out.cpu().numpy(), GOLD[f"ring_d{direction}_f{first}"])


@pytest.mark.parametrize("planes,h,w", [(2, 1, 1), (3, 37, 53), (8, 270, 480), (16, 64, 64)])
def test_layouts_and_ring_vs_oracle(fk, oracle, planes, h, w):
    src = oracle.unit_floats(planes * w, planes * h * w * 3)
    d_src = dev(src)
    for mode in range(4):
        out = torch.full((src.size,), float("nan"), device="cuda")
        fk.tensor_relayout_f32c3(mode, d_src, w, h, planes, out)
        assert same_bits(out.cpu().numpy(), oracle.tensor_relayout_f32c3(mode, src, w, h, planes)), mode
    ring = src.reshape(planes, h, w, 3)
    for direction in (B.ASCENDENT, B.DESCENDENT):
        for first in (0, 1, planes - 1):
            out = torch.full((planes, h, w, 3), float("nan"), device="cuda")
            fk.circular_tensor_read_f32c3(direction, first, dev(ring), out)
            assert same_bits(out.cpu().numpy(), oracle.circular_tensor_read_f32c3(direction, first, ring))


@pytest.mark.parametrize("newest_first", [1, 0])
@pytest.mark.parametrize("batch,size", [(2, (33, 17)), (3, (640, 360)), (4, (1920, 1080)), (8, (224, 224)), (16, (64, 48))])
def test_circular_tensor_update_vs_oracle(fk, oracle, batch, size, newest_first):
    w, h = size
    mul = 1 / 255.0
    tensor = np.full((batch, 3, h, w), -1.0, np.float32)
    ring = np.full((batch, 3, h, w), -2.0, np.float32)
    d_tensor, d_ring = dev(tensor), dev(ring)
    nxt = 0
    for k in range(batch + 3):
        frame = oracle.bytes(300 + k, (h, w, 3))
        oracle.circular_tensor_update_u8c3_split_f32(frame, mul, tensor, ring, nxt, newest_first)
        nxt_gpu = fk.circular_tensor_update_u8c3_split_f32(dev(frame), mul, d_tensor, d_ring, nxt, newest_first)
        nxt = (nxt + 1) % batch
        assert nxt_gpu == nxt
        torch.cuda.synchronize()
        assert same_bits(d_tensor.cpu().numpy(), tensor), k
        assert same_bits(d_ring.cpu().numpy(), ring), k
    # the property the class exists for: the newest plane is the frame just given, scaled
    newest = d_tensor[0 if newest_first else batch - 1].cpu().numpy()
    assert same_bits(newest, frame.astype(np.float32).transpose(2, 0, 1) * np.float32(mul))


def test_argument_errors(fk):
    t = torch.zeros((5, 3, 4, 4), device="cuda")
    frame = torch.zeros((4, 4, 3), dtype=torch.uint8, device="cuda")
    with pytest.raises(fk.FkError, match="unsupported"):
        fk.circular_tensor_update_u8c3_split_f32(frame, 1.0, t, t.clone(), 0, 1)  # no ring of 5 is instantiated
    t4 = torch.zeros((4, 3, 4, 4), device="cuda")
    with pytest.raises(fk.FkError, match="argument"):
        fk.circular_tensor_update_u8c3_split_f32(frame, 1.0, t4, t4.clone(), 4, 1)
