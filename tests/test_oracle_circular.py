"""Pins the tensor-layout / circular part of the oracle (oracle/fk_oracle_circular.c), CPU only:

 1. layouts and circular reads: vectors written by the reference's own headers (tests/golden/make_golden_circular.py),
    that build directly on other shapes where present, and numpy transposes / rolls (the operations are permutations);
 2. CircularTensor::update, which the reference cannot execute (it has no executor for the divergent launch the method
    asks for): the sliding-window property the class exists for, for both orders, every batch size and any number of
    updates, and the composition of the method's two sequences out of the operations pinned in 1.
"""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
from oracle import binding as B  # noqa: E402
import make_golden_circular as G  # noqa: E402

GOLD = np.load(os.path.join(HERE, "golden", "reference_circular_vectors.npz"))


def same_bits(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and a.tobytes() == b.tobytes()


def test_golden_layouts_and_ring(oracle):
    src = oracle.unit_floats(G.SEED, G.PLANES * G.H * G.W * 3)
    for mode in range(4):
        assert same_bits(oracle.tensor_relayout_f32c3(mode, src, G.W, G.H, G.PLANES), GOLD[f"relayout_{mode}"]), mode
    ring = src.reshape(G.PLANES, G.H, G.W, 3)
    for direction in (B.ASCENDENT, B.DESCENDENT):
        for first in range(G.PLANES):
            assert same_bits(oracle.circular_tensor_read_f32c3(direction, first, ring), GOLD[f"ring_d{direction}_f{first}"])


def test_layouts_are_the_transposes_they_name(oracle):
    n, h, w = 3, 4, 6
    packed = oracle.unit_floats(5, n * h * w * 3).reshape(n, h, w, 3)
    split = np.ascontiguousarray(packed.transpose(0, 3, 1, 2))       # n, c, h, w
    transposed = np.ascontiguousarray(packed.transpose(3, 0, 1, 2))  # c, n, h, w
    assert same_bits(oracle.tensor_relayout_f32c3(B.PACKED_TO_SPLIT, packed, w, h, n), split.ravel())
    assert same_bits(oracle.tensor_relayout_f32c3(B.PACKED_TO_TRANSPOSED, packed, w, h, n), transposed.ravel())
    assert same_bits(oracle.tensor_relayout_f32c3(B.SPLIT_TO_PACKED, split, w, h, n), packed.ravel())
    assert same_bits(oracle.tensor_relayout_f32c3(B.TRANSPOSED_TO_PACKED, transposed, w, h, n), packed.ravel())


def test_ring_read_is_a_roll(oracle):
    for planes in (1, 2, 5, 8):
        ring = oracle.unit_floats(planes, planes * 3 * 4 * 3).reshape(planes, 3, 4, 3)
        for first in range(planes):
            assert same_bits(oracle.circular_tensor_read_f32c3(B.ASCENDENT, first, ring), np.roll(ring, -first, axis=0))
            assert same_bits(oracle.circular_tensor_read_f32c3(B.DESCENDENT, first, ring), np.roll(ring[::-1], first + 1, axis=0))


def test_against_reference_build_other_shapes(oracle, reference):
    if reference.circ is None:
        pytest.skip("oracle/_ref/libfkref_circular.so not built")
    for planes, h, w in ((2, 1, 1), (3, 9, 2), (8, 4, 11)):
        src = oracle.unit_floats(planes + w, planes * h * w * 3)
        for mode in range(4):
            assert same_bits(oracle.tensor_relayout_f32c3(mode, src, w, h, planes), reference.tensor_relayout_f32c3(mode, src, w, h, planes))
        ring = src.reshape(planes, h, w, 3)
        for direction in (B.ASCENDENT, B.DESCENDENT):
            for first in range(planes):
                assert same_bits(oracle.circular_tensor_read_f32c3(direction, first, ring), reference.circular_tensor_read_f32c3(direction, first, ring))


@pytest.mark.parametrize("newest_first", [1, 0])
@pytest.mark.parametrize("batch", [1, 2, 3, 4, 8])
def test_update_keeps_the_last_frames_in_age_order(oracle, batch, newest_first):
    h, w, mul = 5, 7, 0.5
    tensor = np.full((batch, 3, h, w), -1.0, np.float32)
    ring = np.full((batch, 3, h, w), -2.0, np.float32)
    frames, nxt = [], 0
    for k in range(2 * batch + 3):
        frame = oracle.bytes(100 + k, (h, w, 3))
        frames.append(frame.astype(np.float32).transpose(2, 0, 1) * np.float32(mul))
        oracle.circular_tensor_update_u8c3_split_f32(frame, mul, tensor, ring, nxt, newest_first)
        nxt = (nxt + 1) % batch
        for age in range(min(batch, k + 1)):  # age 0 = the frame just given
            plane = age if newest_first else batch - 1 - age
            assert same_bits(tensor[plane], frames[k - age]), (k, age)


def test_update_is_its_two_sequences(oracle):
    """The update of circular_tensor.h:107-155 out of operations pinned above: the new frame goes through the chain into
    the tensor's newest plane and into the ring plane `next` (+ that plane index, ascendent); all other planes are the
    circular read of the ring (descendent for NewestFirst, ascendent for OldestFirst) with first = next."""
    batch, h, w, mul = 4, 3, 5, 2.0
    for newest_first in (1, 0):
        tensor = oracle.unit_floats(1, batch * 3 * h * w).reshape(batch, 3, h, w)
        ring = oracle.unit_floats(2, batch * 3 * h * w).reshape(batch, 3, h, w)
        for nxt in range(batch):
            frame = oracle.bytes(50 + nxt, (h, w, 3))
            want_t, want_r = tensor.copy(), ring.copy()
            new_plane = 0 if newest_first else batch - 1
            value = frame.astype(np.float32).transpose(2, 0, 1) * np.float32(mul)
            want_r[(new_plane + nxt) % batch] = value
            # circular read works on packed planes; the ring here is split: convert, read, convert back
            packed = oracle.tensor_relayout_f32c3(B.SPLIT_TO_PACKED, want_r, w, h, batch).reshape(batch, h, w, 3)
            ordered = oracle.circular_tensor_read_f32c3(B.DESCENDENT if newest_first else B.ASCENDENT, nxt, packed)
            ordered = oracle.tensor_relayout_f32c3(B.PACKED_TO_SPLIT, ordered, w, h, batch).reshape(batch, 3, h, w)
            for z in range(batch):
                want_t[z] = value if z == new_plane else ordered[z]
            oracle.circular_tensor_update_u8c3_split_f32(frame, mul, tensor, ring, nxt, newest_first)
            assert same_bits(tensor, want_t) and same_bits(ring, want_r)
