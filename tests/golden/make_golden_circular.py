"""Writes tests/golden/reference_circular_vectors.npz from the REFERENCE's own headers
(oracle/_ref/libfkref_circular.so, built by oracle/Makefile from /root/reference as it lies there; its CPU backend):
the four tensor layout conversions and the circular tensor read in both directions.

Run in the build container only: `python tests/golden/make_golden_circular.py`.  The fixture holds outputs only; the
input is regenerated from the seed below.  Nothing of the reference's source is stored.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import binding as B  # noqa: E402

SEED, W, H, PLANES = 23, 7, 5, 4


def main():
    o, r = B.oracle(), B.reference()
    if r is None or r.circ is None:
        sys.exit("oracle/_ref/libfkref_circular.so is missing: run `make -C oracle` where /root/reference exists")
    src = o.unit_floats(SEED, PLANES * H * W * 3)
    out = {}
    for mode in range(4):
        out[f"relayout_{mode}"] = r.tensor_relayout_f32c3(mode, src, W, H, PLANES)
    ring = src.reshape(PLANES, H, W, 3)
    for direction in (B.ASCENDENT, B.DESCENDENT):
        for first in range(PLANES):
            out[f"ring_d{direction}_f{first}"] = r.circular_tensor_read_f32c3(direction, first, ring)
    np.savez_compressed(os.path.join(HERE, "reference_circular_vectors.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
