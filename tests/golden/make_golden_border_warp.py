"""Writes tests/golden/reference_border_warp_vectors.npz from the REFERENCE's own headers
(oracle/_ref/libfkref_border_warp.so: BorderReader, Warping and Deinterlace; built by oracle/Makefile from /root/reference as it lies there; its CPU backend).

Run in the build container only: `python tests/golden/make_golden_border_warp.py`.  The fixture holds outputs only;
inputs are regenerated from the seed and parameters below.  Nothing of the reference's source is stored.  The source
image is taller than wide, so the reference's host interpolation branch (row index taken from the x coordinate) stays
inside it for every warped coordinate.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import binding as B  # noqa: E402

SEED, SRC = 17, (40, 30, 3)  # rows, columns, channels
WINDOWS = [(5, 7, 44, 60), (-3, -4, 10, 12), (70, 95, 150, 200), (0, 0, 30, 40)]  # left, top, dst_w, dst_h
VALUE = (9, 8, 7)
WARPS = {
    "affine_rot": (B.WARP_AFFINE, [[0.9, 0.1, 2.0], [-0.1, 0.95, 3.0]], (36, 28)),
    "affine_shrink": (B.WARP_AFFINE, [[2.5, 0.0, -3.0], [0.0, 1.75, 0.5]], (16, 30)),
    "perspective": (B.WARP_PERSPECTIVE, [[0.9, 0.05, 1.0], [-0.02, 0.97, 2.0], [1e-3, -5e-4, 1.0]], (36, 28)),
    "perspective_strong": (B.WARP_PERSPECTIVE, [[1.2, 0.3, -4.0], [0.1, 1.4, -2.0], [8e-3, 6e-3, 1.0]], (48, 48)),
}


def main():
    o, r = B.oracle(), B.reference()
    if r is None or r.bw is None:
        sys.exit("oracle/_ref/libfkref_border_warp.so is missing: run `make -C oracle` where /root/reference exists")
    src = o.bytes(SEED, SRC)
    out = {}
    for name, bt in B.BORDER_TYPES.items():
        for i, (left, top, dw, dh) in enumerate(WINDOWS):
            out[f"border_{name}_{i}"] = r.border_crop_u8c3(bt, src, left, top, (dw, dh), VALUE)
    for name, (wt, m, dst) in WARPS.items():
        out[f"warp_{name}"] = r.warp_u8c3_f32c3(wt, m, src, dst)
        out[f"coords_{name}"] = np.array([[r.warp_coords(wt, m, x, y) for x in range(0, dst[0], 5)] for y in range(0, dst[1], 5)], np.float32)
    for kind, even in ((B.DEINTERLACE_BLEND, 1), (B.DEINTERLACE_INTER_LINEAR, 1), (B.DEINTERLACE_INTER_LINEAR, 0)):
        out[f"deinterlace_{kind}_{even}"] = r.deinterlace_u8c3_f32c3(kind, even, src)  # 40 lines: an even number
    np.savez_compressed(os.path.join(HERE, "reference_border_warp_vectors.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
