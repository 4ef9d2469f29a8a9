"""Writes tests/golden/reference_yuv_vectors.npz from the REFERENCE's own headers (oracle/_ref/libfkref_yuv.so, built
by oracle/Makefile from /root/reference as it lies there; its CPU backend).

Run in the build container only: `python tests/golden/make_golden_yuv.py`.  The fixture holds outputs only; inputs are
regenerated from the seeds below with the repository's seeded generator (yuv_case_input).  Nothing of the reference's
source is stored.  The reference is handed RawImages whose data dims carry the image height (see
oracle/ref_driver_yuv.cpp), and the resize case keeps the reference's host interpolation branch (row index taken from
the x coordinate) inside the image.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import binding as B  # noqa: E402

SIZE = (16, 8)            # image width, height
CROP = (2, 0, 6, 8)       # x, y, width, height
DST = (9, 5)
DIV = 255.0


def yuv_case_input(o, name):
    """Seeded raw image and seeded {Y,U,V} pixels for format `name` (every bit of every element random)."""
    fmt = B.YUV_FORMATS[name]
    rows, cols, dt = o.yuv_data_shape(fmt, *SIZE)
    seed = 100 + fmt
    raw = o.bytes(seed, (rows, cols * np.dtype(dt).itemsize)).view(dt)
    pixels = o.bytes(seed + 50, (SIZE[1], SIZE[0] * 3 * np.dtype(dt).itemsize)).view(dt).reshape(SIZE[1], SIZE[0], 3)
    return fmt, raw, pixels


def main():
    o, r = B.oracle(), B.reference()
    if r is None or r.yuv is None:
        sys.exit("oracle/_ref/libfkref_yuv.so is missing: run `make -C oracle` where /root/reference exists")
    out = {}
    for name in B.YUV_FORMATS:
        fmt, raw, pixels = yuv_case_input(o, name)
        out[f"{name}_read"] = r.read_yuv(fmt, raw, *SIZE)
        out[f"{name}_write"] = r.write_yuv(fmt, pixels)
        for rng, prim in B.YUV_MATRICES:
            for alpha in (0, 1):
                for float_out in (0, 1):
                    out[f"{name}_rgb_r{rng}p{prim}a{alpha}f{float_out}"] = r.yuv_to_rgb(fmt, rng, prim, alpha, float_out, raw, *SIZE)
            out[f"{name}_chain_r{rng}p{prim}"] = r.yuv_crop_resize_norm_split(fmt, rng, prim, raw, *SIZE, CROP, DST, DIV)
    np.savez_compressed(os.path.join(HERE, "reference_yuv_vectors.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
