"""Writes tests/golden/reference_paths_vectors.npz from the REFERENCE's own headers (oracle/_ref/libfkref_paths.so,
built by oracle/Makefile from /root/reference as it lies there; its CPU backend): batch reads with
CONDITIONAL_WITH_DEFAULT (copy and resize), a write in the middle of a chain, a batch of output images, a tensor as
the source and the chain of its horizontal-fusion benchmark (a batch of windows of one uchar image).

Run in the build container only: `python tests/golden/make_golden_paths.py`.  The fixture holds outputs only; the inputs
are regenerated from the seeds in CASES.  Nothing of the reference's source is stored.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import binding as B  # noqa: E402

# the source of the resize case is taller than wide: the reference's host branch takes the tap row from the x coordinate
CASES = {
    "copy": {"seed": 31, "shape": (9, 14, 3), "n": 4, "default": (7, 200, 33)},
    "resize": {"seed": 41, "shape": (56, 40, 3), "n": 3, "default": (0.5, -2.0, 300.25), "dst": (24, 30)},
    "midwrite": {"seed": 51, "shape": (11, 17, 3), "mul": 1.75, "add": -0.375},
    "images": {"seed": 61, "shape": (40, 50, 3), "rects": [(0, 0, 13, 9), (37, 31, 13, 9), (5, 20, 13, 9), (20, 3, 13, 9)]},
    "tensor": {"seed": 71, "shape": (3, 6, 10, 3), "mul": (0.5, 3.0, -1.25)},
    # benchmark_horizontal_fusion.h: windows at (i, i); its own constants (1, 1, 3.2) and a set that rounds at every step
    "windows": {"seed": 81, "shape": (48, 70), "rects": [(i, i, 23, 17) for i in range(8)], "ops": [(1.0, 1.0, 3.2), (1.4, 0.3, 255.0)]},
}


def inputs(o, name):
    c = CASES[name]
    if name in ("copy", "resize"):
        return [o.bytes(c["seed"] + i, c["shape"]) for i in range(c["n"])]
    if name in ("images", "windows"):
        return o.bytes(c["seed"], c["shape"])
    n = int(np.prod(c["shape"]))
    return o.unit_floats(c["seed"], n).reshape(c["shape"])


def run(lib, o, quirk=None):
    """Every case through `lib` (the reference driver, or the oracle with the given interpolation rule)."""
    out = {}
    srcs = inputs(o, "copy")
    for used in range(CASES["copy"]["n"] + 1):
        out[f"copy_used{used}"] = lib.conditional_copy_u8c3(srcs, used, CASES["copy"]["default"])
    srcs = inputs(o, "resize")
    for used in range(CASES["resize"]["n"] + 1):
        kw = {} if quirk is None else {"quirk": quirk}
        out[f"resize_used{used}"] = lib.conditional_resize_f32c3(srcs, used, CASES["resize"]["default"], CASES["resize"]["dst"], **kw)
    mid, res = lib.muladd_midwrite_f32c3(inputs(o, "midwrite"), CASES["midwrite"]["mul"], CASES["midwrite"]["add"])
    out["midwrite_mid"], out["midwrite_out"] = mid, res
    for i, img in enumerate(lib.batch_crop_cast_images(inputs(o, "images"), CASES["images"]["rects"])):
        out[f"images_{i}"] = img
    out["tensor"] = lib.tensor_mul_f32c3(inputs(o, "tensor"), CASES["tensor"]["mul"])
    for k, (m, s_, d) in enumerate(CASES["windows"]["ops"]):
        out[f"windows_{k}"] = lib.batch_windows_saturate_muls_f32(inputs(o, "windows"), CASES["windows"]["rects"], m, s_, d)
    return out


def main():
    o, r = B.oracle(), B.reference()
    if r is None or r.paths is None:
        sys.exit("oracle/_ref/libfkref_paths.so is missing: run `make -C oracle` where /root/reference exists")
    out = run(r, o)
    np.savez_compressed(os.path.join(HERE, "reference_paths_vectors.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
