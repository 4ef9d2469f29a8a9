"""Writes tests/golden/reference_vectors.npz from the REFERENCE's own headers (oracle/_ref/libfkref.so, built by
oracle/Makefile from /root/reference as it lies there; its CPU backend, literal host semantics).

Run in the build container only: `python tests/golden/make_golden.py`.  The fixture holds outputs and the seeds /
parameters that regenerate the inputs with the repository's seeded generator; nothing of the reference's source is
stored.  Resize cases are chosen so that the host branch of the reference's bilinear interpolation (row index taken
from the x coordinate) stays inside the source image.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import binding as B  # noqa: E402

CASES = {
    "readme": dict(seed=1, src=(2160, 3840, 3),
                   rects=[(0, 0, 34, 25), (10, 10, 70, 15), (20, 20, 60, 59), (30, 30, 20, 23), (40, 40, 12, 11)],
                   dst=(60, 60), background=(0, 0, 0), mul=(1.4,) * 3, sub=(0.5,) * 3, div=(255.,) * 3),
    "readme_small_bg": dict(seed=11, src=(300, 160, 3), rects=[(3, 1, 40, 17), (7, 2, 16, 33)], dst=(24, 20),
                            background=(0.25, -1.5, 7.0), mul=(1.5, 0.5, 2.0), sub=(0.1, 0.2, 0.3), div=(3.0, 7.0, 255.0)),
    "split": dict(seed=3, src=(600, 300, 3), n=5,
                  rects=[(5, 3, 100, 40), (0, 0, 16, 16), (100, 10, 200, 100), (17, 29, 33, 47), (50, 50, 250, 128)],
                  dst=(32, 32), div1=(255.,) * 3, sub=(.485, .456, .406), div2=(.229, .224, .225)),
    "tiles": dict(seed=4, src=(400, 96), resized=(32, 100), rects=[(0, 0, 8, 8), (8, 4, 8, 8), (16, 8, 8, 8), (24, 0, 8, 8), (3, 5, 8, 8)],
                  tile=(8, 8), mul=(1 / 255.,) * 3),
    "divergent": dict(seed=5, src=(96, 96, 4), resized=(12, 12), mul_b=1 / 255., rect_c=(20, 30, 40, 24), mul_c=2, sub_d=0.5),
    "muladd": dict(seed=2, src=(9, 21, 3), depths=[1, 2, 4, 8, 16], mul_v=1.0001, add_v=1e-4),
    "crops": dict(seed=7, src=(120, 200, 3), rects=[(1, 2, 30, 20), (5, 5, 10, 25), (100, 60, 33, 7)], max_size=(33, 25)),
}


def main():
    o, r = B.oracle(), B.reference()
    if r is None:
        sys.exit("oracle/_ref/libfkref.so is missing: run `make -C oracle` where /root/reference exists")
    out = {}
    c = CASES["readme"]
    src = o.bytes(c["seed"], c["src"])
    for aspect in (B.PRESERVE_AR, B.IGNORE_AR, B.PRESERVE_AR_RN_EVEN, B.PRESERVE_AR_LEFT):
        out[f"readme_ar{aspect}"] = r.crop_resize_muls_bgr_tensor(src, c["rects"], c["dst"], aspect, c["background"], c["mul"], c["sub"], c["div"])
    c = CASES["readme_small_bg"]
    src = o.bytes(c["seed"], c["src"])
    for aspect in (B.PRESERVE_AR, B.PRESERVE_AR_RN_EVEN, B.PRESERVE_AR_LEFT):
        out[f"readme_small_bg_ar{aspect}"] = r.crop_resize_muls_bgr_tensor(src, c["rects"], c["dst"], aspect, c["background"], c["mul"], c["sub"], c["div"])
    c = CASES["split"]
    srcs = [o.bytes(c["seed"] + i, c["src"]) for i in range(c["n"])]
    out["split"] = r.batch_crop_resize_norm_split(srcs, c["rects"], c["dst"], c["div1"], c["sub"], c["div2"])
    c = CASES["tiles"]
    src = o.gradient_noise_u8c3(c["seed"], c["src"][1], c["src"][0])
    out["tiles"] = r.resize_crop_tiles(src, c["resized"], c["rects"], c["tile"], c["mul"])
    c = CASES["divergent"]
    src = o.bytes(c["seed"], c["src"])
    out["div_gray"] = r.rgba2gray_u8c4(src)
    out["div_resized"] = r.resize_mul_u8c4_f32c4(src, c["resized"], c["mul_b"])
    out["div_crop"] = r.crop_mul_saturate_u8c4(src, c["rect_c"], c["mul_c"])
    out["div_bgr"] = r.rgba2bgr_sub_u8c4_f32c3(src, c["sub_d"])
    c = CASES["muladd"]
    src = o.unit_floats(c["seed"], c["src"])
    for d in c["depths"]:
        out[f"muladd_{d}"] = r.muladd_chain_f32c3(src, d, c["mul_v"], c["add_v"])
    out["single_mul"] = r.single_op_f32c3(src, 0, c["mul_v"])
    out["single_add"] = r.single_op_f32c3(src, 1, c["add_v"])
    c = CASES["crops"]
    src = o.bytes(c["seed"], c["src"])
    out["crops"] = r.batch_crop_cast_tensor(src, c["rects"], c["max_size"])
    # single operations of the reference, probed directly
    xs = np.array([-2.5, -1.5, -0.5, -0.49999997, 0.0, 0.49999997, 0.5, 1.5, 2.5, 254.5, 255.49, 1e9, -1e9, 127.5, 63.75], np.float32)
    out["probe_round_in"] = xs
    out["probe_round_out"] = np.array([r.c.fkr_cxp_round(float(x)) for x in xs], np.float32)
    sat = np.array([-300.0, -0.6, -0.5, -0.4, 0.4, 0.5, 1.5, 2.5, 127.5, 254.4, 254.5, 255.0, 255.4, 256.0, 1e6], np.float32)
    out["probe_satf_in"] = sat
    out["probe_satf_out"] = np.array([r.c.fkr_saturate_float_to_u8(float(x)) for x in sat], np.uint8)
    sati = np.array([-2**31, -1, 0, 1, 127, 254, 255, 256, 510, 2**31 - 1], np.int64)
    out["probe_sati_in"] = sati
    out["probe_sati_out"] = np.array([r.c.fkr_saturate_int_to_u8(int(x)) for x in sati], np.uint8)
    rng = np.random.RandomState(0).randint(0, 256, (512, 3)).astype(np.uint8)
    out["probe_gray_in"] = rng
    out["probe_gray_out"] = np.array([r.c.fkr_rgb2gray_u8(int(a), int(b), int(c)) for a, b, c in rng], np.uint8)
    np.savez_compressed(os.path.join(HERE, "reference_vectors.npz"), **out)
    with open(os.path.join(HERE, "reference_cases.json"), "w") as f:
        json.dump(CASES, f, indent=1)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
