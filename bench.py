#!/usr/bin/env python3
"""Benchmark of the fused Transform path on one MI355X.

Headline workload (the vertical-fusion configuration at depth 16): 3840x2160 float3, PerThreadRead -> 16 alternating Mul/Add ->
PerThreadWrite in ONE launch.  One step = one fused launch over the whole image.  Inputs are resident in HBM before
the timed region; three buffer sets (600 MB) are rotated so that the 256 MB Infinity Cache cannot hold a step's data.
Prints ONE JSON line: Gpixel/s, the HBM roofline of the kernel (algorithmic bytes / measured duration vs 8 TB/s),
the reference CPU executor timed on this host, and per-config figures for the other chains.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12
# HBM bytes per launch of the headline kernel from two rocprofv3 --pmc runs (FETCH_SIZE scaled by 1.9994, WRITE_SIZE by
# 1.0, the factors a plain copy of known size shows); the summary lies under profiles/.
MEASURED_TRAFFIC_BYTES = 199.18e6
W, H = 3840, 2160
DEPTH = 16
MUL_V, ADD_V = 1.0001, 1e-4


class StreamTimer:
    """HIP events on the stream the kernels are launched on (through the library's own runtime ABI)."""

    def __init__(self, rt, stream):
        self.rt, self.stream = rt, C.c_void_p(stream)
        self.a, self.b = C.c_void_p(), C.c_void_p()
        assert rt.fkrt_event_create(C.byref(self.a)) == 0 and rt.fkrt_event_create(C.byref(self.b)) == 0

    def start(self):
        assert self.rt.fkrt_event_record(self.a, self.stream) == 0

    def stop_ms(self):
        assert self.rt.fkrt_event_record(self.b, self.stream) == 0
        assert self.rt.fkrt_event_sync(self.b) == 0
        ms = C.c_float()
        assert self.rt.fkrt_event_elapsed_ms(C.byref(ms), self.a, self.b) == 0
        return float(ms.value)


SPINUP_S = 0.2


def spin_up(launch, seconds=None):
    """Untimed launches of the workload itself until the device has been busy for `seconds`: a process starts at idle
    clocks and the first milliseconds of launches run up to 20 % slower than the steady state that is measured."""
    import torch
    seconds = SPINUP_S if seconds is None else seconds
    t0, i = time.perf_counter(), 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(32):
            launch(i)
            i += 1
        torch.cuda.synchronize()


def time_launches(timer, launch, steps, warmup):
    import torch
    spin_up(launch)
    for i in range(warmup):
        launch(i)
    torch.cuda.synchronize()
    timer.start()
    for i in range(steps):
        launch(i)
    ms = timer.stop_ms()
    torch.cuda.synchronize()
    return ms / steps


def cpu_baseline(src_host, budget_s=10.0):
    """The reference's own CPU executor (oracle/_ref, its headers compiled as they are) on the same chain and image,
    one core; falls back to the C restatement when that build is absent."""
    import numpy as np
    from oracle import binding
    ref = binding.reference()
    lib, kind = (ref, "reference") if ref is not None else (binding.oracle(), "port")
    lib.muladd_chain_f32c3(src_host[:64], DEPTH, MUL_V, ADD_V)  # warm-up
    passes, t0 = 0, time.perf_counter()
    while True:
        lib.muladd_chain_f32c3(src_host, DEPTH, MUL_V, ADD_V)
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or passes >= 200:
            break
    return {"value": W * H * passes / dt / 1e9, "unit": "Gpixel/s", "cores": 1, "kind": kind,
            "sample": f"{passes} full passes of the same {W}x{H} float3 depth-{DEPTH} chain in {dt:.1f} s, serial z/y/x loop",
            "ms_per_pass": 1e3 * dt / passes, "host_cores_available": os.cpu_count()}


def other_configs(fk, timer, steps, warmup, only=None):
    """Per-config kernel time, output Gpixel/s and algorithmic GB/s for the remaining chains (device-random inputs).
    `only` restricts the run to the configs whose name starts with it (for counter collection on one kernel)."""
    import torch
    res = {}
    g = torch.Generator(device="cuda").manual_seed(0)

    def rnd_u8(*shape):
        return torch.randint(0, 256, shape, dtype=torch.uint8, device="cuda", generator=g)

    def want(name):
        return only is None or name.startswith(only)

    def record(name, ms, out_px, alg_bytes, note=None):
        res[name] = {"ms": ms, "gpixel_s": out_px / ms / 1e6, "alg_bytes": alg_bytes, "gb_s": alg_bytes / ms / 1e6,
                     "frac_hbm_peak": alg_bytes / (ms * 1e-3) / HBM_PEAK}
        if note:
            res[name]["note"] = note

    # C1: README pipeline at its literal shape (launch-latency bound: 234 KB moved)
    img4k = rnd_u8(2160, 3840, 3)
    rects = [(0, 0, 34, 25), (10, 10, 70, 15), (20, 20, 60, 59), (30, 30, 20, 23), (40, 40, 12, 11)]
    out1 = torch.empty((5, 60, 60, 3), device="cuda")
    a1 = (0, (0, 0, 0), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)
    if want("C1_readme_60x60x5"):
        call = fk.crop_resize_muls_bgr_tensor(img4k, rects, out1, *a1, defer=True)
        ms = time_launches(timer, lambda i: call(), steps, warmup)
        record("C1_readme_60x60x5", ms, 18000, sum(r[2] * r[3] for r in rects) * 3 + 18000 * 12, "launch-latency bound")

    # C1 scaled: same chain, 5 crops of 1024x768 -> 1920x1080 (bandwidth-sized)
    if want("C1_scaled_5x1024x768_to_1920x1080"):
        rects_s = [(64 * i, 48 * i, 1024, 768) for i in range(5)]
        out1s = [torch.empty((5, 1080, 1920, 3), device="cuda") for _ in range(3)]
        calls = [fk.crop_resize_muls_bgr_tensor(img4k, rects_s, o, *a1, defer=True) for o in out1s]
        ms = time_launches(timer, lambda i: calls[i % 3](), steps, warmup)
        record("C1_scaled_5x1024x768_to_1920x1080", ms, 5 * 1920 * 1080, 5 * 1024 * 768 * 3 + 5 * 1920 * 1080 * 12)
        del out1s, calls

    # the same with 16:9 crops: no bars, every output pixel is resampled
    if want("C1_nobars_5x1024x576_to_1920x1080"):
        rects_n = [(64 * i, 48 * i, 1024, 576) for i in range(5)]
        out1n = [torch.empty((5, 1080, 1920, 3), device="cuda") for _ in range(3)]
        calls = [fk.crop_resize_muls_bgr_tensor(img4k, rects_n, o, *a1, defer=True) for o in out1n]
        ms = time_launches(timer, lambda i: calls[i % 3](), steps, warmup)
        record("C1_nobars_5x1024x576_to_1920x1080", ms, 5 * 1920 * 1080, 5 * 1024 * 576 * 3 + 5 * 1920 * 1080 * 12)
        del out1n, calls

    # C3: 50 crops of 50 images -> 224x224x3x50 planar
    if want("C3_batch50_224x224_split"):
        imgs = [rnd_u8(1080, 1920, 3) for _ in range(50)]
        ws = torch.randint(16, 513, (50,), generator=torch.Generator().manual_seed(3)).tolist()
        hs = torch.randint(16, 513, (50,), generator=torch.Generator().manual_seed(4)).tolist()
        rects3 = [((1920 - w) // 2, (1080 - h) // 3, w, h) for w, h in zip(ws, hs)]
        out3 = torch.empty((50, 3, 224, 224), device="cuda")
        a3 = ((255.,) * 3, (.485, .456, .406), (.229, .224, .225))
        call3 = fk.batch_crop_resize_norm_split(imgs, rects3, out3, *a3, defer=True)
        ms = time_launches(timer, lambda i: call3(), steps, warmup)
        record("C3_batch50_224x224_split", ms, 50 * 224 * 224, 50 * 224 * 224 * 12 + sum(3 * r[2] * r[3] for r in rects3))
        del imgs, call3

    # C4: resize 4K -> 1280x720, 32 tiles of 128x128
    if want("C4_resize_crop_32x128x128"):
        rects4 = [(160 * i, 180 * j, 128, 128) for j in range(4) for i in range(8)]
        out4 = torch.empty((32, 128, 128, 3), device="cuda")
        call4 = fk.resize_crop_tiles(img4k, (1280, 720), rects4, out4, (1 / 255.,) * 3, defer=True)
        ms = time_launches(timer, lambda i: call4(), steps, warmup)
        record("C4_resize_crop_32x128x128", ms, 32 * 128 * 128, 32 * 383 * 383 * 3 + 32 * 128 * 128 * 12)

    # Y1..Y4: the YUV front-end at 4K (raw buffers of random bytes: every value is a legal sample)
    n4k = 3840 * 2160
    if want("Y1_nv12_4k_to_rgb_u8c3"):
        nv12 = rnd_u8(3240, 3840)
        outs = [torch.empty((2160, 3840, 3), dtype=torch.uint8, device="cuda") for _ in range(3)]
        calls = [fk.yuv_to_rgb(fk.NV12, fk.RANGE_FULL, fk.BT709, nv12, o, defer=True) for o in outs]
        ms = time_launches(timer, lambda i: calls[i % 3](), steps, warmup)
        record("Y1_nv12_4k_to_rgb_u8c3", ms, n4k, n4k * 3 // 2 + n4k * 3)
        del outs, calls
    if want("Y2_p010_4k_to_rgba_u16c4"):
        p010 = torch.randint(-32768, 32767, (3240, 3840), dtype=torch.int16, device="cuda", generator=g)
        outs = [torch.empty((2160, 3840, 4), dtype=torch.int16, device="cuda") for _ in range(3)]
        calls = [fk.yuv_to_rgb(fk.P010, fk.RANGE_FULL, fk.BT2020, p010, o, defer=True) for o in outs]
        ms = time_launches(timer, lambda i: calls[i % 3](), steps, warmup)
        record("Y2_p010_4k_to_rgba_u16c4", ms, n4k, n4k * 3 + n4k * 8)
        del outs, calls, p010
    if want("Y3_uyvy_4k_to_rgb_f32c3"):
        uyvy = rnd_u8(2160, 7680)
        outs = [torch.empty((2160, 3840, 3), device="cuda") for _ in range(3)]
        calls = [fk.yuv_to_rgb(fk.UYVY, fk.RANGE_FULL, fk.BT601, uyvy, o, defer=True) for o in outs]
        ms = time_launches(timer, lambda i: calls[i % 3](), steps, warmup)
        record("Y3_uyvy_4k_to_rgb_f32c3", ms, n4k, n4k * 2 + n4k * 12)
        del outs, calls, uyvy
    if want("Y4_nv12_crop1920x1080_to_1280x720_split"):
        nv12 = rnd_u8(3240, 3840)
        out_y4 = torch.empty((3, 720, 1280), device="cuda")
        call_y4 = fk.yuv_crop_resize_norm_split(fk.NV12, fk.RANGE_FULL, fk.BT709, nv12, (3840, 2160), (960, 540, 1920, 1080), out_y4, 255.0, defer=True)
        ms = time_launches(timer, lambda i: call_y4(), steps, warmup)
        record("Y4_nv12_crop1920x1080_to_1280x720_split", ms, 1280 * 720, 1920 * 1080 * 3 // 2 + 1280 * 720 * 12,
               "the README's backwards-vertical-fusion example: only the crop's YUV samples are read")
    if want("Y5_nv12_crop640x360_to_1920x1080_split"):
        nv12 = rnd_u8(3240, 3840)
        out_y5 = torch.empty((3, 1080, 1920), device="cuda")
        call_y5 = fk.yuv_crop_resize_norm_split(fk.NV12, fk.RANGE_FULL, fk.BT709, nv12, (3840, 2160), (1600, 900, 640, 360), out_y5, 255.0, defer=True)
        ms = time_launches(timer, lambda i: call_y5(), steps, warmup)
        record("Y5_nv12_crop640x360_to_1920x1080_split", ms, 1920 * 1080, 640 * 360 * 3 // 2 + 1920 * 1080 * 12)

    # B1, W1, W2: border and warp chains over the 4K uchar3 frame
    if want("B1_reflect101_border64_4k_u8c3"):
        outs = [torch.empty((2160 + 128, 3840 + 128, 3), dtype=torch.uint8, device="cuda") for _ in range(3)]
        calls = [fk.border_crop_u8c3(fk.BORDER_REFLECT_101, img4k, 64, 64, o, defer=True) for o in outs]
        ms = time_launches(timer, lambda i: calls[i % 3](), steps, warmup)
        record("B1_reflect101_border64_4k_u8c3", ms, 3968 * 2288, n4k * 3 + 3968 * 2288 * 3)
        del outs, calls
    if want("W1_affine_rot5deg_4k_to_4k_f32c3"):
        import math
        c, s_ = math.cos(math.radians(5.0)), math.sin(math.radians(5.0))
        rot = [[c, -s_, 1920 - c * 1920 + s_ * 1080], [s_, c, 1080 - s_ * 1920 - c * 1080]]  # about the image centre
        outs = [torch.empty((2160, 3840, 3), device="cuda") for _ in range(3)]
        calls = [fk.warp_u8c3_f32c3(fk.WARP_AFFINE, rot, img4k, o, defer=True) for o in outs]
        ms = time_launches(timer, lambda i: calls[i % 3](), steps, warmup)
        record("W1_affine_rot5deg_4k_to_4k_f32c3", ms, n4k, n4k * 3 + n4k * 12, "source bytes counted once for the whole frame")
        del outs, calls
    if want("W2_perspective_4k_to_1920x1080_f32c3"):
        per = [[2.0, 0.1, 0.0], [0.05, 2.0, 0.0], [2e-5, 1e-5, 1.0]]
        out_w2 = torch.empty((1080, 1920, 3), device="cuda")
        call_w2 = fk.warp_u8c3_f32c3(fk.WARP_PERSPECTIVE, per, img4k, out_w2, defer=True)
        ms = time_launches(timer, lambda i: call_w2(), steps, warmup)
        record("W2_perspective_4k_to_1920x1080_f32c3", ms, 1920 * 1080, 1920 * 1080 * 4 * 3 + 1920 * 1080 * 12, "four taps per output pixel, 2x down-scaling: no tap is shared")

    # R1: one update of a ring of eight 1080p frames kept as normalised float planes (new frame through the chain, seven planes re-ordered)
    if want("R1_circular_tensor_update_8x1080p"):
        batch, hh, ww = 8, 1080, 1920
        frame_r = rnd_u8(hh, ww, 3)
        tensor_r = torch.zeros((batch, 3, hh, ww), device="cuda")
        ring_r = torch.zeros((batch, 3, hh, ww), device="cuda")
        calls_r = [fk.circular_tensor_update_u8c3_split_f32(frame_r, 1 / 255., tensor_r, ring_r, i, 1, defer=True) for i in range(batch)]
        ms = time_launches(timer, lambda i: calls_r[i % batch](), steps, warmup)
        px = hh * ww
        record("R1_circular_tensor_update_8x1080p", ms, batch * px, px * 3 + px * 12 * 2 + (batch - 1) * px * 12 * 2,
               "frame read + its planes written to tensor and ring + seven planes copied from the ring")
        del tensor_r, ring_r, calls_r

    # C5: four chains over one 8192x8192 uchar4 image in one launch
    if not want("C5_divergent4_8192x8192"):
        return res
    big = rnd_u8(8192, 8192, 4)
    gray = torch.empty((8192, 8192), dtype=torch.uint8, device="cuda")
    small = torch.empty((512, 512, 4), device="cuda")
    crop = torch.empty((1024, 1024, 4), dtype=torch.uint8, device="cuda")
    bgr = torch.empty((8192, 8192, 3), device="cuda")
    n5 = max(3, steps // 4)
    call5 = fk.divergent4_u8c4(big, gray, small, 1 / 255., (3584, 3584, 1024, 1024), 2, crop, 0.5, bgr, defer=True)
    ms = time_launches(timer, lambda i: call5(), n5, max(1, warmup // 4))
    record("C5_divergent4_8192x8192", ms, 8192 * 8192 * 2 + 512 * 512 + 1024 * 1024, 1426063360,
           "1,157,627,904 B if chains a and d share the source through cache")
    return res


def main():
    global SPINUP_S
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--spinup-s", type=float, default=SPINUP_S,
                    help="seconds of untimed launches of each workload before its warm-up steps (shorter for traces)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sweep", action="store_true", help="skip the depth sweep and the other configs")
    ap.add_argument("--only-config", default=None,
                    help="run only the named secondary config (prefix of C1_readme, C1_scaled, C3, C4, C5) and print its figures: "
                         "for rocprofv3 counter runs on one kernel")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run plain device copies of the same 99.5 MB image (torch copy kernel) before the timed "
                         "region, so that a counter run has a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    SPINUP_S = args.spinup_s
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (planes/row bands would shard with no "
                 "exchange); run with --gpus 1")

    import numpy as np
    import torch
    import fusedkernellibrary_amd as fk
    from oracle import binding

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    rt, _ = fk.load()
    timer = StreamTimer(rt, torch.cuda.current_stream().cuda_stream)

    if args.only_config is not None:
        print(json.dumps(other_configs(fk, timer, args.steps, args.warmup, only=args.only_config)))
        return

    src_host = binding.oracle().unit_floats(2, (H, W, 3))
    sets = 3
    srcs = [torch.from_numpy(src_host).cuda() for _ in range(sets)]
    dsts = [torch.empty((H, W, 3), device="cuda") for _ in range(sets)]
    torch.cuda.synchronize()

    # arguments are marshalled once per buffer set; the timed loop only makes the C calls
    steps_by_set = [fk.muladd_chain_f32c3(srcs[k], dsts[k], DEPTH, MUL_V, ADD_V, defer=True) for k in range(sets)]

    def step(i):
        steps_by_set[i % sets]()

    if args.copy_calibration:
        for i in range(10):
            dsts[i % sets].copy_(srcs[i % sets])
        torch.cuda.synchronize()

    # timed region: exactly `steps` launches, device-synchronised on both sides
    spin_up(step)
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    timer.start()
    for i in range(args.steps):
        step(i)
    kernel_ms = timer.stop_ms() / args.steps
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # the result of the last timed step is the real chain (spot check against the oracle on a few rows)
    want = binding.oracle().muladd_chain_f32c3(src_host[:4], DEPTH, MUL_V, ADD_V)
    got = dsts[(args.steps - 1) % sets][:4].cpu().numpy()
    assert got.tobytes() == want.tobytes(), "benchmark output differs from the oracle"

    alg_bytes = 2 * W * H * 12
    out = {
        "metric": "fused pipeline Gpixel/s + achieved HBM GB/s (% of peak) on 1 MI355X",
        "value": W * H / wall_ms / 1e6, "unit": "Gpixel/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "spinup_s": SPINUP_S, "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"C2 vertical fusion: {W}x{H} float3, PerThreadRead -> {DEPTH} alternating Mul/Add -> "
                               "PerThreadWrite, one fused launch per step, 3 rotating buffer sets"},
        "roofline": {"bound": "hbm", "achieved": alg_bytes / (kernel_ms * 1e-3) / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": alg_bytes / (kernel_ms * 1e-3) / HBM_PEAK, "traffic": MEASURED_TRAFFIC_BYTES,
                     "kernel": "transform_kernel<PointwiseJob<float3 -> float3, depth 16>>", "alg_bytes_per_launch": alg_bytes,
                     "kernel_ms": kernel_ms},
    }

    if not args.no_sweep:
        # the other chains first: the deep end of the sweep below keeps the vector units saturated for seconds, and a
        # launch measured right after it runs at the clock the device has dropped to by then
        out["other_configs"] = other_configs(fk, timer, args.steps, args.warmup)
        sweep = {}
        k = max(10, args.steps // 4)
        for depth in fk.CHAIN_DEPTHS:
            calls = [fk.muladd_chain_f32c3(srcs[q], dsts[q], depth, MUL_V, ADD_V, defer=True) for q in range(sets)]
            fused = time_launches(timer, lambda i: calls[i % sets](), k, 3)
            # the same operations as `depth` separate launches, ping-ponging between two output buffers
            first = [fk.single_op_f32c3(srcs[q], dsts[q], 0, MUL_V, defer=True) for q in range(sets)]
            fwd = [[fk.single_op_f32c3(dsts[q], dsts[(q + 1) % sets], j, ADD_V if j else MUL_V, defer=True) for j in (0, 1)] for q in range(sets)]
            back = [[fk.single_op_f32c3(dsts[(q + 1) % sets], dsts[q], j, ADD_V if j else MUL_V, defer=True) for j in (0, 1)] for q in range(sets)]

            def unfused(i):
                q = i % sets
                first[q]()
                for j in range(1, depth):
                    (fwd if j % 2 else back)[q][j % 2]()
            unf = time_launches(timer, unfused, max(3, k // 4), 1)
            sweep[str(depth)] = {"fused_ms": fused, "unfused_ms": unf, "fused_gb_s": alg_bytes / fused / 1e6,
                                 "fused_frac_hbm_peak": alg_bytes / (fused * 1e-3) / HBM_PEAK, "speedup_vs_unfused": unf / fused}
        out["depth_sweep"] = sweep

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(src_host)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
