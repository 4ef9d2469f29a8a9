#!/usr/bin/env python3
"""Benchmark of the fused Transform path on one MI355X.

Headline workload: the README pipeline (crop -> Resize<INTER_LINEAR, PRESERVE_AR> -> x1.4 -> -0.5 -> /255 -> RGB2BGR ->
float3 tensor) at a bandwidth-sized shape: five 1024x768 crops of a 3840x2160 uchar3 frame, each resized to 1920x1080, one
fused launch per step.  Inputs are resident in HBM before the timed region; source frames and output tensors are rotated
over enough buffer sets that the 256 MB Infinity Cache cannot hold a step's data.
Prints ONE JSON line: Gpixel/s, the HBM roofline of the resize kernel (algorithmic bytes / launch duration by HIP events
on the launch stream, against 8 TB/s), the reference's CPU executor timed on this host, and a roofline object for every
other configuration (the vertical-fusion chain of depth 16 and the divergent launch among them).  Every configuration's
inputs come from the repository's seeded generator, and every configuration's output is checked against the CPU oracle,
on a few rows or planes, after it has been timed.
"""
import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12
# lane operations per second of the vector units for code without FMA and without packed FP32 (this library is built
# without contraction, for bit parity with the reference's CPU results): 256 CUs x 64 lanes x 2.4 GHz
VALU_PEAK = 256 * 64 * 2.4e9
CACHE_BYTES = 256e6  # Infinity Cache
MAX_SETS = 32
W4K, H4K = 3840, 2160
N4K = W4K * H4K
DEPTH = 16
MUL_V, ADD_V = 1.0001, 1e-4
README_ARGS = (0, (0, 0, 0), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)  # PRESERVE_AR, background, mul, sub, div
HEADLINE = "C1_scaled_5x1024x768_to_1920x1080"
CONFIG_NAMES = ["C1_readme_60x60x5", HEADLINE, "C1_nobars_5x1024x576_to_1920x1080", "S0_setto_f32c3_60x60x5", "S1_setto_f32c3_1920x1080x5",
                f"C2_vertical_fusion_depth{DEPTH}", "C3_batch50_224x224_split",
                "C4_resize_crop_32x128x128", "Y1_nv12_4k_to_rgb_u8c3", "Y2_p010_4k_to_rgba_u16c4", "Y3_uyvy_4k_to_rgb_f32c3",
                "Y4_nv12_crop1920x1080_to_1280x720_split", "Y5_nv12_crop640x360_to_1920x1080_split", "B1_reflect101_border64_4k_u8c3",
                "W1_affine_rot5deg_4k_to_4k_f32c3", "W2_perspective_4k_to_1920x1080_f32c3", "R1_circular_tensor_update_8x1080p",
                "K1_conditional_resize_8x1080p_5used", "C5_divergent4_8192x8192"]


class StreamTimer:
    """HIP events on the stream the kernels are launched on (through the library's own runtime ABI)."""

    def __init__(self, rt, stream):
        self.rt, self.stream = rt, C.c_void_p(stream)
        self.a, self.b = C.c_void_p(), C.c_void_p()
        assert rt.fkrt_event_create(C.byref(self.a)) == 0 and rt.fkrt_event_create(C.byref(self.b)) == 0

    def start(self):
        assert self.rt.fkrt_event_record(self.a, self.stream) == 0

    def stop(self):
        assert self.rt.fkrt_event_record(self.b, self.stream) == 0

    def elapsed_ms(self):
        """After the device has been synchronised."""
        assert self.rt.fkrt_event_sync(self.b) == 0
        ms = C.c_float()
        assert self.rt.fkrt_event_elapsed_ms(C.byref(ms), self.a, self.b) == 0
        return float(ms.value)

    def stop_ms(self):
        self.stop()
        return self.elapsed_ms()


SPINUP_S = 0.2
BLOCK_SPINUP_S = 0.01  # untimed launches in front of every timed block after the first


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


def percentile(sorted_values, q):
    """Nearest-rank percentile of an ascending list."""
    return sorted_values[min(len(sorted_values) - 1, max(0, int(math.ceil(q * len(sorted_values))) - 1))]


def time_blocks(timer, launch, steps, warmup, blocks):
    """`blocks` timed blocks of exactly `steps` launches each, every block bracketed by a device synchronisation on both
    sides: per block the wall time per step and the time per launch by HIP events on the launch stream (over the block's
    launches but the first).  Returns the two lists (milliseconds per step), in the order measured."""
    import torch
    spin_up(launch)
    for i in range(warmup):
        launch(i)
    wall, events, n = [], [], 0
    for b in range(blocks):
        # Every timed block starts like the first one: a short run of untimed launches, then the `warmup` launches still in
        # flight when the synchronisation in front of the block is called.  Launches that follow a synchronisation of an
        # ALREADY IDLE device run small kernels about a microsecond slower each for the whole block (measured with blocks of
        # 20 and of 100 launches: 7.3-8.4 against 6.1-6.3 us, 6.1-7.7 against 4.9 us; a stream of launches that never stops
        # gives the lower figures, and so does rocprofv3); with work in flight at the synchronisation they do not.
        if b > 0:
            spin_up(launch, BLOCK_SPINUP_S)
            for i in range(warmup):
                launch(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        # The wall clock covers all `steps` launches.  The event pair covers all but the first: the device is idle when the
        # block starts, so between an event recorded first and the first kernel lies the host's time to issue that launch
        # (10-20 us, which a block of 20 launches would spread over its kernels as a microsecond each).  Recorded behind the
        # first launch, the opening event completes when that kernel ends, and the others follow it back to back.
        if steps > 1:
            launch(n)
            timer.start()
            for i in range(1, steps):
                launch(n + i)
        else:
            timer.start()
            launch(n)
        timer.stop()
        torch.cuda.synchronize()
        wall.append((time.perf_counter() - t0) * 1e3 / steps)
        events.append(timer.elapsed_ms() / max(1, steps - 1))  # (read after the wall clock has stopped)
        n += steps
    return wall, events


def time_launches(timer, launch, steps, warmup, blocks=5):
    """Median over `blocks` timed blocks of `steps` launches each, by HIP events (milliseconds per launch)."""
    _, events = time_blocks(timer, launch, steps, warmup, blocks)
    return percentile(sorted(events), 0.5)


class HostPool:
    """Seeded inputs are generated on the host into one buffer that is reused (the first touch of fresh host memory is
    the slow part of generating them) and copied to the device from there."""

    def __init__(self, oracle):
        import numpy as np
        self.np, self.oracle = np, oracle
        self.buf = np.empty(0, np.uint8)

    def bytes(self, seed, shape):
        """Uniform random bytes (stream `seed` of the oracle's generator): a host array that is valid until the next call."""
        n = int(self.np.prod(shape))
        if self.buf.size < n:
            self.buf = self.np.empty(n, self.np.uint8)
        view = self.buf[:n]
        self.oracle.c.fko_fill_bytes(C.c_uint64(seed), view.ctypes.data_as(C.c_void_p), C.c_size_t(n))
        return view.reshape(shape)

    def device_copies(self, seed, shape, copies, int16=False):
        """`copies` device tensors (distinct allocations) that hold the same seeded bytes."""
        import torch
        nbytes = int(self.np.prod(shape)) * (2 if int16 else 1)
        first = torch.from_numpy(self.bytes(seed, (nbytes,))).cuda()  # a synchronous copy: the pool may be reused after it
        if int16:
            first = first.view(torch.int16)
        first = first.reshape(shape)
        return [first] + [first.clone() for _ in range(copies - 1)]


def sets_for(bytes_per_launch):
    """Buffer sets to rotate so that a launch finds none of its data in the Infinity Cache: the launches between two uses
    of a set move more than 1.5 x the cache (a launch that moves twice the cache by itself needs no second set)."""
    if bytes_per_launch >= 2 * CACHE_BYTES:
        return 1
    return min(MAX_SETS, max(2, int(math.ceil(1.5 * CACHE_BYTES / bytes_per_launch)) + 1))


class Workload:
    def __init__(self, name, launch, out_px, alg_bytes, kernel, sets, verify, note=None):
        self.name, self.launch, self.out_px, self.alg_bytes, self.kernel = name, launch, out_px, alg_bytes, kernel
        self.sets, self.verify, self.note = sets, verify, note
        # what is moved before a buffer set comes round again exceeds the cache, or a single launch already does
        self.cache_resident = alg_bytes < 2 * CACHE_BYTES and sets * alg_bytes < 1.5 * CACHE_BYTES

    def roofline(self, kernel_ms):
        achieved = self.alg_bytes / (kernel_ms * 1e-3)
        traffic, source = measured_traffic(self.name)
        r = {"bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s"}
        # a workload smaller than the cache is served from it however many buffers are rotated: its figure is a rate
        # against the HBM peak, not a fraction of HBM bandwidth in use
        r["frac_peak_cache_resident" if self.cache_resident else "frac"] = achieved / HBM_PEAK
        r.update({"traffic": traffic, "traffic_source": source, "kernel": self.kernel, "alg_bytes_per_launch": self.alg_bytes, "kernel_ms": kernel_ms})
        return r


def measured_traffic(name):
    """(HBM bytes per launch, where it was measured) for a configuration's kernel, from the table in
    profiles/hbm_traffic.md (two rocprofv3 --pmc runs, FETCH_SIZE and WRITE_SIZE, scaled as that file says), or
    (None, None) when the table has no row for it."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.md")
    if os.path.exists(path):
        for line in open(path):
            cells = [c.strip() for c in line.strip().strip("|").split("|")]
            if len(cells) >= 4 and cells[0] == name:
                try:
                    return float(cells[1]) + float(cells[2]), f"profiles/hbm_traffic.md ({cells[3]}): fetch {cells[1]} B + write {cells[2]} B"
                except ValueError:
                    break
    return None, None


def same(a, b):
    return a.shape == b.shape and a.dtype == b.dtype and a.tobytes() == b.tobytes()


def build_workloads(fk, oracle, pool, only=None):
    """The configurations as Workload objects; `only` (a name prefix) limits what is allocated."""
    import numpy as np
    import torch
    from oracle import binding as B
    made = []

    def want(name):
        return only is None or name.startswith(only)

    def add(*a, **k):
        made.append(Workload(*a, **k))

    # ---- C1: the README pipeline (the reference's README example) --------------------------------------------------
    def readme(name, rects, dst, note):
        if not want(name):
            return
        n = len(rects)
        alg = sum(r[2] * r[3] for r in rects) * 3 + n * dst[0] * dst[1] * 12
        k = sets_for(alg)
        frames = pool.device_copies(100, (H4K, W4K, 3), k)
        outs = [torch.empty((n, dst[1], dst[0], 3), device="cuda") for _ in range(k)]
        calls = [fk.crop_resize_muls_bgr_tensor(frames[s], rects, outs[s], *README_ARGS, defer=True) for s in range(k)]

        def verify(last):
            planes = [0, n - 1]
            expect = oracle.crop_resize_muls_bgr_tensor(pool.bytes(100, (H4K, W4K, 3)), [rects[p] for p in planes], dst, *README_ARGS)
            assert same(outs[last % k][planes].cpu().numpy(), expect), name + ": output differs from the oracle"
        add(name, lambda i: calls[i % k](), n * dst[0] * dst[1], alg, "transform_kernel<ResizeJob<uchar3 -> float3, README tail, N = 5>>", k, verify, note)

    readme("C1_readme_60x60x5", [(0, 0, 34, 25), (10, 10, 70, 15), (20, 20, 60, 59), (30, 30, 20, 23), (40, 40, 12, 11)], (60, 60),
           "benchmark configuration 1 at its literal shape: 234 KB moved, bound by launch latency")
    readme(HEADLINE, [(64 * i, 48 * i, 1024, 768) for i in range(5)], (1920, 1080),
           "4:3 crops into a 16:9 target under PRESERVE_AR: a quarter of the output is the bars beside the image")
    readme("C1_nobars_5x1024x576_to_1920x1080", [(64 * i, 48 * i, 1024, 576) for i in range(5)], (1920, 1080),
           "16:9 crops: every output pixel is resampled")

    # ---- S0, S1: fk::setTo on the headline's output tensor and on the literal configuration's: launches that only store ----
    def set_to(name, n, dst, note):
        if not want(name):
            return
        alg = n * dst[0] * dst[1] * 12
        k = sets_for(alg)
        outs = [torch.empty((n, dst[1], dst[0], 3), device="cuda") for _ in range(k)]
        value = (0.25, -1.5, 3.0)
        calls = [fk.set_to_f32c3_tensor(value, outs[s], defer=True) for s in range(k)]

        def verify(last):
            got = outs[last % k].cpu().numpy()
            assert same(got, np.broadcast_to(np.array(value, np.float32), got.shape).copy()), name + ": a fill that is not the value"
        add(name, lambda i: calls[i % k](), n * dst[0] * dst[1], alg, "transform_kernel<GenericJob<ReadSet<float3> -> PerThreadWrite<_3D, float3>>>", k, verify, note)

    set_to("S0_setto_f32c3_60x60x5", 5, (60, 60), "the launch floor of this runtime: 216 KB of stores, nothing read")
    set_to("S1_setto_f32c3_1920x1080x5", 5, (1920, 1080),
           "the store-only ceiling of the headline: the same 124.4 MB tensor written with the same streaming stores, nothing read or computed")

    # ---- C2: vertical fusion, depth 16 (benchmark configuration 2) ----------------------------------------------------
    name = f"C2_vertical_fusion_depth{DEPTH}"
    if want(name):
        alg2 = 2 * N4K * 12
        k2 = sets_for(alg2)
        host2 = oracle.unit_floats(2, (H4K, W4K, 3))
        srcs2 = [torch.from_numpy(host2).cuda() for _ in range(k2)]
        dsts2 = [torch.empty((H4K, W4K, 3), device="cuda") for _ in range(k2)]
        calls2 = [fk.muladd_chain_f32c3(srcs2[s], dsts2[s], DEPTH, MUL_V, ADD_V, defer=True) for s in range(k2)]

        def verify_c2(last):
            assert same(dsts2[last % k2][:4].cpu().numpy(), oracle.muladd_chain_f32c3(host2[:4], DEPTH, MUL_V, ADD_V)), "C2: output differs from the oracle"
        add(name, lambda i: calls2[i % k2](), N4K, alg2, f"transform_kernel<PointwiseJob<float3 -> float3, depth {DEPTH}>>", k2, verify_c2,
            "3840x2160 float3, PerThreadRead -> 16 alternating Mul/Add -> PerThreadWrite in one launch")

    # ---- C3: 50 crops of 50 images -> 224x224x3x50 planar (benchmark configuration 3) ---------------------------------
    if want("C3_batch50_224x224_split"):
        n, w, h = 50, 1920, 1080
        rects3 = []
        for i in range(n):  # crop width and height uniform in [16, 512], origin uniform over the positions that keep it inside
            cw, ch = (int(v) for v in oracle.uniform_ints(103 + i, 16, 512, 2))
            rects3.append((int(oracle.uniform_ints(203 + i, 0, w - cw, 1)[0]), int(oracle.uniform_ints(303 + i, 0, h - ch, 1)[0]), cw, ch))
        alg3 = n * 224 * 224 * 12 + sum(3 * r[2] * r[3] for r in rects3)
        k3 = sets_for(alg3)
        per_image = [pool.device_copies(3 + i, (h, w, 3), k3) for i in range(n)]
        outs3 = [torch.empty((n, 3, 224, 224), device="cuda") for _ in range(k3)]
        a3 = ((255.,) * 3, (.485, .456, .406), (.229, .224, .225))
        calls3 = [fk.batch_crop_resize_norm_split([per_image[i][s] for i in range(n)], rects3, outs3[s], *a3, defer=True) for s in range(k3)]

        def verify_c3(last):
            planes = [0, 17, 49]
            srcs = [pool.bytes(3 + p, (h, w, 3)).copy() for p in planes]
            expect = oracle.batch_crop_resize_norm_split(srcs, [rects3[p] for p in planes], (224, 224), *a3)
            assert same(outs3[last % k3][planes].cpu().numpy(), expect), "C3: output differs from the oracle"
        add("C3_batch50_224x224_split", lambda i: calls3[i % k3](), n * 224 * 224, alg3, "transform_kernel<ResizeJob<uchar3 -> float3 planes, N = 50>>", k3,
            verify_c3, "crops of 16..512 pixels a side at uniform positions inside 50 different 1920x1080 images")

    # ---- C4: resize 4K -> 1280x720, 32 tiles of 128x128 (benchmark configuration 4) -----------------------------------
    if want("C4_resize_crop_32x128x128"):
        rects4 = [(160 * i, 180 * j, 128, 128) for j in range(4) for i in range(8)]
        alg4 = 32 * 383 * 383 * 3 + 32 * 128 * 128 * 12
        k4 = sets_for(alg4)
        host4 = oracle.gradient_noise_u8c3(4, W4K, H4K)  # a smooth gradient plus uniform noise of +-16
        srcs4 = [torch.from_numpy(host4).cuda() for _ in range(k4)]
        outs4 = [torch.empty((32, 128, 128, 3), device="cuda") for _ in range(k4)]
        calls4 = [fk.resize_crop_tiles(srcs4[s], (1280, 720), rects4, outs4[s], (1 / 255.,) * 3, defer=True) for s in range(k4)]

        def verify_c4(last):
            tiles = [0, 31]
            expect = oracle.resize_crop_tiles(host4, (1280, 720), [rects4[t] for t in tiles], (128, 128), (1 / 255.,) * 3)
            assert same(outs4[last % k4][tiles].cpu().numpy(), expect), "C4: output differs from the oracle"
        add("C4_resize_crop_32x128x128", lambda i: calls4[i % k4](), 32 * 128 * 128, alg4, "transform_kernel<ResizeJob<uchar3 -> float3, resize then crop, N = 32>>",
            k4, verify_c4, "the 383x383 source window of each tile counted once")

    # ---- the YUV front-end at 4K -------------------------------------------------------------------------------------
    def first_rows(raw, rows):  # the raw image of the first `rows` lines of a 4:2:0 frame: their luma rows, then their chroma rows
        return np.ascontiguousarray(np.concatenate([raw[:rows], raw[H4K:H4K + rows // 2]]))

    def yuv_full(name, fmt, prim, raw_shape, int16, out_cn, out_dtype, alg, kernel, o_fmt, alpha, float_out, planar420):
        if not want(name):
            return
        k = sets_for(alg)
        raws = pool.device_copies(400, raw_shape, k, int16=int16)
        outs = [torch.empty((H4K, W4K, out_cn), dtype=out_dtype, device="cuda") for _ in range(k)]
        calls = [fk.yuv_to_rgb(fmt, fk.RANGE_FULL, prim[0], raws[s], outs[s], defer=True) for s in range(k)]

        def verify(last):
            host = pool.bytes(400, (raw_shape[0], raw_shape[1] * (2 if int16 else 1)))
            host = host.view(np.uint16) if int16 else host
            raw = first_rows(host, 8) if planar420 else np.ascontiguousarray(host[:8])
            got = outs[last % k][:8].cpu().numpy()
            expect = oracle.yuv_to_rgb(o_fmt, B.RANGE_FULL, prim[1], alpha, float_out, raw, W4K, 8)
            assert same(got.view(expect.dtype), expect), name + ": output differs from the oracle"
        add(name, lambda i: calls[i % k](), N4K, alg, kernel, k, verify)

    yuv_full("Y1_nv12_4k_to_rgb_u8c3", fk.NV12, (fk.BT709, B.BT709), (H4K * 3 // 2, W4K), False, 3, torch.uint8, N4K * 3 // 2 + N4K * 3,
             "transform_kernel<PointwiseJob<NV12 -> uchar3>>", B.NV12, False, False, True)
    yuv_full("Y2_p010_4k_to_rgba_u16c4", fk.P010, (fk.BT2020, B.BT2020), (H4K * 3 // 2, W4K), True, 4, torch.int16, N4K * 3 + N4K * 8,
             "transform_kernel<PointwiseJob<P010 -> ushort4>>", B.P010, True, False, True)
    yuv_full("Y3_uyvy_4k_to_rgb_f32c3", fk.UYVY, (fk.BT601, B.BT601), (H4K, 2 * W4K), False, 3, torch.float32, N4K * 2 + N4K * 12,
             "transform_kernel<PointwiseJob<UYVY -> float3>>", B.UYVY, False, True, False)

    def yuv_resize(name, crop, dst, note=None):
        if not want(name):
            return
        alg = crop[2] * crop[3] * 3 // 2 + dst[0] * dst[1] * 12
        k = sets_for(alg)
        raws = pool.device_copies(460, (H4K * 3 // 2, W4K), k)
        outs = [torch.empty((3, dst[1], dst[0]), device="cuda") for _ in range(k)]
        calls = [fk.yuv_crop_resize_norm_split(fk.NV12, fk.RANGE_FULL, fk.BT709, raws[s], (W4K, H4K), crop, outs[s], 255.0, defer=True) for s in range(k)]

        def verify(last):
            expect = oracle.yuv_crop_resize_norm_split(B.NV12, B.RANGE_FULL, B.BT709, pool.bytes(460, (H4K * 3 // 2, W4K)), W4K, H4K, crop, dst, 255.0)
            assert same(outs[last % k].cpu().numpy(), expect), name + ": output differs from the oracle"
        add(name, lambda i: calls[i % k](), dst[0] * dst[1], alg, "transform_kernel<ResizeJob<NV12 -> RGB -> float3 planes>>", k, verify, note)

    yuv_resize("Y4_nv12_crop1920x1080_to_1280x720_split", (960, 540, 1920, 1080), (1280, 720),
               "the README's backwards-vertical-fusion example: only the crop's YUV samples are read")
    yuv_resize("Y5_nv12_crop640x360_to_1920x1080_split", (1600, 900, 640, 360), (1920, 1080))

    # ---- border and warp chains over the 4K uchar3 frame -------------------------------------------------------------
    if want("B1_reflect101_border64_4k_u8c3"):
        alg_b = N4K * 3 + 3968 * 2288 * 3
        kb = sets_for(alg_b)
        srcs_b = pool.device_copies(500, (H4K, W4K, 3), kb)
        outs_b = [torch.empty((H4K + 128, W4K + 128, 3), dtype=torch.uint8, device="cuda") for _ in range(kb)]
        calls_b = [fk.border_crop_u8c3(fk.BORDER_REFLECT_101, srcs_b[s], 64, 64, outs_b[s], defer=True) for s in range(kb)]

        def verify_b1(last):
            expect = oracle.border_crop_u8c3(B.BORDER_REFLECT_101, pool.bytes(500, (H4K, W4K, 3)), 64, 64, (W4K + 128, 80))
            assert same(outs_b[last % kb][:80].cpu().numpy(), expect), "B1: output differs from the oracle"
        add("B1_reflect101_border64_4k_u8c3", lambda i: calls_b[i % kb](), 3968 * 2288, alg_b, "transform_kernel<GenericJob<BorderReader<REFLECT_101> -> uchar3>>",
            kb, verify_b1)

    def warp(name, kind, o_kind, matrix, dst, alg, note):
        if not want(name):
            return
        k = sets_for(alg)
        srcs = pool.device_copies(520, (H4K, W4K, 3), k)
        outs = [torch.empty((dst[1], dst[0], 3), device="cuda") for _ in range(k)]
        calls = [fk.warp_u8c3_f32c3(kind, matrix, srcs[s], outs[s], defer=True) for s in range(k)]

        def verify(last):
            expect = oracle.warp_u8c3_f32c3(o_kind, matrix, pool.bytes(520, (H4K, W4K, 3)), (dst[0], 16))
            assert same(outs[last % k][:16].cpu().numpy(), expect), name + ": output differs from the oracle"
        add(name, lambda i: calls[i % k](), dst[0] * dst[1], alg, "transform_kernel<GenericJob<Warping -> float3>>", k, verify, note)

    c5, s5 = math.cos(math.radians(5.0)), math.sin(math.radians(5.0))
    warp("W1_affine_rot5deg_4k_to_4k_f32c3", fk.WARP_AFFINE, B.WARP_AFFINE, [[c5, -s5, 1920 - c5 * 1920 + s5 * 1080], [s5, c5, 1080 - s5 * 1920 - c5 * 1080]],
         (W4K, H4K), N4K * 3 + N4K * 12, "a rotation of 5 degrees about the centre; source bytes counted once for the whole frame")
    warp("W2_perspective_4k_to_1920x1080_f32c3", fk.WARP_PERSPECTIVE, B.WARP_PERSPECTIVE, [[2.0, 0.1, 0.0], [0.05, 2.0, 0.0], [2e-5, 1e-5, 1.0]], (1920, 1080),
         1920 * 1080 * 4 * 3 + 1920 * 1080 * 12, "four taps per output pixel, 2x down-scaling: no tap is shared")

    # ---- R1: one update of a ring of eight 1080p frames kept as normalised float planes ------------------------------
    if want("R1_circular_tensor_update_8x1080p"):
        batch, hh, ww = 8, 1080, 1920
        px = hh * ww
        alg_r = px * 3 + px * 12 * 2 + (batch - 1) * px * 12 * 2
        kr = sets_for(alg_r)
        frame_host = pool.bytes(540, (hh, ww, 3)).copy()
        frame = torch.from_numpy(frame_host).cuda()
        tensors = [torch.zeros((batch, 3, hh, ww), device="cuda") for _ in range(kr)]
        rings = [torch.zeros((batch, 3, hh, ww), device="cuda") for _ in range(kr)]
        calls_r = [[fk.circular_tensor_update_u8c3_split_f32(frame, 1 / 255., tensors[s], rings[s], j, 1, defer=True) for j in range(batch)] for s in range(kr)]

        def verify_r1(last):  # newest-first order: plane 0 holds the frame of the last update, through the chain
            expect = np.ascontiguousarray(frame_host.astype(np.float32).transpose(2, 0, 1) * np.float32(1 / 255.))
            assert same(tensors[last % kr][0].cpu().numpy(), expect), "R1: the newest plane differs from the frame through the chain"
        add("R1_circular_tensor_update_8x1080p", lambda i: calls_r[i % kr][(i // kr) % batch](), batch * px, alg_r, "divergent_kernel<new frame, seven planes re-ordered>",
            kr, verify_r1, "frame read + its planes written to tensor and ring + seven planes copied from the ring")

    # ---- K1: a CONDITIONAL_WITH_DEFAULT batch: eight 1080p frames, five in use, resized to 1280x720 ------------------
    if want("K1_conditional_resize_8x1080p_5used"):
        n, used, dst = 8, 5, (1280, 720)
        alg_k = used * 1920 * 1080 * 3 + n * dst[0] * dst[1] * 12
        kk = sets_for(alg_k)
        default = (0.5, 0.25, 0.125)
        per_frame = [pool.device_copies(560 + i, (1080, 1920, 3), kk) for i in range(used)]
        outs_k = [torch.empty((n, dst[1], dst[0], 3), device="cuda") for _ in range(kk)]
        calls_k = [fk.conditional_resize_f32c3([per_frame[i % used][s] for i in range(n)], used, default, outs_k[s], defer=True) for s in range(kk)]

        def verify_k1(last):
            srcs = [pool.bytes(560 + i, (1080, 1920, 3)).copy() for i in (0, 4)]
            expect = oracle.conditional_resize_f32c3(srcs + srcs[:1], 2, default, dst)  # planes 0 and 1 resized, plane 2 the default
            got = outs_k[last % kk].cpu().numpy()
            assert same(got[0], expect[0]) and same(got[4], expect[1]) and same(got[5], expect[2]) and same(got[7], expect[2]), "K1: output differs from the oracle"
        add("K1_conditional_resize_8x1080p_5used", lambda i: calls_k[i % kk](), n * dst[0] * dst[1], alg_k,
            "transform_kernel<ResizeJob<uchar3 -> float3, CONDITIONAL_WITH_DEFAULT, N = 8>>", kk, verify_k1,
            "five planes are resized, three receive the default value")

    # ---- C5: four chains over one 8192x8192 uchar4 image in one launch (benchmark configuration 5) --------------------
    if want("C5_divergent4_8192x8192"):
        big = pool.device_copies(5, (8192, 8192, 4), 1)[0]
        gray = torch.empty((8192, 8192), dtype=torch.uint8, device="cuda")
        small = torch.empty((512, 512, 4), device="cuda")
        crop = torch.empty((1024, 1024, 4), dtype=torch.uint8, device="cuda")
        bgr = torch.empty((8192, 8192, 3), device="cuda")
        rect5 = (3584, 3584, 1024, 1024)
        call5 = fk.divergent4_u8c4(big, gray, small, 1 / 255., rect5, 2, crop, 0.5, bgr, defer=True)

        def verify_c5(last):
            src = pool.bytes(5, (8192, 8192, 4))
            assert same(small.cpu().numpy(), oracle.resize_mul_u8c4_f32c4(src, (512, 512), 1 / 255.)), "C5: the resized chain differs from the oracle"
            assert same(crop.cpu().numpy(), oracle.crop_mul_saturate_u8c4(src, rect5, 2)), "C5: the crop chain differs from the oracle"
            rows = np.ascontiguousarray(src[:16])
            assert same(gray[:16].cpu().numpy(), oracle.rgba2gray_u8c4(rows)), "C5: the gray chain differs from the oracle"
            assert same(bgr[:16].cpu().numpy(), oracle.rgba2bgr_sub_u8c4_f32c3(rows, 0.5)), "C5: the BGR chain differs from the oracle"
        add("C5_divergent4_8192x8192", lambda i: call5(), 8192 * 8192 * 2 + 512 * 512 + 1024 * 1024, 1426063360, "divergent_kernel<gray, resize, crop, BGR>", 1,
            verify_c5, "1.43 GB per launch, five times the Infinity Cache; 1,157,627,904 B if chains a and d share the source through cache")
    return made


def cpu_baseline(binding, budget_s=10.0):
    """The reference's own CPU executor (oracle/_ref: its headers compiled as they are; the C restatement when that build
    is absent) on a bounded sample of the headline workload: one of its five planes (a 1024x768 crop of the 4K frame ->
    1920x1080 through the whole chain), repeated for about `budget_s` seconds on one core."""
    ref = binding.reference()
    lib, kind = (ref, "reference") if ref is not None else (binding.oracle(), "port")
    src = binding.oracle().bytes(100, (H4K, W4K, 3))
    rect, dst = [(0, 0, 1024, 768)], (1920, 1080)
    lib.crop_resize_muls_bgr_tensor(src, [(0, 0, 64, 48)], (120, 68), *README_ARGS)  # warm-up
    passes, t0 = 0, time.perf_counter()
    while True:
        lib.crop_resize_muls_bgr_tensor(src, rect, dst, *README_ARGS)
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or passes >= 1000:
            break
    return {"value": dst[0] * dst[1] * passes / dt / 1e9, "unit": "Gpixel/s", "cores": 1, "kind": kind,
            "sample": f"{passes} passes over one of the workload's five planes (1024x768 crop -> 1920x1080 float3, whole chain) in {dt:.1f} s, serial z/y/x loop",
            "ms_per_plane": 1e3 * dt / passes, "host_cores_available": os.cpu_count()}


def depth_sweep(fk, oracle, timer, steps):
    """benchmark configuration 2: the fused chain at each depth against the same operations as separate launches.
    From 32 operations on, the vector units (no FMA contraction, by design) are busy for more than half of the launch and
    lengthen it: the entry then says that they bound it, and every entry carries the fraction of the vector peak beside
    the HBM figure."""
    import torch
    host = oracle.unit_floats(2, (H4K, W4K, 3))
    sets = 3
    srcs = [torch.from_numpy(host).cuda() for _ in range(sets)]
    dsts = [torch.empty((H4K, W4K, 3), device="cuda") for _ in range(sets)]
    alg_bytes = 2 * N4K * 12
    sweep = {}
    k = max(10, steps // 4)
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
        hbm_frac = alg_bytes / (fused * 1e-3) / HBM_PEAK
        valu_frac = N4K * 3 * depth / (fused * 1e-3) / VALU_PEAK  # one lane operation per channel per Mul or Add
        sweep[str(depth)] = {"fused_ms": fused, "unfused_ms": unf, "speedup_vs_unfused": unf / fused, "fused_gb_s": alg_bytes / fused / 1e6,
                             "bound": "valu" if valu_frac >= 0.5 else "hbm", "frac_hbm_peak": hbm_frac, "frac_valu_peak_no_fma": valu_frac}
    return sweep


def main():
    global SPINUP_S
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--blocks", type=int, default=30,
                    help="timed blocks of --steps launches each for the headline (the median block is reported); the other "
                         "configurations take a third of them")
    ap.add_argument("--spinup-s", type=float, default=SPINUP_S,
                    help="seconds of untimed launches of each workload before its warm-up steps (shorter for traces)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sweep", action="store_true", help="skip the depth sweep and the other configurations")
    ap.add_argument("--no-verify", action="store_true", help="skip the oracle checks of the outputs (for profiler runs)")
    ap.add_argument("--only-config", default=None,
                    help="run only the configurations whose name starts with this (C1_readme, C1_scaled, C1_nobars, C2, C3, C4, C5, "
                         "Y1..Y5, B1, W1, W2, R1, K1) and print their figures: for rocprofv3 runs on one kernel")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="with --only-config: first run ten plain device copies of a 99,532,800-byte tensor (torch's copy kernel), so "
                         "that a counter run holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    SPINUP_S = args.spinup_s
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (planes/row bands would shard with no "
                 "exchange); run with --gpus 1")

    import torch
    import fusedkernellibrary_amd as fk
    from oracle import binding

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    rt, _ = fk.load()
    timer = StreamTimer(rt, torch.cuda.current_stream().cuda_stream)
    oracle = binding.oracle()
    pool = HostPool(oracle)

    def run(w):
        # (blocks of at least 100 launches for these: the first launches after a synchronisation find the device idle, and
        # over a block of 20 launches of a few microseconds each that start-up is a quarter of what is measured)
        big = w.alg_bytes > 1e9
        steps, warmup = (max(3, args.steps // 4), max(1, args.warmup // 4)) if big else (max(100, args.steps), args.warmup)
        blocks = max(1, args.blocks // 6) if big else max(1, args.blocks // 3)
        _, events = time_blocks(timer, w.launch, steps, warmup, blocks)
        events.sort()
        ms = percentile(events, 0.5)
        checked = not args.no_verify
        if checked:
            w.verify(blocks * steps - 1)
        res = {"ms": ms, "ms_p10": percentile(events, 0.1), "ms_p90": percentile(events, 0.9), "timed_blocks": blocks, "steps_per_block": steps,
               "gpixel_s": w.out_px / ms / 1e6, "buffer_sets": w.sets, "checked_against_oracle": checked, "roofline": w.roofline(ms)}
        if w.note:
            res["note"] = w.note
        return res

    if args.only_config is not None:
        if args.copy_calibration:
            a, b = torch.zeros((H4K, W4K, 3), device="cuda"), torch.empty((H4K, W4K, 3), device="cuda")
            for _ in range(10):
                b.copy_(a)
            torch.cuda.synchronize()
            del a, b
        print(json.dumps({w.name: run(w) for w in build_workloads(fk, oracle, pool, only=args.only_config)}))
        return

    # ---- headline: the README pipeline, bandwidth-sized; exactly `steps` launches, device-synchronised on both sides ----
    # `blocks` blocks of exactly `steps` launches, each with a device synchronisation on both sides; the figures are those of
    # the median block (one block of 20 launches is half a millisecond: a single sample of it says little)
    head = build_workloads(fk, oracle, pool, only=HEADLINE)[0]
    blocks = max(1, args.blocks)
    wall, events = time_blocks(timer, head.launch, args.steps, args.warmup, blocks)
    wall.sort()
    events.sort()
    wall_ms, kernel_ms = percentile(wall, 0.5), percentile(events, 0.5)
    if not args.no_verify:
        head.verify(blocks * args.steps - 1)  # the result of the last timed step is the real chain: two of its planes against the oracle

    out = {
        "metric": "fused pipeline Gpixel/s + achieved HBM GB/s (% of peak) on 1 MI355X",
        "value": head.out_px / wall_ms / 1e6, "unit": "Gpixel/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "spinup_s": SPINUP_S, "timed_blocks": blocks, "ms_per_step": wall_ms, "ms_per_step_p10": percentile(wall, 0.1),
        "ms_per_step_p90": percentile(wall, 0.9), "kernel_ms_p10": percentile(events, 0.1), "kernel_ms_p50": kernel_ms,
        "kernel_ms_p90": percentile(events, 0.9), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "README pipeline, bandwidth-sized: five 1024x768 crops of a 3840x2160 uchar3 frame -> Resize<INTER_LINEAR, PRESERVE_AR> to "
                               "1920x1080 -> x1.4 -> -0.5 -> /255 -> RGB2BGR -> float3 tensor 1920x1080x5, one fused launch per step, "
                               f"{head.sets} rotating sets of source frame and output tensor (seeded uniform bytes)"},
        "roofline": head.roofline(kernel_ms),
    }
    del head
    torch.cuda.empty_cache()

    if not args.no_sweep:
        # the other chains first: the deep end of the sweep below keeps the vector units saturated for seconds, and a
        # launch measured right after it runs at the clock the device has dropped to by then
        others = {}
        for name in CONFIG_NAMES:  # one at a time: a configuration's buffers are freed before the next one's are made
            if name == HEADLINE:
                continue
            for w in build_workloads(fk, oracle, pool, only=name):
                others[w.name] = run(w)
            torch.cuda.empty_cache()
        out["other_configs"] = others
        out["depth_sweep"] = depth_sweep(fk, oracle, timer, args.steps)

    out["cpu_baseline"] = None if args.no_cpu else cpu_baseline(binding)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
