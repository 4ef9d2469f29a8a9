"""ctypes bindings of the checker libraries (TEST INFRASTRUCTURE ONLY).

`oracle()` loads oracle/libfkoracle.so, the plain-C restatement of the reference's CPU executor
(fk_oracle.c); `reference()` loads oracle/_ref/libfkref.so, the reference's own headers compiled for
its CPU backend (ref_driver.cpp, plus ref_driver_yuv.cpp and ref_driver_border_warp.cpp in libraries of their own), or returns None when that build is absent.  Both are built by
oracle/Makefile.  Only tests, the smoke check and the CPU-baseline leg of the benchmark import this
module; the shipped library never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

PRESERVE_AR, IGNORE_AR, PRESERVE_AR_RN_EVEN, PRESERVE_AR_LEFT = 0, 1, 2, 3
# PixelFormat / ColorRange / ColorPrimitives values of the reference's raw_image.h
NV12, NV21, P010, P210, Y210, UYVY = 0, 1, 3, 6, 8, 10
YUV_FORMATS = {"NV12": NV12, "NV21": NV21, "P010": P010, "P210": P210, "Y210": Y210, "UYVY": UYVY}
RANGE_LIMITED, RANGE_FULL = 0, 1
BT601, BT709, BT2020 = 0, 1, 2
# the (range, primaries) pairs for which the reference defines a YCbCr -> RGB matrix
BORDER_CONSTANT, BORDER_REPLICATE, BORDER_REFLECT, BORDER_WRAP, BORDER_REFLECT_101 = 0, 1, 2, 3, 4
BORDER_TYPES = {"CONSTANT": 0, "REPLICATE": 1, "REFLECT": 2, "WRAP": 3, "REFLECT_101": 4}
WARP_AFFINE, WARP_PERSPECTIVE = 0, 1
DEINTERLACE_BLEND, DEINTERLACE_INTER_LINEAR = 0, 1
PACKED_TO_SPLIT, PACKED_TO_TRANSPOSED, SPLIT_TO_PACKED, TRANSPOSED_TO_PACKED = 0, 1, 2, 3
ASCENDENT, DESCENDENT = 0, 1
YUV_MATRICES = [(RANGE_FULL, BT601), (RANGE_FULL, BT709), (RANGE_LIMITED, BT709), (RANGE_FULL, BT2020)]


class Rect(C.Structure):
    _fields_ = [("x", C.c_int), ("y", C.c_int), ("width", C.c_int), ("height", C.c_int)]


class ResizeParams(C.Structure):
    _fields_ = [("dst_w", C.c_int), ("dst_h", C.c_int), ("fx", C.c_float), ("fy", C.c_float),
                ("src_w", C.c_int), ("src_h", C.c_int), ("x1", C.c_int), ("y1", C.c_int),
                ("x2", C.c_int), ("y2", C.c_int)]


def rect_array(rects):
    arr = (Rect * len(rects))()
    for i, r in enumerate(rects):
        arr[i] = Rect(*[int(v) for v in r])
    return arr


def _f3(v):
    return (C.c_float * 3)(*[float(x) for x in v])


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


_u8p, _f32p, _sz, _i, _f = C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_float
_f3p = C.POINTER(C.c_float)
_rp = C.POINTER(Rect)

_CHAIN_SIGS = {
    # name: (argtypes for the oracle; the reference driver has the same minus the quirk flag)
    "crop_resize_muls_bgr_tensor": [_u8p, _i, _i, _sz, _rp, _i, _i, _i, _i, _f3p, _f3p, _f3p, _f3p, _i, _f32p],
    "muladd_chain_f32c3": [_f32p, _i, _i, _sz, _i, _f, _f, _f32p, _sz],
    "single_op_f32c3": [_f32p, _i, _i, _sz, _i, _f, _f32p, _sz],
    "batch_crop_resize_norm_split": [C.POINTER(C.c_void_p), _i, _i, _sz, _rp, _i, _i, _i, _f3p, _f3p, _f3p, _i, _f32p],
    "resize_crop_tiles": [_u8p, _i, _i, _sz, _i, _i, _rp, _i, _i, _i, _f3p, _i, _f32p],
    "rgba2gray_u8c4": [_u8p, _i, _i, _sz, _u8p, _sz],
    "resize_mul_u8c4_f32c4": [_u8p, _i, _i, _sz, _i, _i, _f, _i, _f32p, _sz],
    "crop_mul_saturate_u8c4": [_u8p, _i, _i, _sz, Rect, _i, _u8p, _sz],
    "rgba2bgr_sub_u8c4_f32c3": [_u8p, _i, _i, _sz, _f, _f32p, _sz],
    "batch_crop_cast_tensor": [_u8p, _i, _i, _sz, _rp, _i, _i, _i, _i, _f32p],
}
# position of the quirk / exec_all flag that the reference driver's signature does not have
_ORACLE_ONLY_ARG = {
    "crop_resize_muls_bgr_tensor": 13, "batch_crop_resize_norm_split": 11, "resize_crop_tiles": 11,
    "resize_mul_u8c4_f32c4": 7, "batch_crop_cast_tensor": 8,
}


def build(with_reference=True):
    """(Re)build the checker libraries with oracle/Makefile."""
    target = "all" if with_reference else "libfkoracle.so"
    subprocess.run(["make", "-C", _HERE, target], check=True, stdout=subprocess.DEVNULL)


class _Lib:
    """Thin numpy-facing wrapper; `ref=True` talks to the reference driver (literal host semantics)."""

    def __init__(self, cdll, ref, yuv_cdll=None, bw_cdll=None, circ_cdll=None, paths_cdll=None):
        self.c = cdll
        self.ref = ref
        self.yuv = yuv_cdll
        self.bw = bw_cdll
        self.circ = circ_cdll
        self.paths = paths_cdll
        pre = "fkr_" if ref else "fko_"
        if circ_cdll is not None:
            _v = C.c_void_p
            fn = getattr(circ_cdll, pre + "tensor_relayout_f32c3")
            fn.argtypes, fn.restype = [_i, _v, _i, _i, _i, _v], C.c_int
            fn = getattr(circ_cdll, pre + "circular_tensor_read_f32c3")
            fn.argtypes, fn.restype = [_i, _i, _v, _i, _i, _i, _v], C.c_int
            if not ref:
                fn = circ_cdll.fko_circular_tensor_update_u8c3_split_f32
                fn.argtypes, fn.restype = [_v, _i, _i, _sz, _f, _v, _v, _i, _i, _i], C.c_int
        if bw_cdll is not None:
            _v = C.c_void_p
            fn = getattr(bw_cdll, pre + "border_crop_u8c3")
            fn.argtypes, fn.restype = [_i, _v, _i, _i, _sz, _i, _i, _i, _i, _v, _v, _sz], C.c_int
            fn = getattr(bw_cdll, pre + "warp_coords")
            fn.argtypes, fn.restype = [_i, _v, _i, _i, _v], None
            fn = getattr(bw_cdll, pre + "deinterlace_u8c3_f32c3")
            fn.argtypes, fn.restype = [_i, _i, _v, _i, _i, _sz, _v, _sz], C.c_int
            fn = getattr(bw_cdll, pre + "warp_u8c3_f32c3")
            fn.argtypes, fn.restype = [_i, _v, _v, _i, _i, _sz, _i, _i] + ([] if ref else [_i]) + [_v, _sz], C.c_int
            if not ref:
                bw_cdll.fko_border_index.argtypes, bw_cdll.fko_border_index.restype = [_i, _i, _i], C.c_int
        if yuv_cdll is not None:
            _v = C.c_void_p
            for name, sig in {"read_yuv": [_i, _v, _sz, _i, _i, _v, _sz], "write_yuv": [_i, _v, _sz, _i, _i, _v, _sz],
                              "yuv_to_rgb": [_i, _i, _i, _i, _i, _v, _sz, _i, _i, _v, _sz],
                              "yuv_crop_resize_norm_split": [_i, _i, _i, _v, _sz, _i, _i, Rect, _i, _i, _f] +
                                                            ([] if ref else [_i]) + [_v]}.items():
                fn = getattr(yuv_cdll, pre + name)
                fn.argtypes = sig
                fn.restype = C.c_int
        for name, sig in _CHAIN_SIGS.items():
            fn = getattr(cdll, pre + name)
            sig = list(sig)
            if ref and name in _ORACLE_ONLY_ARG:
                del sig[_ORACLE_ONLY_ARG[name]]
            fn.argtypes = sig
            fn.restype = C.c_int if ref else None
        if ref:
            cdll.fkr_cxp_round.argtypes = [_f]
            cdll.fkr_cxp_round.restype = _f
            cdll.fkr_saturate_float_to_u8.argtypes = [_f]
            cdll.fkr_saturate_float_to_u8.restype = C.c_uint8
            cdll.fkr_saturate_int_to_u8.argtypes = [_i]
            cdll.fkr_saturate_int_to_u8.restype = C.c_uint8
            cdll.fkr_rgb2gray_u8.argtypes = [C.c_uint8] * 3
            cdll.fkr_rgb2gray_u8.restype = C.c_uint8
        else:
            cdll.fko_fill_bytes.argtypes = [C.c_uint64, C.c_void_p, _sz]
            cdll.fko_fill_unit_floats.argtypes = [C.c_uint64, C.c_void_p, _sz]
            cdll.fko_fill_uniform_ints.argtypes = [C.c_uint64, _i, _i, C.c_void_p, _sz]
            cdll.fko_fill_gradient_noise_u8c3.argtypes = [C.c_uint64, C.c_void_p, _i, _i]
            cdll.fko_fnv1a64.argtypes = [C.c_void_p, _sz]
            cdll.fko_fnv1a64.restype = C.c_uint64
            cdll.fko_round.argtypes = [_f]
            cdll.fko_round.restype = _f
            cdll.fko_resize_build.argtypes = [_i, _i, _i, _i, _i, C.POINTER(ResizeParams)]
            cdll.fko_bilinear_u8.argtypes = [_u8p, _sz, _i, _i, _i, _i, _i, _f, _f, _i, _f32p]
            cdll.fko_saturate_int_to_u8.argtypes = [_i]
            cdll.fko_saturate_int_to_u8.restype = C.c_uint8
            cdll.fko_saturate_float_to_u8.argtypes = [_f]
            cdll.fko_saturate_float_to_u8.restype = C.c_uint8
            cdll.fko_rgb2gray_u8.argtypes = [C.c_uint8] * 3
            cdll.fko_rgb2gray_u8.restype = C.c_uint8

    def _call(self, name, args):
        args = list(args)
        if self.ref and name in _ORACLE_ONLY_ARG:
            del args[_ORACLE_ONLY_ARG[name]]
        rc = getattr(self.c, ("fkr_" if self.ref else "fko_") + name)(*args)
        if self.ref and rc != 0:
            raise ValueError("reference driver has no instantiation for this batch size / depth")

    # ---- generators (oracle library only) ----
    def bytes(self, seed, shape):
        out = np.empty(shape, np.uint8)
        self.c.fko_fill_bytes(seed, _p(out), out.size)
        return out

    def unit_floats(self, seed, shape):
        out = np.empty(shape, np.float32)
        self.c.fko_fill_unit_floats(seed, _p(out), out.size)
        return out

    def uniform_ints(self, seed, lo, hi, n):
        out = np.empty(n, np.int32)
        self.c.fko_fill_uniform_ints(seed, lo, hi, _p(out), n)
        return out

    def gradient_noise_u8c3(self, seed, w, h):
        out = np.empty((h, w, 3), np.uint8)
        self.c.fko_fill_gradient_noise_u8c3(seed, _p(out), w, h)
        return out

    def fnv1a64(self, a):
        a = np.ascontiguousarray(a)
        return int(self.c.fko_fnv1a64(_p(a), a.nbytes))

    def resize_build(self, aspect, src_w, src_h, dst_w, dst_h):
        p = ResizeParams()
        self.c.fko_resize_build(aspect, src_w, src_h, dst_w, dst_h, C.byref(p))
        return p

    def bilinear_u8(self, img, org, src_size, sx, sy, quirk=0):
        h, w, cn = img.shape
        out = np.empty(cn, np.float32)
        self.c.fko_bilinear_u8(_p(img), img.strides[0], cn, org[0], org[1], src_size[0], src_size[1],
                               float(sx), float(sy), quirk, _p(out))
        return out

    # ---- chains: images are (h, w, c) arrays whose row stride is the pitch ----
    def crop_resize_muls_bgr_tensor(self, src, rects, dst, aspect, background, mul, sub, div, quirk=0):
        h, w, _ = src.shape
        out = np.empty((len(rects), dst[1], dst[0], 3), np.float32)
        self._call("crop_resize_muls_bgr_tensor",
                   [_p(src), w, h, src.strides[0], rect_array(rects), len(rects), dst[0], dst[1], aspect,
                    _f3(background), _f3(mul), _f3(sub), _f3(div), quirk, _p(out)])
        return out

    def muladd_chain_f32c3(self, src, depth, mul_v, add_v):
        h, w, _ = src.shape
        out = np.empty((h, w, 3), np.float32)
        self._call("muladd_chain_f32c3", [_p(src), w, h, src.strides[0], depth, mul_v, add_v, _p(out), out.strides[0]])
        return out

    def single_op_f32c3(self, src, is_add, v):
        h, w, _ = src.shape
        out = np.empty((h, w, 3), np.float32)
        self._call("single_op_f32c3", [_p(src), w, h, src.strides[0], int(is_add), v, _p(out), out.strides[0]])
        return out

    def batch_crop_resize_norm_split(self, srcs, rects, dst, div1, sub, div2, quirk=0):
        n = len(srcs)
        h, w, _ = srcs[0].shape
        ptrs = (C.c_void_p * n)(*[s.ctypes.data for s in srcs])
        out = np.empty((n, 3, dst[1], dst[0]), np.float32)
        self._call("batch_crop_resize_norm_split",
                   [ptrs, w, h, srcs[0].strides[0], rect_array(rects), n, dst[0], dst[1], _f3(div1), _f3(sub),
                    _f3(div2), quirk, _p(out)])
        return out

    def resize_crop_tiles(self, src, resized, rects, tile, mul, quirk=0):
        h, w, _ = src.shape
        out = np.empty((len(rects), tile[1], tile[0], 3), np.float32)
        self._call("resize_crop_tiles",
                   [_p(src), w, h, src.strides[0], resized[0], resized[1], rect_array(rects), len(rects), tile[0],
                    tile[1], _f3(mul), quirk, _p(out)])
        return out

    def rgba2gray_u8c4(self, src):
        h, w, _ = src.shape
        out = np.empty((h, w), np.uint8)
        self._call("rgba2gray_u8c4", [_p(src), w, h, src.strides[0], _p(out), out.strides[0]])
        return out

    def resize_mul_u8c4_f32c4(self, src, dst, mul_v, quirk=0):
        h, w, _ = src.shape
        out = np.empty((dst[1], dst[0], 4), np.float32)
        self._call("resize_mul_u8c4_f32c4", [_p(src), w, h, src.strides[0], dst[0], dst[1], mul_v, quirk, _p(out), out.strides[0]])
        return out

    def crop_mul_saturate_u8c4(self, src, rect, mul_v):
        h, w, _ = src.shape
        out = np.empty((rect[3], rect[2], 4), np.uint8)
        self._call("crop_mul_saturate_u8c4", [_p(src), w, h, src.strides[0], Rect(*rect), mul_v, _p(out), out.strides[0]])
        return out

    def rgba2bgr_sub_u8c4_f32c3(self, src, sub_v):
        h, w, _ = src.shape
        out = np.empty((h, w, 3), np.float32)
        self._call("rgba2bgr_sub_u8c4_f32c3", [_p(src), w, h, src.strides[0], sub_v, _p(out), out.strides[0]])
        return out

    def batch_crop_cast_tensor(self, src, rects, max_size, exec_all=1, fill=None):
        h, w, _ = src.shape
        out = np.empty((len(rects), max_size[1], max_size[0], 3), np.float32)
        if fill is not None:
            out[...] = fill
        self._call("batch_crop_cast_tensor",
                   [_p(src), w, h, src.strides[0], rect_array(rects), len(rects), max_size[0], max_size[1],
                    exec_all, _p(out)])
        return out


    # ---- YUV front-end: `raw` is the (data_h, data_w) buffer of base elements, row stride = pitch ----
    @staticmethod
    def yuv_data_shape(fmt, w, h):
        """(rows, columns, dtype) of the buffer that holds a w x h image of this format."""
        wf, hf, dt = {NV12: (1, 1.5, np.uint8), NV21: (1, 1.5, np.uint8), P010: (1, 1.5, np.uint16),
                      P210: (1, 2, np.uint16), Y210: (2, 1, np.uint16), UYVY: (2, 1, np.uint8)}[fmt]
        return int(h * hf), int(w * wf), dt

    def _yuv_fn(self, name):
        if self.yuv is None:
            raise RuntimeError("the YUV checker library is not built")
        return getattr(self.yuv, ("fkr_" if self.ref else "fko_") + name)

    @staticmethod
    def _check(rc):
        if rc != 0:
            raise ValueError("format or matrix not defined by the reference")

    def read_yuv(self, fmt, raw, w, h):
        out = np.empty((h, w, 3), raw.dtype)
        self._check(self._yuv_fn("read_yuv")(fmt, _p(raw), raw.strides[0], w, h, _p(out), out.strides[0]))
        return out

    def write_yuv(self, fmt, pixels, fill=0):
        h, w, _ = pixels.shape
        rows, cols, dt = self.yuv_data_shape(fmt, w, h)
        raw = np.full((rows, cols), fill, dt)
        self._check(self._yuv_fn("write_yuv")(fmt, _p(pixels), pixels.strides[0], w, h, _p(raw), raw.strides[0]))
        return raw

    def yuv_to_rgb(self, fmt, rng, prim, alpha, float_out, raw, w, h):
        out = np.empty((h, w, 4 if alpha else 3), np.float32 if float_out else raw.dtype)
        self._check(self._yuv_fn("yuv_to_rgb")(fmt, rng, prim, int(alpha), int(float_out), _p(raw), raw.strides[0], w, h,
                                                _p(out), out.strides[0]))
        return out

    def yuv_crop_resize_norm_split(self, fmt, rng, prim, raw, w, h, crop, dst, div_v, quirk=0):
        out = np.empty((3, dst[1], dst[0]), np.float32)
        args = [fmt, rng, prim, _p(raw), raw.strides[0], w, h, Rect(*crop), dst[0], dst[1], float(div_v)]
        if not self.ref:
            args.append(quirk)
        self._check(self._yuv_fn("yuv_crop_resize_norm_split")(*args, _p(out)))
        return out


    # ---- BorderReader and Warping ----
    def _bw_fn(self, name):
        if self.bw is None:
            raise RuntimeError("the border / warp checker library is not built")
        return getattr(self.bw, ("fkr_" if self.ref else "fko_") + name)

    def border_index(self, border_type, i, n):
        return int(self.bw.fko_border_index(border_type, i, n))

    def border_crop_u8c3(self, border_type, src, left, top, dst, value=(0, 0, 0)):
        """src (h, w, 3) uint8 seen through BorderReader<type>, window of dst = (w, h) pixels whose origin is (-left, -top)."""
        h, w, _ = src.shape
        out = np.empty((dst[1], dst[0], 3), np.uint8)
        val = np.array(value, np.uint8)
        self._check(self._bw_fn("border_crop_u8c3")(border_type, _p(src), w, h, src.strides[0], left, top, dst[0], dst[1], _p(val),
                                                     _p(out), out.strides[0]))
        return out

    def warp_coords(self, warp_type, matrix, x, y):
        m = np.ascontiguousarray(matrix, np.float32).ravel()
        out = np.empty(2, np.float32)
        self._bw_fn("warp_coords")(warp_type, _p(m), x, y, _p(out))
        return out

    def warp_u8c3_f32c3(self, warp_type, matrix, src, dst, quirk=0):
        """matrix: 2x3 (affine) or 3x3 (perspective), destination -> source coordinates."""
        h, w, _ = src.shape
        m = np.ascontiguousarray(matrix, np.float32).ravel()
        out = np.empty((dst[1], dst[0], 3), np.float32)
        args = [warp_type, _p(m), _p(src), w, h, src.strides[0], dst[0], dst[1]]
        if not self.ref:
            args.append(quirk)
        self._check(self._bw_fn("warp_u8c3_f32c3")(*args, _p(out), out.strides[0]))
        return out


    def deinterlace_u8c3_f32c3(self, kind, use_even_lines, src):
        h, w, _ = src.shape
        out = np.empty((h, w, 3), np.float32)
        self._check(self._bw_fn("deinterlace_u8c3_f32c3")(kind, int(use_even_lines), _p(src), w, h, src.strides[0], _p(out), out.strides[0]))
        return out

    # ---- tensor layouts, circular reads, CircularTensor::update ----
    def _circ_fn(self, name):
        if self.circ is None:
            raise RuntimeError("the circular checker library is not built")
        return getattr(self.circ, ("fkr_" if self.ref else "fko_") + name)

    def tensor_relayout_f32c3(self, mode, src, w, h, planes):
        """src / result are flat float32 arrays of planes*h*w*3 elements in the layouts the mode names."""
        src = np.ascontiguousarray(src, np.float32)
        out = np.empty(planes * h * w * 3, np.float32)
        self._check(self._circ_fn("tensor_relayout_f32c3")(mode, _p(src), w, h, planes, _p(out)))
        return out

    def circular_tensor_read_f32c3(self, direction, first, ring):
        """ring: (planes, h, w, 3) float32 -> same shape, planes in logical order."""
        planes, h, w, _ = ring.shape
        out = np.empty_like(ring)
        self._check(self._circ_fn("circular_tensor_read_f32c3")(direction, first, _p(ring), w, h, planes, _p(out)))
        return out

    def circular_tensor_update_u8c3_split_f32(self, frame, mul_v, tensor, ring, next_index, newest_first):
        """Updates tensor and ring, both (batch, 3, h, w) float32, in place."""
        h, w, _ = frame.shape
        self._check(self.circ.fko_circular_tensor_update_u8c3_split_f32(_p(frame), w, h, frame.strides[0], float(mul_v), _p(tensor), _p(ring),
                                                                       tensor.shape[0], next_index, int(newest_first)))

    # ---- conditional batches, a write in the middle of a chain, a batch of output images, a tensor as the source ----
    def _paths_fn(self, name):
        if self.paths is None:
            raise RuntimeError("the checker library of the less common chain shapes is not built")
        fn = getattr(self.paths, ("fkr_" if self.ref else "fko_") + name)
        fn.restype = C.c_int
        return fn

    @staticmethod
    def _pointers(arrays):
        return (C.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])

    def conditional_copy_u8c3(self, srcs, used, default):
        """srcs: n images (h, w, 3) uint8 of one size -> (n, h, w, 3) uint8; planes from `used` on hold `default`."""
        h, w, _ = srcs[0].shape
        out = np.empty((len(srcs), h, w, 3), np.uint8)
        d = np.asarray(default, np.uint8)
        self._check(self._paths_fn("conditional_copy_u8c3")(self._pointers(srcs), _i(w), _i(h), _sz(srcs[0].strides[0]), _i(len(srcs)), _i(used),
                                                             _p(d), _p(out)))
        return out

    def conditional_resize_f32c3(self, srcs, used, default, dst, quirk=0):
        """srcs: n images (h, w, 3) uint8 of one size -> (n, dst_h, dst_w, 3) float32; planes from `used` on hold `default`."""
        h, w, _ = srcs[0].shape
        out = np.empty((len(srcs), dst[1], dst[0], 3), np.float32)
        d = np.asarray(default, np.float32)
        args = [self._pointers(srcs), _i(w), _i(h), _sz(srcs[0].strides[0]), _i(len(srcs)), _i(used), _p(d), _i(dst[0]), _i(dst[1])]
        if not self.ref:
            args.append(_i(quirk))
        self._check(self._paths_fn("conditional_resize_f32c3")(*args, _p(out)))
        return out

    def muladd_midwrite_f32c3(self, src, mul_v, add_v):
        """src: (h, w, 3) float32 -> (mid, out)."""
        h, w, _ = src.shape
        mid, out = np.empty_like(src), np.empty_like(src)
        self._check(self._paths_fn("muladd_midwrite_f32c3")(_p(src), _i(w), _i(h), _sz(src.strides[0]), _f(mul_v), _f(add_v), _p(mid),
                                                             _sz(mid.strides[0]), _p(out), _sz(out.strides[0])))
        return mid, out

    def batch_crop_cast_images(self, src, rects):
        """src: (h, w, 3) uint8, rects of one size -> list of (rh, rw, 3) float32 images."""
        h, w, _ = src.shape
        outs = [np.empty((r[3], r[2], 3), np.float32) for r in rects]
        self._check(self._paths_fn("batch_crop_cast_images")(_p(src), _i(w), _i(h), _sz(src.strides[0]), rect_array(rects), _i(len(rects)),
                                                              self._pointers(outs), _sz(outs[0].strides[0])))
        return outs

    def batch_windows_saturate_muls_f32(self, src, rects, mul_v, sub_v, div_v):
        """src: (h, w) uint8, rects of one size -> (n, rh, rw) float32."""
        h, w = src.shape
        out = np.empty((len(rects), rects[0][3], rects[0][2]), np.float32)
        self._check(self._paths_fn("batch_windows_saturate_muls_f32")(_p(src), _i(w), _i(h), _sz(src.strides[0]), rect_array(rects), _i(len(rects)),
                                                                       _f(mul_v), _f(sub_v), _f(div_v), _p(out)))
        return out

    def tensor_mul_f32c3(self, src, mul):
        """src: (planes, h, w, 3) float32 -> same shape."""
        planes, h, w, _ = src.shape
        out = np.empty_like(src)
        self._check(self._paths_fn("tensor_mul_f32c3")(_p(src), _i(w), _i(h), _i(planes), _f3(mul), _p(out)))
        return out


_cache = {}


def oracle():
    if "o" not in _cache:
        path = os.path.join(_HERE, "libfkoracle.so")
        if not os.path.exists(path):
            build(with_reference=False)
        cdll = C.CDLL(path)
        _cache["o"] = _Lib(cdll, ref=False, yuv_cdll=cdll, bw_cdll=cdll, circ_cdll=cdll, paths_cdll=cdll)
    return _cache["o"]


def reference():
    """The reference-headers build, or None when oracle/_ref/libfkref.so has not been built."""
    if "r" not in _cache:
        path = os.path.join(_HERE, "_ref", "libfkref.so")
        yuv_path = os.path.join(_HERE, "_ref", "libfkref_yuv.so")
        yuv = C.CDLL(yuv_path) if os.path.exists(yuv_path) else None
        bw_path = os.path.join(_HERE, "_ref", "libfkref_border_warp.so")
        bw = C.CDLL(bw_path) if os.path.exists(bw_path) else None
        circ_path = os.path.join(_HERE, "_ref", "libfkref_circular.so")
        circ = C.CDLL(circ_path) if os.path.exists(circ_path) else None
        paths_path = os.path.join(_HERE, "_ref", "libfkref_paths.so")
        paths = C.CDLL(paths_path) if os.path.exists(paths_path) else None
        _cache["r"] = _Lib(C.CDLL(path), ref=True, yuv_cdll=yuv, bw_cdll=bw, circ_cdll=circ, paths_cdll=paths) if os.path.exists(path) else None
    return _cache["r"]
